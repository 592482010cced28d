"""FGMS.nn: the autograd Function / Module over FGMS.backend, against torch's own autograd
through the index_add formulation of the same convolution (float64 on the GPU)."""
import numpy as np
import pytest
import torch

from fgms_amd import clouds
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


def reference(x, w, kmap):
    out = torch.zeros(kmap.n_out, w.shape[2], dtype=torch.float64, device=x.device)
    kpos = kmap.kpos.cpu().tolist()
    for k in range(kmap.k_vol):
        i, o = kmap.in_map[kpos[k]:kpos[k + 1]].long(), kmap.out_map[kpos[k]:kpos[k + 1]].long()
        out.index_add_(0, o, x[i] @ w[k])
    return out


def small_layer(seed, c_in, c_out, dtype, strided=False):
    rng = np.random.default_rng(seed)
    pts = np.concatenate([clouds._patch(rng, rng.uniform(6, 18, 3), 9, 9, oblique=False),
                          clouds._sphere_shell(rng, np.array([12., 12, 12]), 7.0, 2500)])
    vox = clouds.dedup(pts, 24)
    if not strided:
        return clouds.submanifold_case(vox, c_in, c_out, dtype, rng)
    coarse = clouds.downsample_coords(vox, 2)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, coarse, clouds.offsets_cube(2), 2)
    return clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(coarse), c_in, c_out, dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("strided", [False, True], ids=["submanifold", "stride2"])
def test_function_matches_torch_autograd(dtype, strided):
    from FGMS import nn as fnn
    L = small_layer(41, 64, 32, dtype, strided)
    D = G.to_dev(L)
    kmap = fnn.KernelMap(D["imap"], D["omap"], L["knnz"], L["n_in"], L["n_out"])
    x = D["in_feats"].clone().requires_grad_(True)
    w = D["kernel"].clone().requires_grad_(True)
    y = fnn.sparse_conv(x, w, kmap)
    (y.float() * D["out_grad"].float()).sum().backward()

    x64 = D["in_feats"].double().requires_grad_(True)
    w64 = D["kernel"].double().requires_grad_(True)
    y64 = reference(x64, w64, kmap)
    (y64 * D["out_grad"].double()).sum().backward()
    mode = G.mode_of(dtype)
    G.assert_close(y.detach().cpu().numpy(), y64.detach().cpu().numpy(), mode, "forward")
    G.assert_close(x.grad.cpu().numpy(), x64.grad.cpu().numpy(), mode, "grad feats")
    G.assert_close(w.grad.cpu().numpy(), w64.grad.cpu().numpy(), mode, "grad weight")

    # the transposed map runs the same pairs backwards: its forward is the input gradient
    yt = fnn.sparse_conv(D["out_grad"], w.detach().transpose(1, 2).contiguous(), kmap.transposed())
    G.assert_close(yt.cpu().numpy(), x64.grad.cpu().numpy(), mode, "transposed forward")


def test_module_trains():
    from FGMS import nn as fnn
    torch.manual_seed(0)
    L = small_layer(42, 16, 32, np.float32)
    D = G.to_dev(L)
    kmap = fnn.KernelMap(D["imap"], D["omap"], L["knnz"], L["n_in"], L["n_out"])
    l1 = fnn.SparseConv(16, 32, 27, bias=True, device="cuda")
    l2 = fnn.SparseConv(32, 8, 27, device="cuda")
    target = torch.randn(L["n_out"], 8, device="cuda")
    opt = torch.optim.SGD(list(l1.parameters()) + list(l2.parameters()), lr=0.05)
    losses = []
    for _ in range(8):
        opt.zero_grad()
        y = l2(torch.relu(l1(D["in_feats"], kmap)), kmap)     # both layers share the map and its plan
        loss = ((y - target) ** 2).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < losses[0] and all(np.isfinite(losses))
    from FGMS import backend
    assert backend.fgms_plan_cache_size() >= 1


def test_kernel_map_from_coordinates():
    from FGMS import nn as fnn
    rng = np.random.default_rng(43)
    vox = clouds.dedup(clouds._sphere_shell(rng, np.array([12., 12, 12]), 7.0, 2500), 24)
    want = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(3))
    kmap = fnn.KernelMap.from_coords(torch.from_numpy(vox).cuda(), torch.from_numpy(vox).cuda(),
                                     clouds.offsets_cube(3))
    assert np.array_equal(kmap.in_map.cpu().numpy(), want[0])
    assert np.array_equal(kmap.out_map.cpu().numpy(), want[1])
    assert np.array_equal(kmap.kernel_nnz.numpy(), want[2])
    y = fnn.sparse_conv(torch.randn(len(vox), 32, device="cuda"), torch.randn(27, 32, 32, device="cuda"), kmap)
    assert y.shape == (len(vox), 32) and torch.isfinite(y).all()


def test_kernel_map_checks_its_sizes():
    from FGMS import nn as fnn
    e = torch.zeros(5, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        fnn.KernelMap(e, e, [2, 2], 10, 10)          # 4 != 5 pairs
    kmap = fnn.KernelMap(e, e, [2, 3], 10, 10)
    with pytest.raises(ValueError):
        fnn.sparse_conv(torch.zeros(9, 4, device="cuda"), torch.zeros(2, 4, 4, device="cuda"), kmap)
