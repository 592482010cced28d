"""fgms_wgrad_static: the weight gradient through the entry point that allocates nothing,
against fgms_wgrad on the same inputs, two calls in a row, the second on a smaller input
(the static accumulator keeps what the first call left behind)."""
import numpy as np
import pytest
import torch

from fgms_amd import clouds
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    from fgms_amd import capi as c
    c.lib()
    assert torch.cuda.is_available()
    c.set_kernel_policy(0)
    return c


def layer(n_vox, c_in, c_out, dtype, seed):
    rng = np.random.default_rng(seed)
    vox = clouds.cloud_indoor(clouds.rng_for(2), target=n_vox)
    return clouds.submanifold_case(vox, c_in, c_out, dtype, rng)


@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["fp16", "fp32"])
@pytest.mark.parametrize("with_plan", [True, False], ids=["plan", "no-plan"])
def test_static_weight_gradient_matches_fgms_wgrad(capi, oracle, dtype, with_plan):
    mode = G.mode_of(dtype)
    # the second call is smaller in rows, pairs AND accumulator size
    for n_vox, c_in, c_out, seed in ((30000, 64, 64, 5), (6000, 32, 64, 6)):
        L = layer(n_vox, c_in, c_out, dtype, seed)
        D = G.to_dev(L)
        plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"]) if with_plan else None
        want = torch.zeros_like(D["kernel"])
        capi.wgrad(D["in_feats"], D["out_grad"], want, D["kpos"], D["imap"], D["omap"], plan=plan)
        got = torch.zeros_like(D["kernel"])
        capi.wgrad_static(D["in_feats"], D["out_grad"], got, D["kpos"], D["imap"], D["omap"], plan=plan)
        torch.cuda.synchronize()
        G.assert_close(got.cpu().numpy(), want.cpu().numpy(), mode, "static vs fgms_wgrad (%d voxels)" % n_vox)
        ref = oracle.np_wgrad(L["in_feats"], L["out_grad"], L["knnz"], L["imap"], L["omap"], L["k_vol"])
        G.assert_close(got.cpu().numpy(), ref, mode, "static vs oracle (%d voxels)" % n_vox)
        if plan is not None:
            plan.close()


def test_static_weight_gradient_accumulates_and_rejects(capi):
    L = layer(6000, 32, 32, np.float16, 9)
    D = G.to_dev(L)
    base = torch.full_like(D["kernel"], 0.25)
    got = base.clone()
    capi.wgrad_static(D["in_feats"], D["out_grad"], got, D["kpos"], D["imap"], D["omap"])
    want = base.clone()
    capi.wgrad(D["in_feats"], D["out_grad"], want, D["kpos"], D["imap"], D["omap"])
    torch.cuda.synchronize()
    G.assert_close(got.cpu().numpy(), want.cpu().numpy(), "fp16", "accumulation on top of a non-zero tensor")
    # beyond the static accumulator: 27 x 512 x 256 floats > 2 Mi
    big_w = torch.zeros(27, 512, 256, dtype=torch.float16, device="cuda")
    x = torch.zeros(D["n_in"], 512, dtype=torch.float16, device="cuda")
    g = torch.zeros(D["n_out"], 256, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError, match="static accumulator"):
        capi.wgrad_static(x, g, big_w, D["kpos"], D["imap"], D["omap"])
    # a shape without an MFMA / skinny kernel is refused, not routed to a kernel that allocates
    odd_w = torch.zeros(27, 24, 40, dtype=torch.float16, device="cuda")
    x = torch.zeros(D["n_in"], 24, dtype=torch.float16, device="cuda")
    g = torch.zeros(D["n_out"], 40, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError, match="only the shapes"):
        capi.wgrad_static(x, g, odd_w, D["kpos"], D["imap"], D["omap"])


def test_static_weight_gradient_allocates_nothing(capi):
    """The entry point's defining property: no device or pinned allocation, also when it is
    the first call to see a fresh plan of a strided (sparse) map -- taking that plan's build
    results would wait for the build and may allocate its pair view, so the call does without."""
    rng = np.random.default_rng(12)
    vin = clouds.cloud_indoor(clouds.rng_for(2), target=20000)
    vout = clouds.downsample_coords(vin, 2)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vin, vout, clouds.offsets_cube(2), stride=2)
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vin), len(vout), 64, 128, np.float16)
    D = G.to_dev(L)
    got = torch.zeros_like(D["kernel"])
    capi.wgrad_static(D["in_feats"], D["out_grad"], got, D["kpos"], D["imap"], D["omap"])       # warm-up: symbol address, LDS limits
    torch.cuda.synchronize()
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])                  # (the build allocates; the call below must not)
    torch.cuda.synchronize()
    before, free_before = capi.allocation_count(), torch.cuda.mem_get_info()[0]
    for _ in range(3):
        got.zero_()
        capi.wgrad_static(D["in_feats"], D["out_grad"], got, D["kpos"], D["imap"], D["omap"], plan=plan)
    torch.cuda.synchronize()
    assert capi.allocation_count() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    want = torch.zeros_like(D["kernel"])
    capi.wgrad(D["in_feats"], D["out_grad"], want, D["kpos"], D["imap"], D["omap"], plan=plan)
    torch.cuda.synchronize()
    G.assert_close(got.cpu().numpy(), want.cpu().numpy(), "fp16", "static (fresh plan of a strided map) vs fgms_wgrad")
    plan.close()
