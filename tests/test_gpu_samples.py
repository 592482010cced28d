"""Layer samples in the reference's on-disk format, replayed through FGMS.backend the way
the reference's scripts do (cpu-check.py:83-127 for checked samples, spconv-test.py:62-122
for timed ones) and checked against the CPU oracle."""
import numpy as np
import pytest
import torch

from fgms_amd import clouds, samples
from fgms_amd.harness import kpos_quantized
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


def layer(seed, c_in, c_out, dtype, kind="subm"):
    rng = np.random.default_rng(seed)
    vox = clouds.dedup(rng.integers(0, 20, size=(2500, 3)), 20)
    if kind == "subm":
        return clouds.submanifold_case(vox, c_in, c_out, dtype, rng)
    coarse = clouds.downsample_coords(vox, 2)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, coarse, clouds.offsets_cube(2), 2)
    return clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(coarse), c_in, c_out, dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("fusion", [True, False], ids=["fused", "seq"])
def test_checked_sample_through_the_backend(tmp_path, oracle, dtype, fusion):
    from FGMS import backend
    L = layer(41, 32, 64, dtype)
    f = tmp_path / "checked.pt"
    samples.save_sample(f, L)
    s = samples.load_sample(f, device="cuda")
    out = torch.zeros((s.n_out, s.c_out), dtype=s.in_feats.dtype, device="cuda")
    qkpos, qsum = kpos_quantized(s.knnz, s.kpos, s.k_vol, 256)
    if fusion:
        backend.fgms_fusion_fwd_cuda(s.in_feats, s.kernel, qsum, out, s.kpos, qkpos, s.imap, s.omap, False, False)
    else:
        backend.fgms_fwd_cuda(s.in_feats, s.kernel, s.sum_nnz, out, s.knnz, s.kpos, s.imap, s.omap, False, False)
    torch.cuda.synchronize()
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    G.assert_close(out.cpu().numpy(), ref, G.mode_of(L["in_feats"].dtype, False), "fwd from a sample file")


@pytest.mark.parametrize("kind", ["subm", "down"])
def test_timed_sample_replay(tmp_path, oracle, kind):
    """The timing protocol: random tensors, and for a submanifold layer (whose dumps leave
    the centre offset empty) the identity pairs spliced in before the call."""
    L = layer(43, 64, 64, np.float16, kind)
    if kind == "subm":          # drop the centre pairs, as the reference's real samples have them
        mid = L["k_vol"] // 2
        a, b = int(L["kpos"][mid]), int(L["kpos"][mid + 1])
        L["imap"] = np.concatenate([L["imap"][:a], L["imap"][b:]])
        L["omap"] = np.concatenate([L["omap"][:a], L["omap"][b:]])
        L["knnz"] = L["knnz"].copy()
        L["knnz"][mid] = 0
        L["kpos"] = np.concatenate([[0], np.cumsum(L["knnz"])]).astype(np.int32)
    f = tmp_path / "timed.pt"
    samples.save_sample(f, L, with_tensors=False)
    s = samples.load_sample(f, device="cuda")
    ms, out, feats, weights = samples.replay(s, dtype=torch.float16, warmup=2, steps=5, return_inputs=True)
    assert ms > 0
    # the oracle on the same random tensors, centre offset included for the submanifold layer
    knnz, imap, omap = L["knnz"].copy(), L["imap"], L["omap"]
    if kind == "subm":
        mid = L["k_vol"] // 2
        a = int(L["kpos"][mid])
        ident = np.arange(L["n_in"], dtype=np.int32)
        imap = np.concatenate([imap[:a], ident, imap[a:]])
        omap = np.concatenate([omap[:a], ident, omap[a:]])
        knnz[mid] = L["n_in"]
    ref = oracle.np_fwd(feats.cpu().numpy(), weights.cpu().numpy(), knnz, imap, omap, L["n_out"])
    G.assert_close(out.cpu().numpy(), ref, "fp16", "replayed forward")
