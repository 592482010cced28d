"""The python extension FGMS.backend called exactly as the reference's scripts
call it (cpu-check.py:108-116, cpu-check-back.py:112-115, spconv-test.py:84-120)."""
import numpy as np
import pytest
import torch

from fgms_amd import clouds, harness
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


def script_inputs(L):
    dev_feats = torch.from_numpy(L["in_feats"]).cuda()
    dev_weights = torch.from_numpy(L["kernel"]).cuda()
    knnz = torch.from_numpy(L["knnz"])
    dev_kpos = torch.from_numpy(L["kpos"]).cuda()
    dev_imap = torch.from_numpy(L["imap"]).cuda()
    dev_omap = torch.from_numpy(L["omap"]).cuda()
    return dev_feats, dev_weights, knnz, dev_kpos, dev_imap, dev_omap


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
def test_cpu_check_flow(oracle, dtype):
    from FGMS.backend import fgms_fwd_cuda, fgms_fusion_fwd_cuda, fgms_bwd_cuda
    rng = np.random.default_rng(30)
    vox = clouds.dedup(np.concatenate([clouds._patch(rng, np.array([10., 10, 10]), 8, 8, False),
                                       clouds._sphere_shell(rng, np.array([10., 10, 10]), 6.0, 2000)]), 20)
    imap, omap, knnz_np, kpos = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(3), skip_offset=13)
    L = clouds.make_layer(rng, imap, omap, knnz_np, kpos, len(vox), len(vox), 16, 16, dtype)
    dev_feats, dev_weights, knnz, dev_kpos, dev_imap, dev_omap = script_inputs(L)
    out_nnz = in_nnz = len(vox)
    separate_mid = in_nnz == out_nnz
    arch80 = True
    dev_qkpos, qsum_nnz = harness.kpos_quantized(knnz, dev_kpos, dev_weights.shape[0], 256)
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], knnz_np, imap, omap, out_nnz, precompute=True)
    mode = "fp16" if dtype == np.float16 else "tf32"
    for fusion in (False, True):
        dev_output = torch.zeros((out_nnz, 16), dtype=dev_feats.dtype, device=dev_feats.device)
        with torch.no_grad():
            if not fusion:
                fgms_fwd_cuda(dev_feats, dev_weights, len(imap), dev_output, knnz.cpu(), dev_kpos,
                              dev_imap, dev_omap, separate_mid, arch80)
            else:
                fgms_fusion_fwd_cuda(dev_feats, dev_weights, qsum_nnz, dev_output, dev_kpos, dev_qkpos,
                                     dev_imap, dev_omap, separate_mid, arch80)
        output = dev_output.clone().cpu()
        G.assert_close(output.numpy(), ref, mode, "fusion=%s" % fusion)
        assert torch.allclose(output.double(), torch.from_numpy(ref), rtol=1e-2, atol=1e-2 if dtype == np.float16 else 1e-4)
    # backward, cpu-check-back.py:100-115
    dev_out_grad = torch.from_numpy(L["out_grad"]).cuda()
    dev_weight_grad = torch.zeros_like(dev_weights)
    dev_in_grad = torch.zeros((in_nnz, 16), dtype=dev_feats.dtype, device=dev_feats.device)
    with torch.no_grad():
        fgms_bwd_cuda(dev_out_grad, dev_feats, dev_weights, qsum_nnz, dev_in_grad, dev_weight_grad,
                      dev_kpos, dev_qkpos, dev_imap, dev_omap, False, False)
    G.assert_close(dev_in_grad.cpu().numpy(), oracle.np_dgrad(L["out_grad"], L["kernel"], knnz_np, imap, omap, in_nnz), mode)
    G.assert_close(dev_weight_grad.cpu().numpy(), oracle.np_wgrad(L["in_feats"], L["out_grad"], knnz_np, imap, omap, 27), mode)


def test_spconv_test_flow_with_remove_mid(oracle):
    """spconv-test.py:84-88: the identity pairs are spliced into the map and the
    timing loop calls the fused entry point repeatedly on the same output."""
    import FGMS.backend as be
    rng = np.random.default_rng(31)
    vox = clouds.dedup(clouds._sphere_shell(rng, np.array([12., 12, 12]), 8.0, 6000), 24)
    imap, omap, knnz_np, kpos = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(3), skip_offset=13)
    n = len(vox)
    knnz = torch.from_numpy(knnz_np.copy())
    dev_kpos = torch.from_numpy(kpos).cuda()
    dev_qkpos, qsum, dev_kpos, dev_imap, dev_omap = harness.remove_mid(
        n, knnz, dev_kpos, 27, 256, torch.from_numpy(imap).cuda(), torch.from_numpy(omap).cuda())
    x = torch.rand((n, 64), dtype=torch.half, device="cuda")
    w = torch.rand((27, 64, 64), dtype=torch.half, device="cuda")
    out = torch.zeros((n, 64), dtype=torch.half, device="cuda")
    be.fgms_plan_cache_clear()
    for _ in range(3):
        be.fgms_fusion_fwd_cuda(x, w, qsum, out, dev_kpos, dev_qkpos, dev_imap, dev_omap, False, True)
    torch.cuda.synchronize()
    assert be.fgms_plan_cache_size() == 1
    ref = 3 * oracle.np_fwd(x.cpu().numpy(), w.cpu().numpy(), knnz.numpy(), dev_imap.cpu().numpy(),
                            dev_omap.cpu().numpy(), n)
    G.assert_close(out.cpu().numpy(), ref, "fp16")


def test_plan_cache_follows_in_place_edits(oracle):
    import FGMS.backend as be
    rng = np.random.default_rng(32)
    vox = clouds.dedup(clouds._sphere_shell(rng, np.array([8., 8, 8]), 5.0, 3000), 16)
    L = clouds.submanifold_case(vox, 32, 32, np.float32, rng)
    x, w, knnz, kpos, imap, omap = script_inputs(L)
    be.fgms_plan_cache_clear()
    out = torch.zeros(L["n_out"], 32, device="cuda")
    be.fgms_fusion_fwd_cuda(x, w, 0, out, kpos, kpos, imap, omap, False, False)
    G.assert_close(out.cpu().numpy(), oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"]), "fp32")
    # rewrite the map in place: same tensors, different pairs
    perm = torch.randperm(L["n_in"], device="cuda").int()
    imap.copy_(perm[imap.long()])
    out.zero_()
    be.fgms_fusion_fwd_cuda(x, w, 0, out, kpos, kpos, imap, omap, False, False)
    G.assert_close(out.cpu().numpy(), oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], imap.cpu().numpy(), L["omap"], L["n_out"]), "fp32")
    assert be.fgms_plan_cache_size() == 1
    be.fgms_plan_cache(False)
    out.zero_()
    be.fgms_fusion_fwd_cuda(x, w, 0, out, kpos, kpos, imap, omap, False, False)
    assert be.fgms_plan_cache_size() == 0
    be.fgms_plan_cache(True)


def test_non_default_stream(oracle):
    import FGMS.backend as be
    rng = np.random.default_rng(33)
    vox = clouds.dedup(clouds._sphere_shell(rng, np.array([8., 8, 8]), 5.0, 3000), 16)
    L = clouds.submanifold_case(vox, 64, 64, np.float16, rng)
    x, w, knnz, kpos, imap, omap = script_inputs(L)
    out = torch.zeros(L["n_out"], 64, device="cuda", dtype=torch.half)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        be.fgms_fusion_fwd_cuda(x, w, 0, out, kpos, kpos, imap, omap, False, False)
    s.synchronize()
    G.assert_close(out.cpu().numpy(), oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"]), "fp16")


def test_calls_can_be_captured_in_a_hip_graph(oracle):
    """After one eager call (workspaces and the cached plan exist), forward and backward
    record into a HIP graph: the library issues kernels only, no allocation, no memset, no
    synchronisation.  Every replay, with eager work in between, must reproduce the eager result."""
    import FGMS.backend as B
    rng = np.random.default_rng(7)
    vox = clouds.dedup(clouds._sphere_shell(rng, np.array([8., 8, 8]), 5.0, 3000), 16)
    L = clouds.submanifold_case(vox, 64, 64, np.float16, rng)
    D = G.to_dev(L)
    qkpos, qsum = harness.kpos_quantized(D["knnz_host"], D["kpos"], L["k_vol"], 256)
    out = torch.zeros(L["n_out"], 64, dtype=torch.float16, device="cuda")
    gi = torch.zeros(L["n_in"], 64, dtype=torch.float16, device="cuda")
    gw = torch.zeros_like(D["kernel"])

    def run():
        out.zero_(); gi.zero_(); gw.zero_()
        B.fgms_fusion_fwd_cuda(D["in_feats"], D["kernel"], qsum, out, D["kpos"], qkpos, D["imap"], D["omap"], False, False)
        B.fgms_bwd_cuda(D["out_grad"], D["in_feats"], D["kernel"], qsum, gi, gw, D["kpos"], qkpos,
                        D["imap"], D["omap"], False, False)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):          # warm-up on the capture stream: plan, workspaces
        run()
    torch.cuda.synchronize()
    want = [t.clone() for t in (out, gi, gw)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run()
    for _ in range(3):
        out.fill_(7); gi.fill_(7); gw.fill_(7)          # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want[0]) and torch.equal(gi, want[1])
        # the weight gradient sums its workgroups' partial tiles with fp32 atomics, whose order
        # is not fixed: equal up to the rounding of that sum
        G.assert_close(gw.cpu().numpy(), want[2].float().cpu().numpy(), "fp16", "replayed weight gradient")
