"""The plan as an object: asynchronous build, transposed views that share a plan's tables,
the python extension's cache recognising a swapped map, HIP-graph capture that includes the
first call on a map, tensors made under inference mode."""
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
    yield c
    c.set_kernel_policy(0)


def strided_layers(dtype=np.float16, n=20000, c_in=64, c_out=128):
    rng = np.random.default_rng(31)
    vin = clouds.cloud_indoor(clouds.rng_for(2), target=n)
    vout = clouds.downsample_coords(vin, 2)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vin, vout, clouds.offsets_cube(2), stride=2)
    down = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vin), len(vout), c_in, c_out, dtype)
    up = clouds.make_layer(rng, omap, imap, knnz, kpos, len(vout), len(vin), c_out, c_in, dtype)
    return down, up


@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["fp16", "fp32"])
def test_transposed_view_shares_the_tables(capi, oracle, dtype):
    """The transposed convolution's map is the same pairs with the sides exchanged: a view of
    the down-sampling layer's plan serves the up-sampling layer, all three passes."""
    down, up = strided_layers(dtype)
    Dd, Du = G.to_dev(down), G.to_dev(up)
    mode = G.mode_of(dtype)
    plan = capi.Plan(Dd["kpos"], Dd["imap"], Dd["omap"], Dd["n_in"], Dd["n_out"])
    view = plan.transposed()
    assert view.usable() == plan.usable(for_dgrad=True) and view.usable(for_dgrad=True) == plan.usable()
    sv, sp = view.stats(), plan.stats()
    assert sv["pairs"] == sp["pairs"] and sv["blocks_fwd"] == sp["blocks_dgrad"] and sv["blocks_dgrad"] == sp["blocks_fwd"]
    a = (up["knnz"], up["imap"], up["omap"])
    capi.profile_reset(); capi.profile_enable(True)
    out = G.run_fwd(capi, Du, plan=view)
    gi, gw = G.run_bwd(capi, Du, plan=view)
    capi.profile_enable(False)
    names = {n for n, _ in capi.profile_records()}
    capi.profile_reset()
    assert any(n.startswith(("gms_rows_kernel", "bwd_fused_kernel")) for n in names), names
    G.assert_close(out, oracle.c_fwd(up["in_feats"], up["kernel"], *a, up["n_out"]), mode, "fwd through the view")
    G.assert_close(gi, oracle.c_dgrad(up["out_grad"], up["kernel"], *a, up["n_in"]), mode, "dgrad through the view")
    G.assert_close(gw, oracle.np_wgrad(up["in_feats"], up["out_grad"], *a, up["k_vol"]), mode, "wgrad through the view")
    # the base can go first: the tables live until the last view does
    plan.close()
    out2 = G.run_fwd(capi, Du, plan=view)
    assert np.array_equal(out, out2)
    view.close()


def test_backend_cache_shares_a_swapped_map(oracle):
    import FGMS.backend as B
    import FGMS.nn as fnn
    down, up = strided_layers()
    Dd = G.to_dev(down)
    B.fgms_plan_cache_clear()
    made = B.fgms_plan_cache_views()
    kmap = fnn.KernelMap(Dd["imap"], Dd["omap"], down["knnz"], Dd["n_in"], Dd["n_out"])
    x = torch.from_numpy(down["in_feats"]).cuda()
    wd = torch.from_numpy(down["kernel"]).cuda()
    wu = torch.from_numpy(up["kernel"]).cuda()
    y = fnn.sparse_conv(x, wd, kmap)
    z = fnn.sparse_conv(y, wu, kmap.transposed())
    torch.cuda.synchronize()
    assert B.fgms_plan_cache_size() == 2 and B.fgms_plan_cache_views() == made + 1
    a = (down["knnz"], down["imap"], down["omap"])
    y_ref = oracle.c_fwd(down["in_feats"], down["kernel"], *a, down["n_out"])
    G.assert_close(y.cpu().numpy(), y_ref, "fp16", "down")
    z_ref = oracle.c_fwd(y.cpu().numpy(), up["kernel"], up["knnz"], up["imap"], up["omap"], up["n_out"])
    G.assert_close(z.cpu().numpy(), z_ref, "fp16", "up through the shared plan")
    B.fgms_plan_cache_clear()


def test_first_call_on_a_map_inside_a_captured_graph(oracle):
    """fgms_plan_create queues the build and returns; a call recorded into a HIP graph right
    behind it cannot wait for the build's findings, so it records the kernels that need no
    plan.  Every replay must give the oracle's result; calls after the capture use the plan."""
    import FGMS.backend as B
    rng = np.random.default_rng(8)
    vox = clouds.dedup(clouds._sphere_shell(rng, np.array([10., 10, 10]), 7.0, 6000), 20)
    L = clouds.submanifold_case(vox, 64, 64, np.float16, rng)
    D = G.to_dev(L)
    out = torch.zeros(L["n_out"], 64, dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    other = clouds.submanifold_case(vox[:2000], 64, 64, np.float16, rng)
    Do = G.to_dev(other)
    oo = torch.zeros(other["n_out"], 64, dtype=torch.float16, device="cuda")
    with torch.cuda.stream(side):      # workspaces of this shape exist before the capture (another map)
        B.fgms_fusion_fwd_cuda(Do["in_feats"], Do["kernel"], 0, oo, Do["kpos"], Do["kpos"], Do["imap"], Do["omap"], False, False)
        B.fgms_plan_cache(False)
        B.fgms_fusion_fwd_cuda(Do["in_feats"], Do["kernel"], 0, oo, Do["kpos"], Do["kpos"], Do["imap"], Do["omap"], False, False)
        B.fgms_plan_cache(True)
    torch.cuda.synchronize()
    want = oracle.c_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side, capture_error_mode="thread_local"):
        out.zero_()
        B.fgms_fusion_fwd_cuda(D["in_feats"], D["kernel"], 0, out, D["kpos"], D["kpos"], D["imap"], D["omap"], False, False)
    for _ in range(3):
        out.fill_(3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        G.assert_close(out.cpu().numpy(), want, "fp16", "replay")
    out.zero_()
    B.fgms_fusion_fwd_cuda(D["in_feats"], D["kernel"], 0, out, D["kpos"], D["kpos"], D["imap"], D["omap"], False, False)
    torch.cuda.synchronize()
    G.assert_close(out.cpu().numpy(), want, "fp16", "eager call after the capture")
    B.fgms_plan_cache_clear()


def test_inference_mode_tensors(oracle):
    import FGMS.backend as B
    rng = np.random.default_rng(9)
    vox = clouds.cloud_indoor(clouds.rng_for(2), target=3000)
    L = clouds.submanifold_case(vox, 32, 32, np.float32, rng)
    with torch.inference_mode():
        D = G.to_dev(L)
        out = torch.zeros(L["n_out"], 32, device="cuda")
        for _ in range(2):          # the second call finds the plan in the cache
            out.zero_()
            B.fgms_fusion_fwd_cuda(D["in_feats"], D["kernel"], 0, out, D["kpos"], D["kpos"], D["imap"], D["omap"], False, False)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
    G.assert_close(got, oracle.c_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"]), "fp32", "fwd")
    B.fgms_plan_cache_clear()


@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["fp16", "fp32"])
def test_more_than_64_offsets_keep_the_output_stationary_kernels(capi, oracle, dtype):
    """A 5 x 5 x 5 kernel has 125 offsets (the reference takes k_vol from kernel.size(0),
    backend/spconv.cu:44-45, without a cap): the plan cuts them into groups of 64, each with
    tables of its own, and forward / input gradient walk the groups with the kernels that
    need no atomics; the weight gradient uses the plan's row bands over all 125."""
    rng = np.random.default_rng(41)
    vox = clouds.cloud_indoor(clouds.rng_for(2), target=6000)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(5))
    assert len(knnz) == 125
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(vox), 32, 64, dtype)
    D = G.to_dev(L)
    mode = G.mode_of(dtype)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    assert plan.usable() and plan.usable(for_dgrad=True)
    assert plan.stats()["pairs"] == len(imap)
    capi.profile_reset(); capi.profile_enable(True)
    out = G.run_fwd(capi, D, plan=plan)
    gi, gw = G.run_bwd(capi, D, plan=plan)
    capi.profile_enable(False)
    names = [n for n, _ in capi.profile_records()]
    capi.profile_reset()
    assert names.count("gms_rows_kernel(fwd)") == 2 and names.count("gms_rows_kernel(dgrad)") == 2, names
    assert not any("pairs" in n or "generic" in n for n in names), names
    a = (L["knnz"], L["imap"], L["omap"])
    G.assert_close(out, oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"]), mode, "fwd")
    G.assert_close(gi, oracle.c_dgrad(L["out_grad"], L["kernel"], *a, L["n_in"]), mode, "dgrad")
    G.assert_close(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *a, L["k_vol"]), mode, "wgrad")
    # the sequential entry point and the omitted-centre form go the same way
    out_seq = G.run_fwd(capi, D, fused=False, plan=plan)
    G.assert_close(out_seq, out.astype(np.float32), mode, "seq fwd")
    plan.close()


def _two_clouds(n=6000):
    a = clouds.cloud_indoor(clouds.rng_for(2), target=n)
    b = clouds.cloud_indoor(clouds.rng_for(7), target=n)
    m = min(len(a), len(b))
    return np.ascontiguousarray(a[:m], dtype=np.int32), np.ascontiguousarray(b[:m], dtype=np.int32)


def test_rewritten_map_is_noticed_by_the_plan(capi, oracle):
    """A map rewritten through raw pointers (how a native builder fills a pre-allocated tensor)
    leaves the plan with last iteration's neighbour tables.  fgms_plan_check queues a
    fingerprint check; the call after it raises."""
    va, vb = _two_clouds()
    offs = clouds.offsets_cube(3)
    n, k_vol = len(va), len(offs)
    cap = n * k_vol
    into = (torch.empty(cap, dtype=torch.int32, device="cuda"), torch.empty(cap, dtype=torch.int32, device="cuda"),
            torch.empty(k_vol, dtype=torch.int32, device="cuda"), torch.empty(k_vol + 1, dtype=torch.int32, device="cuda"))
    ca, cb = torch.from_numpy(va).cuda(), torch.from_numpy(vb).cuda()
    imap, omap, knnz, kpos = capi.build_kernel_map(ca, ca, offs, 1, into=into)
    plan = capi.Plan(kpos, imap, omap, n, n)
    plan.check(); plan.check()
    torch.cuda.synchronize()
    plan.check()                                  # unchanged lists: nothing to report
    capi.build_kernel_map(cb, cb, offs, 1, into=into)      # same tensors, new content
    plan.check()                                  # queues the check that finds it
    torch.cuda.synchronize()
    with pytest.raises(capi.StalePlanError):
        plan.check()
    x = torch.zeros(n, 32, dtype=torch.float16, device="cuda")
    w = torch.zeros(k_vol, 32, 32, dtype=torch.float16, device="cuda")
    out = torch.zeros(n, 32, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.StalePlanError):      # every entry point refuses the plan from now on
        capi.fusion_fwd(x, w, 0, out, kpos, None, imap, omap, False, False, plan=plan)
    plan.close()
    # the same with the check carried by the forward / backward launches themselves
    g = torch.zeros(n, 32, dtype=torch.float16, device="cuda")
    gi, gw = torch.zeros_like(x), torch.zeros_like(w)
    for use in ("fwd", "bwd"):
        capi.build_kernel_map(ca, ca, offs, 1, into=into)
        plan = capi.Plan(kpos, imap, omap, n, n)

        def call():
            plan.check(with_next_launch=True)
            if use == "fwd":
                capi.fusion_fwd(x, w, 0, out, kpos, None, imap, omap, False, False, plan=plan)
            else:
                capi.bwd(g, x, w, 0, gi, gw, kpos, None, imap, omap, False, False, plan=plan)
            torch.cuda.synchronize()

        call(); call()
        capi.build_kernel_map(cb, cb, offs, 1, into=into)
        call()                                    # old tables; the launch's extra workgroup notices
        with pytest.raises(capi.StalePlanError):
            call()
        plan.close()


def test_backend_cache_drops_a_plan_whose_map_was_rewritten(capi, oracle):
    import FGMS.backend as backend
    backend.fgms_plan_cache(True)
    backend.fgms_plan_cache_clear()
    va, vb = _two_clouds()
    offs = clouds.offsets_cube(3)
    n, k_vol = len(va), len(offs)
    cap = n * k_vol
    into = (torch.empty(cap, dtype=torch.int32, device="cuda"), torch.empty(cap, dtype=torch.int32, device="cuda"),
            torch.empty(k_vol, dtype=torch.int32, device="cuda"), torch.empty(k_vol + 1, dtype=torch.int32, device="cuda"))
    rng = np.random.default_rng(3)
    x_np = rng.standard_normal((n, 32)).astype(np.float16)
    w_np = (rng.standard_normal((k_vol, 32, 32)) * 0.1).astype(np.float16)
    x, w = torch.from_numpy(x_np).cuda(), torch.from_numpy(w_np).cuda()

    def forward():
        out = torch.zeros(n, 32, dtype=torch.float16, device="cuda")
        backend.fgms_fusion_fwd_cuda(x, w, 0, out, into[3], torch.zeros_like(into[3]), into[0], into[1], False, False)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    def reference():
        kp = into[3].cpu().numpy()
        m = int(kp[-1])
        return oracle.c_fwd(x_np, w_np, into[2].cpu().numpy(), into[0][:m].cpu().numpy(), into[1][:m].cpu().numpy(), n)

    capi.build_kernel_map(torch.from_numpy(va).cuda(), torch.from_numpy(va).cuda(), offs, 1, into=into)
    G.assert_close(forward(), reference(), "fp16", "first map")
    G.assert_close(forward(), reference(), "fp16", "first map, plan from the cache")
    capi.build_kernel_map(torch.from_numpy(vb).cuda(), torch.from_numpy(vb).cuda(), offs, 1, into=into)
    forward()                                     # computes with the old tables; its check notices
    with pytest.raises(RuntimeError, match="rewritten in place"):
        forward()
    G.assert_close(forward(), reference(), "fp16", "second map, after the stale plan was dropped")
    backend.fgms_plan_cache_clear()
