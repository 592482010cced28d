"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle
on identical seeded inputs.  Tolerances: fp32 rel 1e-5, tf32 / fp16 rel 1e-2
(see gpu_util.assert_close); index handling bit-exact."""
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


def cloud(seed, n=3000, grid=24):
    rng = np.random.default_rng(seed)
    pts = np.concatenate([
        clouds._patch(rng, rng.uniform(6, 18, 3), 9, 9, oblique=False),
        clouds._patch(rng, rng.uniform(6, 18, 3), 9, 9, oblique=True),
        clouds._sphere_shell(rng, np.array([12., 12, 12]), 7.0, n),
    ])
    return clouds.dedup(pts, grid)


def layer(seed, c_in, c_out, dtype, kind="subm"):
    rng = np.random.default_rng(seed)
    vox = cloud(seed)
    if kind == "subm":
        return clouds.submanifold_case(vox, c_in, c_out, dtype, rng)
    coarse = clouds.downsample_coords(vox, 2)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, coarse, clouds.offsets_cube(2), 2)
    if kind == "down":
        return clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(coarse), c_in, c_out, dtype)
    return clouds.make_layer(rng, omap, imap, knnz, kpos, len(coarse), len(vox), c_in, c_out, dtype)


def check_all(capi, oracle, L, policy, use_plan, arch80=False):
    capi.set_kernel_policy(policy)
    D = G.to_dev(L)
    mode = G.mode_of(L["in_feats"].dtype, arch80)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"]) if use_plan else None
    args = (L["knnz"], L["imap"], L["omap"])
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], *args, L["n_out"])
    G.assert_close(G.run_fwd(capi, D, fused=True, arch80=arch80, plan=plan), ref, mode, "fused fwd")
    G.assert_close(G.run_fwd(capi, D, fused=False, arch80=arch80, plan=plan), ref, mode, "seq fwd")
    gi, gw = G.run_bwd(capi, D, plan=plan)
    bmode = mode if mode != "fp32" else "fp32"
    G.assert_close(gi, oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"]), bmode, "dgrad")
    G.assert_close(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"]), bmode, "wgrad")
    if plan is not None:
        plan.close()


SHAPES = [(32, 32), (64, 64), (16, 16), (4, 32), (3, 5), (128, 128), (64, 128), (128, 64), (48, 80), (8, 8)]


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "%dx%d" % s)
def test_submanifold_auto(capi, oracle, shape, dtype):
    L = layer(11, shape[0], shape[1], dtype)
    check_all(capi, oracle, L, policy=0, use_plan=False)
    check_all(capi, oracle, L, policy=0, use_plan=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("shape", [(32, 32), (64, 64), (3, 5), (128, 64)], ids=lambda s: "%dx%d" % s)
def test_submanifold_generic_kernels(capi, oracle, shape, dtype):
    check_all(capi, oracle, layer(12, shape[0], shape[1], dtype), policy=1, use_plan=False)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("shape", [(32, 32), (64, 64), (128, 128), (64, 128)], ids=lambda s: "%dx%d" % s)
def test_submanifold_pair_stationary_mfma(capi, oracle, shape, dtype):
    check_all(capi, oracle, layer(13, shape[0], shape[1], dtype), policy=2, use_plan=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("shape", [(128, 128), (64, 128), (256, 256), (16, 128)], ids=lambda s: "%dx%d" % s)
def test_submanifold_wide_wave_tiles(capi, oracle, shape, dtype):
    """The 128-column wave tiles of the output-stationary kernel, which the automatic
    dispatch reserves for large fp16 layers, forced on at test size."""
    check_all(capi, oracle, layer(14, shape[0], shape[1], dtype), policy=3, use_plan=True)


@pytest.mark.parametrize("use_plan", [True, False], ids=["plan", "noplan"])
@pytest.mark.parametrize("kind,shape", [("subm", (256, 256)), ("subm", (128, 256)), ("subm", (256, 512)),
                                        ("subm", (512, 256)), ("down", (128, 256)), ("up", (256, 128))])
def test_wide_pair_stationary_kernel(capi, oracle, kind, shape, use_plan):
    """The pair-stationary kernel with 256-column workgroups (fp16, a multiple of 256
    destination channels in the pass at hand), forced where the automatic dispatch would take a
    plan-driven kernel: forward of the (c, 256 n) layers, input gradient of the (256 n, c) ones,
    whole and partial 256-pair tiles, several tiles per workgroup."""
    check_all(capi, oracle, layer(31, shape[0], shape[1], np.float16, kind), policy=7, use_plan=use_plan)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("parts", [1, 2, 4])
@pytest.mark.parametrize("shape", [(4, 32), (16, 16), (64, 8)], ids=lambda s: "%dx%d" % s)
def test_skinny_layers_by_waves_per_block(capi, oracle, monkeypatch, shape, parts, dtype):
    """The skinny-channel kernel with one, two and four waves sharing a 64-row block (the
    library picks by the size of the launch; FGMS_SMALL_PARTS, read on every call, overrides)."""
    monkeypatch.setenv("FGMS_SMALL_PARTS", str(parts))
    check_all(capi, oracle, layer(17, *shape, dtype), policy=0, use_plan=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("use_plan", [True, False], ids=["plan", "noplan"])
@pytest.mark.parametrize("shape", [(4, 16), (4, 64), (8, 32), (16, 64), (16, 16)], ids=lambda s: "%dx%d" % s)
def test_skinny_weight_gradient_shapes(capi, oracle, shape, use_plan, dtype):
    """Layers with 4 / 8 / 16 input channels: forward, input gradient and the skinny
    weight-gradient kernel (lanes share a pair, four output channels each), sliced by the
    plan's row bands or, without a plan, by pair count."""
    check_all(capi, oracle, layer(29, *shape, dtype), policy=0, use_plan=use_plan)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("kind,shape", [("down", (64, 128)), ("up", (128, 64)), ("down", (16, 32)), ("up", (5, 3))])
def test_strided_and_transposed(capi, oracle, kind, shape, dtype):
    L = layer(14, shape[0], shape[1], dtype, kind)
    check_all(capi, oracle, L, policy=0, use_plan=False)
    check_all(capi, oracle, L, policy=0, use_plan=True)


def test_tf32_mode_flag(capi, oracle):
    check_all(capi, oracle, layer(15, 64, 64, np.float32), policy=0, use_plan=True, arch80=True)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "seq"])
def test_separate_mid(capi, oracle, fused, dtype):
    """Centre offset left out of the map (knnz[13] == 0) and added as a dense
    product, the form the reference's tiny samples take (cpu-check.py:100)."""
    rng = np.random.default_rng(16)
    vox = cloud(16)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(3), skip_offset=13)
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(vox), 32, 64, dtype)
    D = G.to_dev(L)
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], knnz, imap, omap, len(vox), precompute=True)
    mode = G.mode_of(dtype)
    for use_plan in (False, True):
        plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"]) if use_plan else None
        G.assert_close(G.run_fwd(capi, D, fused=fused, separate_mid=True, plan=plan), ref, mode)
    if fused:
        # the fused form overwrites (GEMM beta = 0, backend/spconv.cu:56): junk in out must vanish
        junk = torch.full((len(vox), 64), 7.0, dtype=D["in_feats"].dtype, device="cuda")
        G.assert_close(G.run_fwd(capi, D, fused=True, separate_mid=True, out_init=junk), ref, mode)


@pytest.mark.parametrize("fused", [True, False], ids=["fused", "seq"])
def test_separate_mid_wide_layer(capi, oracle, fused):
    """The same with 256 output channels in fp16: the centre product and the scattered map both
    run the pair-stationary kernel with 256-column workgroups."""
    rng = np.random.default_rng(18)
    vox = cloud(18)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(3), skip_offset=13)
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(vox), 128, 256, np.float16)
    D = G.to_dev(L)
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], knnz, imap, omap, len(vox), precompute=True)
    capi.set_kernel_policy(0)
    G.assert_close(G.run_fwd(capi, D, fused=fused, separate_mid=True, plan=None), ref, "fp16")
    if fused:
        junk = torch.full((len(vox), 256), 7.0, dtype=D["in_feats"].dtype, device="cuda")
        G.assert_close(G.run_fwd(capi, D, fused=True, separate_mid=True, out_init=junk), ref, "fp16")


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
def test_accumulates_in_place(capi, oracle, dtype):
    L = layer(17, 32, 32, dtype)
    D = G.to_dev(L)
    base = torch.randn(D["n_out"], 32, device="cuda").to(D["in_feats"].dtype)
    ref = base.float().cpu().numpy().astype(np.float64) + oracle.np_fwd(
        L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    for use_plan in (False, True):
        plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"]) if use_plan else None
        G.assert_close(G.run_fwd(capi, D, plan=plan, out_init=base), ref, G.mode_of(dtype))


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
def test_index_handling_bit_exact(capi, dtype):
    """W[k] = identity and every output row hit by exactly one pair: the result
    is a permutation copy, so any index slip shows as a bit difference."""
    rng = np.random.default_rng(18)
    n_in, n_out, c, k_vol = 5000, 4000, 64, 8
    knnz = np.array([0, 700, 1, 0, 2000, 255, 257, 787], np.int32)
    kpos = np.concatenate([[0], np.cumsum(knnz)]).astype(np.int32)
    omap = rng.permutation(n_out).astype(np.int32)
    imap = rng.integers(0, n_in, n_out).astype(np.int32)
    x = rng.standard_normal((n_in, c)).astype(dtype)
    w = np.broadcast_to(np.eye(c, dtype=dtype), (k_vol, c, c)).copy()
    D = dict(in_feats=torch.from_numpy(x).cuda(), kernel=torch.from_numpy(w).cuda(),
             kpos=torch.from_numpy(kpos).cuda(), imap=torch.from_numpy(imap).cuda(),
             omap=torch.from_numpy(omap).cuda(), n_in=n_in, n_out=n_out, c_in=c, c_out=c,
             knnz_host=torch.from_numpy(knnz))
    want = np.zeros((n_out, c), dtype)
    want[omap] = x[imap]
    for policy in (0, 1, 2):
        capi.set_kernel_policy(policy)
        for use_plan in (False, True):
            plan = capi.Plan(D["kpos"], D["imap"], D["omap"], n_in, n_out) if use_plan else None
            for fused in (True, False):
                got = G.run_fwd(capi, D, fused=fused, plan=plan)
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (policy, use_plan, fused)
    capi.set_kernel_policy(0)


def test_duplicate_rows_inside_an_offset(capi, oracle):
    """Not a sparse-conv map (an offset hits one output row twice): the plan
    reports itself unusable and the atomic kernels still give the right sums."""
    rng = np.random.default_rng(19)
    n_in, n_out, k_vol = 900, 300, 3
    knnz = np.array([500, 0, 700], np.int32)
    kpos = np.concatenate([[0], np.cumsum(knnz)]).astype(np.int32)
    imap = rng.integers(0, n_in, 1200).astype(np.int32)
    omap = rng.integers(0, n_out, 1200).astype(np.int32)
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, n_in, n_out, 64, 64, np.float32)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], n_in, n_out)
    assert not plan.usable(False) and not plan.usable(True)
    G.assert_close(G.run_fwd(capi, D, plan=plan), oracle.np_fwd(L["in_feats"], L["kernel"], knnz, imap, omap, n_out), "fp32")
    gi, gw = G.run_bwd(capi, D, plan=plan)
    G.assert_close(gi, oracle.np_dgrad(L["out_grad"], L["kernel"], knnz, imap, omap, n_in), "fp32")
    G.assert_close(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], knnz, imap, omap, k_vol), "fp32")


def test_out_of_range_map_is_rejected_by_plan(capi):
    kpos = torch.tensor([0, 2, 4], dtype=torch.int32, device="cuda")
    imap = torch.tensor([0, 1, 2, 99], dtype=torch.int32, device="cuda")
    omap = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device="cuda")
    # the build is asynchronous: the plan is handed out at once, what the build found is
    # known (and reported) when the plan is first asked about or used
    plan = capi.Plan(kpos, imap, omap, 10, 10)
    assert not plan.usable() and not plan.usable(for_dgrad=True)
    x = torch.zeros(10, 32, device="cuda")
    w = torch.zeros(2, 32, 32, device="cuda")
    out = torch.zeros(10, 32, device="cuda")
    with pytest.raises(ValueError, match="outside"):
        capi.fusion_fwd(x, w, 0, out, kpos, None, imap, omap, False, False, plan=plan)
    with pytest.raises(ValueError, match="outside"):
        plan.stats()
    plan.close()


def test_empty_inputs(capi):
    for dtype in (torch.float32, torch.float16):
        x = torch.randn(10, 32, device="cuda").to(dtype)
        w = torch.randn(27, 32, 32, device="cuda").to(dtype)
        out = torch.zeros(10, 32, device="cuda", dtype=dtype)
        kpos = torch.zeros(28, dtype=torch.int32, device="cuda")
        e = torch.zeros(0, dtype=torch.int32, device="cuda")
        capi.fusion_fwd(x, w, 0, out, kpos, kpos, e, e, False, False)
        capi.seq_fwd(x, w, 0, out, torch.zeros(27, dtype=torch.int32), kpos, e, e, False, False)
        gi, gw = torch.zeros_like(x), torch.zeros_like(w)
        capi.bwd(out, x, w, 0, gi, gw, kpos, kpos, e, e, False, False)
        plan = capi.Plan(kpos, e, e, 10, 10)
        capi.fusion_fwd(x, w, 0, out, kpos, kpos, e, e, False, False, plan=plan)
        torch.cuda.synchronize()
        assert not out.any() and not gi.any() and not gw.any()
    with pytest.raises(ValueError):
        capi.fusion_fwd(x, w[:, :16], 0, out, kpos, kpos, e, e, False, False)


@pytest.mark.parametrize("cfg,variant", [(1, None), (3, None), (4, None), (4, "up"), (5, "skinny"), (5, "wide")])
def test_baseline_configs_scaled(capi, oracle, cfg, variant):
    """The benchmark configurations at a size the oracle finishes in seconds."""
    L = clouds.config_case(cfg, variant, scale=0.08 if cfg != 1 else 0.5)
    check_all(capi, oracle, L, policy=0, use_plan=True)
    check_all(capi, oracle, L, policy=0, use_plan=False)


@pytest.mark.parametrize("dtype,arch80", [(np.float32, False), (np.float32, True), (np.float16, False)],
                         ids=["fp32", "fp32-tf32-mode", "fp16"])
@pytest.mark.parametrize("shape", [(32, 32), (64, 64), (128, 128), (64, 128), (256, 256), (96, 32)], ids=lambda s: "%dx%d" % s)
def test_pair_view(capi, oracle, shape, dtype, arch80):
    """Policy 5: forward and input gradient run the output-stationary kernel over the plan's
    pair view (pair lists padded per offset to whole 64-row blocks, atomic sums); dense
    submanifold map, strided map and a map with empty offsets."""
    capi.set_kernel_policy(5)
    try:
        L = layer(14, shape[0], shape[1], dtype)
        D = G.to_dev(L)
        plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
        capi.profile_reset()
        capi.profile_enable(True)
        G.run_fwd(capi, D, fused=True, arch80=arch80, plan=plan)
        G.run_bwd(capi, D, plan=plan, arch80=arch80)
        torch.cuda.synchronize()
        capi.profile_enable(False)
        names = [n for n, _ in capi.profile_records()]
        capi.profile_reset()
        plan.close()
        assert any("pair view" in n and "fwd" in n for n in names), names
        assert any("pair view" in n and "dgrad" in n for n in names), names
        check_all(capi, oracle, L, policy=5, use_plan=True, arch80=arch80)
        if shape == (64, 128):
            check_all(capi, oracle, clouds.config_case(4, None, scale=0.08), policy=5, use_plan=True)
            check_all(capi, oracle, clouds.config_case(4, "up", scale=0.08), policy=5, use_plan=True)
            check_all(capi, oracle, clouds.config_case(3, None, scale=0.05), policy=5, use_plan=True)
    finally:
        capi.set_kernel_policy(0)


def test_plan_stats(capi):
    """fgms_plan_stats against a count in numpy: pairs, and the (64-row block, offset)
    combinations in use, which lie between pairs / 64 (and the number of offsets in use) and
    the pair count (and blocks x offsets)."""
    L = layer(15, 32, 32, np.float32)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    st = plan.stats()
    plan.close()
    assert st["pairs"] == len(L["imap"])
    floor = max(-(-len(L["imap"]) // 64), int((L["knnz"] > 0).sum()))
    assert floor <= st["blocks_fwd"] <= min(len(L["imap"]), -(-L["n_out"] // 64) * L["k_vol"])
    assert floor <= st["blocks_dgrad"] <= min(len(L["imap"]), -(-L["n_in"] // 64) * L["k_vol"])
    assert st["pair_view_rows"] % 256 == 0


@pytest.mark.parametrize("dtype", ["wide", "wide-fp32"], ids=["fp16", "fp32"])
def test_scattered_wide_layer_takes_the_pair_stationary_kernel(capi, oracle, dtype):
    """A 256 -> 256 layer over a scattered cloud (few pairs per 64-row block and offset):
    automatic dispatch weighs the empty row slots of the output-stationary kernel against
    the atomics of the pair-stationary one and picks the latter; a dense 64 -> 64 layer
    stays output-stationary.  Results against the oracle either way."""
    L = clouds.config_case(5, dtype, scale=0.08)
    D = G.to_dev(L)
    capi.set_kernel_policy(0)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    capi.profile_reset()
    capi.profile_enable(True)
    out = G.run_fwd(capi, D, fused=True, plan=plan)
    torch.cuda.synchronize()
    capi.profile_enable(False)
    names = [n for n, _ in capi.profile_records()]
    capi.profile_reset()
    plan.close()
    # (fp16: the pair-stationary kernel with 256-column workgroups; fp32: the output-stationary
    # kernel's body over the plan's pair view; both with atomics)
    want = "gms_wide_kernel(fwd)" if dtype == "wide" else "gms_rows_kernel(fwd, pair view)"
    assert want in names and "gms_rows_kernel(fwd)" not in names, names
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    G.assert_close(out, ref, G.mode_of(L["in_feats"].dtype, False), "fwd")

    # policy 4 keeps the scattered layer on the output-stationary kernel: same bits every run
    capi.set_kernel_policy(4)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    capi.profile_enable(True)
    first = G.run_fwd(capi, D, fused=True, plan=plan)
    second = G.run_fwd(capi, D, fused=True, plan=plan)
    torch.cuda.synchronize()
    capi.profile_enable(False)
    names = [n for n, _ in capi.profile_records()]
    capi.profile_reset()
    plan.close()
    capi.set_kernel_policy(0)
    assert "gms_rows_kernel(fwd)" in names and "gms_pairs_kernel(fwd)" not in names, names
    assert np.array_equal(first, second)
    G.assert_close(first, ref, G.mode_of(L["in_feats"].dtype, False), "fwd, policy 4")

    L = layer(5, 64, 64, np.float16)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    capi.profile_enable(True)
    G.run_fwd(capi, D, fused=True, plan=plan)
    torch.cuda.synchronize()
    capi.profile_enable(False)
    names = [n for n, _ in capi.profile_records()]
    capi.profile_reset()
    plan.close()
    assert "gms_rows_kernel(fwd)" in names, names


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("shape", [(64, 64), (128, 128), (32, 64)], ids=lambda s: "%dx%d" % s)
def test_backward_in_one_call_equals_its_two_halves(capi, shape, dtype):
    """fgms_bwd runs the weight gradient first and lets the two main launches carry the
    weight re-layout and the fp32 -> fp16 rounding of the weight gradient along; fgms_dgrad
    and fgms_wgrad launch those steps by themselves.  Same input gradient bit for bit, same
    weight gradient up to the order of its atomic sums; twice in a row, so that the fp32
    accumulator is seen to come back empty.  (Policy 4: the kernels without atomics, also
    where automatic dispatch would send this small scattered cloud to the pair-stationary one.)"""
    L = layer(23, *shape, dtype)
    D = G.to_dev(L)
    capi.set_kernel_policy(4)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    gi_s, gw_s = G.run_bwd(capi, D, plan=plan, split=True)
    for _ in range(2):
        gi_f, gw_f = G.run_bwd(capi, D, plan=plan, split=False)
        assert np.array_equal(gi_f, gi_s)
        G.assert_close(gw_f, gw_s, G.mode_of(L["in_feats"].dtype, False), "wgrad")
    plan.close()
    capi.set_kernel_policy(0)


def test_config2_scaled_fp32_and_tf32(capi, oracle):
    L = clouds.config_case(2, scale=0.08)
    check_all(capi, oracle, L, policy=0, use_plan=True, arch80=False)
    check_all(capi, oracle, L, policy=0, use_plan=True, arch80=True)


def test_gather_probe_runs_and_is_timed(capi):
    """The diagnostic gather-only pass: launches over a plan for both directions,
    leaves the tensors untouched and shows up in the per-kernel timing records."""
    L = layer(31, 64, 32, np.float16)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    before_in, before_g = D["in_feats"].clone(), D["out_grad"].clone()
    capi.profile_reset()
    capi.profile_enable(True)
    capi.probe_gather(D["in_feats"], plan, for_dgrad=False)
    capi.probe_gather(D["out_grad"], plan, for_dgrad=True)
    torch.cuda.synchronize()
    capi.profile_enable(False)
    names = [n for n, _ in capi.profile_records()]
    capi.profile_reset()
    assert names == ["gather_probe_kernel(fwd)", "gather_probe_kernel(dgrad)"]
    assert torch.equal(before_in, D["in_feats"]) and torch.equal(before_g, D["out_grad"])
    with pytest.raises(ValueError):
        capi.probe_gather(D["in_feats"][:, :3].contiguous(), plan)     # 6-byte rows


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
def test_pairs_in_any_order_inside_an_offset(capi, oracle, dtype):
    """The reference fixes no order of the pairs inside an offset.  Shuffled lists
    make the plan drop its output-row bands (the weight gradient then slices by
    pair count); every result must stay the same."""
    L = layer(15, 64, 64, dtype)
    rng = np.random.default_rng(15)
    kpos = np.concatenate([[0], np.cumsum(L["knnz"])])
    for k in range(L["k_vol"]):
        p = kpos[k] + rng.permutation(kpos[k + 1] - kpos[k])
        L["imap"][kpos[k]:kpos[k + 1]] = L["imap"][p]
        L["omap"][kpos[k]:kpos[k + 1]] = L["omap"][p]
    check_all(capi, oracle, L, policy=0, use_plan=True)
    check_all(capi, oracle, L, policy=0, use_plan=False)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=["fp32", "fp16"])
def test_result_rows_not_16_byte_aligned(capi, oracle, dtype):
    """A result tensor that starts 4 bytes (fp16) / 8 bytes (fp32) past a 16-byte
    boundary cannot take the planned kernel's vector updates: the call must fall
    back to the pair-stationary kernels and still be right."""
    L = layer(16, 64, 64, np.float16 if dtype == torch.float16 else np.float32)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    buf = torch.zeros(D["n_out"] * 64 + 8, dtype=dtype, device="cuda")
    out = buf[2:2 + D["n_out"] * 64].view(D["n_out"], 64)
    assert out.data_ptr() % 16 != 0 and out.is_contiguous()
    capi.fusion_fwd(D["in_feats"], D["kernel"], 0, out, D["kpos"], None, D["imap"], D["omap"],
                    False, False, plan=plan)
    torch.cuda.synchronize()
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    G.assert_close(out.cpu().numpy(), ref, G.mode_of(dtype), "fwd into an unaligned result")
    assert not buf[:2].any() and not buf[2 + D["n_out"] * 64:].any()


@pytest.mark.parametrize("shape", [(64, 64), (32, 64), (96, 32)], ids=lambda s: "%dx%d" % s)
def test_tf32_mode_multiplies_in_split_bf16(capi, oracle, shape):
    """fp32 tensors with arch80 set (the reference's tf32 mode): the output-stationary
    forward kernel splits every value into two bf16 numbers and multiplies with three
    16-bit MFMAs.  That path is the one that runs, and it is far inside the mode's
    tolerance: at most 1e-4 of the result's rms where tf32 itself would be allowed 1e-2
    (measured 5e-6).  Non-finite inputs stay non-finite only where they are used."""
    L = layer(19, shape[0], shape[1], np.float32)
    D = G.to_dev(L)
    capi.set_kernel_policy(4)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    capi.profile_reset()
    capi.profile_enable(True)
    for fused in (True, False):
        out = G.run_fwd(capi, D, fused=fused, arch80=True, plan=plan)
        G.assert_close(out, ref, "tf32", "tf32-mode forward")
        rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        assert np.abs(out - ref).max() <= 1e-4 * rms
    capi.profile_enable(False)
    names = {n for n, _ in capi.profile_records()}
    capi.profile_reset()
    assert names == {"gms_rows_kernel(fwd, bf16x3)"}, names
    # an infinite input value reaches exactly the output rows that use its row
    D2 = dict(D)
    x = D["in_feats"].clone()
    x[5, 3] = float("inf")
    D2["in_feats"] = x
    out = G.run_fwd(capi, D2, fused=True, arch80=True, plan=plan)
    users = np.unique(L["omap"][L["imap"] == 5])
    bad = np.where(~np.isfinite(out).all(axis=1))[0]
    assert set(bad) == set(users)
    plan.close()
    capi.set_kernel_policy(0)


@pytest.mark.parametrize("kind", ["subm", "down"])
@pytest.mark.parametrize("shape", [(64, 64), (32, 64), (96, 32), (64, 128), (128, 128)], ids=lambda s: "%dx%d" % s)
def test_tf32_mode_backward_in_split_bf16(capi, oracle, shape, kind):
    """fgms_bwd of fp32 tensors with arch80 set (the reference's backward is tf32 whenever the
    tensors are fp32, backend/spconv.cu:551-569): the input gradient and the weight gradient
    (per-wave and workgroup-level kernel bodies alike) multiply in split bf16.  Both stay
    within 1e-4 of the result's rms (tf32 would be allowed 1e-2), on two calls in a row."""
    L = layer(29, shape[0], shape[1], np.float32, kind)
    D = G.to_dev(L)
    capi.set_kernel_policy(4)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    args = (L["knnz"], L["imap"], L["omap"])
    want_gi = oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"])
    want_gw = oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"])
    exact_gi, exact_gw = G.run_bwd(capi, D, plan=plan, arch80=False)
    for _ in range(2):
        gi, gw = G.run_bwd(capi, D, plan=plan, arch80=True)
        for got, want, what in ((gi, want_gi, "dgrad"), (gw, want_gw, "wgrad")):
            G.assert_close(got, want, "tf32", "tf32-mode " + what)
            rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
            assert np.abs(got - want).max() <= 1e-4 * rms, what
    # the split path is the one that ran: both gradients differ from the fp32 kernels' in their last bits
    assert not np.array_equal(gi, exact_gi) and not np.array_equal(gw, exact_gw)
    G.assert_close(exact_gi, want_gi, "fp32", "fp32 dgrad")
    G.assert_close(exact_gw, want_gw, "fp32", "fp32 wgrad")
    plan.close()
    capi.set_kernel_policy(0)


@pytest.mark.parametrize("shape", [(64, 64), (96, 32), (256, 256)], ids=lambda s: "%dx%d" % s)
def test_tf32_mode_without_a_plan(capi, oracle, shape):
    """The pair-stationary kernels (calls without a plan) multiply in split bf16 as well,
    forward (also with the centre offset taken apart) and backward."""
    L = layer(37, shape[0], shape[1], np.float32)
    D = G.to_dev(L)
    capi.set_kernel_policy(0)
    args = (L["knnz"], L["imap"], L["omap"])
    want = oracle.np_fwd(L["in_feats"], L["kernel"], *args, L["n_out"])
    capi.profile_reset()
    capi.profile_enable(True)
    out = G.run_fwd(capi, D, fused=True, arch80=True, plan=None)
    gi, gw = G.run_bwd(capi, D, plan=None, arch80=True)
    capi.profile_enable(False)
    names = {n for n, _ in capi.profile_records()}
    capi.profile_reset()
    assert {"gms_pairs_kernel(fwd, bf16x3)", "gms_pairs_kernel(dgrad, bf16x3)"} <= names, names
    for got, ref, what in ((out, want, "fwd"),
                           (gi, oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"]), "dgrad"),
                           (gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"]), "wgrad")):
        G.assert_close(got, ref, "tf32", "tf32-mode " + what)
        assert np.abs(got - ref).max() <= 1e-4 * float(np.sqrt(np.mean(ref.astype(np.float64) ** 2))), what
    # the centre offset left out of the map and added as a dense product (separate_mid)
    rng = np.random.default_rng(38)
    vox = cloud(38)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(3), skip_offset=13)
    Ls = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(vox), shape[0], shape[1], np.float32)
    Ds = G.to_dev(Ls)
    ref = oracle.np_fwd(Ls["in_feats"], Ls["kernel"], knnz, imap, omap, len(vox), precompute=True)
    for fused in (True, False):
        G.assert_close(G.run_fwd(capi, Ds, fused=fused, separate_mid=True, arch80=True, plan=None), ref, "tf32",
                       "tf32-mode forward, centre apart")


@pytest.mark.parametrize("shape", [(32, 32), (64, 64)], ids=["32x32", "64x64"])
def test_fp32_with_half_the_rms_floor(capi, oracle, shape):
    """assert_close allows rtol * rms(reference) on top of the relative bound, which for
    small-magnitude elements is most of the allowance.  Here the fp32 path is held to
    |d| <= 1e-5 |ref| + 5e-6 rms(ref) against the float64 formulation, half the usual floor, and
    the error of the typical element to a tenth of it.  (A sum of a thousand fp32 products
    carries rounding noise of 2-3e-6 of the result's rms in its worst elements, whatever the
    order of summation: a floor below that would test the number format, not the kernel.)"""
    L = layer(43, shape[0], shape[1], np.float32)
    D = G.to_dev(L)
    args = (L["knnz"], L["imap"], L["omap"])
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])

    def tight(got, ref, what):
        got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
        rms = float(np.sqrt(np.mean(ref ** 2)))
        err = np.abs(got - ref)
        bad = err > 1e-5 * np.abs(ref) + 5e-6 * rms
        assert not bad.any(), "%s: %d / %d outside 1e-5 |ref| + 5e-6 rms (worst %.3g of rms)" % (
            what, int(bad.sum()), bad.size, float(err.max() / rms))
        assert float(np.median(err)) <= 1e-6 * rms, (what, float(np.median(err)) / rms)

    for p, tag in ((plan, "plan"), (None, "no plan")):
        tight(G.run_fwd(capi, D, plan=p), oracle.np_fwd(L["in_feats"], L["kernel"], *args, L["n_out"]), "fwd, " + tag)
        gi, gw = G.run_bwd(capi, D, plan=p)
        tight(gi, oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"]), "dgrad, " + tag)
        tight(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"]), "wgrad, " + tag)
    plan.close()
