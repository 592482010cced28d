"""GPU checks at the full BASELINE sizes, where the CPU oracle is too slow to be the
checker for every case: size-independent properties of the three products.

With T(x, W, g) = sum_j  g[omap[j]] . (x[imap[j]] @ W[k(j)])  (a trilinear form):
    <g, fwd(x, W)>  =  <dgrad(g, W), x>  =  <wgrad(x, g), W>  =  T(x, W, g)
so the three kernels must agree on one number; forward is linear in x; the planned
(output-stationary) and the pair-stationary kernels must agree with each other; and on
the one configuration the C oracle finishes in a second it is compared directly."""
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


def run_all(capi, D, plan):
    dt = D["in_feats"].dtype
    out = torch.zeros(D["n_out"], D["c_out"], dtype=dt, device="cuda")
    gi = torch.zeros(D["n_in"], D["c_in"], dtype=dt, device="cuda")
    gw = torch.zeros_like(D["kernel"])
    capi.fusion_fwd(D["in_feats"], D["kernel"], 0, out, D["kpos"], None, D["imap"], D["omap"],
                    False, False, plan=plan)
    capi.dgrad(D["out_grad"], D["kernel"], gi, D["kpos"], D["imap"], D["omap"], plan=plan)
    capi.wgrad(D["in_feats"], D["out_grad"], gw, D["kpos"], D["imap"], D["omap"], plan=plan)
    torch.cuda.synchronize()
    return out, gi, gw


def dot(a, b):
    return float((a.double() * b.double()).sum())


CASES = [(2, "fp16", 2e-3), (2, None, 2e-5), (3, None, 2e-3), (4, None, 2e-3), (4, "up", 2e-3), (5, "wide", 2e-3)]


@pytest.mark.parametrize("cfg,variant,tol", CASES, ids=lambda v: str(v))
def test_trilinear_form_agrees_full_size(capi, cfg, variant, tol):
    L = clouds.config_case(cfg, variant, scale=1.0)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    out, gi, gw = run_all(capi, D, plan)
    t_f, t_d, t_w = dot(D["out_grad"], out), dot(gi, D["in_feats"]), dot(gw, D["kernel"])
    # scale of the form: sqrt(#terms) * typical term, from the forward result itself
    scale = float(out.double().norm() * D["out_grad"].double().norm())
    assert abs(t_f - t_d) <= tol * scale, (t_f, t_d, scale)
    assert abs(t_f - t_w) <= tol * scale, (t_f, t_w, scale)
    assert torch.isfinite(out).all() and torch.isfinite(gi).all() and torch.isfinite(gw).all()

    # linearity: fwd(2 x) = 2 fwd(x) bit for bit, scaling by two being exact, except where
    # the fp16 result is subnormal (there the doubled sum keeps one more bit).  A property
    # of the kernels without atomics: policy 4 keeps automatic dispatch from handing a
    # scattered wide layer (cfg 5) to the pair-stationary kernel, whose sums depend on order.
    capi.set_kernel_policy(4)
    out = torch.zeros_like(out)
    capi.fusion_fwd(D["in_feats"], D["kernel"], 0, out, D["kpos"], None, D["imap"], D["omap"],
                    False, False, plan=plan)
    D2 = dict(D)
    D2["in_feats"] = D["in_feats"] * 2
    out2 = torch.zeros_like(out)
    capi.fusion_fwd(D2["in_feats"], D["kernel"], 0, out2, D["kpos"], None, D["imap"], D["omap"],
                    False, False, plan=plan)
    torch.cuda.synchronize()
    capi.set_kernel_policy(0)
    if out.dtype == torch.float16:
        assert float((out2.float() - 2 * out.float()).abs().max()) <= 2.0 ** -23
        normal = out.abs() > 2.0 ** -14      # 2^-14 itself can be a subnormal-range sum rounded up
        assert torch.equal(out2[normal], (out * 2)[normal])
    else:
        assert torch.equal(out2, out * 2)

    # the pair-stationary (atomic) kernels, no plan: same results within the mode's tolerance
    mode = G.mode_of(D["in_feats"].dtype)
    out_p, gi_p, gw_p = run_all(capi, D, None)
    G.assert_close(out_p.cpu().numpy(), out.cpu().numpy(), mode, "fwd planned vs pair-stationary")
    G.assert_close(gi_p.cpu().numpy(), gi.cpu().numpy(), mode, "dgrad planned vs pair-stationary")
    G.assert_close(gw_p.cpu().numpy(), gw.cpu().numpy(), mode, "wgrad bands vs equal slices")
    plan.close()


def test_config1_full_size_against_oracle(capi, oracle):
    """20 k voxels, 32 -> 32 fp32: small enough for the C oracle at full size."""
    L = clouds.config_case(1, None, scale=1.0)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    out, gi, gw = run_all(capi, D, plan)
    a = (L["knnz"], L["imap"], L["omap"])
    G.assert_close(out.cpu().numpy(), oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"]), "fp32", "fwd")
    G.assert_close(gi.cpu().numpy(), oracle.c_dgrad(L["out_grad"], L["kernel"], *a, L["n_in"]), "fp32", "dgrad")
    G.assert_close(gw.cpu().numpy(), oracle.c_wgrad(L["in_feats"], L["out_grad"], *a, L["k_vol"]), "fp32", "wgrad")
    plan.close()


# Every BASELINE configuration at the size it is benchmarked at, element by element against
# the C oracle (cpu-check.py:121-127 compares whole outputs the same way).  These are the
# launches that take the full-size-only paths: tile tables with XCD homes, first offsets
# from the tile table, 128-column wave tiles, split bf16 at 200 k voxels, the scattered
# wide layer's dispatch.
FULL = [
    # cfg, variant, arch80, passes
    (2, "fp16", False, "f"), (2, None, False, "f"), (2, None, True, "f"),
    (3, None, False, "fdw"),
    (4, None, False, "fdw"), (4, "up", False, "fdw"),
    (5, "wide", False, "f"), (5, "wide-fp32", False, "f"),
    (5, "skinny", False, "fdw"), (5, "skinny-fp32", False, "fdw"),
]


@pytest.mark.parametrize("cfg,variant,arch80,passes", FULL,
                         ids=["cfg%d-%s%s" % (c, v or "default", "-tf32" if a else "") for c, v, a, _ in FULL])
@pytest.mark.parametrize("with_plan", [True, False], ids=["plan", "no-plan"])
def test_configs_full_size_against_oracle(capi, oracle, cfg, variant, arch80, passes, with_plan):
    L = clouds.config_case(cfg, variant, scale=1.0)
    D = G.to_dev(L)
    capi.set_kernel_policy(0)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"]) if with_plan else None
    mode = G.mode_of(L["in_feats"].dtype, arch80)
    a = (L["knnz"], L["imap"], L["omap"])
    out = G.run_fwd(capi, D, fused=True, arch80=arch80, plan=plan)
    G.assert_close(out, oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"]), mode, "fwd")
    if "d" in passes:
        gi, gw = G.run_bwd(capi, D, plan=plan, arch80=arch80)
        G.assert_close(gi, oracle.c_dgrad(L["out_grad"], L["kernel"], *a, L["n_in"]), mode, "dgrad")
        # (a weight-gradient element sums tens of thousands of pairs: the float64 formulation)
        G.assert_close(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *a, L["k_vol"]), mode, "wgrad")
    if plan is not None:
        plan.close()


@pytest.mark.parametrize("side,c,dtype,tol", [(100, 64, torch.float16, 2e-3), (96, 32, torch.float32, 2e-5)],
                         ids=["1M-fp16", "885k-fp32"])
def test_dense_grid_built_and_convolved_on_the_device(capi, side, c, dtype, tol):
    """A full side^3 grid (every voxel has all its in-grid neighbours): the map comes from
    the device builder and its size has a closed form, sum over offsets of
    (side-|dx|)(side-|dy|)(side-|dz|); the three kernels must agree on the trilinear form at
    a size (26 M pairs) far beyond the oracle's reach."""
    n = side ** 3
    g = torch.arange(side, dtype=torch.int32, device="cuda")
    coords = torch.stack(torch.meshgrid(g, g, g, indexing="ij"), -1).reshape(-1, 3).contiguous()
    offs = np.array([(a, b, d) for a in (-1, 0, 1) for b in (-1, 0, 1) for d in (-1, 0, 1)], np.int32)
    imap, omap, knnz, kpos = capi.build_kernel_map(coords, coords, offs, 1)
    expect = [(side - abs(a)) * (side - abs(b)) * (side - abs(d)) for a, b, d in offs]
    assert [int(v) for v in knnz] == expect and int(imap.numel()) == sum(expect)
    gen = torch.Generator(device="cuda").manual_seed(side)
    x = torch.randn(n, c, device="cuda", dtype=dtype, generator=gen)
    w = (torch.randn(27, c, c, device="cuda", generator=gen) * 0.05).to(dtype)
    go = torch.randn(n, c, device="cuda", dtype=dtype, generator=gen)
    plan = capi.Plan(kpos, imap, omap, n, n)
    out = torch.zeros(n, c, device="cuda", dtype=dtype)
    gi, gw = torch.zeros_like(x), torch.zeros_like(w)
    capi.fusion_fwd(x, w, 0, out, kpos, None, imap, omap, False, False, plan=plan)
    capi.bwd(go, x, w, 0, gi, gw, kpos, None, imap, omap, False, False, plan=plan)
    torch.cuda.synchronize()
    t_f, t_d, t_w = dot(go, out), dot(gi, x), dot(gw, w)
    scale = float(out.double().norm() * go.double().norm())
    assert abs(t_f - t_d) <= tol * scale and abs(t_f - t_w) <= tol * scale, (t_f, t_d, t_w, scale)
    # an interior voxel against the definition: sum over offsets of x[neighbour] @ w[k]
    v = (side // 2 * side + side // 2) * side + side // 2
    ref = torch.zeros(c, dtype=torch.float64, device="cuda")
    for k, (a, b, d) in enumerate(offs):
        u = v + (int(a) * side + int(b)) * side + int(d)
        ref += x[u].double() @ w[k].double()
    assert torch.allclose(out[v].double(), ref, rtol=1e-2 if dtype == torch.float16 else 1e-5,
                          atol=1e-2 if dtype == torch.float16 else 1e-5)
    plan.close()


@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["fp16", "fp32"])
@pytest.mark.parametrize("shape", [(64, 64), (32, 64), (64, 32), (32, 32)], ids=lambda s: "%dx%d" % s)
def test_backward_in_one_launch_full_size(capi, oracle, shape, dtype):
    """On a launch that fills the chip fgms_bwd runs both gradients of a 32/64-channel layer
    in ONE grid (input-gradient workgroups first, weight-gradient workgroups behind them).
    Over the 200k-voxel cloud: that kernel is the one that ran, the input gradient equals
    the separate fgms_dgrad call bit for bit, both gradients match the CPU oracle, and a
    second call gives the same (the fp32 scratch of the fp16 weight gradient came back
    empty)."""
    rng = np.random.default_rng(77)
    vox = clouds.cloud_indoor(clouds.rng_for(2), target=200000)
    L = clouds.submanifold_case(vox, shape[0], shape[1], dtype, rng)
    D = G.to_dev(L)
    capi.set_kernel_policy(0)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    mode = G.mode_of(L["in_feats"].dtype, False)
    args = (L["knnz"], L["imap"], L["omap"])
    want_gi = oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"])
    want_gw = oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"])
    gi_s, _ = G.run_bwd(capi, D, plan=plan, split=True)
    capi.profile_reset()
    capi.profile_enable(True)
    for _ in range(2):
        gi_f, gw_f = G.run_bwd(capi, D, plan=plan, split=False)
        assert np.array_equal(gi_f, gi_s)
        G.assert_close(gi_f, want_gi, mode, "dgrad")
        G.assert_close(gw_f, want_gw, mode, "wgrad")
    capi.profile_enable(False)
    names = {n for n, _ in capi.profile_records()}
    capi.profile_reset()
    plan.close()
    assert names == {"bwd_fused_kernel"}, names


@pytest.mark.parametrize("voxels", [9000, 30000, 62000, 70000, 100000, 128000, 140000])
@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["fp16", "fp32"])
def test_every_grid_choice_against_oracle(capi, oracle, voxels, dtype):
    """The output-stationary launch picks its grid by the number of rows: tiles of 128 rows
    shared by two workgroups (9 k, 30 k, 62 k), the plan's tile table with 256-row tiles shared
    by two workgroups (70 k), plain 128-row tiles although a table exists (100 k, 128 k:
    forward only), the table again (140 k and up).  Forward, input and
    weight gradient of a 64 -> 64 layer against the oracle at each size, the input gradient of
    the one-grid backward call bit for bit equal to the separate call's."""
    rng = np.random.default_rng(91)
    vox = clouds.cloud_indoor(clouds.rng_for(2), target=voxels)
    L = clouds.submanifold_case(vox, 64, 64, dtype, rng)
    D = G.to_dev(L)
    capi.set_kernel_policy(4)      # the kernels with a plan, whatever the cloud's row-slot fill
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    mode = G.mode_of(L["in_feats"].dtype, False)
    a = (L["knnz"], L["imap"], L["omap"])
    out = G.run_fwd(capi, D, fused=True, plan=plan)
    G.assert_close(out, oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"]), mode, "fwd")
    gi_s, _ = G.run_bwd(capi, D, plan=plan, split=True)
    gi, gw = G.run_bwd(capi, D, plan=plan)
    capi.set_kernel_policy(0)
    plan.close()
    assert np.array_equal(gi, gi_s)
    G.assert_close(gi, oracle.c_dgrad(L["out_grad"], L["kernel"], *a, L["n_in"]), mode, "dgrad")
    G.assert_close(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *a, L["k_vol"]), mode, "wgrad")
