"""Pins the CPU oracle (oracle/fgms_oracle.c and its float64 numpy twin) without
the reference's data files, which do not exist offline: closed forms, library
routines that the sparse convolution reduces to, autograd, adjoint identities
and brute-force python loops restating cpu-check.py:27-44 and
cpu-check-back.py:28-41 literally."""
import bisect

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fgms_amd import clouds


def dense_grid(d, h, w):
    g = np.stack(np.meshgrid(np.arange(d), np.arange(h), np.arange(w), indexing="ij"), -1)
    return g.reshape(-1, 3).astype(np.int32)


def rand_layer(rng, coords_in, coords_out, offsets, stride, c_in, c_out, dtype=np.float32):
    imap, omap, knnz, kpos = clouds.build_kernel_map(coords_in, coords_out, offsets, stride)
    return clouds.make_layer(rng, imap, omap, knnz, kpos, len(coords_in), len(coords_out),
                             c_in, c_out, dtype)


# ---------------------------------------------------------------- conversions
def test_half_to_float_all_bit_patterns(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.fgms_oracle_half_to_float(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_float_to_half_rounding(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 20000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                  2.0 ** -25 * 1.0001, 6.1e-5, 6.0975e-5, np.inf, -np.inf], np.float32),
        # exact ties between neighbouring halves
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) * np.float32(2.0 ** -10),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.fgms_oracle_float_to_half(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- index helpers
def test_qkpos_closed_form(oracle):
    rng = np.random.default_rng(1)
    for q in (1, 32, 256):
        knnz = rng.integers(0, 2000, 27).astype(np.int32)
        knnz[[3, 13]] = 0
        qk, total = oracle.c_qkpos(knnz, q)
        assert qk[0] == 0 and total == qk[-1]
        d = np.diff(qk)
        assert np.all(d % q == 0) and np.all(d >= knnz) and np.all(d - knnz < q)


def test_offset_lookup_matches_bisect(oracle):
    rng = np.random.default_rng(2)
    for _ in range(40):
        k_vol = int(rng.integers(1, 12))
        knnz = rng.integers(0, 4, k_vol) * 4
        pos = np.concatenate([[0], np.cumsum(knnz)]).astype(np.int32)
        for eid in range(0, int(pos[-1]) + 3):
            want = min(max(bisect.bisect_right(list(pos), eid) - 1, 0), k_vol)
            assert oracle.c_offset_of(pos, eid, 0, k_vol) == want


# ---------------------------------------------------------------- brute force
def loops_fwd(x, w, knnz, imap, omap, n_out, precompute):
    """cpu-check.py:27-44, literally."""
    k_vol, c_in, c_out = w.shape
    mid = k_vol // 2 if k_vol % 2 == 1 else 0
    out = np.zeros((n_out, c_out), np.float64)
    nb = 0
    for k in range(k_vol):
        for _ in range(int(knnz[k])):
            i, o = imap[nb], omap[nb]
            for co in range(c_out):
                for ci in range(c_in):
                    out[o, co] += float(x[i, ci]) * float(w[k, ci, co])
            nb += 1
    if precompute:
        for i in range(n_out):
            for co in range(c_out):
                for ci in range(c_in):
                    out[i, co] += float(x[i, ci]) * float(w[mid, ci, co])
    return out


def loops_bwd(g, w, x, n_in, knnz, imap, omap):
    """cpu-check-back.py:28-41, literally."""
    k_vol, c_in, c_out = w.shape
    gi = np.zeros((n_in, c_in), np.float64)
    gw = np.zeros((k_vol, c_in, c_out), np.float64)
    nb = 0
    for k in range(k_vol):
        for _ in range(int(knnz[k])):
            i, o = imap[nb], omap[nb]
            for ci in range(c_in):
                for co in range(c_out):
                    gi[i, ci] += float(g[o, co]) * float(w[k, ci, co])
                    gw[k, ci, co] += float(x[i, ci]) * float(g[o, co])
            nb += 1
    return gi, gw


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_bruteforce_tiny(oracle, dtype):
    rng = np.random.default_rng(3)
    coords = clouds.dedup(rng.uniform(0, 5, (60, 3)), 5)
    L = rand_layer(rng, coords, coords, clouds.offsets_cube(3), 1, 5, 3, dtype)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == np.float32 else dict(rtol=2e-3, atol=2e-3)
    for pre in (False, True):
        want = loops_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"], pre)
        got = oracle.c_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"], pre)
        np.testing.assert_allclose(got.astype(np.float64), want, **tol)
        np.testing.assert_allclose(
            oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"], pre),
            want, rtol=1e-12, atol=1e-12)
    gi, gw = loops_bwd(L["out_grad"], L["kernel"], L["in_feats"], L["n_in"], L["knnz"], L["imap"], L["omap"])
    np.testing.assert_allclose(
        oracle.c_dgrad(L["out_grad"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_in"]).astype(np.float64),
        gi, **tol)
    np.testing.assert_allclose(
        oracle.c_wgrad(L["in_feats"], L["out_grad"], L["knnz"], L["imap"], L["omap"], L["k_vol"]).astype(np.float64),
        gw, **(tol if dtype == np.float32 else dict(rtol=5e-3, atol=2e-2)))
    np.testing.assert_allclose(oracle.np_dgrad(L["out_grad"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_in"]), gi, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(oracle.np_wgrad(L["in_feats"], L["out_grad"], L["knnz"], L["imap"], L["omap"], L["k_vol"]), gw, rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------- dense-grid reductions
def conv_weight(w, ks):
    k_vol, c_in, c_out = w.shape
    return torch.from_numpy(w.astype(np.float64)).reshape(ks, ks, ks, c_in, c_out).permute(4, 3, 0, 1, 2)


def test_dense_submanifold_equals_conv3d(oracle):
    rng = np.random.default_rng(4)
    d, h, w_ = 5, 4, 6
    coords = dense_grid(d, h, w_)
    L = rand_layer(rng, coords, coords, clouds.offsets_cube(3), 1, 7, 5)
    x = torch.from_numpy(L["in_feats"].astype(np.float64)).reshape(d, h, w_, 7).permute(3, 0, 1, 2)[None]
    want = F.conv3d(x, conv_weight(L["kernel"], 3), padding=1)[0].permute(1, 2, 3, 0).reshape(-1, 5).numpy()
    got = oracle.c_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"]),
                               want, rtol=1e-12, atol=1e-12)


def test_dense_separate_mid_equals_conv3d(oracle):
    """Map without the centre offset + precompute == the full convolution."""
    rng = np.random.default_rng(5)
    coords = dense_grid(4, 4, 4)
    imap, omap, knnz, kpos = clouds.build_kernel_map(coords, coords, clouds.offsets_cube(3), skip_offset=13)
    assert knnz[13] == 0
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, 64, 64, 6, 4, np.float32)
    x = torch.from_numpy(L["in_feats"].astype(np.float64)).reshape(4, 4, 4, 6).permute(3, 0, 1, 2)[None]
    want = F.conv3d(x, conv_weight(L["kernel"], 3), padding=1)[0].permute(1, 2, 3, 0).reshape(-1, 4).numpy()
    got = oracle.c_fwd(L["in_feats"], L["kernel"], knnz, imap, omap, 64, precompute=True)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_dense_stride2_and_transposed(oracle):
    rng = np.random.default_rng(6)
    fine = dense_grid(4, 6, 4)
    coarse = clouds.downsample_coords(fine, 2)
    imap, omap, knnz, kpos = clouds.build_kernel_map(fine, coarse, clouds.offsets_cube(2), stride=2)
    assert len(imap) == len(fine)
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, len(fine), len(coarse), 3, 5, np.float32)
    x = torch.from_numpy(L["in_feats"].astype(np.float64)).reshape(4, 6, 4, 3).permute(3, 0, 1, 2)[None]
    want = F.conv3d(x, conv_weight(L["kernel"], 2), stride=2)[0].permute(1, 2, 3, 0).reshape(-1, 5).numpy()
    got = oracle.c_fwd(L["in_feats"], L["kernel"], knnz, imap, omap, len(coarse))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    # transposed: the two maps swap roles
    T = clouds.make_layer(rng, omap, imap, knnz, kpos, len(coarse), len(fine), 5, 3, np.float32)
    xc = torch.from_numpy(T["in_feats"].astype(np.float64)).reshape(2, 3, 2, 5).permute(3, 0, 1, 2)[None]
    wt = torch.from_numpy(T["kernel"].astype(np.float64)).reshape(2, 2, 2, 5, 3).permute(3, 4, 0, 1, 2)
    want_t = F.conv_transpose3d(xc, wt, stride=2)[0].permute(1, 2, 3, 0).reshape(-1, 3).numpy()
    got_t = oracle.c_fwd(T["in_feats"], T["kernel"], knnz, omap, imap, len(fine))
    np.testing.assert_allclose(got_t, want_t, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- gradients
def test_gradients_match_autograd(oracle):
    rng = np.random.default_rng(7)
    coords = clouds.dedup(rng.uniform(0, 8, (300, 3)), 8)
    L = rand_layer(rng, coords, coords, clouds.offsets_cube(3), 1, 6, 9)
    x = torch.tensor(L["in_feats"], dtype=torch.float64, requires_grad=True)
    w = torch.tensor(L["kernel"], dtype=torch.float64, requires_grad=True)
    out = torch.zeros(L["n_out"], 9, dtype=torch.float64)
    kpos = L["kpos"]
    for k in range(L["k_vol"]):
        a, b = int(kpos[k]), int(kpos[k + 1])
        if b > a:
            im = torch.from_numpy(L["imap"][a:b].astype(np.int64))
            om = torch.from_numpy(L["omap"][a:b].astype(np.int64))
            out = out.index_add(0, om, x[im] @ w[k])
    g = torch.tensor(L["out_grad"], dtype=torch.float64)
    gx, gw = torch.autograd.grad(out, (x, w), g)
    np.testing.assert_allclose(
        oracle.c_dgrad(L["out_grad"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_in"]),
        gx.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(
        oracle.c_wgrad(L["in_feats"], L["out_grad"], L["knnz"], L["imap"], L["omap"], L["k_vol"]),
        gw.numpy(), rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(
        oracle.c_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"]),
        out.detach().numpy(), rtol=1e-4, atol=1e-5)


def test_adjoint_identities(oracle):
    """<g, fwd(x)> == <dgrad(g), x> == <wgrad(x, g), W> in float64."""
    rng = np.random.default_rng(8)
    fine = clouds.dedup(rng.uniform(0, 12, (500, 3)), 12)
    coarse = clouds.downsample_coords(fine, 2)
    L = rand_layer(rng, fine, coarse, clouds.offsets_cube(2), 2, 4, 7)
    args = (L["knnz"], L["imap"], L["omap"])
    y = oracle.np_fwd(L["in_feats"], L["kernel"], *args, L["n_out"])
    gi = oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"])
    gw = oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"])
    lhs = float(np.sum(L["out_grad"].astype(np.float64) * y))
    assert abs(lhs - float(np.sum(gi * L["in_feats"]))) < 1e-9 * max(1.0, abs(lhs))
    assert abs(lhs - float(np.sum(gw * L["kernel"]))) < 1e-9 * max(1.0, abs(lhs))


def test_threads_and_duplicates(oracle):
    """Thread count does not change the result; duplicate output rows inside an
    offset (not a sparse-conv map, but legal input) accumulate."""
    rng = np.random.default_rng(9)
    n_in, n_out, c_in, c_out, k_vol = 50, 20, 8, 8, 3
    knnz = np.array([40, 0, 25], np.int32)
    imap = rng.integers(0, n_in, 65).astype(np.int32)
    omap = rng.integers(0, n_out, 65).astype(np.int32)
    x = rng.standard_normal((n_in, c_in)).astype(np.float32)
    w = rng.standard_normal((k_vol, c_in, c_out)).astype(np.float32)
    g = rng.standard_normal((n_out, c_out)).astype(np.float32)
    ref = oracle.np_fwd(x, w, knnz, imap, omap, n_out)
    a = oracle.c_fwd(x, w, knnz, imap, omap, n_out, threads=1)
    b = oracle.c_fwd(x, w, knnz, imap, omap, n_out, threads=4)
    assert np.array_equal(a, b)
    np.testing.assert_allclose(a, ref, rtol=1e-5, atol=1e-5)
    assert np.array_equal(oracle.c_dgrad(g, w, knnz, imap, omap, n_in, threads=1),
                          oracle.c_dgrad(g, w, knnz, imap, omap, n_in, threads=3))
    assert np.array_equal(oracle.c_wgrad(x, g, knnz, imap, omap, k_vol, threads=1),
                          oracle.c_wgrad(x, g, knnz, imap, omap, k_vol, threads=5))
    np.testing.assert_allclose(oracle.c_wgrad(x, g, knnz, imap, omap, k_vol),
                               oracle.np_wgrad(x, g, knnz, imap, omap, k_vol), rtol=1e-5, atol=1e-5)


def test_accumulates_onto_existing_output(oracle):
    rng = np.random.default_rng(10)
    coords = clouds.dedup(rng.uniform(0, 6, (100, 3)), 6)
    L = rand_layer(rng, coords, coords, clouds.offsets_cube(3), 1, 4, 4)
    base = rng.standard_normal((L["n_out"], 4)).astype(np.float32)
    got = oracle.c_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"], out_init=base)
    want = base + oracle.np_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_config1_c_vs_numpy(oracle):
    """The CPU-runnable configuration at full size: the C loop nest against the
    float64 numpy formulation."""
    L = clouds.config_case(1)
    args = (L["knnz"], L["imap"], L["omap"])
    y = oracle.c_fwd(L["in_feats"], L["kernel"], *args, L["n_out"])
    ref = oracle.np_fwd(L["in_feats"], L["kernel"], *args, L["n_out"])
    assert np.max(np.abs(y - ref)) <= 1e-5 * np.sqrt(np.mean(ref ** 2)) + 1e-5 * np.max(np.abs(ref))
    gi = oracle.c_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"])
    ref = oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"])
    assert np.max(np.abs(gi - ref)) <= 2e-5 * np.max(np.abs(ref))
    gw = oracle.c_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"])
    ref = oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"])
    assert np.max(np.abs(gw - ref)) <= 1e-4 * np.max(np.abs(ref))
