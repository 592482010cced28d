"""fgms_build_kernel_map against the numpy builder of the harness (itself pinned by the
brute-force dictionary builder in tests/test_harness.py): bit-exact, order included."""
import numpy as np
import pytest
import torch

from fgms_amd import clouds

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    from fgms_amd import capi as c
    c.lib()
    assert torch.cuda.is_available()
    return c


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a.astype(np.int32))).cuda()


def check(capi, vin, vout, offsets, stride=1, skip=None):
    want = clouds.build_kernel_map(vin, vout, offsets, stride, skip)
    got = capi.build_kernel_map(dev(vin), dev(vout), offsets, stride, skip)
    for g, w, name in zip(got, want, ("in_map", "out_map", "kernel_nnz", "kpos")):
        assert np.array_equal(g.cpu().numpy(), w), name
    return got


def random_cloud(seed, n=4000, grid=40, shift=0):
    rng = np.random.default_rng(seed)
    pts = np.concatenate([clouds._patch(rng, rng.uniform(8, 30, 3), 14, 14, oblique=True),
                          clouds._sphere_shell(rng, np.array([20., 20, 20]), 11.0, n)])
    return clouds.dedup(pts, grid) + shift


def test_submanifold_3x3x3(capi):
    vox = random_cloud(51)
    check(capi, vox, vox, clouds.offsets_cube(3))
    check(capi, vox, vox, clouds.offsets_cube(3), skip=13)          # centre left to separate_mid


def test_negative_coordinates_and_5x5x5(capi):
    vox = random_cloud(52, shift=-25)
    assert vox.min() < 0
    check(capi, vox, vox, clouds.offsets_cube(5))                    # 125 offsets: more than the plan's 64


def test_stride_two_down_and_up(capi):
    vox = random_cloud(53)
    coarse = clouds.downsample_coords(vox, 2)
    imap, omap, knnz, kpos = check(capi, vox, coarse, clouds.offsets_cube(2), stride=2)
    assert int(kpos[-1]) == len(vox)                                 # every input voxel has exactly one parent


def test_duplicate_input_coordinates_take_the_smallest_row(capi):
    vox = random_cloud(54, n=1500)
    twice = np.concatenate([vox, vox[::3]])                          # repeats come later: never chosen
    check(capi, twice, vox, clouds.offsets_cube(3))


def check_one_list(capi, vox, offsets, skip=None):
    """One device tensor on both sides: the builder may then take half of the lookups from the
    other half (a submanifold map is its own mirror image)."""
    want = clouds.build_kernel_map(vox, vox, offsets, 1, skip)
    d = dev(vox)
    got = capi.build_kernel_map(d, d, offsets, 1, skip)
    for g, w, name in zip(got, want, ("in_map", "out_map", "kernel_nnz", "kpos")):
        assert np.array_equal(g.cpu().numpy(), w), name
    return got


def test_one_coordinate_list_on_both_sides(capi):
    vox = random_cloud(56)
    check_one_list(capi, vox, clouds.offsets_cube(3))
    check_one_list(capi, vox, clouds.offsets_cube(3), skip=13)
    check_one_list(capi, random_cloud(57, shift=-25), clouds.offsets_cube(5))
    check_one_list(capi, vox, clouds.offsets_cube(2))               # offsets without mirror images
    check_one_list(capi, vox, clouds.offsets_cube(3)[::-1][[1, 0] + list(range(2, 27))])   # ... in an order that is not mirrored
    check_one_list(capi, vox[:1], clouds.offsets_cube(3))
    twice = np.concatenate([vox, vox[::3]])                          # rows that share coordinates: no mirroring
    check_one_list(capi, twice, clouds.offsets_cube(3))


def test_empty_sides(capi):
    vox = random_cloud(55, n=300)
    none = np.zeros((0, 3), np.int32)
    for vin, vout in ((none, vox), (vox, none), (none, none)):
        imap, omap, knnz, kpos = capi.build_kernel_map(dev(vin), dev(vout), clouds.offsets_cube(3))
        assert imap.numel() == 0 and omap.numel() == 0 and not knnz.any() and not kpos.any()


def test_errors(capi):
    vox = random_cloud(56, n=500)
    with pytest.raises(ValueError, match="capacity"):
        capi.build_kernel_map(dev(vox), dev(vox), clouds.offsets_cube(3), capacity=len(vox))
    far = vox.copy()
    far[0, 0] = 1 << 20
    with pytest.raises(ValueError, match="outside"):
        capi.build_kernel_map(dev(far), dev(vox), clouds.offsets_cube(3))
    with pytest.raises(ValueError):
        capi.build_kernel_map(dev(vox).long(), dev(vox), clouds.offsets_cube(3))


def test_headline_cloud_full_size_and_feeds_the_kernels(capi, oracle):
    """200 k voxels, 27 offsets: the map of the headline benchmark, rebuilt on the device,
    equals the harness's bit for bit and drives a forward pass."""
    vox = clouds.indoor_cloud()
    imap, omap, knnz, kpos = check(capi, vox, vox, clouds.offsets_cube(3))
    assert imap.numel() == 2112390
    for g, w in zip(check_one_list(capi, vox, clouds.offsets_cube(3)), (imap, omap, knnz, kpos)):
        assert torch.equal(g, w)
    n = len(vox)
    x = torch.randn(n, 32, device="cuda").half()
    w = (torch.randn(27, 32, 32, device="cuda") * 0.05).half()
    out = torch.zeros(n, 32, device="cuda", dtype=torch.float16)
    plan = capi.Plan(kpos, imap, omap, n, n)
    capi.fusion_fwd(x, w, 0, out, kpos, None, imap, omap, False, False, plan=plan)
    torch.cuda.synchronize()
    # centre offset alone is x @ w[13]; all offsets: spot-check 64 rows against the C oracle's formula
    rows = np.arange(0, n, n // 64)[:64]
    kp = kpos.cpu().numpy(); im = imap.cpu().numpy(); om = omap.cpu().numpy()
    xf, wf = x.float().cpu().numpy(), w.float().cpu().numpy()
    ref = np.zeros((len(rows), 32))
    for k in range(27):
        o = om[kp[k]:kp[k + 1]]; i = im[kp[k]:kp[k + 1]]
        sel = np.isin(o, rows)
        for oo, ii in zip(o[sel], i[sel]):
            ref[np.searchsorted(rows, oo)] += xf[ii] @ wf[k]
    got = out[torch.from_numpy(rows).cuda()].float().cpu().numpy()
    assert np.allclose(got, ref, rtol=1e-2, atol=1e-2 * np.sqrt((ref ** 2).mean()))
