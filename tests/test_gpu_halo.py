"""The kernel that keeps a tile's neighbourhood rows in LDS (kernel policy 6, plans made with
voxel coordinates) against the CPU oracle: submanifold, strided and dense-grid maps, wide
destination sides, neighbourhoods larger than one LDS round, and the fall-back when a
tile's row list does not fit."""
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


def dev_coords(c):
    return torch.from_numpy(np.ascontiguousarray(c, dtype=np.int32)).cuda()


def run_and_check(capi, oracle, L, in_c, out_c, coord_bits, expect_halo=("fwd", "dgrad")):
    D = G.to_dev(L)
    ic, oc = dev_coords(in_c), dev_coords(out_c)
    if in_c is out_c:
        oc = ic
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"], in_coords=ic, out_coords=oc,
                     coord_bits=coord_bits)
    capi.set_kernel_policy(6)
    capi.profile_reset()
    capi.profile_enable(True)
    try:
        out = G.run_fwd(capi, D, plan=plan)
        gi, gw = G.run_bwd(capi, D, plan=plan)
    finally:
        capi.profile_enable(False)
        names = {n for n, _ in capi.profile_records()}
        capi.profile_reset()
        capi.set_kernel_policy(0)
    a = (L["knnz"], L["imap"], L["omap"])
    G.assert_close(out, oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"]), "fp16", "fwd")
    G.assert_close(gi, oracle.c_dgrad(L["out_grad"], L["kernel"], *a, L["n_in"]), "fp16", "dgrad")
    G.assert_close(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *a, L["k_vol"]), "fp16", "wgrad")
    for what in ("fwd", "dgrad"):
        ran = ("gms_halo_kernel(%s)" % what) in names
        assert ran == (what in expect_halo), (what, names)
    # a second call on top of the first: the rows are accumulated in place (which wave drew
    # which offset differs from run to run, so sums may differ in their last bit)
    capi.set_kernel_policy(6)
    out2 = G.run_fwd(capi, D, plan=plan, out_init=torch.from_numpy(out).cuda())
    capi.set_kernel_policy(0)
    G.assert_close(out2, 2.0 * out.astype(np.float32), "fp16", "accumulation in place")
    plan.close()


@pytest.mark.parametrize("shape", [(64, 64), (64, 128), (128, 64), (64, 192)], ids=lambda s: "%dx%d" % s)
def test_submanifold_surface_cloud(capi, oracle, shape):
    """12 k voxels of the indoor-like cloud: 64 source channels on either side take the
    kernel (forward needs c_in = 64, the input gradient c_out = 64)."""
    rng = np.random.default_rng(21)
    vox = clouds.cloud_indoor(clouds.rng_for(2), target=12000)
    L = clouds.submanifold_case(vox, shape[0], shape[1], np.float16, rng)
    expect = [w for w, c in (("fwd", shape[0]), ("dgrad", shape[1])) if c == 64]
    run_and_check(capi, oracle, L, vox, vox, 9, expect)


def test_strided_map_has_two_coordinate_sets(capi, oracle):
    rng = np.random.default_rng(22)
    vin = clouds.cloud_indoor(clouds.rng_for(2), target=20000)
    vout = clouds.downsample_coords(vin, 2)
    imap, omap, knnz, kpos = clouds.build_kernel_map(vin, vout, clouds.offsets_cube(2), stride=2)
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vin), len(vout), 64, 64, np.float16)
    run_and_check(capi, oracle, L, vin, vout, 9)


def test_dense_grid_needs_two_rounds(capi, oracle):
    """Every voxel of a 24^3 grid has all its neighbours: a tile of 128 rows reads more than the
    320 rows one LDS round holds, so its offsets are walked twice."""
    rng = np.random.default_rng(23)
    g = np.arange(24)
    vox = np.stack(np.meshgrid(g, g, g, indexing="ij"), -1).reshape(-1, 3).astype(np.int32)
    L = clouds.submanifold_case(vox, 64, 64, np.float16, rng)
    run_and_check(capi, oracle, L, vox, vox, 5)


def test_row_list_overflow_falls_back(capi, oracle):
    """Coordinates that have nothing to do with the map (here: shuffled) give tiles whose rows
    are scattered; their neighbourhood lists overflow, the tables are marked unusable and the
    usual kernels run."""
    rng = np.random.default_rng(24)
    g = np.arange(20)
    vox = np.stack(np.meshgrid(g, g, g, indexing="ij"), -1).reshape(-1, 3).astype(np.int32)
    L = clouds.submanifold_case(vox, 64, 64, np.float16, rng)
    wrong = vox[rng.permutation(len(vox))]
    run_and_check(capi, oracle, L, wrong, wrong, 5, expect_halo=())


def test_ragged_and_empty(capi, oracle):
    """Row counts that are no multiple of the tile, offsets without pairs, and coordinates over
    the full signed range (coord_bits = 0)."""
    rng = np.random.default_rng(25)
    vox = clouds.cloud_indoor(clouds.rng_for(2), target=1500)[:1333] - 300
    imap, omap, knnz, kpos = clouds.build_kernel_map(vox, vox, clouds.offsets_cube(3), skip_offset=4)
    L = clouds.make_layer(rng, imap, omap, knnz, kpos, len(vox), len(vox), 64, 64, np.float16)
    run_and_check(capi, oracle, L, vox, vox, 0)
