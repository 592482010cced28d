"""Caller-side helpers (fgms_amd.harness) and the synthetic clouds / kernel maps."""
import numpy as np
import torch

from fgms_amd import clouds, harness


def test_kpos_quantized_matches_reference_formula():
    # cpu-check.py:6-14 on tensors
    knnz = torch.tensor([5, 0, 256, 257, 1000], dtype=torch.int32)
    kpos = torch.zeros(6, dtype=torch.int32)
    kpos[1:] = torch.cumsum(knnz, 0)
    qk, total = harness.kpos_quantized(knnz, kpos, 5, 256)
    assert qk.dtype == kpos.dtype
    assert qk.tolist() == [0, 256, 256, 512, 1024, 2048] and total == 2048
    qk2, total2 = harness.kpos_quantized(knnz.numpy(), kpos.numpy(), 5, 256)
    assert qk2.tolist() == qk.tolist() and total2 == total


def test_remove_mid_splices_identity():
    # spconv-test.py:17-38
    nnz, k_vol = 6, 3
    knnz = torch.tensor([2, 0, 3], dtype=torch.int32)
    kpos = torch.tensor([0, 2, 2, 5], dtype=torch.int32)
    imap = torch.tensor([1, 2, 0, 3, 4], dtype=torch.int32)
    omap = torch.tensor([0, 1, 3, 4, 5], dtype=torch.int32)
    qk, qsum, kpos_new, im, om = harness.remove_mid(nnz, knnz, kpos, k_vol, 4, imap, omap)
    assert knnz.tolist() == [2, 6, 3]
    assert kpos_new.tolist() == [0, 2, 8, 11]
    assert im.tolist() == [1, 2, 0, 1, 2, 3, 4, 5, 0, 3, 4]
    assert om.tolist() == [0, 1, 0, 1, 2, 3, 4, 5, 3, 4, 5]
    assert qk.tolist() == [0, 4, 12, 16] and qsum == 16
    assert im.dtype == torch.int32


def test_remove_mid_keeps_nonzero_mid_count():
    knnz = np.array([1, 2, 1], np.int32)
    kpos = np.array([0, 1, 3, 4], np.int32)
    imap = np.arange(4, dtype=np.int32)
    omap = np.arange(4, dtype=np.int32)
    _, _, kpos_new, im, _ = harness.remove_mid(3, knnz, kpos, 3, 2, imap, omap)
    # as in the reference, a non-empty centre count is left alone
    assert knnz.tolist() == [1, 2, 1] and kpos_new.tolist() == [0, 1, 3, 4] and len(im) == 7


def test_channel_transform():
    f = torch.arange(6.).reshape(2, 3)
    w = torch.arange(2 * 3 * 2.).reshape(2, 3, 2)
    f2, w2 = harness.channel_transform(f, w, 5, 3)
    assert f2.shape == (2, 5) and w2.shape == (2, 5, 3)
    assert torch.equal(f2[:, 3:], f[:, :2]) and torch.equal(w2[:, :3, 2], w[:, :, 0])
    assert f2.is_contiguous() and w2.is_contiguous()


def test_kernel_map_equals_bruteforce():
    rng = np.random.default_rng(0)
    pts = clouds.dedup(rng.uniform(0, 9, (400, 3)), 9)
    for offs, stride, outc in ((clouds.offsets_cube(3), 1, pts),
                               (clouds.offsets_cube(2), 2, clouds.downsample_coords(pts, 2))):
        a = clouds.build_kernel_map(pts, outc, offs, stride)
        b = clouds.build_kernel_map_bruteforce(pts, outc, offs, stride)
        for x, y in zip(a, b):
            assert x.dtype == np.int32 and np.array_equal(x, y)


def test_kernel_map_properties():
    L = clouds.config_case(1, scale=0.1)
    k_vol, n = L["k_vol"], L["n_in"]
    assert k_vol == 27 and L["knnz"][13] == n          # centre offset = identity
    a, b = L["kpos"][13], L["kpos"][14]
    assert np.array_equal(L["imap"][a:b], np.arange(n)) and np.array_equal(L["omap"][a:b], np.arange(n))
    assert np.array_equal(L["knnz"], L["knnz"][::-1])  # offset symmetry of a submanifold map
    for k in range(k_vol):                             # rows unique inside an offset
        o = L["omap"][L["kpos"][k]:L["kpos"][k + 1]]
        assert len(np.unique(o)) == len(o)
    assert L["kpos"][-1] == len(L["imap"]) == len(L["omap"])


def test_stride2_map_has_one_pair_per_input():
    L = clouds.config_case(4, scale=0.05)
    assert len(L["imap"]) == L["n_in"] and np.array_equal(np.sort(L["imap"]), np.arange(L["n_in"]))
    U = clouds.config_case(4, "up", scale=0.05)
    assert U["n_in"] == L["n_out"] and U["n_out"] == L["n_in"] and U["c_in"] == 128 and U["c_out"] == 64


def test_clouds_are_deterministic_and_sized():
    a = clouds.config_case(3, scale=0.05)
    b = clouds.config_case(3, scale=0.05)
    assert np.array_equal(a["imap"], b["imap"]) and np.array_equal(a["in_feats"], b["in_feats"])
    assert a["in_feats"].dtype == np.float16 and a["c_in"] == 128
    s = clouds.config_case(5, "skinny", scale=0.05)
    assert s["c_in"] == 4 and s["c_out"] == 32 and s["in_feats"].min() >= 0 and s["in_feats"].max() <= 1  # fp16 rounding can reach 1.0
    w = clouds.config_case(5, "wide", scale=0.05)
    assert w["c_in"] == 256 and w["n_in"] == 2500
    bound = 1 / np.sqrt(27 * 256)
    assert np.abs(w["kernel"].astype(np.float32)).max() <= bound * 1.001


def test_full_size_clouds():
    v = clouds.indoor_cloud()
    assert len(v) == 200000 and v.min() >= 0 and v.max() < 512
    imap, omap, knnz, kpos = clouds.build_kernel_map(v, v, clouds.offsets_cube(3))
    assert 8.0 < len(imap) / len(v) < 12.0            # ~9-10 active neighbours per voxel
    lid = clouds.cloud_lidar(clouds.rng_for(3))
    assert 100000 < len(lid) < 140000
