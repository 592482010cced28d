"""The on-disk layer-sample format of the reference's scripts (cpu-check.py:83-94,
spconv-test.py:64-73): writer / reader round trip and the reader's consistency checks.
No sample data ships with the reference, so the files are written here from the
package's own generators."""
import numpy as np
import pytest
import torch

from fgms_amd import clouds, samples


def small_layer(seed=3, c_in=8, c_out=16, dtype=np.float32):
    rng = np.random.default_rng(seed)
    pts = rng.integers(0, 12, size=(400, 3))
    vox = clouds.dedup(pts, 12)
    return clouds.submanifold_case(vox, c_in, c_out, dtype, rng)


def test_checked_sample_round_trip(tmp_path):
    L = small_layer()
    f = tmp_path / "layer.pt"
    samples.save_sample(f, L)
    s = samples.load_sample(f)
    assert (s.n_in, s.n_out, s.k_vol, s.c_in, s.c_out) == (L["n_in"], L["n_out"], 27, 8, 16)
    assert s.sum_nnz == len(L["imap"]) and s.submanifold
    assert s.knnz.dtype == torch.int32 and s.knnz.device.type == "cpu"
    assert np.array_equal(s.imap.numpy(), L["imap"]) and np.array_equal(s.omap.numpy(), L["omap"])
    assert np.array_equal(s.kpos.numpy(), L["kpos"]) and np.array_equal(s.knnz.numpy(), L["knnz"])
    assert np.array_equal(s.in_feats.numpy(), L["in_feats"]) and np.array_equal(s.kernel.numpy(), L["kernel"])


def test_timed_sample_has_the_map_only(tmp_path):
    L = small_layer(c_in=4, c_out=32)
    f = tmp_path / "map.pt"
    samples.save_sample(f, L, with_tensors=False)
    s = samples.load_sample(f)
    assert s.in_feats is None and s.kernel is None
    assert (s.n_in, s.c_in, s.c_out, s.k_vol) == (L["n_in"], 4, 32, 27)


def test_reader_flattens_and_narrows_the_maps(tmp_path):
    """The scripts reshape imap / omap themselves (cpu-check.py:93-94): files may hold them
    as columns, or as int64."""
    L = small_layer()
    f = tmp_path / "cols.pt"
    samples.save_sample(f, L)
    d = torch.load(f, weights_only=True)
    d["imap"] = d["imap"].reshape(-1, 1).long()
    d["omap"] = d["omap"].reshape(1, -1).long()
    d["sum_nnz"] = torch.tensor(d["sum_nnz"])
    torch.save(d, f)
    s = samples.load_sample(f)
    assert s.imap.dtype == torch.int32 and s.imap.dim() == 1 and np.array_equal(s.imap.numpy(), L["imap"])
    assert s.omap.dtype == torch.int32 and s.omap.dim() == 1 and np.array_equal(s.omap.numpy(), L["omap"])


@pytest.mark.parametrize("breakage", ["kpos", "range", "missing", "count", "shape", "notdict"])
def test_reader_rejects_inconsistent_files(tmp_path, breakage):
    L = small_layer()
    f = tmp_path / "bad.pt"
    samples.save_sample(f, L)
    d = torch.load(f, weights_only=True)
    if breakage == "kpos":
        d["kpos"][3] += 1
    elif breakage == "range":
        d["omap"][5] = L["n_out"]
    elif breakage == "missing":
        del d["knnz"]
    elif breakage == "count":
        d["sum_nnz"] += 1
    elif breakage == "shape":
        d["kernel"] = d["kernel"][:, :4]
    else:
        d = [1, 2, 3]
    torch.save(d, f)
    with pytest.raises(ValueError):
        samples.load_sample(f)
