"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py
from torch's dense conv3d / conv_transpose3d and autograd in float64): the CPU
oracle must reproduce them, and so must the HIP kernels."""
import glob
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def load(path):
    z = np.load(path)
    return {k: (z[k].item() if z[k].shape == () else z[k]) for k in z.files}


def test_fixtures_exist():
    assert len(FIXTURES) >= 4


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p)[:-4] for p in FIXTURES])
def test_oracle_reproduces_golden(oracle, path):
    z = load(path)
    args = (z["knnz"], z["imap"], z["omap"])
    tol = dict(rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(oracle.c_fwd(z["in_feats"], z["kernel"], *args, z["n_out"]), z["out"], **tol)
    np.testing.assert_allclose(oracle.c_dgrad(z["out_grad"], z["kernel"], *args, z["n_in"]), z["in_grad"], **tol)
    np.testing.assert_allclose(oracle.c_wgrad(z["in_feats"], z["out_grad"], *args, len(z["knnz"])),
                               z["kernel_grad"], rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(oracle.np_fwd(z["in_feats"], z["kernel"], *args, z["n_out"]), z["out"],
                               rtol=1e-6, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p)[:-4] for p in FIXTURES])
def test_gpu_reproduces_golden(path, dtype):
    import torch
    from fgms_amd import capi
    from tests import gpu_util as G
    z = load(path)
    L = dict(in_feats=z["in_feats"].astype(dtype), kernel=z["kernel"].astype(dtype),
             out_grad=z["out_grad"].astype(dtype), imap=z["imap"], omap=z["omap"], knnz=z["knnz"],
             kpos=z["kpos"], n_in=z["n_in"], n_out=z["n_out"], c_in=z["kernel"].shape[1],
             c_out=z["kernel"].shape[2], k_vol=len(z["knnz"]))
    D = G.to_dev(L)
    mode = G.mode_of(dtype)
    for use_plan in (False, True):
        plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"]) if use_plan else None
        G.assert_close(G.run_fwd(capi, D, plan=plan), z["out"], mode, "fwd")
        gi, gw = G.run_bwd(capi, D, plan=plan)
        G.assert_close(gi, z["in_grad"], mode, "dgrad")
        G.assert_close(gw, z["kernel_grad"], mode, "wgrad")
