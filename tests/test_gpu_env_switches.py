"""The library reads a few switches from the environment once per process (they exist for
comparisons and experiments).  Each alternative path still has to give the right answer:
a child process per setting runs forward and backward of four layers through the C ABI,
checks them against the CPU oracle and reports which kernels ran."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import json, sys
import numpy as np, torch
sys.path.insert(0, %r)
from fgms_amd import capi
from oracle import fgms_oracle as oracle
from tests import gpu_util as G
from tests.test_gpu_parity import layer
names = set()
for shape, dtype in (((64, 64), np.float16), ((128, 128), np.float16), ((64, 128), np.float16), ((32, 64), np.float32)):
    L = layer(41, shape[0], shape[1], dtype)
    D = G.to_dev(L)
    capi.set_kernel_policy(4)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    mode = G.mode_of(L["in_feats"].dtype, False)
    args = (L["knnz"], L["imap"], L["omap"])
    capi.profile_reset(); capi.profile_enable(True)
    out = G.run_fwd(capi, D, fused=True, plan=plan)
    for _ in range(2):      # twice: scratch must come back clean
        gi, gw = G.run_bwd(capi, D, plan=plan)
        G.assert_close(gi, oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"]), mode, "dgrad")
        G.assert_close(gw, oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"]), mode, "wgrad")
    want = oracle.np_fwd(L["in_feats"], L["kernel"], *args, L["n_out"])
    G.assert_close(out, want, mode, "fwd")
    if dtype == np.float32:
        G.assert_close(G.run_fwd(capi, D, fused=True, arch80=True, plan=plan), want, "tf32", "tf32-mode fwd")
    capi.profile_enable(False)
    names |= {n for n, _ in capi.profile_records()}
    plan.close()
print("KERNELS " + json.dumps(sorted(names)))
""" % ROOT


def run_child(env_extra):
    env = dict(os.environ)
    env.update(env_extra)
    r = subprocess.run([sys.executable, "-c", CHILD], env=env, cwd=ROOT, stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-3000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("KERNELS ")][-1]
    return set(json.loads(line[len("KERNELS "):]))


def test_default_settings_run_the_backward_in_one_grid():
    names = run_child({})
    assert "bwd_fused_kernel" in names and "wgrad_wave_kernel" not in names, names
    assert "gms_rows_kernel(fwd, bf16x3)" in names, names


def test_tf32_mode_on_fp32_matrix_instructions():
    """FGMS_SPLIT_BF16=0: fp32 tensors in tf32 mode run the fp32 kernels."""
    names = run_child({"FGMS_SPLIT_BF16": "0"})
    assert "gms_rows_kernel(fwd, bf16x3)" not in names and "gms_rows_kernel(fwd)" in names, names


def test_backward_on_two_launches():
    """FGMS_FUSED_BWD=0: weight gradient first (its launch re-lays the weights for the input
    gradient), then the input gradient (its launch rounds an fp16 weight gradient)."""
    names = run_child({"FGMS_FUSED_BWD": "0"})
    assert "bwd_fused_kernel" not in names, names
    assert {"gms_rows_kernel(dgrad)", "wgrad_wave_kernel", "wgrad_kernel"} <= names, names


def test_weights_re_laid_instead_of_read_as_they_lie():
    """FGMS_RAW_WEIGHTS=0: every pass works on a re-laid copy of the weights (which also
    rules out the one-grid backward, whose input gradient reads them as they lie)."""
    names = run_child({"FGMS_RAW_WEIGHTS": "0"})
    assert "bwd_fused_kernel" not in names and "gms_rows_kernel(fwd)" in names, names


def test_small_launches_on_256_row_tiles():
    """FGMS_HALF_TILES=0: launches too small to fill the chip keep tiles of 256 rows instead of
    128 (the test clouds are that small, so the default run above went through the 128-row
    tiles and this one through the others; both meet the oracle)."""
    names = run_child({"FGMS_HALF_TILES": "0"})
    assert "bwd_fused_kernel" in names and "gms_rows_kernel(fwd)" in names, names


FULL_SIZE_CHILD = r"""
import sys
import numpy as np, torch
sys.path.insert(0, %r)
import bench
from fgms_amd import capi
from oracle import fgms_oracle as oracle
from tests import gpu_util as G
L, passes, arch80 = bench.make_case("cfg2-indoor200k-k27-64x64-tf32-fwd", 1.0)
assert arch80 and L["in_feats"].dtype == np.float32 and L["n_in"] >= 190000
D = G.to_dev(L)
plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
capi.profile_reset(); capi.profile_enable(True)
out = G.run_fwd(capi, D, fused=True, arch80=True, plan=plan)
capi.profile_enable(False)
names = sorted({n for n, _ in capi.profile_records()})
want = oracle.c_fwd(L["in_feats"], L["kernel"], L["knnz"], L["imap"], L["omap"], L["n_out"])
G.assert_close(out, want, "tf32", "cfg2 at full size, tf32 mode on fp32 matrix instructions")
G.assert_close(out, want, "fp32", "the same, held to the fp32 tolerance (the arithmetic is fp32)")
print("KERNELS " + " ".join(names))
""" % ROOT


def test_tf32_mode_on_fp32_matrix_instructions_at_full_size():
    """The arithmetic the task prescribes for tf32 mode (fp32 MFMA, FGMS_SPLIT_BF16=0) on the
    200 000-voxel cloud of BASELINE config 2, element by element against the C oracle."""
    env = dict(os.environ)
    env["FGMS_SPLIT_BF16"] = "0"
    r = subprocess.run([sys.executable, "-c", FULL_SIZE_CHILD], env=env, cwd=ROOT, stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("KERNELS ")][-1]
    assert "bf16x3" not in line and "gms_rows_kernel(fwd)" in line, line
