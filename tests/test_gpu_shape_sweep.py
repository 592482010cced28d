"""Every combination of the channel counts a voxel network uses (and a few it does not:
3, 12, 24, 160), fp16 and fp32, submanifold and strided, with and without a plan: forward,
input gradient and weight gradient through the C ABI against the CPU oracle.  The dispatch
has a dozen branches (skinny, output-stationary with 64- and 128-column wave tiles, raw or
re-laid weights, pair-stationary, generic, three weight-gradient kernels, backward in one
call); this walks all of them at sizes the oracle finishes in milliseconds."""
import itertools

import numpy as np
import pytest
import torch

from tests import gpu_util as G
from tests.test_gpu_parity import layer

pytestmark = pytest.mark.gpu

CHANNELS = [3, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 160, 256]


@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["fp16", "fp32"])
def test_all_channel_shapes(oracle, dtype):
    from fgms_amd import capi
    capi.set_kernel_policy(0)
    failures, n = [], 0
    for ci, co in itertools.product(CHANNELS, CHANNELS):
        if ci * co > 128 * 160:
            continue
        for kind in ("subm", "down"):
            if kind == "down" and (ci + co) % 3:          # a third of the shapes also strided
                continue
            L = layer(100 + n, ci, co, dtype, kind)
            n += 1
            D = G.to_dev(L)
            mode = G.mode_of(L["in_feats"].dtype, False)
            args = (L["knnz"], L["imap"], L["omap"])
            ref = (oracle.np_fwd(L["in_feats"], L["kernel"], *args, L["n_out"]),
                   oracle.np_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"]),
                   oracle.np_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"]))
            for use_plan in (True, False):
                plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"]) if use_plan else None
                try:
                    out = G.run_fwd(capi, D, fused=True, plan=plan)
                    gi, gw = G.run_bwd(capi, D, plan=plan)
                    for got, want, what in zip((out, gi, gw), ref, ("fwd", "dgrad", "wgrad")):
                        G.assert_close(got, want, mode, what)
                except AssertionError as e:
                    failures.append("%d -> %d %s %s: %s" % (ci, co, kind, "plan" if use_plan else "no plan", str(e)[:160]))
                finally:
                    if plan is not None:
                        plan.close()
    torch.cuda.synchronize()
    assert n > 200 and not failures, "\n".join(failures[:20])
