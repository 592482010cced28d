"""Pinned weights (fgms_weights_pin): the re-laid copy of a weight tensor is made once, later
calls find it, results do not change by a bit; pinning again after a write drops the copy; the
python extension pins again by itself when the tensor's version counter has moved."""
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
    c.weights_unpin(None)
    c.set_kernel_policy(0)


def layer(dtype, c_in, c_out, n=12000):
    rng = np.random.default_rng(77)
    coords = clouds.cloud_indoor(clouds.rng_for(5), target=n)
    return clouds.submanifold_case(coords, c_in, c_out, dtype, rng)


# shapes whose forward kernel reads re-laid weights: 128-column wave tiles (fp16), fp32, fp32 in
# the reference's tf32 mode (split-bf16 layout)
CASES = [(np.float16, 256, 256, False), (np.float32, 64, 64, False), (np.float32, 64, 64, True)]
IDS = ["fp16-256x256", "fp32-64x64", "fp32-64x64-tf32mode"]


@pytest.mark.parametrize("dtype,c_in,c_out,arch80", CASES, ids=IDS)
def test_pinned_copy_is_made_once_and_changes_nothing(capi, oracle, dtype, c_in, c_out, arch80):
    L = layer(dtype, c_in, c_out)
    D = G.to_dev(L)
    # (128-column wave tiles are for large layers: asked for by hand on this small one)
    capi.set_kernel_policy(3 if c_out == 256 else 0)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    base = G.run_fwd(capi, D, plan=plan, arch80=arch80)
    a = (L["knnz"], L["imap"], L["omap"])
    G.assert_close(base, oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"]), G.mode_of(dtype, arch80), "unpinned")

    capi.weights_pin(D["kernel"])
    h0 = capi.relaid_weights_hits()
    first = G.run_fwd(capi, D, plan=plan, arch80=arch80)      # makes the copy
    assert capi.relaid_weights_hits() == h0
    n0 = capi.allocation_count()
    second = G.run_fwd(capi, D, plan=plan, arch80=arch80)     # finds it
    assert capi.relaid_weights_hits() == h0 + 1, "the launch did not go through re-laid weights"
    assert capi.allocation_count() == n0
    assert np.array_equal(first, base) and np.array_equal(second, base)

    # another stream waits for the copy's fill and reads the same copy
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        third = G.run_fwd(capi, D, plan=plan, arch80=arch80)
    assert capi.relaid_weights_hits() == h0 + 2
    assert np.array_equal(third, base)

    # new bytes, pinned again: the copy is made anew
    w2 = (L["kernel"].astype(np.float32) * 0.5 + 0.01).astype(dtype)
    D["kernel"].copy_(torch.from_numpy(w2))
    capi.weights_pin(D["kernel"])
    fresh = G.run_fwd(capi, D, plan=plan, arch80=arch80)
    assert capi.relaid_weights_hits() == h0 + 2
    G.assert_close(fresh, oracle.c_fwd(L["in_feats"], w2, *a, L["n_out"]), G.mode_of(dtype, arch80), "pinned again")
    again = G.run_fwd(capi, D, plan=plan, arch80=arch80)
    assert capi.relaid_weights_hits() == h0 + 3 and np.array_equal(again, fresh)

    # unpinned: back to a copy per call
    capi.weights_unpin(D["kernel"])
    last = G.run_fwd(capi, D, plan=plan, arch80=arch80)
    assert capi.relaid_weights_hits() == h0 + 3 and np.array_equal(last, fresh)
    plan.close()
    capi.set_kernel_policy(0)


def test_pinned_fp16_forward_reads_the_copy_and_the_backward_call_does_not(capi, oracle):
    """64 -> 64 fp16 reads the weight tensor as it lies; pinned, the forward pass takes the kept
    re-laid copy instead (plain instead of transposing fragment reads), the backward call still
    reads the tensor itself."""
    L = layer(np.float16, 64, 64)
    D = G.to_dev(L)
    plan = capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    a = (L["knnz"], L["imap"], L["omap"])
    raw = G.run_fwd(capi, D, plan=plan)
    capi.weights_pin(D["kernel"])
    h0 = capi.relaid_weights_hits()
    out = G.run_fwd(capi, D, plan=plan)
    out2 = G.run_fwd(capi, D, plan=plan)
    assert capi.relaid_weights_hits() == h0 + 1
    gi, gw = G.run_bwd(capi, D, plan=plan)
    assert capi.relaid_weights_hits() == h0 + 1
    ref = oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"])
    G.assert_close(raw, ref, "fp16", "fwd, weights as they lie")
    G.assert_close(out, ref, "fp16", "fwd, pinned")
    assert np.array_equal(out, out2)
    G.assert_close(gi, oracle.c_dgrad(L["out_grad"], L["kernel"], *a, L["n_in"]), "fp16", "dgrad")
    capi.weights_unpin(D["kernel"])
    plan.close()


def test_backend_pins_again_when_the_version_counter_moves(capi, oracle):
    import FGMS.backend as B
    L = layer(np.float16, 256, 256, n=8000)
    D = G.to_dev(L)
    a = (L["knnz"], L["imap"], L["omap"])
    w = D["kernel"]

    def fwd():
        out = torch.zeros(D["n_out"], D["c_out"], dtype=w.dtype, device="cuda")
        B.fgms_fusion_fwd_cuda(D["in_feats"], w, 0, out, D["kpos"], D["kpos"][:0], D["imap"], D["omap"], False, False)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    capi.set_kernel_policy(3)
    B.fgms_weights_pin(w)
    h0 = capi.relaid_weights_hits()
    y0 = fwd()
    y1 = fwd()
    assert capi.relaid_weights_hits() == h0 + 1 and np.array_equal(y0, y1)
    G.assert_close(y0, oracle.c_fwd(L["in_feats"], L["kernel"], *a, L["n_out"]), "fp16", "pinned through the backend")
    w.mul_(0.5)                                    # bumps the version counter
    y2 = fwd()
    assert capi.relaid_weights_hits() == h0 + 1, "the stale copy was used"
    G.assert_close(y2, oracle.c_fwd(L["in_feats"], (L["kernel"].astype(np.float32) * 0.5).astype(np.float16), *a, L["n_out"]),
                   "fp16", "after an in-place update")
    y3 = fwd()
    assert capi.relaid_weights_hits() == h0 + 2 and np.array_equal(y2, y3)
    B.fgms_weights_unpin(w)
    y4 = fwd()
    assert capi.relaid_weights_hits() == h0 + 2 and np.array_equal(y2, y4)
    capi.set_kernel_policy(0)
