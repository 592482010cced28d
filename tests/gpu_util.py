"""Shared helpers of the GPU parity tests: move a numpy layer to the card, call
the C ABI (fgms_amd.capi) and compare with the CPU oracle."""
import numpy as np
import torch

RTOL = {"fp32": 1e-5, "tf32": 1e-2, "fp16": 1e-2}


def to_dev(L):
    d = {}
    for k, v in L.items():
        d[k] = torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) and k != "knnz" else v
    d["knnz_host"] = torch.from_numpy(L["knnz"].astype(np.int32))
    return d


def assert_close(got, ref, mode, what=""):
    """|got - ref| <= rtol * |ref| + rtol * rms(ref): the relative tolerance the
    task states (fp32 1e-5, tf32 / fp16 1e-2), with the absolute floor tied to
    the result's own scale so near-zero sums of signed terms are judged fairly
    (the reference's script uses rtol=1e-2, atol=1e-4, cpu-check.py:127)."""
    rtol = RTOL[mode]
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.all(np.isfinite(got)), what + ": non-finite values"
    scale = float(np.sqrt(np.mean(ref ** 2))) if ref.size else 0.0
    err = np.abs(got - ref)
    bound = rtol * np.abs(ref) + rtol * scale
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError("%s: %d / %d outside tolerance (worst at %s: got %r want %r, rms %g)"
                             % (what, int(bad.sum()), err.size, i, got[i], ref[i], scale))


def mode_of(dtype, arch80=False):
    if dtype == np.float16 or dtype == torch.float16:
        return "fp16"
    return "tf32" if arch80 else "fp32"


def run_fwd(capi, D, fused=True, separate_mid=False, arch80=False, plan=None, out_init=None):
    out = (torch.zeros(D["n_out"], D["c_out"], dtype=D["in_feats"].dtype, device="cuda")
           if out_init is None else out_init.clone())
    if fused:
        capi.fusion_fwd(D["in_feats"], D["kernel"], 0, out, D["kpos"], None, D["imap"], D["omap"],
                        separate_mid, arch80, plan=plan)
    else:
        capi.seq_fwd(D["in_feats"], D["kernel"], len(D["imap"]), out, D["knnz_host"], D["kpos"],
                     D["imap"], D["omap"], separate_mid, arch80, plan=plan)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def run_bwd(capi, D, plan=None, split=False, arch80=False):
    gi = torch.zeros(D["n_in"], D["c_in"], dtype=D["in_feats"].dtype, device="cuda")
    gw = torch.zeros_like(D["kernel"])
    if split:
        capi.dgrad(D["out_grad"], D["kernel"], gi, D["kpos"], D["imap"], D["omap"], plan=plan)
        capi.wgrad(D["in_feats"], D["out_grad"], gw, D["kpos"], D["imap"], D["omap"], plan=plan)
    else:
        capi.bwd(D["out_grad"], D["in_feats"], D["kernel"], 0, gi, gw, D["kpos"], None,
                 D["imap"], D["omap"], False, arch80, plan=plan)
    torch.cuda.synchronize()
    return gi.cpu().numpy(), gw.cpu().numpy()
