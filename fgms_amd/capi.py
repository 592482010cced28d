"""ctypes binding of ``include/fgms.h`` (libfgms_hip.so).

The functions take torch GPU tensors only to read their ``data_ptr()`` and
shapes; nothing torch-specific crosses the C boundary.  There is no CPU
fallback: if the shared library is missing or a call fails this raises.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfgms_hip.so")

F32, F16 = 0, 1
SYMBOLS = [
    "fgms_version", "fgms_last_error", "fgms_plan_create", "fgms_plan_check", "fgms_plan_transposed", "fgms_plan_destroy",
    "fgms_plan_usable", "fgms_plan_stats", "fgms_fusion_fwd", "fgms_fwd", "fgms_bwd", "fgms_dgrad",
    "fgms_wgrad", "fgms_wgrad_static", "fgms_set_kernel_policy", "fgms_profile_enable", "fgms_profile_read",
    "fgms_profile_reset", "fgms_probe_gather", "fgms_build_kernel_map", "fgms_allocation_count",
    "fgms_weights_pin", "fgms_weights_unpin", "fgms_relaid_weights_hits",
]

_lib = None


class FgmsError(RuntimeError):
    pass


class StalePlanError(FgmsError):
    """FGMS_E_STALE: the pair lists were rewritten after the plan was made."""


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FgmsError("%s is missing: run `python -m fgms_amd.build` (there is no CPU fallback)"
                        % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.fgms_version.restype = ctypes.c_char_p
    L.fgms_last_error.restype = ctypes.c_char_p
    L.fgms_plan_create.argtypes = [ctypes.POINTER(vp), vp, vp, vp, i64, i64, i32, i64, vp]
    L.fgms_plan_transposed.argtypes = [ctypes.POINTER(vp), vp]
    L.fgms_plan_check.argtypes = [vp, vp, i32]
    L.fgms_plan_destroy.argtypes = [vp]
    L.fgms_plan_destroy.restype = None
    L.fgms_plan_usable.argtypes = [vp, i32]
    L.fgms_plan_stats.argtypes = [vp, ctypes.POINTER(ctypes.c_int64)]
    L.fgms_plan_stats.restype = i32
    L.fgms_fusion_fwd.argtypes = [vp, vp, i32, vp, vp, vp, vp, vp, i32, i32,
                                  i64, i64, i32, i32, i32, i64, i32, vp, vp]
    L.fgms_fwd.argtypes = [vp, vp, i32, vp, vp, vp, vp, vp, i32, i32,
                           i64, i64, i32, i32, i32, i64, i32, vp, vp]
    L.fgms_bwd.argtypes = [vp, vp, vp, i32, vp, vp, vp, vp, vp, vp, i32, i32,
                           i64, i64, i32, i32, i32, i64, i32, vp, vp]
    L.fgms_dgrad.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i32, i32, i32, i64, i32, vp, vp]
    L.fgms_wgrad.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i32, i32, i32, i64, i32, vp, vp]
    L.fgms_wgrad_static.argtypes = L.fgms_wgrad.argtypes
    L.fgms_build_kernel_map.argtypes = [vp, i64, vp, i64, vp, i32, i32, i32, vp, vp, i64, vp, vp,
                                        ctypes.POINTER(ctypes.c_int64), vp]
    L.fgms_build_kernel_map.restype = i32
    L.fgms_probe_gather.argtypes = [vp, i32, i32, i32, vp, vp]
    L.fgms_probe_gather.restype = i32
    L.fgms_set_kernel_policy.argtypes = [i32]
    L.fgms_set_kernel_policy.restype = None
    L.fgms_allocation_count.restype = ctypes.c_longlong
    L.fgms_relaid_weights_hits.restype = ctypes.c_longlong
    L.fgms_weights_pin.argtypes = [vp]
    L.fgms_weights_pin.restype = i32
    L.fgms_weights_unpin.argtypes = [vp]
    L.fgms_weights_unpin.restype = i32
    L.fgms_profile_enable.argtypes = [i32]
    L.fgms_profile_enable.restype = None
    L.fgms_profile_reset.restype = None
    L.fgms_profile_read.argtypes = [i32, ctypes.c_char_p, i32, ctypes.POINTER(ctypes.c_float)]
    _lib = L
    return L


def version():
    return lib().fgms_version().decode()


def _check(rc):
    if rc != 0:
        msg = lib().fgms_last_error().decode()
        if rc == -1:
            raise ValueError(msg)
        if rc == -4:
            raise StalePlanError(msg)
        raise FgmsError("fgms error %d: %s" % (rc, msg))


def _dtype(t):
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.float32:
        return F32
    raise ValueError("FGMS handles float32 and float16 tensors")


def _p(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None and t.numel() else None)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(t, name, dtype=None):
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError("%s must be a contiguous GPU tensor" % name)
    if dtype is not None and t.dtype != dtype:
        raise ValueError("%s must be %s" % (name, dtype))


def set_kernel_policy(policy):
    """0 automatic, 1 generic kernels only, 2 pair-stationary MFMA even with a plan."""
    lib().fgms_set_kernel_policy(int(policy))


def allocation_count():
    """Device / pinned allocations the library has made so far (``fgms_allocation_count``)."""
    return int(lib().fgms_allocation_count())


def weights_pin(kernel):
    """Promise that ``kernel``'s bytes stay as they are until the next pin / unpin of the tensor:
    the library keeps its re-laid copies (``fgms_weights_pin``).  The caller keeps the tensor alive."""
    _check(lib().fgms_weights_pin(ctypes.c_void_p(kernel.data_ptr())))


def weights_unpin(kernel=None):
    """Drop the re-laid copies of ``kernel`` (None: of every pinned tensor on the current device)."""
    _check(lib().fgms_weights_unpin(ctypes.c_void_p(kernel.data_ptr() if kernel is not None else None)))


def relaid_weights_hits():
    return int(lib().fgms_relaid_weights_hits())


def profile_enable(on=True):
    lib().fgms_profile_enable(int(on))


def profile_reset():
    lib().fgms_profile_reset()


def profile_records():
    """[(kernel name, milliseconds)] of every main-kernel launch since the last
    reset, timed with HIP events on the launch stream."""
    out, i = [], 0
    name = ctypes.create_string_buffer(96)
    ms = ctypes.c_float()
    while lib().fgms_profile_read(i, name, 96, ctypes.byref(ms)) == 0:
        out.append((name.value.decode(), float(ms.value)))
        i += 1
    return out


class Plan:
    """Neighbour tables for one kernel map (``fgms_plan_create``)."""

    def __init__(self, kpos, in_map, out_map, n_in, n_out):
        for t, n in ((kpos, "kpos"), (in_map, "in_map"), (out_map, "out_map")):
            _need(t, n, torch.int32)
        self._keep = (kpos, in_map, out_map)
        self._h = ctypes.c_void_p()
        _check(lib().fgms_plan_create(ctypes.byref(self._h), _p(kpos), _p(in_map), _p(out_map),
                                      int(n_in), int(n_out), kpos.numel() - 1, in_map.numel(),
                                      _stream()))

    @property
    def handle(self):
        return self._h

    def transposed(self):
        """A plan for the same pairs with in_map and out_map exchanged (the transposed
        convolution's map); shares this plan's tables."""
        view = Plan.__new__(Plan)
        view._keep = (self,) + tuple(self._keep)
        view._h = ctypes.c_void_p()
        _check(lib().fgms_plan_transposed(ctypes.byref(view._h), self._h))
        return view

    def check(self, with_next_launch=False):
        """Has the pair lists checked against the fingerprint the plan was built with
        (``fgms_plan_check``): by a small kernel queued now, or as part of the next launch that
        reads the plan; raises StalePlanError once an earlier check has found them changed."""
        _check(lib().fgms_plan_check(self._h, _stream(), int(with_next_launch)))

    def usable(self, for_dgrad=False):
        return bool(lib().fgms_plan_usable(self._h, int(for_dgrad)))

    def stats(self):
        """dict(pairs, blocks_fwd, blocks_dgrad, pair_view_rows) as counted by the build; the
        output-stationary kernels run 64 row slots per (64-row block, offset) in use."""
        out = (ctypes.c_int64 * 4)()
        _check(lib().fgms_plan_stats(self._h, out))
        return {"pairs": out[0], "blocks_fwd": out[1], "blocks_dgrad": out[2], "pair_view_rows": out[3]}

    def close(self):
        if self._h:
            lib().fgms_plan_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _ph(plan):
    return plan.handle if plan is not None else ctypes.c_void_p()


def _check_feats(in_feats, kernel):
    if in_feats.shape[1] != kernel.shape[1]:
        raise ValueError("Input feature size and kernel size mismatch")


def fusion_fwd(in_feats, kernel, sum_nnz, out_feats, kpos, qkpos, in_map, out_map,
               separate_mid, arch80, plan=None):
    _check_feats(in_feats, kernel)
    for t, n in ((in_feats, "in_feats"), (kernel, "kernel"), (out_feats, "out_feats")):
        _need(t, n, in_feats.dtype)
    for t, n in ((kpos, "kpos"), (in_map, "in_map"), (out_map, "out_map")):
        _need(t, n, torch.int32)
    _check(lib().fgms_fusion_fwd(
        _p(in_feats), _p(kernel), int(sum_nnz), _p(out_feats), _p(kpos), _p(qkpos), _p(in_map),
        _p(out_map), int(separate_mid), int(arch80), in_feats.shape[0], out_feats.shape[0],
        kernel.shape[1], kernel.shape[2], kernel.shape[0], in_map.numel(), _dtype(in_feats),
        _ph(plan), _stream()))


def seq_fwd(in_feats, kernel, sum_nnz, out_feats, kernel_nnz, kernel_pos, in_map, out_map,
            separate_mid, arch80, plan=None):
    _check_feats(in_feats, kernel)
    if kernel_nnz.is_cuda:
        raise ValueError("kernel_nnz must be a CPU int32 tensor")
    knnz = kernel_nnz.to(torch.int32).contiguous()
    for t, n in ((in_feats, "in_feats"), (kernel, "kernel"), (out_feats, "out_feats")):
        _need(t, n, in_feats.dtype)
    for t, n in ((kernel_pos, "kernel_pos"), (in_map, "in_map"), (out_map, "out_map")):
        _need(t, n, torch.int32)
    _check(lib().fgms_fwd(
        _p(in_feats), _p(kernel), int(sum_nnz), _p(out_feats), ctypes.c_void_p(knnz.data_ptr()),
        _p(kernel_pos), _p(in_map), _p(out_map), int(separate_mid), int(arch80),
        in_feats.shape[0], out_feats.shape[0], kernel.shape[1], kernel.shape[2], kernel.shape[0],
        in_map.numel(), _dtype(in_feats), _ph(plan), _stream()))


def bwd(out_grad, in_feats, kernel, sum_nnz, in_grad, kernel_grad, kpos, qkpos, in_map,
        out_map, separate_mid, arch80, plan=None):
    _check_feats(in_feats, kernel)
    for t, n in ((out_grad, "out_feats_grad"), (in_feats, "in_feats"), (kernel, "kernel"),
                 (in_grad, "in_feats_grad"), (kernel_grad, "kernel_grad")):
        _need(t, n, in_feats.dtype)
    for t, n in ((kpos, "kpos"), (in_map, "in_map"), (out_map, "out_map")):
        _need(t, n, torch.int32)
    _check(lib().fgms_bwd(
        _p(out_grad), _p(in_feats), _p(kernel), int(sum_nnz), _p(in_grad), _p(kernel_grad),
        _p(kpos), _p(qkpos), _p(in_map), _p(out_map), int(separate_mid), int(arch80),
        in_feats.shape[0], out_grad.shape[0], kernel.shape[1], kernel.shape[2], kernel.shape[0],
        in_map.numel(), _dtype(in_feats), _ph(plan), _stream()))


def dgrad(out_grad, kernel, in_grad, kpos, in_map, out_map, plan=None):
    for t, n in ((out_grad, "out_feats_grad"), (kernel, "kernel"), (in_grad, "in_feats_grad")):
        _need(t, n, out_grad.dtype)
    _check(lib().fgms_dgrad(
        _p(out_grad), _p(kernel), _p(in_grad), _p(kpos), _p(in_map), _p(out_map),
        in_grad.shape[0], out_grad.shape[0], kernel.shape[1], kernel.shape[2], kernel.shape[0],
        in_map.numel(), _dtype(out_grad), _ph(plan), _stream()))


def build_kernel_map(in_coords, out_coords, offsets, stride=1, skip_offset=None, capacity=None, into=None):
    """Pair lists of a kernel map from int32 voxel coordinates on the device.
    Returns (in_map, out_map, kernel_nnz, kpos): device int32 tensors, the maps trimmed
    to the number of pairs found.  into=(in_map, out_map, kernel_nnz, kpos): write into these
    tensors (through their data pointers, as a native builder does) and return them untrimmed."""
    import numpy as np
    import torch
    for t, n in ((in_coords, "in_coords"), (out_coords, "out_coords")):
        if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous() or t.dim() != 2 or t.shape[1] != 3:
            raise ValueError("%s must be a contiguous int32 [N, 3] tensor on the GPU" % n)
    offs = np.ascontiguousarray(np.asarray(offsets, dtype=np.int32).reshape(-1, 3))
    k_vol = len(offs)
    n_in, n_out = in_coords.shape[0], out_coords.shape[0]
    cap = k_vol * n_out if capacity is None else int(capacity)
    if into is not None:
        in_map, out_map, knnz, kpos = into
        cap = min(in_map.numel(), out_map.numel())
    else:
        in_map = torch.empty(max(cap, 1), dtype=torch.int32, device=in_coords.device)
        out_map = torch.empty(max(cap, 1), dtype=torch.int32, device=in_coords.device)
        knnz = torch.empty(k_vol, dtype=torch.int32, device=in_coords.device)
        kpos = torch.empty(k_vol + 1, dtype=torch.int32, device=in_coords.device)
    found = ctypes.c_int64(0)
    _check(lib().fgms_build_kernel_map(
        _p(in_coords), n_in, _p(out_coords), n_out, offs.ctypes.data_as(ctypes.c_void_p), k_vol,
        int(stride), -1 if skip_offset is None else int(skip_offset), _p(in_map), _p(out_map), cap,
        _p(knnz), _p(kpos), ctypes.byref(found), _stream()))
    if into is not None:
        return in_map, out_map, knnz, kpos
    return in_map[:found.value], out_map[:found.value], knnz, kpos


def probe_gather(feats, plan, for_dgrad=False):
    """Gather-only pass over the rows the planned kernel reads (diagnostic)."""
    _check(lib().fgms_probe_gather(_p(feats), feats.shape[1], _dtype(feats), int(for_dgrad),
                                   _ph(plan), _stream()))


def wgrad(in_feats, out_grad, kernel_grad, kpos, in_map, out_map, plan=None):
    for t, n in ((in_feats, "in_feats"), (out_grad, "out_feats_grad"), (kernel_grad, "kernel_grad")):
        _need(t, n, in_feats.dtype)
    _check(lib().fgms_wgrad(
        _p(in_feats), _p(out_grad), _p(kernel_grad), _p(kpos), _p(in_map), _p(out_map),
        in_feats.shape[0], out_grad.shape[0], kernel_grad.shape[1], kernel_grad.shape[2],
        kernel_grad.shape[0], in_map.numel(), _dtype(in_feats), _ph(plan), _stream()))


def wgrad_static(in_feats, out_grad, kernel_grad, kpos, in_map, out_map, plan=None):
    """fgms_wgrad_static: the weight gradient without any device allocation."""
    for t, n in ((in_feats, "in_feats"), (out_grad, "out_feats_grad"), (kernel_grad, "kernel_grad")):
        _need(t, n, in_feats.dtype)
    _check(lib().fgms_wgrad_static(
        _p(in_feats), _p(out_grad), _p(kernel_grad), _p(kpos), _p(in_map), _p(out_map),
        in_feats.shape[0], out_grad.shape[0], kernel_grad.shape[1], kernel_grad.shape[2],
        kernel_grad.shape[0], in_map.numel(), _dtype(in_feats), _ph(plan), _stream()))
