"""TEST INFRASTRUCTURE ONLY -- python face of the CPU oracle.

Two independent restatements of what hkeee21/FGMS computes:

* ``c_*``   : ctypes calls into ``libfgms_oracle.so`` (``fgms_oracle.c``), the
              loop nests of ``cpu-check.py:16-44`` and ``cpu-check-back.py:16-44``
              in fp32 arithmetic.  This is also the timed CPU baseline.
* ``np_*``  : float64 numpy ``add.at`` formulations of the same sums, written
              independently of the C code; the tests pin one against the other
              and both against closed forms (dense conv3d, autograd, adjoints).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import
this module; the shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfgms_oracle.so")
_lib = None

F32, F16 = 0, 1


def build(force=False):
    """Compile libfgms_oracle.so with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "libfgms_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i32p = ctypes.c_void_p, ctypes.c_void_p
        i64, i32 = ctypes.c_int64, ctypes.c_int
        L.fgms_oracle_fwd.argtypes = [vp, vp, vp, i32p, i32p, i32p, i64, i64,
                                      i32, i32, i32, i32, i32, i32]
        L.fgms_oracle_dgrad.argtypes = [vp, vp, vp, i32p, i32p, i32p, i64, i64,
                                        i32, i32, i32, i32, i32]
        L.fgms_oracle_wgrad.argtypes = [vp, vp, vp, i32p, i32p, i32p, i64, i64,
                                        i32, i32, i32, i32, i32]
        L.fgms_oracle_qkpos.argtypes = [i32p, i32, i32, i32p]
        L.fgms_oracle_qkpos.restype = i64
        L.fgms_oracle_offset_of.argtypes = [i32p, i32, i32, i32]
        L.fgms_oracle_offset_of.restype = i32
        L.fgms_oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.fgms_oracle_half_to_float.restype = ctypes.c_float
        L.fgms_oracle_float_to_half.argtypes = [ctypes.c_float]
        L.fgms_oracle_float_to_half.restype = ctypes.c_uint16
        L.fgms_oracle_max_threads.restype = i32
        _lib = L
    return _lib


def _dtype_code(a):
    if a.dtype == np.float32:
        return F32
    if a.dtype == np.float16:
        return F16
    raise TypeError("oracle handles float32 / float16, got %s" % a.dtype)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a, a.ctypes.data


def _i32(a):
    return _c(np.asarray(a), np.int32)


def mid_offset(k_vol):
    """cpu-check.py:26 / backend/spconv.cu:52."""
    return k_vol // 2 if k_vol % 2 == 1 else 0


# --------------------------------------------------------------------- C calls
def c_fwd(in_feats, kernel, knnz, imap, omap, n_out, precompute=False,
          out_init=None, threads=0):
    in_feats, pi = _c(in_feats)
    kernel, pw = _c(kernel, in_feats.dtype)
    k_vol, c_in, c_out = kernel.shape
    assert in_feats.shape[1] == c_in
    out = (np.zeros((n_out, c_out), in_feats.dtype) if out_init is None
           else np.array(out_init, dtype=in_feats.dtype, order="C", copy=True))
    knnz, pk = _i32(knnz)
    imap, pim = _i32(imap)
    omap, pom = _i32(omap)
    rc = lib().fgms_oracle_fwd(pi, pw, out.ctypes.data, pk, pim, pom,
                               in_feats.shape[0], n_out, c_in, c_out, k_vol,
                               _dtype_code(in_feats), int(precompute), threads)
    assert rc == 0
    return out


def c_dgrad(out_grad, kernel, knnz, imap, omap, n_in, threads=0):
    out_grad, pg = _c(out_grad)
    kernel, pw = _c(kernel, out_grad.dtype)
    k_vol, c_in, c_out = kernel.shape
    assert out_grad.shape[1] == c_out
    gi = np.zeros((n_in, c_in), out_grad.dtype)
    knnz, pk = _i32(knnz)
    imap, pim = _i32(imap)
    omap, pom = _i32(omap)
    rc = lib().fgms_oracle_dgrad(pg, pw, gi.ctypes.data, pk, pim, pom, n_in,
                                 out_grad.shape[0], c_in, c_out, k_vol,
                                 _dtype_code(out_grad), threads)
    assert rc == 0
    return gi


def c_wgrad(in_feats, out_grad, knnz, imap, omap, k_vol, threads=0):
    in_feats, pi = _c(in_feats)
    out_grad, pg = _c(out_grad, in_feats.dtype)
    c_in, c_out = in_feats.shape[1], out_grad.shape[1]
    gw = np.zeros((k_vol, c_in, c_out), in_feats.dtype)
    knnz, pk = _i32(knnz)
    imap, pim = _i32(imap)
    omap, pom = _i32(omap)
    rc = lib().fgms_oracle_wgrad(pi, pg, gw.ctypes.data, pk, pim, pom,
                                 in_feats.shape[0], out_grad.shape[0], c_in,
                                 c_out, k_vol, _dtype_code(in_feats), threads)
    assert rc == 0
    return gw


def c_qkpos(knnz, q):
    knnz, pk = _i32(knnz)
    qk = np.zeros(len(knnz) + 1, np.int32)
    total = lib().fgms_oracle_qkpos(pk, len(knnz), q, qk.ctypes.data)
    return qk, int(total)


def c_offset_of(pos, eid, start, end):
    pos, pp = _i32(pos)
    return lib().fgms_oracle_offset_of(pp, int(eid), int(start), int(end))


def max_threads():
    return lib().fgms_oracle_max_threads()


# ----------------------------------------------------------- numpy, float64
def _runs(knnz):
    kpos = np.concatenate([[0], np.cumsum(np.asarray(knnz, np.int64))])
    return [(k, int(kpos[k]), int(kpos[k + 1])) for k in range(len(knnz))]


def np_fwd(in_feats, kernel, knnz, imap, omap, n_out, precompute=False):
    x = np.asarray(in_feats, np.float64)
    w = np.asarray(kernel, np.float64)
    out = np.zeros((n_out, w.shape[2]))
    for k, a, b in _runs(knnz):
        if b > a:
            np.add.at(out, omap[a:b], x[imap[a:b]] @ w[k])
    if precompute:
        out += x[:n_out] @ w[mid_offset(w.shape[0])]
    return out


def np_dgrad(out_grad, kernel, knnz, imap, omap, n_in):
    g = np.asarray(out_grad, np.float64)
    w = np.asarray(kernel, np.float64)
    gi = np.zeros((n_in, w.shape[1]))
    for k, a, b in _runs(knnz):
        if b > a:
            np.add.at(gi, imap[a:b], g[omap[a:b]] @ w[k].T)
    return gi


def np_wgrad(in_feats, out_grad, knnz, imap, omap, k_vol):
    x = np.asarray(in_feats, np.float64)
    g = np.asarray(out_grad, np.float64)
    gw = np.zeros((k_vol, x.shape[1], g.shape[1]))
    for k, a, b in _runs(knnz):
        if b > a:
            gw[k] = x[imap[a:b]].T @ g[omap[a:b]]
    return gw
