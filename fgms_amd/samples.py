"""On-disk layer samples in the format hkeee21/FGMS's scripts read.

The reference's scripts replay dumps of real network layers: one ``torch.save``-d dict per
layer, fetched by ``download_data.sh`` into ``sample-data/``.  Two flavours exist:

* checked samples (``sample-data/tiny-samples``, ``cpu-check.py:83-94``,
  ``cpu-check-back.py:80-92``): ``in_feats [N_in, C_in]``, ``kernel [K, C_in, C_out]``,
  ``sum_nnz`` (pairs), ``out_nnz`` (output rows), ``knnz [K]``, ``kpos [K + 1]``,
  ``imap`` / ``omap`` (any shape, flattened by the reader);
* timed samples (``sample-data/real-samples``, ``spconv-test.py:64-73``): the map only --
  ``sum_nnz``, ``out_nnz``, ``knnz``, ``kpos``, ``imap``, ``omap`` plus ``in_nnz``, ``c_in``,
  ``c_out``, ``k_vol``; features and weights are drawn at random by the script.

The data itself is not available offline, so this module is written against that schema
alone: :func:`load_sample` reads either flavour (with ``weights_only=True``: nothing from
the file is executed), checks it (counts add up, indices in range) and normalises dtypes;
:func:`save_sample` writes the same schema from a layer of this package's generators, which
is what the tests round-trip.  :func:`replay` times a sample the way ``spconv-test.py`` does
(centre offset spliced in with ``remove_mid`` for submanifold layers, 10 + 100 calls by
default).  ``python -m fgms_amd.samples DIR [--precision fp16] [--no-fusion]`` replays a
directory.
"""
import argparse
import os
import time
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch

from .harness import kpos_quantized, remove_mid

_MAP_KEYS = ("sum_nnz", "out_nnz", "knnz", "kpos", "imap", "omap")


@dataclass
class Sample:
    """One layer: the kernel map (host int32 ``knnz``; ``kpos``, ``imap``, ``omap`` int32 on
    ``device``) and, for checked samples, its features and weights."""
    n_in: int
    n_out: int
    k_vol: int
    c_in: int
    c_out: int
    sum_nnz: int
    knnz: torch.Tensor
    kpos: torch.Tensor
    imap: torch.Tensor
    omap: torch.Tensor
    in_feats: Optional[torch.Tensor] = None
    kernel: Optional[torch.Tensor] = None

    @property
    def submanifold(self):
        """What the reference's scripts test before they treat the centre offset apart
        (``cpu-check.py:100``, ``spconv-test.py:79``)."""
        return self.n_in == self.n_out


def _as_int(v, name):
    if isinstance(v, torch.Tensor):
        if v.numel() != 1:
            raise ValueError("sample field %r should be a single number" % name)
        return int(v.item())
    if isinstance(v, (int, np.integer)):
        return int(v)
    raise ValueError("sample field %r should be an integer, got %s" % (name, type(v).__name__))


def load_sample(path, device="cpu"):
    """Reads one sample file.  Raises ``ValueError`` when the dict does not follow the
    schema or its numbers contradict each other."""
    d = torch.load(path, map_location="cpu", weights_only=True)
    if not isinstance(d, dict):
        raise ValueError("%s: expected a dict, got %s" % (path, type(d).__name__))
    missing = [k for k in _MAP_KEYS if k not in d]
    if missing:
        raise ValueError("%s: missing fields %s" % (path, ", ".join(missing)))
    knnz = torch.as_tensor(d["knnz"]).reshape(-1).to(torch.int32).cpu()
    imap = torch.as_tensor(d["imap"]).reshape(-1).to(torch.int32)
    omap = torch.as_tensor(d["omap"]).reshape(-1).to(torch.int32)
    kpos = torch.as_tensor(d["kpos"]).reshape(-1).to(torch.int32)
    k_vol = int(knnz.numel())
    sum_nnz, n_out = _as_int(d["sum_nnz"], "sum_nnz"), _as_int(d["out_nnz"], "out_nnz")
    feats, kernel = d.get("in_feats"), d.get("kernel")
    if (feats is None) != (kernel is None):
        raise ValueError("%s: in_feats and kernel come together or not at all" % path)
    if feats is not None:
        if feats.dim() != 2 or kernel.dim() != 3 or kernel.shape[1] != feats.shape[1]:
            raise ValueError("%s: in_feats [N, C_in] / kernel [K, C_in, C_out] shapes do not fit" % path)
        n_in, c_in, c_out = int(feats.shape[0]), int(kernel.shape[1]), int(kernel.shape[2])
        if int(kernel.shape[0]) != k_vol:
            raise ValueError("%s: kernel has %d offsets, knnz %d" % (path, kernel.shape[0], k_vol))
        for key, have in (("in_nnz", n_in), ("c_in", c_in), ("c_out", c_out), ("k_vol", k_vol)):
            if key in d and _as_int(d[key], key) != have:
                raise ValueError("%s: %s = %d contradicts the tensors (%d)" % (path, key, _as_int(d[key], key), have))
    else:
        need = [k for k in ("in_nnz", "c_in", "c_out", "k_vol") if k not in d]
        if need:
            raise ValueError("%s: a sample without tensors needs %s" % (path, ", ".join(need)))
        n_in, c_in, c_out = (_as_int(d[k], k) for k in ("in_nnz", "c_in", "c_out"))
        if _as_int(d["k_vol"], "k_vol") != k_vol:
            raise ValueError("%s: k_vol = %d, knnz has %d entries" % (path, _as_int(d["k_vol"], "k_vol"), k_vol))
    # the numbers must agree with each other
    m = int(knnz.to(torch.int64).sum())
    if kpos.numel() != k_vol + 1:
        raise ValueError("%s: kpos has %d entries for %d offsets" % (path, kpos.numel(), k_vol))
    expect = torch.zeros(k_vol + 1, dtype=torch.int64)
    expect[1:] = torch.cumsum(knnz.to(torch.int64), 0)
    if not torch.equal(kpos.to(torch.int64), expect):
        raise ValueError("%s: kpos is not the running sum of knnz" % path)
    if imap.numel() != m or omap.numel() != m:
        raise ValueError("%s: %d pairs by knnz, %d / %d map entries" % (path, m, imap.numel(), omap.numel()))
    if sum_nnz != m:
        raise ValueError("%s: sum_nnz = %d, knnz adds up to %d" % (path, sum_nnz, m))
    if m and (int(imap.min()) < 0 or int(imap.max()) >= n_in or int(omap.min()) < 0 or int(omap.max()) >= n_out):
        raise ValueError("%s: a map index is outside [0, %d) x [0, %d)" % (path, n_in, n_out))
    return Sample(n_in, n_out, k_vol, c_in, c_out, sum_nnz, knnz, kpos.to(device), imap.to(device),
                  omap.to(device), None if feats is None else feats.to(device),
                  None if kernel is None else kernel.to(device))


def save_sample(path, layer, with_tensors=True):
    """Writes a layer dict of this package's generators (``fgms_amd.clouds``) in the
    reference's schema: a checked sample with ``with_tensors``, a timed one without."""
    d = {
        "sum_nnz": int(len(layer["imap"])),
        "out_nnz": int(layer["n_out"]),
        "knnz": torch.as_tensor(np.asarray(layer["knnz"]), dtype=torch.int32),
        "kpos": torch.as_tensor(np.asarray(layer["kpos"]), dtype=torch.int32),
        "imap": torch.as_tensor(np.asarray(layer["imap"]), dtype=torch.int32),
        "omap": torch.as_tensor(np.asarray(layer["omap"]), dtype=torch.int32),
        "in_nnz": int(layer["n_in"]),
        "c_in": int(layer["c_in"]),
        "c_out": int(layer["c_out"]),
        "k_vol": int(layer["k_vol"]),
    }
    if with_tensors:
        d["in_feats"] = torch.as_tensor(np.asarray(layer["in_feats"]))
        d["kernel"] = torch.as_tensor(np.asarray(layer["kernel"]))
    torch.save(d, path)


def replay(sample, dtype=torch.float16, fusion=True, arch80=False, warmup=10, steps=100, seed=0,
           return_inputs=False):
    """Times the forward pass of one sample on its device the way ``spconv-test.py:75-122``
    does: random features and weights, the centre offset of a submanifold layer spliced into
    the maps, ``warmup`` untimed and ``steps`` timed calls between synchronisations.
    Returns (milliseconds per call, output of one call on a zeroed tensor), with
    ``return_inputs`` also the features and weights that were drawn."""
    from FGMS import backend
    dev = sample.imap.device
    gen = torch.Generator(device=dev).manual_seed(seed)
    feats = torch.rand((sample.n_in, sample.c_in), dtype=dtype, device=dev, generator=gen)
    weights = torch.rand((sample.k_vol, sample.c_in, sample.c_out), dtype=dtype, device=dev, generator=gen)
    out = torch.zeros((sample.n_out, sample.c_out), dtype=dtype, device=dev)
    knnz, kpos, imap, omap = sample.knnz.clone(), sample.kpos, sample.imap, sample.omap
    if sample.submanifold:
        qkpos, qsum, kpos, imap, omap = remove_mid(sample.n_in, knnz, kpos, sample.k_vol, 256, imap, omap)
    else:
        qkpos, qsum = kpos_quantized(knnz, kpos, sample.k_vol, 256)
    sum_nnz = int(imap.numel())

    def call():
        if fusion:
            backend.fgms_fusion_fwd_cuda(feats, weights, qsum, out, kpos, qkpos, imap, omap, False, arch80)
        else:
            backend.fgms_fwd_cuda(feats, weights, sum_nnz, out, knnz, kpos, imap, omap, False, arch80)

    with torch.no_grad():
        for _ in range(warmup):
            call()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            call()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        out.zero_()
        call()
        torch.cuda.synchronize()
    ms = (t1 - t0) * 1e3 / max(steps, 1)
    return (ms, out, feats, weights) if return_inputs else (ms, out)


def main(argv=None):
    ap = argparse.ArgumentParser(description="replay a directory of FGMS layer samples")
    ap.add_argument("dir")
    ap.add_argument("--precision", choices=("fp16", "fp32"), default="fp32")
    ap.add_argument("--no-fusion", action="store_true", help="one launch per offset (fgms_fwd_cuda)")
    ap.add_argument("--tf32", action="store_true", help="the reference's arch80 flag for fp32 tensors")
    args = ap.parse_args(argv)
    dtype = torch.float16 if args.precision == "fp16" else torch.float32
    for name in sorted(os.listdir(args.dir)):
        s = load_sample(os.path.join(args.dir, name), device="cuda")
        ms, _ = replay(s, dtype=dtype, fusion=not args.no_fusion, arch80=args.tf32)
        print("[input size=%d, mapping size=%d, in channel=%d, out channel=%d, fusion=%s] duration: %.4f ms"
              % (s.n_in, s.sum_nnz, s.c_in, s.c_out, not args.no_fusion, ms))


if __name__ == "__main__":
    main()
