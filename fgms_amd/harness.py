"""Caller-side helpers every FGMS script repeats before it calls the extension.

These mirror the python prologue of the reference's three scripts so a caller
can switch libraries without touching its own code:

* ``kpos_quantized``  -- ``cpu-check.py:6-14`` (identical copies at
  ``cpu-check-back.py:6-14``, ``spconv-test.py:7-15``)
* ``remove_mid``      -- ``spconv-test.py:17-38``
* ``channel_transform`` -- ``cpu-check.py:47-65``

They accept torch tensors (as the scripts do) or numpy arrays.
"""
import numpy as np

try:  # torch is only needed when the caller passes tensors
    import torch
except Exception:  # pragma: no cover
    torch = None


def _is_tensor(x):
    return torch is not None and isinstance(x, torch.Tensor)


def kpos_quantized(knnz, kpos, k_vol, q):
    """qkpos[k+1] = qkpos[k] + ceil(knnz[k] / q) * q ; returns (qkpos, qkpos[K]).
    The result has kpos's type, dtype and device."""
    kn = knnz.detach().cpu().numpy() if _is_tensor(knnz) else np.asarray(knnz)
    acc = np.zeros(len(kpos), np.int64)
    for k in range(k_vol):
        acc[k + 1] = acc[k] + (int(kn[k]) + q - 1) // q * q
    total = int(acc[k_vol])
    if _is_tensor(kpos):
        return torch.as_tensor(acc, dtype=kpos.dtype, device=kpos.device), total
    return acc.astype(np.asarray(kpos).dtype), total


def mid_offset(k_vol):
    return k_vol // 2 if k_vol % 2 == 1 else 0


def remove_mid(nnz, knnz, kpos, k_vol, q, imap, omap):
    """Splice the identity pairs 0..nnz-1 in at the centre offset's position and
    rebuild kpos / qkpos.  As in the reference, ``knnz[mid]`` is set to ``nnz``
    (in place) only when it was 0.  Returns (qkpos, qsum, kpos_new, imap_new,
    omap_new)."""
    mid = mid_offset(k_vol)
    if _is_tensor(imap):
        change = int(kpos[mid])
        ident = torch.arange(nnz, device=imap.device, dtype=imap.dtype)
        imap_new = torch.cat([imap[:change], ident, imap[change:]]).int().contiguous()
        omap_new = torch.cat([omap[:change], ident.to(omap.dtype), omap[change:]]).int().contiguous()
    else:
        change = int(kpos[mid])
        ident = np.arange(nnz, dtype=np.int32)
        imap_new = np.concatenate([imap[:change], ident, imap[change:]]).astype(np.int32)
        omap_new = np.concatenate([omap[:change], ident, omap[change:]]).astype(np.int32)
    if int(knnz[mid]) == 0:
        knnz[mid] = nnz
    kn = knnz.detach().cpu().numpy() if _is_tensor(knnz) else np.asarray(knnz)
    kp = np.zeros(k_vol + 1, np.int64)
    kp[1:] = np.cumsum(kn[:k_vol].astype(np.int64))
    if _is_tensor(kpos):
        kpos_new = torch.as_tensor(kp, dtype=kpos.dtype, device=kpos.device)
    else:
        kpos_new = kp.astype(np.asarray(kpos).dtype)
    qkpos, qsum = kpos_quantized(knnz, kpos_new, k_vol, q)
    return qkpos, qsum, kpos_new, imap_new, omap_new


def channel_transform(feats, weights, ci_tgt, co_tgt):
    """Tile, then crop, the channel axes to (ci_tgt, co_tgt)."""
    cat = torch.cat if _is_tensor(feats) else (lambda xs, dim: np.concatenate(xs, axis=dim))
    ci, co = weights.shape[1], weights.shape[2]
    while ci < ci_tgt:
        feats = cat([feats, feats], dim=1)
        weights = cat([weights, weights], dim=1)
        ci *= 2
    while co < co_tgt:
        weights = cat([weights, weights], dim=2)
        co *= 2
    feats = feats[:, :ci_tgt]
    weights = weights[:, :ci_tgt, :co_tgt]
    if _is_tensor(feats):
        return feats.contiguous(), weights.contiguous()
    return np.ascontiguousarray(feats), np.ascontiguousarray(weights)
