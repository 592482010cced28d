"""Autograd wrapper over ``FGMS.backend``: the caller side that hkeee21/FGMS leaves to
an external library (``README.md:3``).  It owns exactly what the reference's scripts
repeat by hand before every call: the padded offset table ``qkpos``
(``cpu-check.py:6-14``), zero-initialised outputs (``cpu-check.py:107-108``,
``cpu-check-back.py:104-107``) and the pairing of the forward call with the backward one
(``spconv-test.py:96-120``).

    y = sparse_conv(feats, weight, kmap)          # differentiable in feats and weight
    layer = SparseConv(64, 64, k_vol=27); y = layer(feats, kmap)

``kmap`` is a :class:`KernelMap`: the pair lists of one kernel map on the device.  Every
layer, pass and iteration that shares a map shares its plan through ``FGMS.backend``'s
cache, which is keyed on these tensors.
"""
import math

import torch

from . import backend
from fgms_amd.harness import kpos_quantized

_Q = 256   # padding quantum of the reference's scripts (cpu-check.py:106); advisory here


class KernelMap:
    """Pair lists of one kernel map: ``in_map[j] -> out_map[j]`` for j in
    ``[kpos[k], kpos[k+1])`` through offset k.  int32, on the device of the features."""

    def __init__(self, in_map, out_map, kernel_nnz, n_in, n_out):
        kn = torch.as_tensor(kernel_nnz, dtype=torch.int32).cpu()
        self.k_vol = int(kn.numel())
        self.kernel_nnz = kn                                        # host, as fgms_fwd_cuda wants it
        kpos = torch.zeros(self.k_vol + 1, dtype=torch.int32)
        kpos[1:] = torch.cumsum(kn, 0)
        if int(kpos[-1]) != in_map.numel() or in_map.numel() != out_map.numel():
            raise ValueError("kernel_nnz does not add up to the length of the pair lists")
        self.in_map = in_map.to(torch.int32).contiguous()
        self.out_map = out_map.to(torch.int32).contiguous()
        self.kpos = kpos.to(self.in_map.device)
        self.qkpos, self.qsum = kpos_quantized(kn, self.kpos, self.k_vol, _Q)
        self.n_in, self.n_out = int(n_in), int(n_out)

    @classmethod
    def from_coords(cls, in_coords, out_coords, offsets, stride=1):
        """Builds the map on the device from int32 voxel coordinates ``[N, 3]``: pairs
        (i, o) with ``in_coords[i] == out_coords[o] * stride + offsets[k]``."""
        from fgms_amd import capi
        in_map, out_map, knnz, _ = capi.build_kernel_map(in_coords, out_coords, offsets, stride)
        return cls(in_map, out_map, knnz, in_coords.shape[0], out_coords.shape[0])

    def transposed(self):
        """The map of the transposed convolution: the same pairs, roles swapped.  It keeps
        this map's tensors (not copies), so ``FGMS.backend`` recognises the pair lists and lets
        both maps share one plan."""
        t = KernelMap.__new__(KernelMap)
        t.k_vol, t.kernel_nnz = self.k_vol, self.kernel_nnz
        t.in_map, t.out_map = self.out_map, self.in_map
        t.kpos, t.qkpos, t.qsum = self.kpos, self.qkpos, self.qsum
        t.n_in, t.n_out = self.n_out, self.n_in
        return t


class _SparseConvFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, feats, weight, kmap, allow_tf32):
        if feats.dim() != 2 or weight.dim() != 3 or weight.shape[0] != kmap.k_vol:
            raise ValueError("expected feats [N, Cin] and weight [K, Cin, Cout] with K = the map's offsets")
        if feats.shape[0] != kmap.n_in:
            raise ValueError("feats has %d rows, the kernel map expects %d" % (feats.shape[0], kmap.n_in))
        feats = feats.contiguous()
        weight = weight.contiguous()
        out = torch.zeros(kmap.n_out, weight.shape[2], dtype=feats.dtype, device=feats.device)
        backend.fgms_fusion_fwd_cuda(feats, weight, kmap.qsum, out, kmap.kpos, kmap.qkpos,
                                     kmap.in_map, kmap.out_map, False, bool(allow_tf32))
        ctx.save_for_backward(feats, weight)
        ctx.kmap = kmap
        ctx.allow_tf32 = bool(allow_tf32)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        feats, weight = ctx.saved_tensors
        kmap = ctx.kmap
        grad_out = grad_out.contiguous()
        grad_feats = torch.zeros_like(feats)
        grad_weight = torch.zeros_like(weight)
        backend.fgms_bwd_cuda(grad_out, feats, weight, kmap.qsum, grad_feats, grad_weight,
                              kmap.kpos, kmap.qkpos, kmap.in_map, kmap.out_map, False, ctx.allow_tf32)
        return grad_feats, grad_weight, None, None


def sparse_conv(feats, weight, kmap, allow_tf32=False):
    """out[out_map[j]] += feats[in_map[j]] @ weight[k]; differentiable in feats and weight."""
    return _SparseConvFunction.apply(feats, weight, kmap, allow_tf32)


class SparseConv(torch.nn.Module):
    """A sparse convolution layer over a precomputed :class:`KernelMap`.  Weights
    ``[k_vol, c_in, c_out]``, Kaiming-uniform with fan-in ``k_vol * c_in``; optional bias."""

    def __init__(self, c_in, c_out, k_vol=27, bias=False, dtype=None, device=None, allow_tf32=False):
        super().__init__()
        self.c_in, self.c_out, self.k_vol = c_in, c_out, k_vol
        self.allow_tf32 = allow_tf32
        self.weight = torch.nn.Parameter(torch.empty(k_vol, c_in, c_out, dtype=dtype, device=device))
        self.bias = torch.nn.Parameter(torch.zeros(c_out, dtype=dtype, device=device)) if bias else None
        self.reset_parameters()

    def reset_parameters(self):
        bound = 1.0 / math.sqrt(self.k_vol * self.c_in)
        with torch.no_grad():
            self.weight.uniform_(-bound, bound)
            if self.bias is not None:
                self.bias.zero_()

    def forward(self, feats, kmap):
        out = sparse_conv(feats, self.weight, kmap, self.allow_tf32)
        return out if self.bias is None else out + self.bias
