"""Writes the golden fixtures in this directory.

The reference ships no data and no golden vectors (its samples are downloaded,
download_data.sh:1-5), so the expected values here come from library routines
the sparse convolution reduces to on a fully occupied grid, computed in
float64 and independent of both the oracle and the HIP kernels:
  * 3x3x3 submanifold conv      == torch.nn.functional.conv3d(padding=1)
  * 2x2x2 stride-2 conv         == conv3d(stride=2)
  * its transposed counterpart  == conv_transpose3d(stride=2)
gradients by torch.autograd.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from fgms_amd import clouds  # noqa: E402


def dense_grid(d, h, w):
    g = np.stack(np.meshgrid(np.arange(d), np.arange(h), np.arange(w), indexing="ij"), -1)
    return g.reshape(-1, 3).astype(np.int32)


def conv_weight(w, ks):
    k_vol, c_in, c_out = w.shape
    return w.reshape(ks, ks, ks, c_in, c_out).permute(4, 3, 0, 1, 2)


def make(name, shape, ksize, stride, c_in, c_out, seed, transposed=False):
    rng = np.random.default_rng(seed)
    d, h, w_ = shape
    fine = dense_grid(d, h, w_)
    offs = clouds.offsets_cube(ksize)
    if stride == 1:
        imap, omap, knnz, kpos = clouds.build_kernel_map(fine, fine, offs)
        in_shape = out_shape = shape
    else:
        coarse = clouds.downsample_coords(fine, stride)
        imap, omap, knnz, kpos = clouds.build_kernel_map(fine, coarse, offs, stride)
        in_shape, out_shape = shape, tuple(s // stride for s in shape)
        if transposed:
            imap, omap = omap, imap
            in_shape, out_shape = out_shape, in_shape
    n_in, n_out = int(np.prod(in_shape)), int(np.prod(out_shape))
    x = torch.tensor(rng.standard_normal((n_in, c_in)), dtype=torch.float64, requires_grad=True)
    w = torch.tensor(rng.uniform(-0.3, 0.3, (len(offs), c_in, c_out)), dtype=torch.float64, requires_grad=True)
    g = torch.tensor(rng.standard_normal((n_out, c_out)), dtype=torch.float64)
    xg = x.reshape(*in_shape, c_in).permute(3, 0, 1, 2)[None]
    if stride == 1:
        y = F.conv3d(xg, conv_weight(w, ksize), padding=ksize // 2)
    elif not transposed:
        y = F.conv3d(xg, conv_weight(w, ksize), stride=stride)
    else:
        y = F.conv_transpose3d(xg, w.reshape(ksize, ksize, ksize, c_in, c_out).permute(3, 4, 0, 1, 2), stride=stride)
    out = y[0].permute(1, 2, 3, 0).reshape(n_out, c_out)
    gx, gw = torch.autograd.grad(out, (x, w), g)
    np.savez_compressed(
        os.path.join(HERE, name + ".npz"),
        in_feats=x.detach().numpy().astype(np.float32), kernel=w.detach().numpy().astype(np.float32),
        out_grad=g.numpy().astype(np.float32), imap=imap, omap=omap, knnz=knnz, kpos=kpos,
        n_in=n_in, n_out=n_out, out=out.detach().numpy().astype(np.float32),
        in_grad=gx.numpy().astype(np.float32), kernel_grad=gw.numpy().astype(np.float32))


if __name__ == "__main__":
    make("dense_subm_k3_8x16", (4, 5, 6), 3, 1, 8, 16, seed=1)
    make("dense_subm_k3_32x32", (5, 5, 6), 3, 1, 32, 32, seed=2)
    make("dense_down_k2_16x32", (6, 4, 8), 2, 2, 16, 32, seed=3)
    make("dense_up_k2_32x16", (6, 4, 8), 2, 2, 32, 16, seed=4, transposed=True)
    print(sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
