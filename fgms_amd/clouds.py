"""Seeded synthetic voxel clouds and the kernel maps built on them.

hkeee21/FGMS ships no kernel-map builder and no data: its scripts load
``imap / omap / knnz / kpos`` from downloaded files (``cpu-check.py:83-94``,
``spconv-test.py:64-73``).  This module is the caller-side stand-in for those
files: deterministic coordinate generators (numpy PCG64) for the benchmark
configurations and a sort/search kernel-map builder that emits the flat
``int32`` pair lists in the layout the entry points take (pairs of offset ``k``
in ``[kpos[k], kpos[k+1])``, centre offset = ``K // 2``, ``backend/spconv.cu:52``).

Everything here is host-side numpy; none of it is on the GPU hot path.
"""
import itertools

import numpy as np

_BIAS = 1 << 20


def rng_for(cfg_id):
    return np.random.Generator(np.random.PCG64(1000 + int(cfg_id)))


# ----------------------------------------------------------------- voxel sets
def dedup(points, grid):
    """floor -> clip to [0, grid) -> unique rows (lexicographic order)."""
    v = np.floor(points).astype(np.int64)
    keep = np.all((v >= 0) & (v < grid), axis=1)
    return np.unique(v[keep], axis=0).astype(np.int32)


def _frame(rng, oblique):
    """Two orthonormal tangents of a random plane."""
    if not oblique:
        axes = np.eye(3)[rng.permutation(3)]
        return axes[0], axes[1]
    n = rng.normal(size=3)
    n /= np.linalg.norm(n)
    a = np.cross(n, np.eye(3)[np.argmin(np.abs(n))])
    a /= np.linalg.norm(a)
    return a, np.cross(n, a)


def _patch(rng, centre, half_u, half_v, oblique, step=0.5):
    u, v = _frame(rng, oblique)
    a = np.arange(-half_u, half_u + step, step)
    b = np.arange(-half_v, half_v + step, step)
    aa, bb = np.meshgrid(a, b, indexing="ij")
    return centre + aa.reshape(-1, 1) * u + bb.reshape(-1, 1) * v


def _sphere_shell(rng, centre, radius, n):
    d = rng.normal(size=(n, 3))
    d /= np.linalg.norm(d, axis=1, keepdims=True)
    return centre + radius * d


def _box_surface(centre, half, step=0.5):
    pts = []
    for ax in range(3):
        o = [i for i in range(3) if i != ax]
        a = np.arange(-half[o[0]], half[o[0]] + step, step)
        b = np.arange(-half[o[1]], half[o[1]] + step, step)
        aa, bb = np.meshgrid(a, b, indexing="ij")
        for s in (-1.0, 1.0):
            p = np.zeros((aa.size, 3))
            p[:, o[0]] = aa.ravel()
            p[:, o[1]] = bb.ravel()
            p[:, ax] = s * half[ax]
            pts.append(p)
    return centre + np.concatenate(pts)


def _cylinder_surface(centre, radius, half_h, axis, step=0.5):
    th = np.arange(0.0, 2 * np.pi, step / max(radius, 1.0))
    h = np.arange(-half_h, half_h + step, step)
    tt, hh = np.meshgrid(th, h, indexing="ij")
    o = [i for i in range(3) if i != axis]
    p = np.zeros((tt.size, 3))
    p[:, o[0]] = radius * np.cos(tt.ravel())
    p[:, o[1]] = radius * np.sin(tt.ravel())
    p[:, axis] = hh.ravel()
    return centre + p


def cloud_planes_spheres(rng, grid=128, target=20000):
    """6 random planes + 4 sphere shells in a grid^3 box, ~target unique voxels."""
    pts = []
    for i in range(6):
        c = rng.uniform(0.3 * grid, 0.7 * grid, size=3)
        pts.append(_patch(rng, c, 0.19 * grid, 0.19 * grid, oblique=(i % 2 == 1)))
    for _ in range(4):
        c = rng.uniform(0.3 * grid, 0.7 * grid, size=3)
        r = rng.uniform(0.08 * grid, 0.16 * grid)
        pts.append(_sphere_shell(rng, c, r, 60000))
    vox = dedup(np.concatenate(pts), grid)
    return _trim(rng, vox, target)


def cloud_indoor(rng, grid=512, target=200000):
    """~40 planar patches (axis-aligned and oblique) + 20 box / cylinder
    surfaces in a grid^3 box: an indoor-scan-like set of 2-D sheets."""
    pts = []
    for i in range(40):
        c = rng.uniform(0.15 * grid, 0.85 * grid, size=3)
        hu, hv = rng.uniform(22, 42, size=2)
        pts.append(_patch(rng, c, hu, hv, oblique=(i % 2 == 1)))
    for i in range(20):
        c = rng.uniform(0.15 * grid, 0.85 * grid, size=3)
        if i % 2 == 0:
            pts.append(_box_surface(c, rng.uniform(8, 18, size=3)))
        else:
            pts.append(_cylinder_surface(c, rng.uniform(8, 16), rng.uniform(10, 24),
                                         int(rng.integers(3))))
    vox = dedup(np.concatenate(pts), grid)
    return _trim(rng, vox, target)


def cloud_lidar(rng, voxel=0.05, beams=64, azimuths=2048, rmin=2.0, rmax=50.0,
                sweeps=5):
    """Sweeps of a spinning multi-beam sensor 1.73 m above a ground plane with
    random box obstacles, hits voxelised at `voxel` metres.  One 64 x 2048 sweep
    collapses to ~50 k voxels at 5 cm (the near rings are denser than the voxel
    pitch), so `sweeps` consecutive positions of a moving sensor are merged, as
    multi-sweep LiDAR pipelines do, to land near 120 k voxels."""
    elev = np.deg2rad(np.linspace(-25.0, 3.0, beams))
    azim = np.linspace(0.0, 2 * np.pi, azimuths, endpoint=False)
    ee, aa = np.meshgrid(elev, azim, indexing="ij")
    d = np.stack([np.cos(ee) * np.cos(aa), np.cos(ee) * np.sin(aa), np.sin(ee)], -1)
    d = d.reshape(-1, 3)
    nbox = 60
    ang = rng.uniform(0, 2 * np.pi, nbox)
    rad = rng.uniform(5.0, 45.0, nbox)
    half = np.stack([rng.uniform(0.8, 5.0, nbox), rng.uniform(0.8, 5.0, nbox),
                     rng.uniform(0.7, 4.0, nbox)], 1)
    cen = np.stack([rad * np.cos(ang), rad * np.sin(ang), half[:, 2]], 1)
    pts = []
    for s in range(sweeps):
        origin = np.array([2.3 * s, 0.6 * s, 1.73])
        t_hit = np.full(len(d), np.inf)
        down = d[:, 2] < -1e-9
        t_hit[down] = -origin[2] / d[down, 2]
        with np.errstate(divide="ignore", invalid="ignore"):
            inv = 1.0 / d
            for b in range(nbox):
                t0 = (cen[b] - half[b] - origin) * inv
                t1 = (cen[b] + half[b] - origin) * inv
                tn = np.nanmax(np.minimum(t0, t1), axis=1)
                tf = np.nanmin(np.maximum(t0, t1), axis=1)
                ok = (tn <= tf) & (tn > 0)
                t_hit = np.where(ok & (tn < t_hit), tn, t_hit)
        ok = (t_hit >= rmin) & (t_hit <= rmax)
        t = t_hit[ok] + rng.normal(0.0, 0.01, ok.sum())
        pts.append(origin + d[ok] * t[:, None])
    v = np.floor(np.concatenate(pts) / voxel).astype(np.int64)
    v -= v.min(axis=0)
    return np.unique(v, axis=0).astype(np.int32)


def _trim(rng, vox, target):
    """Keep the cloud's sheets intact: drop whole x-slabs from the top until at
    most ~target voxels remain (random thinning would destroy the neighbour
    structure the benchmark is about)."""
    if target is None or len(vox) <= target:
        return vox
    order = np.argsort(vox[:, 0], kind="stable")
    return np.unique(vox[order[:target]], axis=0).astype(np.int32)


def subsample(rng, vox, n):
    """Uniform random subset of n voxels (the wide-channel case)."""
    if len(vox) <= n:
        return vox
    idx = np.sort(rng.choice(len(vox), size=n, replace=False))
    return vox[idx]


# ----------------------------------------------------------------- kernel maps
def offsets_cube(ksize):
    """Lexicographic offsets: {-1,0,1}^3 for ksize 3 (centre = index 13),
    {0,1}^3 for ksize 2."""
    r = range(-(ksize // 2), ksize // 2 + 1) if ksize % 2 == 1 else range(ksize)
    return np.array(list(itertools.product(r, r, r)), np.int32)


def _keys(c):
    c = c.astype(np.int64) + _BIAS
    return (c[:, 0] << 42) | (c[:, 1] << 21) | c[:, 2]


def build_kernel_map(in_coords, out_coords, offsets, stride=1, skip_offset=None):
    """Pairs (i, o) with in_coords[i] == out_coords[o] * stride + offsets[k],
    grouped by k, ascending o inside a group.  Returns imap, omap, knnz, kpos."""
    in_keys = _keys(in_coords)
    order = np.argsort(in_keys, kind="stable")
    sk = in_keys[order]
    imaps, omaps, knnz = [], [], []
    base = out_coords.astype(np.int64) * stride
    for k, off in enumerate(offsets):
        if skip_offset is not None and k == skip_offset:
            knnz.append(0)
            continue
        q = _keys(base + off.astype(np.int64))
        pos = np.searchsorted(sk, q)
        pos[pos == len(sk)] = 0
        hit = sk[pos] == q if len(sk) else np.zeros(len(q), bool)
        o = np.nonzero(hit)[0]
        imaps.append(order[pos[o]].astype(np.int32))
        omaps.append(o.astype(np.int32))
        knnz.append(len(o))
    knnz = np.array(knnz, np.int32)
    kpos = np.concatenate([[0], np.cumsum(knnz)]).astype(np.int32)
    cat = lambda xs: (np.concatenate(xs) if xs else np.zeros(0, np.int32)).astype(np.int32)
    return cat(imaps), cat(omaps), knnz, kpos


def build_kernel_map_bruteforce(in_coords, out_coords, offsets, stride=1):
    """Dictionary lookup, one python loop per (offset, output voxel)."""
    table = {tuple(int(v) for v in c): i for i, c in enumerate(in_coords)}
    imap, omap, knnz = [], [], []
    for off in offsets:
        n = 0
        for o, c in enumerate(out_coords):
            key = tuple(int(c[d]) * stride + int(off[d]) for d in range(3))
            i = table.get(key)
            if i is not None:
                imap.append(i)
                omap.append(o)
                n += 1
        knnz.append(n)
    knnz = np.array(knnz, np.int32)
    kpos = np.concatenate([[0], np.cumsum(knnz)]).astype(np.int32)
    return (np.array(imap, np.int32), np.array(omap, np.int32), knnz, kpos)


def downsample_coords(in_coords, stride=2):
    return np.unique(in_coords // stride, axis=0).astype(np.int32)


# ----------------------------------------------------------------- tensors
def kaiming_uniform(rng, k_vol, c_in, c_out):
    """U(-b, b), b = 1/sqrt(K*Cin): torch's kaiming_uniform_(a=sqrt(5)) with
    fan-in K*Cin."""
    b = 1.0 / np.sqrt(k_vol * c_in)
    return rng.uniform(-b, b, size=(k_vol, c_in, c_out)).astype(np.float32)


def make_layer(rng, imap, omap, knnz, kpos, n_in, n_out, c_in, c_out, dtype,
               feats="normal"):
    k_vol = len(knnz)
    if feats == "normal":
        x = rng.standard_normal((n_in, c_in), dtype=np.float32)
    else:
        x = rng.random((n_in, c_in), dtype=np.float32)
    w = kaiming_uniform(rng, k_vol, c_in, c_out)
    g = rng.standard_normal((n_out, c_out), dtype=np.float32)
    return dict(in_feats=x.astype(dtype), kernel=w.astype(dtype), out_grad=g.astype(dtype),
                imap=imap, omap=omap, knnz=knnz, kpos=kpos, n_in=int(n_in),
                n_out=int(n_out), c_in=c_in, c_out=c_out, k_vol=k_vol)


_CLOUD_CACHE = {}


def indoor_cloud(target=200000):
    key = ("indoor", target)
    if key not in _CLOUD_CACHE:
        _CLOUD_CACHE[key] = cloud_indoor(rng_for(2), target=target)
    return _CLOUD_CACHE[key]


def submanifold_case(coords, c_in, c_out, dtype, rng, feats="normal"):
    imap, omap, knnz, kpos = build_kernel_map(coords, coords, offsets_cube(3))
    n = len(coords)
    return make_layer(rng, imap, omap, knnz, kpos, n, n, c_in, c_out, dtype, feats)


def config_case(cfg_id, variant=None, scale=1.0):
    """The benchmark configurations.  `scale` < 1 shrinks the voxel target for
    CPU-sized parity runs; shapes and structure stay the same."""
    rng = rng_for(cfg_id)
    if cfg_id == 1:
        vox = cloud_planes_spheres(rng, 128, int(20000 * scale))
        return submanifold_case(vox, 32, 32, np.float32, rng)
    if cfg_id == 2:
        vox = cloud_indoor(rng_for(2), target=int(200000 * scale))
        dtype = np.float16 if variant == "fp16" else np.float32
        return submanifold_case(vox, 64, 64, dtype, rng)
    if cfg_id == 3:
        vox = cloud_lidar(rng, azimuths=max(64, int(2048 * scale)))
        return submanifold_case(vox, 128, 128, np.float16, rng)
    if cfg_id == 4:
        vin = cloud_indoor(rng_for(2), target=int(200000 * scale))
        vout = downsample_coords(vin, 2)
        imap, omap, knnz, kpos = build_kernel_map(vin, vout, offsets_cube(2), stride=2)
        if variant == "up":   # transposed conv: roles of the two maps swap
            return make_layer(rng, omap, imap, knnz, kpos, len(vout), len(vin),
                              128, 64, np.float16)
        return make_layer(rng, imap, omap, knnz, kpos, len(vin), len(vout),
                          64, 128, np.float16)
    if cfg_id == 5:
        vox = cloud_indoor(rng_for(2), target=int(200000 * scale))
        dtype = np.float32 if variant and variant.endswith("fp32") else np.float16
        if variant and variant.startswith("wide"):
            vox = subsample(rng, vox, int(50000 * scale))
            return submanifold_case(vox, 256, 256, dtype, rng)
        return submanifold_case(vox, 4, 32, dtype, rng, feats="uniform")
    raise ValueError("unknown config %r" % (cfg_id,))
