// MFMA weight-gradient kernel for gfx950.
//
//   dW[k][ci][co] += sum over the pairs j of offset k of in[imap[j]][ci] * gout[omap[j]][co]
//
// The contraction runs over pairs.  A workgroup takes a run of pairs of one
// offset ("chunk") and a CI x CO tile of dW[k] (the whole matrix up to
// 128 x 128), stages the gathered `in` rows and `gout` rows of 64 (fp16) or 32
// (fp32) pairs at a time in LDS with 16-byte loads, double-buffered so the next
// stage's gathers are in flight while the current one is multiplied, and keeps
// the tile in MFMA accumulators until the chunk ends; one fp32 atomic flush per
// workgroup.  Each row is gathered once per chunk, not once per 32x32 tile of dW
// as in the reference (backend/bwd_kernels.cuh:935-954).
//
// fp16: both MFMA operands need 8 consecutive PAIRS of one channel per lane,
// the transpose of how rows sit in LDS; ds_read_b64_tr_b16 does that transpose
// on the way out of LDS (16 lanes hand in the addresses of a 4-row x 16-column
// block, lane i gets column i).  fp32: v_mfma_f32_32x32x2_f32 takes one element
// per lane, so plain ds_read_b32 along a row is already the right shape.
#include <type_traits>

#include <stdlib.h>

#include <map>
#include <mutex>

#include "fgms_device.h"
#include "fgms_internal.h"
#include "fgms_wgrad_bodies.h"

namespace fgms {
namespace {


constexpr int kThreads = 256;
constexpr int kSkinnyThreads = 256;    // the skinny weight-gradient kernel

// The workgroup-level variant (wgrad_wg_body) in a launch of its own.
template <typename T, int BI, int BJ, bool SPLIT>
__global__ __launch_bounds__(kThreads) void wgrad_kernel(
    const T *__restrict__ in, const T *__restrict__ gout, float *__restrict__ gw32,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
    const int32_t *__restrict__ omap, int k_vol, int c_in, int c_out, SliceMap smap, SideJob side) {
  // the leading workgroups of the grid run the side job, if there is one
  int block_x = blockIdx.x;
  if (side.blocks) {
    if (block_x < side.blocks) {
      if (blockIdx.y == 0) run_side_job(side, block_x);
      return;
    }
    block_x -= side.blocks;
  }
  wgrad_wg_body<T, BI, BJ, SPLIT>(in, gout, gw32, kpos, imap, omap, k_vol, c_in, c_out, smap, block_x, blockIdx.y);
}

// The per-wave variant (wgrad_wave_body) in a launch of its own.
template <typename T, int BI, int BJ, bool SPLIT>
__global__ __launch_bounds__(kThreads, 3) void wgrad_wave_kernel(
    const T *__restrict__ in, const T *__restrict__ gout, float *__restrict__ gw32,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
    const int32_t *__restrict__ omap, int k_vol, int c_in, int c_out, SliceMap smap, SideJob side,
    unsigned in_bytes, unsigned gout_bytes) {
  // the leading workgroups of the grid run the side job, if there is one
  int block_x = blockIdx.x;
  if (side.blocks) {
    if (block_x < side.blocks) {
      if (blockIdx.y == 0) run_side_job(side, block_x);
      return;
    }
    block_x -= side.blocks;
  }
  wgrad_wave_body<T, BI, BJ, SPLIT>(in, gout, gw32, kpos, imap, omap, k_vol, c_in, c_out, smap, block_x, blockIdx.y,
                                    in_bytes, gout_bytes);
}

// ---------------------------------------------------------------------------
// Skinny layers (4 / 8 / 16 input channels, e.g. the 4 -> 32 first layer of a voxel
// network): a 4 x 32 tile of dW[k] is no work for the matrix cores and the pass is all
// gathers, 8 + 64 bytes a pair in fp16 -- so few bytes per pair that the number of load
// INSTRUCTIONS is what counts.  A wave takes 64 pairs a round: lane l fetches the two
// indices and the whole input row of pair l (one instruction each for the wave), then the
// round is worked off in U steps of 64 / U pairs, GD = U lanes sharing a pair with 16 bytes
// of its output-gradient row each (one load instruction a step); the pair's index and
// input row reach those lanes by shuffles.  A lane keeps a CS x KD block of products in
// registers.  Everything is loaded unconditionally (clamped to the slice; pairs past its
// end count with weight 0).  At the end the lanes that hold the same channels add up
// (shuffles), then the four waves (LDS), then one atomic add per tile element and
// workgroup.
// N consecutive elements (a multiple of four; 8- or 16-byte aligned) widened to fp32.
template <typename T, int N>
__device__ __forceinline__ void load_elems(float (&x)[N], const T *__restrict__ p) {
  static_assert(N % 4 == 0, "rows are read four elements at a time");
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int i = 0; i < N / 4; ++i) {
      const float4v v = reinterpret_cast<const float4v *>(p)[i];
      x[4 * i] = v[0]; x[4 * i + 1] = v[1]; x[4 * i + 2] = v[2]; x[4 * i + 3] = v[3];
    }
  } else if constexpr (N % 8 == 0) {
#pragma unroll
    for (int i = 0; i < N / 8; ++i) {
      const half8 v = reinterpret_cast<const half8 *>(p)[i];
#pragma unroll
      for (int j = 0; j < 8; ++j) x[8 * i + j] = (float)v[j];
    }
  } else {
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int i = 0; i < N / 4; ++i) {
      const half4 v = reinterpret_cast<const half4 *>(p)[i];
      x[4 * i] = (float)v[0]; x[4 * i + 1] = (float)v[1]; x[4 * i + 2] = (float)v[2]; x[4 * i + 3] = (float)v[3];
    }
  }
}

template <typename T, int CS, int CD>
__global__ __launch_bounds__(kSkinnyThreads) void wgrad_skinny_kernel(
    const T *__restrict__ in, const T *__restrict__ gout, float *__restrict__ gw32,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
    const int32_t *__restrict__ omap, int k_vol, SliceMap smap) {
  constexpr int KD = 16 / (int)sizeof(T);     // output channels per lane: one 16-byte load
  constexpr int GD = CD / KD;                 // lanes per pair = steps per round
  constexpr int PPS = 64 / GD;                // pairs per step
  constexpr int XW = CS * (int)sizeof(T) / 4; // 32-bit words of an input row
  static_assert(CD % KD == 0 && 64 % GD == 0 && XW >= 1, "shape");
  extern __shared__ float red[];            // [waves - 1][CS][CD]
  constexpr int kWavesS = kSkinnyThreads / 64;
  int k, first, count;
  if (!locate_slice(kpos, smap, k_vol, blockIdx.x, k, first, count)) return;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int sub = lane / GD, cg = lane % GD;
  const int rounds = (count + kSkinnyThreads - 1) / kSkinnyThreads;

  float acc[CS][KD];
#pragma unroll
  for (int i = 0; i < CS; ++i)
#pragma unroll
    for (int j = 0; j < KD; ++j) acc[i][j] = 0.f;

  // pair lane l fetches in round rd
  auto my_pair = [&](int rd) { return (rd * kWavesS + wave) * 64 + lane; };
  auto load_x = [&](uint32_t (&xw)[XW], int row) {
    const uint32_t *p = reinterpret_cast<const uint32_t *>(in + (size_t)row * CS);
    if constexpr (XW % 4 == 0) {
#pragma unroll
      for (int i = 0; i < XW / 4; ++i) {
        const int4v v = reinterpret_cast<const int4v *>(p)[i];
        xw[4 * i] = v[0]; xw[4 * i + 1] = v[1]; xw[4 * i + 2] = v[2]; xw[4 * i + 3] = v[3];
      }
    } else {
      typedef unsigned uint2v __attribute__((ext_vector_type(2)));
#pragma unroll
      for (int i = 0; i < XW / 2; ++i) {
        const uint2v v = reinterpret_cast<const uint2v *>(p)[i];
        xw[2 * i] = v[0]; xw[2 * i + 1] = v[1];
      }
    }
  };
  // Pipeline over the rounds: entering round rd the input rows and output-gradient rows
  // of rd and the indices of rd + 1 are there (or on their way); the round issues the
  // indices of rd + 2 and the rows of rd + 1 in one block, then multiplies.  The
  // scheduling barrier keeps the loads together in front of the arithmetic (left alone,
  // the compiler feeds them in one at a time between the multiply-adds, each waiting for
  // the one before).
  auto load_g = [&](float (&g)[GD][KD], int gi_lane) {
#pragma unroll
    for (int u = 0; u < GD; ++u) {
      const int row = __shfl(gi_lane, u * PPS + sub);
      load_elems<T, KD>(g[u], gout + (size_t)row * CD + cg * KD);
    }
  };
  uint32_t xw[XW], xw_n[XW];
  float g[GD][KD], g_n[GD][KD];
  {
    const int p0 = first + min(my_pair(0), count - 1);
    load_x(xw, imap[p0]);
    load_g(g, omap[p0]);
  }
  int xi_n = imap[first + min(my_pair(1), count - 1)], gi_n = omap[first + min(my_pair(1), count - 1)];
  for (int rd = 0; rd < rounds; ++rd) {
    const int p_nn = first + min(my_pair(rd + 2), count - 1);
    const int xi_nn = imap[p_nn], gi_nn = omap[p_nn];
    load_x(xw_n, xi_n);
    load_g(g_n, gi_n);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < GD; ++u) {
      const int src = u * PPS + sub;
      const float live = (rd * kWavesS + wave) * 64 + src < count ? 1.f : 0.f;
      float x[CS];
#pragma unroll
      for (int i = 0; i < XW; ++i) {
        const uint32_t word = (uint32_t)__shfl((int)xw[i], src);
        if constexpr (sizeof(T) == 4) {
          x[i] = __builtin_bit_cast(float, word) * live;
        } else {
          x[2 * i] = (float)__builtin_bit_cast(_Float16, (unsigned short)(word & 0xffffu)) * live;
          x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(word >> 16)) * live;
        }
      }
#pragma unroll
      for (int i = 0; i < CS; ++i)
#pragma unroll
        for (int j = 0; j < KD; ++j) acc[i][j] += x[i] * g[u][j];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < XW; ++i) xw[i] = xw_n[i];
#pragma unroll
    for (int u = 0; u < GD; ++u)
#pragma unroll
      for (int j = 0; j < KD; ++j) g[u][j] = g_n[u][j];
    xi_n = xi_nn;
    gi_n = gi_nn;
  }
  // lanes sub = 0 .. PPS-1 with the same cg hold the same channels
#pragma unroll
  for (int off = GD; off < 64; off <<= 1)
#pragma unroll
    for (int i = 0; i < CS; ++i)
#pragma unroll
      for (int j = 0; j < KD; ++j) acc[i][j] += __shfl_xor(acc[i][j], off);
  if (wave > 0 && sub == 0) {
#pragma unroll
    for (int i = 0; i < CS; ++i)
#pragma unroll
      for (int j = 0; j < KD; ++j) red[((wave - 1) * CS + i) * CD + cg * KD + j] = acc[i][j];
  }
  __syncthreads();
  if (wave == 0 && sub == 0) {
#pragma unroll
    for (int i = 0; i < CS; ++i)
#pragma unroll
      for (int j = 0; j < KD; ++j) {
        float v = acc[i][j];
        for (int w = 0; w < kWavesS - 1; ++w) v += red[(w * CS + i) * CD + cg * KD + j];
        atomic_add(gw32 + ((size_t)k * CS + i) * CD + cg * KD + j, v);
      }
  }
}

// dst[i] += acc[i] rounded once to fp16 and acc[i] = 0, in a launch of its own.
__global__ void add_and_clear_kernel(__half *__restrict__ dst, float *__restrict__ acc, size_t n) {
  add_and_clear_elements(dst, acc, n, (size_t)blockIdx.x * blockDim.x + threadIdx.x,
                         (size_t)gridDim.x * blockDim.x);
}

int blocks_of(int c) { return c % 128 == 0 ? 4 : (c % 64 == 0 ? 2 : 1); }

// 32-column blocks (BI x BJ) of the tile a wave or workgroup holds of dW[k].  A 128 x 128 fp16 tile
// in a launch of its own is cut into four 64 x 64 tiles for the per-wave body (rows gathered twice,
// twelve independent waves per CU instead of two workgroups of four: 110 -> 100 us at 128 -> 128
// over 120k voxels); in the backward launch, next to the input gradient's workgroups, the
// workgroup-level body stays ahead (163 against 166 us).
void tile_blocks(const WgradArgs &a, bool shares_grid, int *bi, int *bj) {
  *bi = blocks_of(a.c_in);
  *bj = blocks_of(a.c_out);
  if (!shares_grid && a.dtype == FGMS_F16 && *bi * *bj == 16) {
    *bi = 2;
    *bj = 2;
  }
}

// Slices per offset: from the plan's row bands when it has them, `stride` bands to
// a slice so that about `want_wgs` workgroups result; else equal pair counts,
// enough to fill the chip a few times with at least ~16 stages of pairs per slice
// on average.  A multiple of 8 (one per XCD).
SliceMap choose_slices(const WgradArgs &a, int ty, int stage_pairs, int64_t want_wgs) {
  SliceMap m{};
  if (a.plan && a.plan->bands_ok && a.plan->band_start && a.plan->k_vol == a.k_vol &&
      a.plan->n_pairs == a.n_pairs && a.plan->n_out == a.n_out) {
    m.band_start = a.plan->band_start;
    m.bands = a.plan->band_count;
    m.stride = 1;
    while (m.stride < 8 && (int64_t)(m.bands / (m.stride * 2)) * a.k_vol * ty >= want_wgs &&
           (m.bands / (m.stride * 2)) % 8 == 0)
      m.stride *= 2;
    m.slices = (m.bands + m.stride - 1) / m.stride;
    if (m.stride == 1) {
      // as many bands in flight per XCD as fit its 4 MB L2 (both feature matrices' rows)
      const size_t band_bytes = (size_t)a.plan->band_rows * (a.c_in + a.c_out) * (a.dtype == FGMS_F16 ? 2 : 4);
      int t = 3;
      while (t > 0 && (((size_t)1 << t) * band_bytes > (size_t)7 << 19 || (1 << t) > m.bands / 8)) --t;
      m.cells = a.plan->band_cells + (size_t)t * m.bands * a.k_vol;
    }
    return m;
  }
  int64_t slices = want_wgs / ((int64_t)a.k_vol * ty);
  const int64_t by_work = a.n_pairs / ((int64_t)a.k_vol * 16 * stage_pairs);
  if (slices > by_work) slices = by_work;
  slices = (slices + 7) / 8 * 8;
  m.slices = (int)(slices < 8 ? 8 : slices);
  return m;
}

template <typename T, int BI, int BJ>
int launch(const WgradArgs &a, float *acc32) {
  WgradGeometry g;
  int rc = wgrad_geometry(a, &g);
  if (rc != FGMS_OK) return rc;
  constexpr bool kCanSplit = sizeof(T) == 4;
  auto kern = g.split ? wgrad_kernel<T, BI, BJ, kCanSplit> : wgrad_kernel<T, BI, BJ, false>;
  { const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)g.lds); if (rc_lds != FGMS_OK) return rc_lds; }
  {
    ProfileScope prof(g.split ? "wgrad_kernel(bf16x3)" : "wgrad_kernel", a.stream);
    kern<<<dim3((unsigned)g.tiles + (unsigned)a.side.blocks, (unsigned)g.ty), kThreads, g.lds, a.stream>>>(
        (const T *)a.in, (const T *)a.gout, acc32, a.kpos, a.imap, a.omap, a.k_vol, a.c_in,
        a.c_out, g.smap, a.side);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

template <typename T, int BI, int BJ>
int launch_wave(const WgradArgs &a, float *acc32) {
  WgradGeometry g;
  int rc = wgrad_geometry(a, &g);
  if (rc != FGMS_OK) return rc;
  constexpr bool kCanSplit = sizeof(T) == 4;
  auto kern = g.split ? wgrad_wave_kernel<T, BI, BJ, kCanSplit> : wgrad_wave_kernel<T, BI, BJ, false>;
  { const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)g.lds); if (rc_lds != FGMS_OK) return rc_lds; }
  {
    ProfileScope prof(g.split ? "wgrad_wave_kernel(bf16x3)" : "wgrad_wave_kernel", a.stream);
    kern<<<dim3((unsigned)g.tiles + (unsigned)a.side.blocks, (unsigned)g.ty), kThreads, g.lds, a.stream>>>(
        (const T *)a.in, (const T *)a.gout, acc32, a.kpos, a.imap, a.omap, a.k_vol, a.c_in,
        a.c_out, g.smap, a.side, (unsigned)((size_t)a.n_in * a.c_in * sizeof(T)),
        (unsigned)((size_t)a.n_out * a.c_out * sizeof(T)));
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

bool skinny_shape(const WgradArgs &a) {
  const size_t esz = a.dtype == FGMS_F16 ? 2 : 4;
  return (a.c_in == 4 || a.c_in == 8 || a.c_in == 16) && (a.c_out == 16 || a.c_out == 32 || a.c_out == 64) &&
         reinterpret_cast<uintptr_t>(a.in) % 16 == 0 && reinterpret_cast<uintptr_t>(a.gout) % 16 == 0 &&
         (size_t)a.c_in * esz % 8 == 0;
}

template <typename T, int CS, int CD>
int launch_skinny(const WgradArgs &a, float *acc32) {
  if (a.side.kind != 0) {       // nothing rides along with this launch
    int rc = launch_side_job(a.side, a.stream);
    if (rc != FGMS_OK) return rc;
  }
  // Few, big workgroups (about two to a CU): measured on the 4 -> 32 layer over 2.1 M
  // pairs, 34 us against 40 us with six to a CU, 36-72 us with equal runs of the pair list
  // instead of the plan's (offset, band) cells (workgroups that run at the same time then
  // work on the same offset and their closing atomic adds queue on the same addresses),
  // and 40-68 us with 16-wave workgroups.
  static const int wgs_per_cu = getenv("FGMS_SKINNY_WGS") ? atoi(getenv("FGMS_SKINNY_WGS")) : 2;
  const SliceMap smap = choose_slices(a, 1, 64, (int64_t)num_cus() * wgs_per_cu);
  const int64_t tiles = (int64_t)smap.slices * a.k_vol;
  const size_t lds = (size_t)(kSkinnyThreads / 64 - 1) * CS * CD * sizeof(float);
  auto kern = wgrad_skinny_kernel<T, CS, CD>;
  { const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)lds); if (rc_lds != FGMS_OK) return rc_lds; }
  {
    ProfileScope prof("wgrad_skinny_kernel", a.stream);
    kern<<<(unsigned)tiles, kSkinnyThreads, lds, a.stream>>>(
        (const T *)a.in, (const T *)a.gout, acc32, a.kpos, a.imap, a.omap, a.k_vol, smap);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

template <typename T>
int dispatch(const WgradArgs &a, float *acc32) {
  if (skinny_shape(a)) {
#define FGMS_WS(I, J) if (a.c_in == I && a.c_out == J) return launch_skinny<T, I, J>(a, acc32);
    FGMS_WS(4, 16) FGMS_WS(4, 32) FGMS_WS(4, 64)
    FGMS_WS(8, 16) FGMS_WS(8, 32) FGMS_WS(8, 64)
    FGMS_WS(16, 16) FGMS_WS(16, 32) FGMS_WS(16, 64)
#undef FGMS_WS
  }
  int bi, bj;
  tile_blocks(a, false, &bi, &bj);
#define FGMS_WW(I, J) if (bi == I && bj == J) return launch_wave<T, I, J>(a, acc32);
  FGMS_WW(1, 1) FGMS_WW(1, 2) FGMS_WW(2, 1) FGMS_WW(2, 2)
#undef FGMS_WW
#define FGMS_WG(I, J) if (bi == I && bj == J) return launch<T, I, J>(a, acc32);
  FGMS_WG(1, 4) FGMS_WG(2, 4)
  FGMS_WG(4, 1) FGMS_WG(4, 2) FGMS_WG(4, 4)
#undef FGMS_WG
  set_error("launch_mfma_wgrad: unsupported shape");
  return FGMS_E_INVALID;
}

}  // namespace

bool mfma_wgrad_supported(const WgradArgs &a) {
  if (skinny_shape(a)) return true;     // (no MFMA there: the skinny kernel shares this path's accumulator)
  if (a.c_in % 32 != 0 || a.c_out % 32 != 0) return false;
  if (reinterpret_cast<uintptr_t>(a.in) % 16 || reinterpret_cast<uintptr_t>(a.gout) % 16) return false;
  // (rows are addressed by 32-bit byte offsets through buffer resources)
  const size_t esz = a.dtype == FGMS_F16 ? 2 : 4;
  if ((size_t)a.n_in * a.c_in * esz > kMaxBufferBytes || (size_t)a.n_out * a.c_out * esz > kMaxBufferBytes) return false;
  return true;
}

int wgrad_geometry(const WgradArgs &a, WgradGeometry *g, bool shares_grid) {
  if (skinny_shape(a) || !mfma_wgrad_supported(a)) {
    set_error("wgrad_geometry: not a shape of the MFMA weight-gradient kernels");
    return FGMS_E_INVALID;
  }
  const bool f16 = a.dtype == FGMS_F16;
  const size_t esz = f16 ? 2 : 4;
  int bi, bj;
  tile_blocks(a, shares_grid, &bi, &bj);
  const int pad = f16 ? WT<__half>::pad : WT<float>::pad;
  *g = WgradGeometry{};
  g->bi = bi;
  g->bj = bj;
  g->ty = (a.c_in / (32 * bi)) * (a.c_out / (32 * bj));
  g->wave = bi <= 2 && bj <= 2;
  if (g->wave) {
    const int sp = f16 ? WTW<__half>::stage_pairs : WTW<float>::stage_pairs;
    g->smap = choose_slices(a, g->ty, sp, (int64_t)num_cus() * 6);
    g->tiles = (int64_t)g->smap.slices * a.k_vol;
    // fp32 tensors whose caller allows tf32 precision: four 16-bit tiles per wave instead
    g->split = !f16 && a.reduced && split_bf16_enabled();
    const size_t lds = (g->split ? 4 * (size_t)sp * 2 * ((bi * 32 + 16) + (bj * 32 + 16)) * 2
                                 : 4 * (size_t)sp * ((bi * 32 + (f16 ? 0 : pad)) + (bj * 32 + (f16 ? 0 : pad))) * esz)
                       + 4 * 64 * sizeof(int);                           // + the waves' index exchange
    const size_t red = 3 * (size_t)bi * bj * 16 * 64 * sizeof(float);     // the partial tiles' exchange
    g->lds = lds < red ? red : lds;
    return FGMS_OK;
  }
  const int sp = f16 ? WT<__half>::stage_pairs : WT<float>::stage_pairs;
  if (bi * bj == 16) {
    // whole 128 x 128 tiles (64 KB to flush per workgroup, 2 workgroups per CU):
    // equal tiles in pair-list order, measured faster than row bands; about 4 per CU in a
    // launch of their own, 2 where the input gradient's workgroups share the grid and keep
    // the chip busy (128 -> 128 over 120k voxels: 160 us against 169 with 4, 179 with 1)
    const int per_cu = shares_grid ? 2 : 4;
    int64_t chunk = (a.n_pairs + (int64_t)num_cus() * per_cu - 1) / ((int64_t)num_cus() * per_cu);
    chunk = (chunk + sp - 1) / sp * sp;
    if (chunk < 4 * sp) chunk = 4 * sp;
    g->smap.chunk = (int)chunk;
    g->tiles = (a.n_pairs + chunk - 1) / chunk + a.k_vol;
  } else {
    g->smap = choose_slices(a, g->ty, sp, (int64_t)num_cus() * 4);
    g->tiles = (int64_t)g->smap.slices * a.k_vol;
  }
  g->split = !f16 && a.reduced && split_bf16_enabled();
  g->lds = g->split ? 2 * (size_t)sp * 2 * ((bi * 32 + 16) + (bj * 32 + 16)) * 2
                    : 2 * (size_t)sp * ((bi * 32 + pad) + (bj * 32 + pad)) * esz;
  return FGMS_OK;
}

int wgrad_accumulator(const WgradArgs &a, float **acc32) {
  if (a.dtype != FGMS_F16) {
    *acc32 = (float *)a.gw;
    return FGMS_OK;
  }
  if (a.acc_override) {
    *acc32 = a.acc_override;
    return FGMS_OK;
  }
  // partial sums of all workgroups meet in fp32 and are rounded to fp16 once.
  // The accumulator is zero-filled when it is (re)allocated and left zero by
  // every call, so no fill launch is needed per call.
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  void *ws = nullptr;
  bool fresh = false;
  int rc = workspace_get(a.stream, 1, n * sizeof(float), &ws, &fresh);
  if (rc != FGMS_OK) return rc;
  if (fresh && (rc = launch_fill_zero(ws, workspace_bytes(a.stream, 1), a.stream))) return rc;
  *acc32 = (float *)ws;
  return FGMS_OK;
}

int wgrad_finish(const WgradArgs &a, float *acc32) {
  if (a.dtype != FGMS_F16) return FGMS_OK;
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  add_and_clear_kernel<<<(unsigned)((n + 255) / 256), 256, 0, a.stream>>>((__half *)a.gw, acc32, n);
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

int launch_mfma_wgrad(const WgradArgs &a) {
  float *acc32 = nullptr;
  int rc = wgrad_accumulator(a, &acc32);
  if (rc != FGMS_OK) return rc;
  if (a.dtype != FGMS_F16) return dispatch<float>(a, acc32);
  if ((rc = dispatch<__half>(a, acc32))) {
    const size_t bytes = a.acc_override ? (size_t)a.k_vol * a.c_in * a.c_out * sizeof(float)
                                        : workspace_bytes(a.stream, 1);
    (void)launch_fill_zero(acc32, bytes, a.stream);
    return rc;
  }
  if (a.deferred_flush) {
    // the caller attaches the flush to its next launch on the stream
    const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
    SideJob &f = *a.deferred_flush;
    f = SideJob{};
    f.kind = 2;
    f.dst = a.gw;
    f.acc = acc32;
    f.n = n;
    f.dtype = a.dtype;
    size_t blocks = ((n + 2047) / 2048 + 7) / 8 * 8;   // about 8 elements per thread
    f.blocks = (int)(blocks > 1024 ? 1024 : blocks);
    return FGMS_OK;
  }
  return wgrad_finish(a, acc32);
}

// ---------------------------------------------------------------------------
// The weight gradient for callers that cannot allocate (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc): the fp32 accumulator of the fp16 path
// lives in a file-scope device array instead of the stream's grown-on-demand workspace.
// Every GPU holds its own copy of the array at its own address until the process ends; the
// array's name is only a host-side handle, so its device address is asked for once per
// device and kept.
constexpr size_t kScratchFloats = (size_t)2 << 20;       // 8 MiB: 27 offsets of 256 x 256 fit
static __device__ __align__(256) float scratch[kScratchFloats];

namespace {
std::mutex g_scratch_mutex;
std::map<int, float *> g_scratch_ptr;       // device -> address of that device's copy

int scratch_address(float **ptr) {
  int dev = 0;
  FGMS_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  auto it = g_scratch_ptr.find(dev);
  if (it != g_scratch_ptr.end()) {
    *ptr = it->second;
    return FGMS_OK;
  }
  float *p = nullptr;
  FGMS_HIP_TRY(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
  g_scratch_ptr[dev] = p;
  *ptr = p;
  return FGMS_OK;
}
}  // namespace

int wgrad_static(WgradArgs a) {
  if (a.n_pairs == 0) return FGMS_OK;
  if (kernel_policy() == 1 || !mfma_wgrad_supported(a)) {
    set_error("fgms_wgrad_static: only the shapes of the MFMA / skinny weight-gradient kernels "
              "(channel counts that are multiples of 32, or 4/8/16 -> 16/32/64; 16-byte aligned rows)");
    return FGMS_E_INVALID;
  }
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  if (a.dtype == FGMS_F16) {
    if (n > kScratchFloats) {
      set_error("fgms_wgrad_static: k_vol * c_in * c_out = %zu exceeds the static accumulator's %zu floats",
                n, kScratchFloats);
      return FGMS_E_INVALID;
    }
    float *ptr = nullptr;
    int rc = scratch_address(&ptr);
    if (rc != FGMS_OK) return rc;
    // the array keeps what the last call left (a failed or overlapping call may have left
    // sums behind): the part this call uses starts from zero
    if ((rc = launch_fill_zero(ptr, n * sizeof(float), a.stream))) return rc;
    a.acc_override = ptr;
  }
  a.side = SideJob{};
  a.deferred_flush = nullptr;
  if (a.plan) plan_touch(a.plan, a.stream);
  return launch_mfma_wgrad(a);
}

}  // namespace fgms
