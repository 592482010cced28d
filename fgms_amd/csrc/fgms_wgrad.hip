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

#include "fgms_device.h"
#include "fgms_internal.h"

namespace fgms {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kSkinnyThreads = 256;    // the skinny weight-gradient kernel

template <typename T> struct WT;
template <> struct WT<__half> {
  static constexpr int E = 8;          // elements per 16-byte chunk
  static constexpr int stage_pairs = 64;
  static constexpr int step_pairs = 16; // pairs per k-step (one 32x32x16 MFMA)
  static constexpr int pad = 16;        // row padding in elements (32 bytes)
};
template <> struct WT<float> {
  static constexpr int E = 4;
  static constexpr int stage_pairs = 32;
  static constexpr int step_pairs = 8;  // four 32x32x2 MFMAs
  static constexpr int pad = 4;
};

template <int BI, int BJ> struct WaveGrid {
  static constexpr int WI = BI >= 2 ? (BJ == 1 && BI == 4 ? 4 : 2) : 1;
  static constexpr int WJ = BJ >= 2 ? (BI == 1 && BJ == 4 ? 4 : (WI == 4 ? 1 : 2)) : 1;
  static constexpr int WK = 4 / (WI * WJ);
  static constexpr int TI = BI / WI;
  static constexpr int TJ = BJ / WJ;
  static_assert(WI * WJ * WK == 4 && TI * WI == BI && TJ * WJ == BJ, "wave grid");
};

// One k-step (16 pairs) of one 32-wide operand block, fp16: returns the 8
// pair-values of channel (lane % 32) for pairs p0 + 8 * (lane / 32) + 0..7.
__device__ __forceinline__ half8 tr_frag(const __half *tile, int ld, int p0, int c0, int lane) {
  const int b = lane >> 4, i = lane & 15, h = lane >> 5;
  const __half *base = tile + (size_t)(p0 + h * 8 + (i >> 2)) * ld + c0 + (b & 1) * 16 + (i & 3) * 4;
  typedef __attribute__((address_space(3))) short4v lds_v4;
  const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4 *)(base));
  const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4 *)(base + 4 * ld));
  const short8v v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(half8, v);
}

// Workgroup -> (slice sl of the pair list, offset k) and the slice's pair range.
// Workgroups go to the 8 XCDs round-robin; numbering them so that one XCD gets
// all the offsets of a slice lets the rows one offset pulled into that XCD's L2
// serve the other offsets of the slice, provided slice sl of every offset covers
// the same band of rows.  With a plan whose pair lists are ordered by output row
// a slice is `stride` consecutive row bands of the plan (band_start, found by
// bisection when the plan was built); without one every offset is cut into equal
// pair counts, which only approximates it.  slices is a multiple of 8.
struct SliceMap {
  const int32_t *band_start;   // [k_vol][bands + 1] or nullptr
  const int32_t *cells;        // the plan's dispatch order of the (offset, band) cells, or nullptr
  int bands, stride;           // slice sl = bands [sl * stride, (sl + 1) * stride)
  int slices;
  int chunk;                   // > 0: plain tiles of `chunk` pairs in pair-list order instead
};

__device__ __forceinline__ bool locate_slice(const int32_t *__restrict__ kpos, const SliceMap &m,
                                             int k_vol, int block, int &k, int &first, int &count) {
  if (m.chunk > 0) return locate_tile(kpos, k_vol, m.chunk, block, k, first, count);
  int sl;
  if (m.cells) {                    // biggest cells of this XCD first
    const int cell = m.cells[block];
    k = cell >> 16;
    sl = cell & 0xffff;
  } else {
    const int xcd = block % 8, idx = block / 8;
    sl = (idx / k_vol) * 8 + xcd;
    k = idx % k_vol;
  }
  if (sl >= m.slices) return false;
  const int k_first = kpos[k], k_count = kpos[k + 1] - k_first;
  if (m.band_start) {
    const int32_t *row = m.band_start + (size_t)k * (m.bands + 1);
    const int b0 = row[min(sl * m.stride, m.bands)], b1 = row[min((sl + 1) * m.stride, m.bands)];
    first = k_first + b0;
    count = b1 - b0;
  } else {
    const int per = (k_count + m.slices - 1) / m.slices;
    first = k_first + sl * per;
    count = min(per, k_count - sl * per);
  }
  return count > 0;
}

template <typename T, int BI, int BJ>
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
  using W = WT<T>;
  using G = WaveGrid<BI, BJ>;
  constexpr int E = W::E, SP = W::stage_pairs, KP = W::step_pairs;
  constexpr int CI = BI * 32, CO = BJ * 32;
  constexpr int LDI = CI + W::pad, LDO = CO + W::pad;
  constexpr int NCI = CI / E, NCO = CO / E;   // 16-byte chunks per staged row
  constexpr int NX = BI, NG = BJ;             // chunks per thread and stage
  extern __shared__ int4v lds[];
  // two staging buffers, each SP rows of `in` followed by SP rows of `dOut`.  (Addressed
  // by arithmetic on the LDS base: through an array of pointers the compiler loses the
  // address space and falls back to flat loads and stores, which also wait on the
  // global loads in flight.)
  T *const stage0 = reinterpret_cast<T *>(lds);
  constexpr int kBufElems = SP * (LDI + LDO);

  int k, first, count;
  if (!locate_slice(kpos, smap, k_vol, block_x, k, first, count)) return;
  const int tiles_co = c_out / CO;
  const int ci0 = (blockIdx.y / tiles_co) * CI;
  const int co0 = (blockIdx.y % tiles_co) * CO;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wi = wave % G::WI, wj = (wave / G::WI) % G::WJ, wk = wave / (G::WI * G::WJ);

  float16v acc[G::TI][G::TJ];
#pragma unroll
  for (int a = 0; a < G::TI; ++a)
#pragma unroll
    for (int b = 0; b < G::TJ; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  const int nstages = (count + SP - 1) / SP;
  int xi[NX], gi[NG];                  // gather rows of the stage about to be loaded
  int4v xa[NX], ga[NG], xb[NX], gb[NG];  // rows in flight: even stages in (xa, ga), odd ones in (xb, gb)

  // Everything below is issued unconditionally and nothing touches a loaded register
  // before its consumer: an index or a row that is selected, copied or loaded under a
  // branch makes the compiler wait for ALL loads in flight at that point, and the row
  // loads would no longer run under the MFMAs.  Past the end of the slice the last pair
  // is read again; store_rows zeroes those rows by their position instead.
  // Two stages of rows are in flight: loads complete in order, so the indices of stage
  // s + 1 are issued BEFORE the rows of stage s -- waiting for those indices then leaves
  // the rows behind them in flight.
  auto load_idx = [&](int st) {
#pragma unroll
    for (int i = 0; i < NX; ++i)
      xi[i] = imap[first + min(st * SP + (tid + kThreads * i) / NCI, count - 1)];
#pragma unroll
    for (int i = 0; i < NG; ++i)
      gi[i] = omap[first + min(st * SP + (tid + kThreads * i) / NCO, count - 1)];
  };
  auto load_rows = [&](int4v (&xr)[NX], int4v (&gr)[NG], const int (&xrow)[NX], const int (&grow)[NG]) {
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int cc = (tid + kThreads * i) % NCI;
      xr[i] = *reinterpret_cast<const int4v *>(in + (size_t)xrow[i] * c_in + ci0 + cc * E);
    }
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int cc = (tid + kThreads * i) % NCO;
      gr[i] = *reinterpret_cast<const int4v *>(gout + (size_t)grow[i] * c_out + co0 + cc * E);
    }
  };
  auto store_rows = [&](int buf, int st, const int4v (&xr)[NX], const int4v (&gr)[NG]) {
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int e = tid + kThreads * i;
      *reinterpret_cast<int4v *>(stage0 + buf * kBufElems + (e / NCI) * LDI + (e % NCI) * E) =
          st * SP + e / NCI < count ? xr[i] : int4v{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int e = tid + kThreads * i;
      *reinterpret_cast<int4v *>(stage0 + buf * kBufElems + SP * LDI + (e / NCO) * LDO + (e % NCO) * E) =
          st * SP + e / NCO < count ? gr[i] : int4v{0, 0, 0, 0};
    }
  };
  auto multiply = [&](int cur) {
    const T *x = stage0 + cur * kBufElems, *g = x + SP * LDI;
#pragma unroll
    for (int ks = wk; ks < SP / KP; ks += G::WK) {
      const int p0 = ks * KP;
      if constexpr (sizeof(T) == 2) {
        half8 a[G::TI], b[G::TJ];
#pragma unroll
        for (int ti = 0; ti < G::TI; ++ti) a[ti] = tr_frag(x, LDI, p0, (wi * G::TI + ti) * 32, lane);
#pragma unroll
        for (int tj = 0; tj < G::TJ; ++tj) b[tj] = tr_frag(g, LDO, p0, (wj * G::TJ + tj) * 32, lane);
#pragma unroll
        for (int ti = 0; ti < G::TI; ++ti)
#pragma unroll
          for (int tj = 0; tj < G::TJ; ++tj)
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ti], b[tj], acc[ti][tj], 0, 0, 0);
      } else {
        const int h = lane >> 5, c = lane & 31;
#pragma unroll
        for (int m = 0; m < KP / 2; ++m) {
          float a[G::TI], b[G::TJ];
#pragma unroll
          for (int ti = 0; ti < G::TI; ++ti) a[ti] = x[(p0 + 2 * m + h) * LDI + (wi * G::TI + ti) * 32 + c];
#pragma unroll
          for (int tj = 0; tj < G::TJ; ++tj) b[tj] = g[(p0 + 2 * m + h) * LDO + (wj * G::TJ + tj) * 32 + c];
#pragma unroll
          for (int ti = 0; ti < G::TI; ++ti)
#pragma unroll
            for (int tj = 0; tj < G::TJ; ++tj)
              acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ti], b[tj], acc[ti][tj], 0, 0, 0);
        }
      }
    }
  };
  // one stage: LDS buffer `cur` holds stage st; the rows of st + 1 are in flight in
  // (xn, gn), the index registers hold stage st + 2; (xf, gf) is free
  auto stage = [&](int st, int cur, int4v (&xf)[NX], int4v (&gf)[NG], const int4v (&xn)[NX],
                   const int4v (&gn)[NG]) {
    int xrow[NX], grow[NG];
#pragma unroll
    for (int i = 0; i < NX; ++i) xrow[i] = xi[i];
#pragma unroll
    for (int i = 0; i < NG; ++i) grow[i] = gi[i];
    load_idx(st + 3);                       // indices first ...
    __builtin_amdgcn_sched_barrier(0);
    load_rows(xf, gf, xrow, grow);          // ... then the rows of stage st + 2
    __builtin_amdgcn_sched_barrier(0);
    multiply(cur);
    // the stores wait for the rows of st + 1: keep them (and that wait) behind the MFMAs
    __builtin_amdgcn_sched_barrier(0);
    store_rows(cur ^ 1, st + 1, xn, gn);
    __syncthreads();
  };

  load_idx(0);
  {
    int xrow[NX], grow[NG];
#pragma unroll
    for (int i = 0; i < NX; ++i) xrow[i] = xi[i];
#pragma unroll
    for (int i = 0; i < NG; ++i) grow[i] = gi[i];
    load_idx(1);
    load_rows(xa, ga, xrow, grow);          // stage 0
  }
  {
    int xrow[NX], grow[NG];
#pragma unroll
    for (int i = 0; i < NX; ++i) xrow[i] = xi[i];
#pragma unroll
    for (int i = 0; i < NG; ++i) grow[i] = gi[i];
    load_idx(2);
    load_rows(xb, gb, xrow, grow);          // stage 1
  }
  store_rows(0, 0, xa, ga);
  __syncthreads();
  for (int st = 0; st < nstages; st += 2) {
    stage(st, 0, xa, ga, xb, gb);
    if (st + 1 >= nstages) break;
    stage(st + 1, 1, xb, gb, xa, ga);
  }

  // flush: accumulator register r of lane l is row (r/4)*8 + (l/32)*4 + r%4, column l%32
  const int h = lane >> 5, c = lane & 31;
#pragma unroll
  for (int ti = 0; ti < G::TI; ++ti)
#pragma unroll
    for (int tj = 0; tj < G::TJ; ++tj) {
      float *tile = gw32 + ((size_t)k * c_in + ci0 + (wi * G::TI + ti) * 32) * c_out + co0 +
                    (wj * G::TJ + tj) * 32 + c;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        atomic_add(tile + (size_t)((r / 4) * 8 + h * 4 + (r % 4)) * c_out, acc[ti][tj][r]);
    }
}

// Variant for dW tiles up to 64 x 64: every wave stages its own pairs in its own
// LDS region and multiplies them into a private copy of the whole tile, so the
// pair loop has no workgroup barrier at all (the four waves take the chunk's
// 32-pair stages round-robin); the four partial tiles are summed through LDS
// once, after the loop.  Each operand fragment read from LDS then feeds two
// MFMAs instead of one.
template <typename T> struct WTW;
template <> struct WTW<__half> { static constexpr int stage_pairs = 32; };
template <> struct WTW<float> { static constexpr int stage_pairs = 16; };

template <typename T, int BI, int BJ>
__global__ __launch_bounds__(kThreads, 3) void wgrad_wave_kernel(
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
  using W = WT<T>;
  constexpr int E = W::E, SP = WTW<T>::stage_pairs, KP = W::step_pairs;
  constexpr int CI = BI * 32, CO = BJ * 32;
  constexpr int LDI = CI + W::pad, LDO = CO + W::pad;
  constexpr int NCI = CI / E, NCO = CO / E;
  constexpr int NX = SP * NCI / 64, NG = SP * NCO / 64;   // chunks per lane and stage
  static_assert(NX >= 1 && NG >= 1, "stage too small");
  extern __shared__ int4v lds[];
  int k, first, count;
  if (!locate_slice(kpos, smap, k_vol, block_x, k, first, count)) return;
  const int tiles_co = c_out / CO;
  const int ci0 = (blockIdx.y / tiles_co) * CI;
  const int co0 = (blockIdx.y % tiles_co) * CO;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  T *x = reinterpret_cast<T *>(lds) + (size_t)wave * SP * (LDI + LDO);
  T *g = x + SP * LDI;

  float16v acc[BI][BJ];
#pragma unroll
  for (int a = 0; a < BI; ++a)
#pragma unroll
    for (int b = 0; b < BJ; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  const int nstages = (count + SP - 1) / SP;
  int xi[NX], gi[NG];        // gather rows of the next stage to load
  int4v xr[NX], gr[NG];      // the rows in flight

  // Everything is issued unconditionally and nothing touches a loaded register before
  // its consumer: an index or a row that is selected, copied or loaded under a branch
  // makes the compiler wait for ALL loads in flight at that point, and the row loads
  // would no longer run under the MFMAs.  Past the end of the slice the last pair is
  // read again; store_rows zeroes those rows by their position instead.
  auto load_idx = [&](int st) {
#pragma unroll
    for (int i = 0; i < NX; ++i)
      xi[i] = imap[first + min(st * SP + (lane + 64 * i) / NCI, count - 1)];
#pragma unroll
    for (int i = 0; i < NG; ++i)
      gi[i] = omap[first + min(st * SP + (lane + 64 * i) / NCO, count - 1)];
  };
  auto load_rows = [&]() {
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int cc = (lane + 64 * i) % NCI;
      xr[i] = *reinterpret_cast<const int4v *>(in + (size_t)xi[i] * c_in + ci0 + cc * E);
    }
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int cc = (lane + 64 * i) % NCO;
      gr[i] = *reinterpret_cast<const int4v *>(gout + (size_t)gi[i] * c_out + co0 + cc * E);
    }
  };
  auto store_rows = [&](int st) {     // st: the stage the rows in flight belong to
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int e = lane + 64 * i;
      *reinterpret_cast<int4v *>(x + (e / NCI) * LDI + (e % NCI) * E) =
          st * SP + e / NCI < count ? xr[i] : int4v{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int e = lane + 64 * i;
      *reinterpret_cast<int4v *>(g + (e / NCO) * LDO + (e % NCO) * E) =
          st * SP + e / NCO < count ? gr[i] : int4v{0, 0, 0, 0};
    }
  };
  auto wave_fence = [] {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  int st = wave;
  load_idx(st);
  load_rows();
  load_idx(st + 4);
  while (st < nstages) {
    store_rows(st);                 // waits for the stage's rows
    wave_fence();
    load_rows();                    // stage st + 4, in flight during the MFMAs
    __builtin_amdgcn_sched_barrier(0);   // (rows first, then indices, both before the MFMAs:
    load_idx(st + 8);                    //  the wait for the rows then leaves the indices in flight)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < SP / KP; ++ks) {
      const int p0 = ks * KP;
      if constexpr (sizeof(T) == 2) {
        half8 a[BI], b[BJ];
#pragma unroll
        for (int ti = 0; ti < BI; ++ti) a[ti] = tr_frag(x, LDI, p0, ti * 32, lane);
#pragma unroll
        for (int tj = 0; tj < BJ; ++tj) b[tj] = tr_frag(g, LDO, p0, tj * 32, lane);
#pragma unroll
        for (int ti = 0; ti < BI; ++ti)
#pragma unroll
          for (int tj = 0; tj < BJ; ++tj)
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ti], b[tj], acc[ti][tj], 0, 0, 0);
      } else {
        const int h = lane >> 5, c = lane & 31;
#pragma unroll
        for (int m = 0; m < KP / 2; ++m) {
          float a[BI], b[BJ];
#pragma unroll
          for (int ti = 0; ti < BI; ++ti) a[ti] = x[(p0 + 2 * m + h) * LDI + ti * 32 + c];
#pragma unroll
          for (int tj = 0; tj < BJ; ++tj) b[tj] = g[(p0 + 2 * m + h) * LDO + tj * 32 + c];
#pragma unroll
          for (int ti = 0; ti < BI; ++ti)
#pragma unroll
            for (int tj = 0; tj < BJ; ++tj)
              acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ti], b[tj], acc[ti][tj], 0, 0, 0);
        }
      }
    }
    wave_fence();                   // the tile is rewritten at the top of the loop
    st += 4;
  }

  // sum the four waves' tiles: (2, 3) -> (0, 1), then 1 -> 0, through LDS
  float *red = reinterpret_cast<float *>(lds);
  constexpr int kTileFloats = BI * BJ * 16 * 64;
  auto put = [&](int slot) {
#pragma unroll
    for (int ti = 0; ti < BI; ++ti)
#pragma unroll
      for (int tj = 0; tj < BJ; ++tj)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          red[(size_t)slot * kTileFloats + ((ti * BJ + tj) * 16 + r) * 64 + lane] = acc[ti][tj][r];
  };
  auto take = [&](int slot) {
#pragma unroll
    for (int ti = 0; ti < BI; ++ti)
#pragma unroll
      for (int tj = 0; tj < BJ; ++tj)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[ti][tj][r] += red[(size_t)slot * kTileFloats + ((ti * BJ + tj) * 16 + r) * 64 + lane];
  };
  __syncthreads();
  if (wave >= 2) put(wave - 2);
  __syncthreads();
  if (wave < 2) take(wave);
  __syncthreads();
  if (wave == 1) put(0);
  __syncthreads();
  if (wave != 0) return;
  take(0);
  const int h = lane >> 5, c = lane & 31;
#pragma unroll
  for (int ti = 0; ti < BI; ++ti)
#pragma unroll
    for (int tj = 0; tj < BJ; ++tj) {
      float *tile = gw32 + ((size_t)k * c_in + ci0 + ti * 32) * c_out + co0 + tj * 32 + c;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        atomic_add(tile + (size_t)((r / 4) * 8 + h * 4 + (r % 4)) * c_out, acc[ti][tj][r]);
    }
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

int num_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess)
      cus = p.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
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
  using W = WT<T>;
  constexpr int SP = W::stage_pairs;
  const int ty = (a.c_in / (32 * BI)) * (a.c_out / (32 * BJ));
  SliceMap smap{};
  int64_t tiles;
  if (BI * BJ == 16) {
    // whole 128 x 128 tiles (64 KB to flush per workgroup, 2 workgroups per CU):
    // equal tiles in pair-list order, about 4 per CU, measured faster than row bands
    int64_t chunk = (a.n_pairs + (int64_t)num_cus() * 4 - 1) / ((int64_t)num_cus() * 4);
    chunk = (chunk + SP - 1) / SP * SP;
    if (chunk < 4 * SP) chunk = 4 * SP;
    smap.chunk = (int)chunk;
    tiles = (a.n_pairs + chunk - 1) / chunk + a.k_vol;
  } else {
    smap = choose_slices(a, ty, SP, (int64_t)num_cus() * 4);
    tiles = (int64_t)smap.slices * a.k_vol;
  }
  const size_t lds = 2 * (size_t)SP * ((BI * 32 + W::pad) + (BJ * 32 + W::pad)) * sizeof(T);
  auto kern = wgrad_kernel<T, BI, BJ>;
  FGMS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  {
    ProfileScope prof("wgrad_kernel", a.stream);
    kern<<<dim3((unsigned)tiles + (unsigned)a.side.blocks, (unsigned)ty), kThreads, lds, a.stream>>>(
        (const T *)a.in, (const T *)a.gout, acc32, a.kpos, a.imap, a.omap, a.k_vol, a.c_in,
        a.c_out, smap, a.side);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

template <typename T, int BI, int BJ>
int launch_wave(const WgradArgs &a, float *acc32) {
  using W = WT<T>;
  constexpr int SP = WTW<T>::stage_pairs;
  const int ty = (a.c_in / (32 * BI)) * (a.c_out / (32 * BJ));
  const SliceMap smap = choose_slices(a, ty, SP, (int64_t)num_cus() * 6);
  const int64_t tiles = (int64_t)smap.slices * a.k_vol;
  size_t lds = 4 * (size_t)SP * ((BI * 32 + W::pad) + (BJ * 32 + W::pad)) * sizeof(T);
  const size_t red = 2 * (size_t)BI * BJ * 16 * 64 * sizeof(float);
  if (lds < red) lds = red;
  auto kern = wgrad_wave_kernel<T, BI, BJ>;
  FGMS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  {
    ProfileScope prof("wgrad_wave_kernel", a.stream);
    kern<<<dim3((unsigned)tiles + (unsigned)a.side.blocks, (unsigned)ty), kThreads, lds, a.stream>>>(
        (const T *)a.in, (const T *)a.gout, acc32, a.kpos, a.imap, a.omap, a.k_vol, a.c_in,
        a.c_out, smap, a.side);
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
  FGMS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
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
  const int bi = blocks_of(a.c_in), bj = blocks_of(a.c_out);
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
  return true;
}

int launch_mfma_wgrad(const WgradArgs &a) {
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  if (a.dtype == FGMS_F16) {
    // partial sums of all workgroups meet in fp32 and are rounded to fp16 once.
    // The accumulator is zero-filled when it is (re)allocated and left zero by
    // every call, so no fill launch is needed per call.
    void *ws = nullptr;
    bool fresh = false;
    int rc = workspace_get(a.stream, 1, n * sizeof(float), &ws, &fresh);
    if (rc != FGMS_OK) return rc;
    if (fresh && (rc = launch_fill_zero(ws, workspace_bytes(a.stream, 1), a.stream))) return rc;
    if ((rc = dispatch<__half>(a, (float *)ws))) {
      (void)launch_fill_zero(ws, workspace_bytes(a.stream, 1), a.stream);
      return rc;
    }
    if (a.deferred_flush) {
      // the caller attaches the flush to its next launch on the stream
      SideJob &f = *a.deferred_flush;
      f = SideJob{};
      f.kind = 2;
      f.dst = a.gw;
      f.acc = (float *)ws;
      f.n = n;
      f.dtype = a.dtype;
      size_t blocks = ((n + 2047) / 2048 + 7) / 8 * 8;   // about 8 elements per thread
      f.blocks = (int)(blocks > 1024 ? 1024 : blocks);
      return FGMS_OK;
    }
    add_and_clear_kernel<<<(unsigned)((n + 255) / 256), 256, 0, a.stream>>>((__half *)a.gw, (float *)ws, n);
    FGMS_HIP_TRY(hipGetLastError());
    return FGMS_OK;
  }
  return dispatch<float>(a, (float *)a.gw);
}

}  // namespace fgms
