// The bodies of the MFMA weight-gradient kernels and what they need, shared by the
// weight-gradient launch of its own and by the backward launch that runs them next to the
// input gradient.
#pragma once

#include "fgms_device.h"
#include "fgms_internal.h"
#include "fgms_mma.h"

namespace fgms {

typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));

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

// The same from a tile without row padding (rows of exactly `ld` = 32 or 64 halfs).  One
// transposing read touches rows p .. p + 3 and p + 8 .. p + 11, 64 bytes of each; with 128-byte
// rows, rows p and p + 2 would meet in the same banks, so the writer exchanges the two 64-byte
// halves of every row whose (row >> 1) is odd (wave tile below) and the read does the same.
template <int LD>
__device__ __forceinline__ half8 tr_frag_dense(const __half *tile, int p0, int c0, int lane) {
  static_assert(LD == 32 || LD == 64, "dense tile: 32 or 64 channels a row");
  const int b = lane >> 4, i = lane & 15, h = lane >> 5;
  const int sw = LD == 64 ? ((lane >> 3) & 1) * 32 : 0;
  const __half *base = tile + (size_t)(p0 + h * 8 + (i >> 2)) * LD + (c0 ^ sw) + (b & 1) * 16 + (i & 3) * 4;
  typedef __attribute__((address_space(3))) short4v lds_v4;
  const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4 *)(base));
  const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4 *)(base + 4 * LD));
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

// Split staging (fp32 rows whose caller allows tf32 precision): chunk c (4 fp32 values) of a
// staged row becomes 4 hi and 4 lo bf16 values in two 16-bit tiles laid out like the fp16
// path's.  Lane pairs hold neighbouring chunks and exchange halves, so the even lane writes
// 8 hi values and the odd one 8 lo values, 16 bytes each.
__device__ __forceinline__ void store_split_chunk(__half *hi_tile, __half *lo_tile, int ld, int row, int c,
                                                  const int4v &raw, bool valid, int lane) {
  const bool odd = lane & 1;
  const float4v v = valid ? __builtin_bit_cast(float4v, raw) : float4v{0.f, 0.f, 0.f, 0.f};
  bf16x4 hi, lo;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    __bf16 h, l;
    split_bf16(v[q], h, l);
    hi[q] = h;
    lo[q] = l;
  }
  const int2v h2 = __builtin_bit_cast(int2v, hi), l2 = __builtin_bit_cast(int2v, lo);
  const int got0 = __builtin_bit_cast(int, swap_with_neighbour(__builtin_bit_cast(float, odd ? h2[0] : l2[0])));
  const int got1 = __builtin_bit_cast(int, swap_with_neighbour(__builtin_bit_cast(float, odd ? h2[1] : l2[1])));
  if (odd) *reinterpret_cast<int4v *>(lo_tile + row * ld + (c - 1) * 4) = int4v{got0, got1, l2[0], l2[1]};
  else *reinterpret_cast<int4v *>(hi_tile + row * ld + c * 4) = int4v{h2[0], h2[1], got0, got1};
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

// (block_x, block_y): the workgroup's place in a grid of cells x tiles of dW[k]; 256 threads.
// SPLIT (fp32 tensors whose caller allows tf32 precision): the staged rows are split into
// bf16 pairs, x = hi + lo, on their way to LDS -- four 16-bit tiles per wave, laid out like
// the fp16 path's two -- and a product is three bf16 MFMAs, hi*hi + hi*lo + lo*hi, fed
// through the same transposing LDS reads as fp16.
template <typename T, int BI, int BJ, bool SPLIT = false>
__device__ __forceinline__ void wgrad_wave_body(
    const T *__restrict__ in, const T *__restrict__ gout, float *__restrict__ gw32,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
    const int32_t *__restrict__ omap, int k_vol, int c_in, int c_out, const SliceMap &smap,
    int block_x, int block_y, unsigned in_bytes, unsigned gout_bytes) {
  using W = WT<T>;
  constexpr int E = W::E, SP = WTW<T>::stage_pairs, KP = W::step_pairs;
  // fp16: rows through buffer loads (32-bit offsets; a slot past the end of the slice is loaded
  // from kAbsentRow and arrives as zeros) and all of a stage's fragments requested from LDS
  // before its first MFMA
  constexpr bool kBufW = sizeof(T) == 2 && !SPLIT;
  const __amdgpu_buffer_rsrc_t in_rsrc = rows_resource(in, in_bytes), gout_rsrc = rows_resource(gout, gout_bytes);
  constexpr int CI = BI * 32, CO = BJ * 32;
  // (fp16: rows without padding, 64-byte halves exchanged by row instead, see tr_frag_dense)
  constexpr int LDI = CI + (kBufW ? 0 : W::pad), LDO = CO + (kBufW ? 0 : W::pad);
  constexpr int NCI = CI / E, NCO = CO / E;
  constexpr int NX = SP * NCI / 64, NG = SP * NCO / 64;   // chunks per lane and stage
  static_assert(NX >= 1 && NG >= 1, "stage too small");
  extern __shared__ int4v lds[];
  int k, first, count;
  if (!locate_slice(kpos, smap, k_vol, block_x, k, first, count)) return;
  const int tiles_co = c_out / CO;
  const int ci0 = (block_y / tiles_co) * CI;
  const int co0 = (block_y % tiles_co) * CO;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  T *x = reinterpret_cast<T *>(lds) + (size_t)wave * SP * (LDI + LDO);
  T *g = x + SP * LDI;
  // SPLIT: 16-bit tiles with the fp16 path's row padding (32 bytes)
  constexpr int LDIh = CI + 16, LDOh = CO + 16;
  __half *xh = reinterpret_cast<__half *>(lds) + (size_t)wave * SP * 2 * (LDIh + LDOh);
  __half *xl = xh + SP * LDIh, *gh = xl + SP * LDIh, *gl = gh + SP * LDOh;
  static_assert(!SPLIT || (sizeof(T) == 4 && SP == 16), "split tiles: fp32 rows, one 16-pair MFMA step a stage");

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
  // fp16: a stage's 2 x SP indices arrive through ONE load (lanes 0..SP-1 read the input rows'
  // indices, lanes 32.. the output rows') and are handed round through 256 bytes of LDS behind
  // the staging tiles, instead of one load instruction per row instruction: a lane's chunks then
  // belong to NX (NG) consecutive pairs, whose indices it reads back with one LDS read each.
  static_assert(!kBufW || (SP == 32 && (NX == 2 || NX == 4) && (NG == 2 || NG == 4)), "index exchange: 32 pairs a stage");
  int *ibuf = reinterpret_cast<int *>(reinterpret_cast<T *>(lds) + (size_t)4 * SP * (LDI + LDO)) + wave * 64;
  const int32_t *const my_map = lane < 32 ? imap : omap;
  int idx_raw = 0;
  // chunk i of this lane: pair `row`, 16-byte piece `cc` of its row
  auto x_row = [&](int i) { return kBufW ? (lane / NCI) * NX + i : (lane + 64 * i) / NCI; };
  auto g_row = [&](int i) { return kBufW ? (lane / NCO) * NG + i : (lane + 64 * i) / NCO; };

  // Everything is issued unconditionally and nothing touches a loaded register before
  // its consumer: an index or a row that is selected, copied or loaded under a branch
  // makes the compiler wait for ALL loads in flight at that point, and the row loads
  // would no longer run under the MFMAs.  Past the end of the slice the last pair is
  // read again; store_rows zeroes those rows by their position instead.
  auto load_idx = [&](int st) {
    if constexpr (kBufW) {
      idx_raw = my_map[first + min(st * SP + (lane & 31), count - 1)];
      return;
    }
#pragma unroll
    for (int i = 0; i < NX; ++i)
      xi[i] = imap[first + min(st * SP + (lane + 64 * i) / NCI, count - 1)];
#pragma unroll
    for (int i = 0; i < NG; ++i)
      gi[i] = omap[first + min(st * SP + (lane + 64 * i) / NCO, count - 1)];
  };
  // fp16: the indices that load_idx fetched last, from idx_raw through LDS into xi / gi
  auto hand_round = [&]() {
    ibuf[lane] = idx_raw;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if constexpr (NX == 4) {
      const int4v v = *reinterpret_cast<const int4v *>(ibuf + (lane / NCI) * 4);
      xi[0] = v[0]; xi[1] = v[1]; xi[2] = v[2]; xi[3] = v[3];
    } else {
      const int2v v = *reinterpret_cast<const int2v *>(ibuf + (lane / NCI) * 2);
      xi[0] = v[0]; xi[1] = v[1];
    }
    if constexpr (NG == 4) {
      const int4v v = *reinterpret_cast<const int4v *>(ibuf + 32 + (lane / NCO) * 4);
      gi[0] = v[0]; gi[1] = v[1]; gi[2] = v[2]; gi[3] = v[3];
    } else {
      const int2v v = *reinterpret_cast<const int2v *>(ibuf + 32 + (lane / NCO) * 2);
      gi[0] = v[0]; gi[1] = v[1];
    }
  };
  auto load_rows = [&](int st_) {      // st_: the stage the indices in xi / gi belong to
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int cc = kBufW ? lane % NCI : (lane + 64 * i) % NCI;
      if constexpr (kBufW) {
        const bool live = st_ * SP + x_row(i) < count;
        const unsigned off = live ? (unsigned)xi[i] * (unsigned)(c_in * (int)sizeof(T)) : kAbsentRow;
        xr[i] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(
                                              in_rsrc, off + (unsigned)((ci0 + cc * E) * (int)sizeof(T)), 0, 0));
      } else {
        xr[i] = *reinterpret_cast<const int4v *>(in + (size_t)xi[i] * c_in + ci0 + cc * E);
      }
    }
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int cc = kBufW ? lane % NCO : (lane + 64 * i) % NCO;
      if constexpr (kBufW) {
        const bool live = st_ * SP + g_row(i) < count;
        const unsigned off = live ? (unsigned)gi[i] * (unsigned)(c_out * (int)sizeof(T)) : kAbsentRow;
        gr[i] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(
                                              gout_rsrc, off + (unsigned)((co0 + cc * E) * (int)sizeof(T)), 0, 0));
      } else {
        gr[i] = *reinterpret_cast<const int4v *>(gout + (size_t)gi[i] * c_out + co0 + cc * E);
      }
    }
  };
  auto store_rows = [&](int st) {     // st: the stage the rows in flight belong to
#pragma unroll
    for (int i = 0; i < NX; ++i) {
      const int e = lane + 64 * i;
      if constexpr (SPLIT)
        store_split_chunk(xh, xl, LDIh, e / NCI, e % NCI, xr[i], st * SP + e / NCI < count, lane);
      else if constexpr (kBufW)
        *reinterpret_cast<int4v *>(x + x_row(i) * LDI + (((lane % NCI) ^ (CI == 64 ? ((x_row(i) >> 1) & 1) * 4 : 0)) * E)) = xr[i];
      else
        *reinterpret_cast<int4v *>(x + (e / NCI) * LDI + (e % NCI) * E) =
            st * SP + e / NCI < count ? xr[i] : int4v{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int e = lane + 64 * i;
      if constexpr (SPLIT)
        store_split_chunk(gh, gl, LDOh, e / NCO, e % NCO, gr[i], st * SP + e / NCO < count, lane);
      else if constexpr (kBufW)
        *reinterpret_cast<int4v *>(g + g_row(i) * LDO + (((lane % NCO) ^ (CO == 64 ? ((g_row(i) >> 1) & 1) * 4 : 0)) * E)) = gr[i];
      else
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
  if constexpr (kBufW) hand_round();
  load_rows(st);
  load_idx(st + 4);
  while (st < nstages) {
    store_rows(st);                 // waits for the stage's rows
    if constexpr (kBufW) hand_round();   // (the indices of stage st + 4 came in behind them)
    else wave_fence();
    load_rows(st + 4);              // stage st + 4, in flight during the MFMAs
    __builtin_amdgcn_sched_barrier(0);   // (rows first, then indices, both before the MFMAs:
    load_idx(st + 8);                    //  the wait for the rows then leaves the indices in flight)
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (SPLIT) {
      bf16x8 ah[BI], al[BI], bh[BJ], bl[BJ];
#pragma unroll
      for (int ti = 0; ti < BI; ++ti) {
        ah[ti] = __builtin_bit_cast(bf16x8, tr_frag(xh, LDIh, 0, ti * 32, lane));
        al[ti] = __builtin_bit_cast(bf16x8, tr_frag(xl, LDIh, 0, ti * 32, lane));
      }
#pragma unroll
      for (int tj = 0; tj < BJ; ++tj) {
        bh[tj] = __builtin_bit_cast(bf16x8, tr_frag(gh, LDOh, 0, tj * 32, lane));
        bl[tj] = __builtin_bit_cast(bf16x8, tr_frag(gl, LDOh, 0, tj * 32, lane));
      }
#pragma unroll
      for (int ti = 0; ti < BI; ++ti)
#pragma unroll
        for (int tj = 0; tj < BJ; ++tj) {
          acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[ti], bh[tj], acc[ti][tj], 0, 0, 0);
          acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ti], bl[tj], acc[ti][tj], 0, 0, 0);
          acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ti], bh[tj], acc[ti][tj], 0, 0, 0);
        }
    } else if constexpr (kBufW) {
      constexpr int KS = SP / KP;
      half8 a[KS][BI], b[KS][BJ];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int ti = 0; ti < BI; ++ti) a[ks][ti] = tr_frag_dense<CI>(x, ks * KP, ti * 32, lane);
#pragma unroll
        for (int tj = 0; tj < BJ; ++tj) b[ks][tj] = tr_frag_dense<CO>(g, ks * KP, tj * 32, lane);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int ti = 0; ti < BI; ++ti)
#pragma unroll
          for (int tj = 0; tj < BJ; ++tj)
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks][ti], b[ks][tj], acc[ti][tj], 0, 0, 0);
    } else {
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
    }
    wave_fence();                   // the tile is rewritten at the top of the loop
    st += 4;
  }

  // Sum the four waves' tiles through LDS and flush.  Every wave ends up with a quarter of the
  // summed tile (accumulator registers q * R / 4 ... of the R = BI * BJ * 16 a lane holds) and
  // flushes that: one barrier, and the atomic updates of the tile issued by four waves instead
  // of one.  red: [quarter][contribution 0..2][register of the quarter][lane].
  float *red = reinterpret_cast<float *>(lds);
  constexpr int R = BI * BJ * 16, RQ = R / 4;
  __syncthreads();                  // every wave is done with its staging tiles
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (q == wave) continue;
    const int slot = wave < q ? wave : wave - 1;
#pragma unroll
    for (int j = 0; j < RQ; ++j) {
      const int idx = q * RQ + j, t = idx / 16;
      red[(size_t)((q * 3 + slot) * RQ + j) * 64 + lane] = acc[t / BJ][t % BJ][idx % 16];
    }
  }
  __syncthreads();
  const int h = lane >> 5, c = lane & 31;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (q != wave) continue;
#pragma unroll
    for (int j = 0; j < RQ; ++j) {
      const int idx = q * RQ + j, t = idx / 16, r = idx % 16, ti = t / BJ, tj = t % BJ;
      float v = acc[ti][tj][r];
#pragma unroll
      for (int slot = 0; slot < 3; ++slot) v += red[(size_t)((q * 3 + slot) * RQ + j) * 64 + lane];
      // accumulator register r of lane l is row (r/4)*8 + (l/32)*4 + r%4, column l%32 of its 32 x 32 tile
      atomic_add(gw32 + ((size_t)k * c_in + ci0 + ti * 32 + (r / 4) * 8 + h * 4 + (r % 4)) * c_out + co0 + tj * 32 + c, v);
    }
  }
}


template <int BI, int BJ> struct WaveGrid {
  static constexpr int WI = BI >= 2 ? (BJ == 1 && BI == 4 ? 4 : 2) : 1;
  static constexpr int WJ = BJ >= 2 ? (BI == 1 && BJ == 4 ? 4 : (WI == 4 ? 1 : 2)) : 1;
  static constexpr int WK = 4 / (WI * WJ);
  static constexpr int TI = BI / WI;
  static constexpr int TJ = BJ / WJ;
  static_assert(WI * WJ * WK == 4 && TI * WI == BI && TJ * WJ == BJ, "wave grid");
};

// The workgroup-level weight-gradient kernel body (dW tiles wider than 64 x 64): the four
// waves share the staged pairs and split the tile.  (block_x, block_y): the workgroup's
// place in a grid of cells x tiles of dW[k]; 256 threads.
// SPLIT: as in wgrad_wave_body (fp32 rows staged as hi / lo bf16 tiles, three bf16 MFMAs a product).
template <typename T, int BI, int BJ, bool SPLIT = false>
__device__ __forceinline__ void wgrad_wg_body(
    const T *__restrict__ in, const T *__restrict__ gout, float *__restrict__ gw32,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
    const int32_t *__restrict__ omap, int k_vol, int c_in, int c_out, const SliceMap &smap,
    int block_x, int block_y) {
  constexpr int kThreads = 256;
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
  // SPLIT: a buffer holds four 16-bit tiles, x hi, x lo, g hi, g lo, rows padded as in the fp16 path
  constexpr int LDIh = CI + 16, LDOh = CO + 16;
  constexpr int kBufHalfs = SP * 2 * (LDIh + LDOh);
  __half *const stage0h = reinterpret_cast<__half *>(lds);
  static_assert(!SPLIT || (sizeof(T) == 4 && G::WK == 1 && SP % 16 == 0), "split tiles: fp32 rows, whole 16-pair steps");

  int k, first, count;
  if (!locate_slice(kpos, smap, k_vol, block_x, k, first, count)) return;
  const int tiles_co = c_out / CO;
  const int ci0 = (block_y / tiles_co) * CI;
  const int co0 = (block_y % tiles_co) * CO;
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
      if constexpr (SPLIT) {
        __half *xh = stage0h + buf * kBufHalfs;
        store_split_chunk(xh, xh + SP * LDIh, LDIh, e / NCI, e % NCI, xr[i], st * SP + e / NCI < count, lane);
      } else {
        *reinterpret_cast<int4v *>(stage0 + buf * kBufElems + (e / NCI) * LDI + (e % NCI) * E) =
            st * SP + e / NCI < count ? xr[i] : int4v{0, 0, 0, 0};
      }
    }
#pragma unroll
    for (int i = 0; i < NG; ++i) {
      const int e = tid + kThreads * i;
      if constexpr (SPLIT) {
        __half *gh = stage0h + buf * kBufHalfs + SP * 2 * LDIh;
        store_split_chunk(gh, gh + SP * LDOh, LDOh, e / NCO, e % NCO, gr[i], st * SP + e / NCO < count, lane);
      } else {
        *reinterpret_cast<int4v *>(stage0 + buf * kBufElems + SP * LDI + (e / NCO) * LDO + (e % NCO) * E) =
            st * SP + e / NCO < count ? gr[i] : int4v{0, 0, 0, 0};
      }
    }
  };
  auto multiply = [&](int cur) {
    if constexpr (SPLIT) {
      const __half *xh = stage0h + cur * kBufHalfs, *xl = xh + SP * LDIh;
      const __half *gh = xl + SP * LDIh, *gl = gh + SP * LDOh;
#pragma unroll
      for (int p0 = 0; p0 < SP; p0 += 16) {
        bf16x8 ah[G::TI], al[G::TI], bh[G::TJ], bl[G::TJ];
#pragma unroll
        for (int ti = 0; ti < G::TI; ++ti) {
          ah[ti] = __builtin_bit_cast(bf16x8, tr_frag(xh, LDIh, p0, (wi * G::TI + ti) * 32, lane));
          al[ti] = __builtin_bit_cast(bf16x8, tr_frag(xl, LDIh, p0, (wi * G::TI + ti) * 32, lane));
        }
#pragma unroll
        for (int tj = 0; tj < G::TJ; ++tj) {
          bh[tj] = __builtin_bit_cast(bf16x8, tr_frag(gh, LDOh, p0, (wj * G::TJ + tj) * 32, lane));
          bl[tj] = __builtin_bit_cast(bf16x8, tr_frag(gl, LDOh, p0, (wj * G::TJ + tj) * 32, lane));
        }
#pragma unroll
        for (int ti = 0; ti < G::TI; ++ti)
#pragma unroll
          for (int tj = 0; tj < G::TJ; ++tj) {
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[ti], bh[tj], acc[ti][tj], 0, 0, 0);
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ti], bl[tj], acc[ti][tj], 0, 0, 0);
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[ti], bh[tj], acc[ti][tj], 0, 0, 0);
          }
      }
      return;
    }
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


// ---- host side (fgms_wgrad.hip) ----
// Which of the two MFMA bodies serves a layer and the grid it wants.
struct WgradGeometry {
  SliceMap smap;
  int64_t tiles;   // grid x: cells (or plain tiles of the pair list)
  int ty;          // grid y: BI*32 x BJ*32 tiles of dW[k]
  int bi, bj;
  bool wave;       // wgrad_wave_body, else wgrad_wg_body
  bool split;      // wgrad_wave_body in split bf16
  size_t lds;      // dynamic LDS
};
// shares_grid: the launch also holds the input gradient's workgroups.
int wgrad_geometry(const WgradArgs &a, WgradGeometry *g, bool shares_grid = false);
// Where the kernels accumulate: the caller's fp32 tensor, or for fp16 the stream's fp32
// scratch (zero between calls), which wgrad_finish rounds into the caller's tensor and
// clears again in a launch of its own.
int wgrad_accumulator(const WgradArgs &a, float **acc32);
int wgrad_finish(const WgradArgs &a, float *acc32);

}  // namespace fgms
