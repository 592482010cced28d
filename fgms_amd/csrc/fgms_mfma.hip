// MFMA gather-GEMM-scatter kernels for gfx950 (forward and input gradient).
//
// Two dataflows share one fragment scheme:
//
//  * pair-stationary ("pairs"): a workgroup walks a run of 256-pair tiles of the
//    flat pair list, keeps op(W[k]) in LDS while the offset k does not change,
//    gathers the source rows through LDS and scatters the products with
//    atomics.  Works for any map.  This is the dataflow of the reference's fused
//    kernels (backend/spconv.cuh:1328-1477, backend/fwd_kernels.cuh:17-144,
//    backend/bwd_kernels.cuh:13-142, 281-408) re-tiled for 64-wide waves.
//  * output-stationary ("rows"): a workgroup owns 256 destination rows, walks the
//    offsets k through the plan's neighbour table, sums everything in MFMA
//    accumulators and writes each destination row once: no atomics, run-to-run
//    identical results.  Needs a plan whose map is functional.
//
// Fragment scheme.  A source row is cut into slabs of 2*S 16-byte chunks
// (S = 4, 2 or 1; a chunk is 8 halfs or 4 floats).  Lanes 0-31 of a wave carry
// the first S chunks of the slab, lanes 32-63 the last S, so one MFMA
// (v_mfma_f32_32x32x16_f16, or four v_mfma_f32_32x32x2_f32) contracts chunk s of
// both halves.  The order of the contraction index is free as long as both
// operands agree, and it lets every lane read one contiguous 16-byte piece.
// Weights are re-laid on the device into exactly that per-lane order before the
// main kernel runs (pack_weights_kernel), transposed for the input gradient.
//
// Gathered rows reach LDS with 16-byte loads, 2*S lanes per row (full 128-byte
// lines for S = 4), in an XOR-swizzled layout so that the b128 reads of the MFMA
// operand do not collide on banks.
#include <stdlib.h>

#include <type_traits>

#include "fgms_device.h"
#include "fgms_internal.h"
#include "fgms_mma.h"
#include "fgms_tile_ops.h"
#include "fgms_wgrad_bodies.h"

namespace fgms {
namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kWaveRows = 64;                 // two 32-row MFMA tiles per wave
constexpr int kTileRows = kWaves * kWaveRows; // 256 rows per workgroup tile

// ---------------------------------------------------------------------------
// Weight re-layout (see pack_weight_elements) in a launch of its own.
template <typename T>
__global__ void pack_weights_kernel(const T *__restrict__ w, T *__restrict__ packed, int k_vol,
                                    int c_in, int c_out, int S, bool transpose) {
  pack_weight_elements<T>(w, packed, k_vol, c_in, c_out, S, transpose,
                          (size_t)blockIdx.x * blockDim.x + threadIdx.x,
                          (size_t)gridDim.x * blockDim.x);
}

__global__ void side_job_kernel(SideJob job) { run_side_job(job, blockIdx.x); }

// Copies the packed weights of offset k, destination tiles [nt0, nt0 + NT), to LDS.
template <int NT>
__device__ __forceinline__ void load_weights(int4v *__restrict__ w_lds,
                                             const int4v *__restrict__ packed_k, int qs, int nts,
                                             int nt0) {
  const int n = qs * NT * 64;
  for (int i = threadIdx.x; i < n; i += kThreads) {
    const int q = i / (NT * 64), rem = i % (NT * 64);
    w_lds[i] = packed_k[((size_t)q * nts + nt0) * 64 + rem];
  }
}

// The same for split weights (pack_weights_bf3_kernel): per (slab, k-step) NT * 128 chunks.
template <int NT>
__device__ __forceinline__ void load_weights_bf3(int4v *__restrict__ w_lds,
                                                 const int4v *__restrict__ packed_k, int slabs, int nts,
                                                 int nt0) {
  const int n = slabs * 2 * NT * 128;
  for (int i = threadIdx.x; i < n; i += kThreads) {
    const int q = i / (NT * 128), rem = i % (NT * 128);
    w_lds[i] = packed_k[((size_t)q * nts + nt0) * 128 + rem];
  }
}

// acc[mt][nt] += A(slab) x W(slab).
template <typename T, int NT, int S, int MT>
__device__ __forceinline__ void mma_slab(float16v (&acc)[MT][NT], const int4v *__restrict__ a_lds,
                                         const int4v *__restrict__ w_lds, int slab, int lane) {
  const int h = lane / 32, r = lane % 32;
  if constexpr (sizeof(T) == 2 && NT <= 2) {
    // (pipelined like mma_slab_raw below: the next k-step's fragments are requested first)
    int4v a[2][MT], b[2][NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) b[0][nt] = w_lds[((slab * S) * NT + nt) * 64 + lane];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) a[0][mt] = a_lds[a_slot<S>(mt * 32 + r, h * S)];
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if (s + 1 < S) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) b[(s + 1) & 1][nt] = w_lds[((slab * S + s + 1) * NT + nt) * 64 + lane];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a[(s + 1) & 1][mt] = a_lds[a_slot<S>(mt * 32 + r, h * S + s + 1)];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) mma<T>(acc[mt][nt], a[s & 1][mt], b[s & 1][nt]);
      __builtin_amdgcn_sched_barrier(0);
    }
    return;
  }
#pragma unroll
  for (int s = 0; s < S; ++s) {
    int4v b[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) b[nt] = w_lds[((slab * S + s) * NT + nt) * 64 + lane];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int4v a = a_lds[a_slot<S>(mt * 32 + r, h * S + s)];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) mma<T>(acc[mt][nt], a, b[nt]);
    }
  }
}

// The MFMA phase of a stage, software-pipelined by hand: the fragments of k-step s + 1 are
// requested from LDS before the MFMAs of k-step s are issued (two sets of fragment registers),
// so that a wave's matrix instructions follow each other instead of each pair waiting out an
// LDS round trip.  The scheduling barriers keep the compiler from sinking the reads back to
// their uses (left alone it emits read, wait, two MFMAs, read, wait, ... in source order).
// acc[mt][nt] += A(slab) x W(slab), weights as raw_weight_frag reads them.
template <typename T, int NT, int S, int MT>
__device__ __forceinline__ void mma_slab_raw(float16v (&acc)[MT][NT], const int4v *__restrict__ a_lds,
                                             const int4v *__restrict__ w_lds, int lane) {
  const int h = lane / 32, r = lane % 32;
  int4v a[2][MT], b[2][NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) b[0][nt] = raw_weight_frag<NT, S>(w_lds, 0, nt, lane);
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) a[0][mt] = a_lds[a_slot<S>(mt * 32 + r, h * S)];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    if (s + 1 < S) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) b[(s + 1) & 1][nt] = raw_weight_frag<NT, S>(w_lds, s + 1, nt, lane);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) a[(s + 1) & 1][mt] = a_lds[a_slot<S>(mt * 32 + r, h * S + s + 1)];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) mma<T>(acc[mt][nt], a[s & 1][mt], b[s & 1][nt]);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// --- input-gradient weights straight from the caller's tensor --------------------------
// The input gradient contracts over the COLUMNS of W[k] (dIn[ci] = sum over co of
// dOut[co] * W[k][ci][co]), and those are contiguous in memory: the 8 halfs (4 floats) an
// MFMA lane wants are one 16-byte piece of row ci.  A stage's weight tile (NT*32 rows ci x
// 2*S chunks of the co slab) goes to LDS as it lies in memory, swizzled like a wave's
// staging tile of gathered rows, and a fragment is one 16-byte read.  No re-layout at all.
template <typename T, int NT, int S, int MT>
__device__ __forceinline__ void mma_slab_rawt(float16v (&acc)[MT][NT], const int4v *__restrict__ a_lds,
                                              const int4v *__restrict__ w_lds, int lane) {
  const int h = lane / 32, r = lane % 32;
  if constexpr (sizeof(T) == 4) {
    // (fp32: a k-step is sixteen MFMAs of 64 cycles, long enough to cover the next reads)
#pragma unroll
    for (int s = 0; s < S; ++s) {
      int4v b[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) b[nt] = w_lds[a_slot<S>(nt * 32 + r, h * S + s)];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int4v a = a_lds[a_slot<S>(mt * 32 + r, h * S + s)];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) mma<T>(acc[mt][nt], a, b[nt]);
      }
    }
    return;
  }
  int4v a[2][MT], b[2][NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) b[0][nt] = w_lds[a_slot<S>(nt * 32 + r, h * S)];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) a[0][mt] = a_lds[a_slot<S>(mt * 32 + r, h * S)];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    if (s + 1 < S) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) b[(s + 1) & 1][nt] = w_lds[a_slot<S>(nt * 32 + r, h * S + s + 1)];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) a[(s + 1) & 1][mt] = a_lds[a_slot<S>(mt * 32 + r, h * S + s + 1)];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) mma<T>(acc[mt][nt], a[s & 1][mt], b[s & 1][nt]);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// --- fp32 tensors, products in split bf16 ("tf32" mode) ------------------------------------
// gfx950 has no tf32 matrix instruction, and its fp32 one runs at a sixteenth of the 16-bit
// rate.  Where the caller allows tf32 precision for the products (10 mantissa bits), every
// fp32 value is split into two bf16 numbers, x = hi + lo + O(2^-17 x), and a product becomes
// three bf16 MFMAs into the fp32 accumulator: hi*hi + hi*lo + lo*hi.  The dropped lo*lo term
// is below 2^-16 of the product, so this is more exact than tf32, at 3/16 of the fp32 matrix
// time.  Rows are split when they go from registers to LDS, the weights by their re-layout
// kernel.
// Slot (16 bytes = 8 bf16) of a wave's split staging tile: row-major, a row holds its 32
// values of the slab as 4 chunks of hi followed by 4 chunks of lo (128 bytes, as the fp32
// row did); the XOR spreads the 8 rows one b128 read pass touches over all banks.
__device__ __forceinline__ int a_bf_slot(int row, int part, int j) {
  return row * 8 + part * 4 + (j ^ ((row >> 1) & 3));
}

// One fp32 chunk (4 values; chunk c of its row's slab) split and written to a split tile.
// Lane pairs hold the two fp32 chunks that make one bf16 chunk; they exchange halves, so the
// even lane ends up with the 8 hi values and the odd one with the 8 lo values and each
// still writes one 16-byte chunk.
__device__ __forceinline__ void split_and_store(int4v *__restrict__ tile, const float4v &x, int row, int c,
                                                int lane) {
  const bool odd = lane & 1;
  bf16x4 hi, lo;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    __bf16 h, l;
    split_bf16(x[i], h, l);
    hi[i] = h;
    lo[i] = l;
  }
  const int2v h2 = __builtin_bit_cast(int2v, hi), l2 = __builtin_bit_cast(int2v, lo);
  // the even lane hands over its lo half and takes the odd lane's hi half
  const int got0 = __builtin_bit_cast(int, swap_with_neighbour(__builtin_bit_cast(float, odd ? h2[0] : l2[0])));
  const int got1 = __builtin_bit_cast(int, swap_with_neighbour(__builtin_bit_cast(float, odd ? h2[1] : l2[1])));
  tile[a_bf_slot(row, odd ? 1 : 0, c / 2)] = odd ? int4v{got0, got1, l2[0], l2[1]} : int4v{h2[0], h2[1], got0, got1};
}

// registers -> LDS for the split tile of gathered rows (absent rows as zeros).
template <int N>
__device__ __forceinline__ void gather_commit_bf3(int4v *__restrict__ a_lds, int4v (&v)[N],
                                                  const int (&g)[N], int lane) {
#pragma unroll
  for (int it = 0; it < N; ++it) {
    const int slot = it * 64 + lane;
    const float4v x = g[it] < 0 ? float4v{0.f, 0.f, 0.f, 0.f} : __builtin_bit_cast(float4v, v[it]);
    split_and_store(a_lds, x, slot / 8, slot % 8, lane);
  }
}

// acc[mt][nt] += A(slab) x W(slab), both split; weights in LDS as [k-step][nt][hi, lo][lane].
template <int NT, int MT>
__device__ __forceinline__ void mma_slab_bf3(float16v (&acc)[MT][NT], const int4v *__restrict__ a_lds,
                                             const int4v *__restrict__ w_lds, int lane) {
  const int h = lane / 32, r = lane % 32;
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    bf16x8 bh[NT], bl[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      bh[nt] = __builtin_bit_cast(bf16x8, w_lds[((s * NT + nt) * 2 + 0) * 64 + lane]);
      bl[nt] = __builtin_bit_cast(bf16x8, w_lds[((s * NT + nt) * 2 + 1) * 64 + lane]);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8 ah = __builtin_bit_cast(bf16x8, a_lds[a_bf_slot(mt * 32 + r, 0, s * 2 + h)]);
      const bf16x8 al = __builtin_bit_cast(bf16x8, a_lds[a_bf_slot(mt * 32 + r, 1, s * 2 + h)]);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh[nt], acc[mt][nt], 0, 0, 0);
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl[nt], acc[mt][nt], 0, 0, 0);
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh[nt], acc[mt][nt], 0, 0, 0);
      }
    }
  }
}

// The same for the input gradient: the weight tile (NT*32 rows of W[k], the slab's 32 columns)
// was split on its way to LDS like a tile of gathered rows (RAW = 4).
template <int NT, int MT>
__device__ __forceinline__ void mma_slab_bf3t(float16v (&acc)[MT][NT], const int4v *__restrict__ a_lds,
                                              const int4v *__restrict__ w_lds, int lane) {
  const int h = lane / 32, r = lane % 32;
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    bf16x8 bh[NT], bl[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      bh[nt] = __builtin_bit_cast(bf16x8, w_lds[a_bf_slot(nt * 32 + r, 0, s * 2 + h)]);
      bl[nt] = __builtin_bit_cast(bf16x8, w_lds[a_bf_slot(nt * 32 + r, 1, s * 2 + h)]);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bf16x8 ah = __builtin_bit_cast(bf16x8, a_lds[a_bf_slot(mt * 32 + r, 0, s * 2 + h)]);
      const bf16x8 al = __builtin_bit_cast(bf16x8, a_lds[a_bf_slot(mt * 32 + r, 1, s * 2 + h)]);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh[nt], acc[mt][nt], 0, 0, 0);
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl[nt], acc[mt][nt], 0, 0, 0);
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh[nt], acc[mt][nt], 0, 0, 0);
      }
    }
  }
}

// Split weights in the order mma_slab_bf3 reads them: chunk
//   ((((k * slabs + slab) * 2 + s) * nts + nt) * 2 + part) * 64 + lane
// holds the 8 values op(W[k])[slab*32 + s*16 + (lane/32)*8 + 0..7][nt*32 + lane%32], hi (part 0)
// or lo (part 1).  One thread per chunk pair.
__global__ void pack_weights_bf3_kernel(const float *__restrict__ w, int4v *__restrict__ packed,
                                        int k_vol, int c_in, int c_out, bool transpose) {
  // (transpose: the input gradient's view, W[k]^T -- source channels are the columns of W[k])
  const int slabs = (transpose ? c_out : c_in) / 32, nts = (transpose ? c_in : c_out) / 32;
  const size_t total = (size_t)k_vol * slabs * 2 * nts * 64;
  for (size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x; t < total;
       t += (size_t)gridDim.x * blockDim.x) {
    const int lane = (int)(t % 64);
    size_t q = t / 64;
    const int nt = (int)(q % nts); q /= nts;
    const int s = (int)(q % 2); q /= 2;
    const int slab = (int)(q % slabs);
    const int k = (int)(q / slabs);
    const int cs0 = slab * 32 + s * 16 + (lane / 32) * 8, cd = nt * 32 + lane % 32;
    bf16x8 hi, lo;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      __bf16 h, l;
      split_bf16(transpose ? w[((size_t)k * c_in + cd) * c_out + cs0 + e] : w[((size_t)k * c_in + cs0 + e) * c_out + cd], h, l);
      hi[e] = h;
      lo[e] = l;
    }
    const size_t base = (t / 64) * 128 + lane;
    packed[base] = __builtin_bit_cast(int4v, hi);
    packed[base + 64] = __builtin_bit_cast(int4v, lo);
  }
}

// ---------------------------------------------------------------------------
// Row gathers in two steps, so that the loads of one slab run under the MFMAs of the
// previous one: issue (global -> registers, absent rows read row 0) and commit
// (registers -> the wave's LDS tile, absent rows as zeros; waits for the loads).
// (N chunks per lane: 2 * S for a wave tile of 64 rows, S for one of 32)
template <typename T, int S, int N>
__device__ __forceinline__ void gather_issue(int4v (&v)[N], int (&g)[N],
                                             const int *__restrict__ idx,
                                             const T *__restrict__ src, int c_src, int slab,
                                             int lane) {
  constexpr int E = Elem<T>::per_chunk;
  constexpr int C = 2 * S;
#pragma unroll
  for (int it = 0; it < N; ++it) g[it] = idx[(it * 64 + lane) / C];
#pragma unroll
  for (int it = 0; it < N; ++it) {
    const int c = (it * 64 + lane) % C;
    v[it] = *reinterpret_cast<const int4v *>(src + (size_t)max(g[it], 0) * c_src +
                                             (size_t)(slab * C + c) * E);
  }
}

template <int S, int N>
__device__ __forceinline__ void gather_commit(int4v *__restrict__ a_lds, int4v (&v)[N],
                                              const int (&g)[N], int lane) {
  constexpr int C = 2 * S;
#pragma unroll
  for (int it = 0; it < N; ++it) {
    const int slot = it * 64 + lane;
    a_lds[a_slot<S>(slot / C, slot % C)] = g[it] < 0 ? int4v{0, 0, 0, 0} : v[it];
  }
}

// The same two steps for the output-stationary kernel, through buffer loads (see kAbsentRow):
// `offs` holds a byte offset per row of the wave's tile, kAbsentRow for a row that has no
// neighbour through this offset, which then arrives as zeros by itself: no select on the way
// to LDS, no row index kept per load, 32-bit address arithmetic.
template <int S, int N>
__device__ __forceinline__ void gather_issue_buf(int4v (&v)[N], const unsigned *__restrict__ offs,
                                                 __amdgpu_buffer_rsrc_t rsrc, int slab, int lane) {
  constexpr int C = 2 * S;
  unsigned off[N];
#pragma unroll
  for (int it = 0; it < N; ++it) off[it] = offs[(it * 64 + lane) / C] + (unsigned)((lane % C) * 16);
#pragma unroll
  for (int it = 0; it < N; ++it)
    v[it] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off[it], slab * (C * 16), 0));
}

template <int S, int N>
__device__ __forceinline__ void gather_commit_buf(int4v *__restrict__ a_lds, const int4v (&v)[N], int lane) {
  constexpr int C = 2 * S;
  if constexpr (C == 8) {
    // a_slot(it * 8 + lane / 8, lane % 8) spelled out: the swizzle term (row >> 1) & 7 is
    // lane / 16 for even `it` and lane / 16 + 4 for odd ones, so two per-lane bases and
    // immediate offsets address all N writes
    const int base = (lane / 8) * 8, c = lane % 8, x = lane / 16;
    const int even = base + (c ^ x), odd = base + (c ^ (x + 4));
#pragma unroll
    for (int it = 0; it < N; ++it) a_lds[((it & 1) ? odd : even) + it * 64] = v[it];
  } else {
#pragma unroll
    for (int it = 0; it < N; ++it) {
      const int slot = it * 64 + lane;
      a_lds[a_slot<S>(slot / C, slot % C)] = v[it];
    }
  }
}

template <int N>
__device__ __forceinline__ void gather_commit_bf3_buf(int4v *__restrict__ a_lds, const int4v (&v)[N], int lane) {
#pragma unroll
  for (int it = 0; it < N; ++it) {
    const int slot = it * 64 + lane;
    split_and_store(a_lds, __builtin_bit_cast(float4v, v[it]), slot / 8, slot % 8, lane);
  }
}

// ---------------------------------------------------------------------------
// Pair-stationary kernel.
// SPLIT: fp32 tensors whose caller allows tf32 precision, products in split bf16 (see
// mma_slab_bf3); `packed` from pack_weights_bf3_kernel.
template <typename T, int NT, int S, bool SPLIT>
__global__ __launch_bounds__(kThreads) void gms_pairs_kernel(
    const T *__restrict__ src, const T *__restrict__ packed, T *__restrict__ dst,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ gmap,
    const int32_t *__restrict__ smap, int k_vol, int c_src, int c_dst, int tiles_per_wg,
    int dense_k, int dense_rows) {
  constexpr int E = Elem<T>::per_chunk;
  extern __shared__ int4v lds[];
  const int slabs = c_src / (2 * S * E);
  const int qs = slabs * S;
  const int nts = c_dst / 32;
  int4v *w_lds = lds;                                   // qs * NT * 64 chunks
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  int4v *a_lds = lds + qs * NT * 64 + wave * (kWaveRows * 2 * S);
  int *idx_all = reinterpret_cast<int *>(lds + qs * NT * 64 + kWaves * (kWaveRows * 2 * S));
  int *gidx = idx_all + wave * 2 * kWaveRows;
  int *sidx = gidx + kWaveRows;
  const int nt0 = blockIdx.y * NT;
  const size_t packed_per_k = (size_t)c_src * c_dst / E;  // chunks

  int cur_k = -1;
  const int t_begin = blockIdx.x * tiles_per_wg;
  for (int t = t_begin; t < t_begin + tiles_per_wg; ++t) {
    int k, first, count;
    if (dense_k >= 0) {
      k = dense_k;
      first = t * kTileRows;
      if (first >= dense_rows) break;
      count = min(kTileRows, dense_rows - first);
    } else if (!locate_tile(kpos, k_vol, kTileRows, t, k, first, count)) {
      break;
    }
    if (k != cur_k) {  // uniform over the workgroup
      __syncthreads();
      if constexpr (SPLIT)
        load_weights_bf3<NT>(w_lds, reinterpret_cast<const int4v *>(packed) + packed_per_k * k, slabs, nts, nt0);
      else
        load_weights<NT>(w_lds, reinterpret_cast<const int4v *>(packed) + packed_per_k * k, qs, nts, nt0);
      __syncthreads();
      cur_k = k;
    }
    const int wfirst = wave * kWaveRows;
    const int nrows = min(kWaveRows, count - wfirst);
    if (nrows <= 0) continue;
    const bool live = lane < nrows;
    const int j = first + wfirst + lane;
    gidx[lane] = !live ? -1 : (gmap ? gmap[j] : j);
    sidx[lane] = !live ? -1 : (smap ? smap[j] : j);
    wave_lds_fence();

    float16v acc[2][NT];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.f;

    int4v v[2 * S];
    int gsel[2 * S];
    gather_issue<T, S>(v, gsel, gidx, src, c_src, 0, lane);
    for (int slab = 0; slab < slabs; ++slab) {
      if constexpr (SPLIT) gather_commit_bf3(a_lds, v, gsel, lane);
      else gather_commit<S>(a_lds, v, gsel, lane);
      wave_lds_fence();
      if (slab + 1 < slabs) gather_issue<T, S>(v, gsel, gidx, src, c_src, slab + 1, lane);   // under the MFMAs
      if constexpr (SPLIT) mma_slab_bf3<NT>(acc, a_lds, w_lds + slab * (2 * NT * 128), lane);
      else mma_slab<T, NT, S>(acc, a_lds, w_lds, slab, lane);
      wave_lds_fence();
    }
    write_tile<T, NT, true>(acc, dst, sidx, c_dst, nt0 * 32, lane);
    wave_lds_fence();
  }
}

// ---------------------------------------------------------------------------
// Output-stationary kernel.  nbr is the plan's table laid out [k_vol][n_dst]:
// nbr[k][d] = source row that reaches destination row d through offset k, or -1.
//
// The work of a workgroup is a list of stages (offset k, slab of the source
// row).  Stages are software-pipelined: while the MFMAs of stage t run, the
// weights and the gathered rows of stage t + 1 are already in flight in
// registers (the row index of the offset after that is in flight too); they are
// written to LDS after the MFMAs and one barrier closes the stage.  Weights are
// double-buffered in LDS, each wave's row tile is single-buffered (only its own
// wave reads it).
// RAW = 1: `packed` is the caller's weight tensor itself, forward (fp16: see raw_weight_frag);
// RAW = 2: the same for the input gradient (see mma_slab_rawt); RAW = 3: fp32 tensors with
// products in split bf16 (see mma_slab_bf3), `packed` from pack_weights_bf3_kernel; RAW = 4:
// the input gradient in split bf16, weights read as they lie and split on their way to LDS;
// RAW = 0: the re-laid copy pack_weight_elements makes.
// (block_x, block_y, block_z) of a grid (tiles, column tiles, grid_z parts of a tile).
// MT: 32-row MFMA tiles per wave.  2 (a workgroup tile of 256 rows) is the layout every plan
// table is made for; 1 (tiles of 128 rows, half the work per wave and stage) serves launches
// too small to fill the chip, where a tile's chain of stages is all there is to the duration.
template <typename T, int NT, int S, int RAW, int MT = 2>
__device__ __forceinline__ void gms_rows_body(
    const T *__restrict__ src, const T *__restrict__ packed, T *__restrict__ dst,
    const int32_t *__restrict__ nbr, const unsigned long long *__restrict__ block_masks,
    const int32_t *__restrict__ perm, const int32_t *__restrict__ tile_order, int n_dst, int k_vol,
    int c_src, int c_dst, int part_stages, int block_x, int block_y, int block_z, int grid_z,
    unsigned src_bytes, int pair_view = 0) {
  constexpr int E = Elem<T>::per_chunk;
  constexpr int C = 2 * S;
  // 16-bit matrix instructions (fp16 tensors, fp32 tensors in split bf16): rows and weights come
  // through buffer loads and the MFMA phase is pipelined by hand; plain fp32, whose MFMA phase is
  // eight times as long, keeps pointer loads and interleaves them with its MFMAs instead
  constexpr bool kBuf = sizeof(T) == 2 || RAW == 3 || RAW == 4;
  const __amdgpu_buffer_rsrc_t rsrc = rows_resource(src, src_bytes);
  const unsigned row_bytes = (unsigned)c_src * (unsigned)sizeof(T);
  // byte offset of source row g in the buffer (kAbsentRow: no neighbour, the loads return zeros)
  auto row_offset = [&](int g) { return !kBuf ? (unsigned)g : g < 0 ? kAbsentRow : (unsigned)g * row_bytes; };
  // pair view: `nbr` is one list of source rows for all offsets (a 64-row block belongs to
  // the one offset its mask names), `perm` the destination rows; results are added atomically
  const size_t nbr_stride = pair_view ? 0 : (size_t)n_dst;
  constexpr int WCH = S * NT * 64;                        // 16-byte chunks of one stage's weights
  constexpr int NW = (WCH + kThreads - 1) / kThreads;     // ... per thread
  extern __shared__ int4v lds[];
  __shared__ unsigned long long wg_mask;
  // fp32 only: its MFMA phase is long enough (4 k clocks a stage) to absorb the loads'
  // issue waits; for fp16 the interleaved stage measured 2 us slower per launch
  constexpr bool kInterleave = sizeof(T) == 4 && RAW != 3 && RAW != 4;
  const int slabs = c_src / (C * E);
  const int nts = c_dst / 32;
  int4v *w_lds = lds;                                     // [2][WCH]
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  constexpr int WR = MT * 32;                             // rows per wave
  constexpr int TR = kWaves * WR;                         // rows per workgroup tile
  int4v *a_lds = lds + 2 * WCH + wave * (WR * C);
  int *idx_all = reinterpret_cast<int *>(lds + 2 * WCH + kWaves * (WR * C));
  // per wave: the rows to gather -- byte offsets, two sets (this offset's and the next one's), or
  // plain indices (!kBuf, one set) -- and the destination rows
  unsigned *goff = reinterpret_cast<unsigned *>(idx_all + wave * 3 * WR);
  const int *gidx = idx_all + wave * 3 * WR;
  int *didx = idx_all + wave * 3 * WR + 2 * WR;
  const int nt0 = block_y * NT;
  const int4v *packed4 = reinterpret_cast<const int4v *>(packed);
  const size_t packed_per_k = (size_t)c_src * c_dst / E;  // chunks

  // the plan's table gives the tile and the first offset it uses
  int tile = block_x, k_first = -1;
  if (tile_order) {
    const int entry = tile_order[block_x];
    if (entry < 0) return;
    tile = entry & 0xFFFFFF;
    if (grid_z == 1) k_first = entry >> 24;
  }
  const int row0 = tile * TR + wave * WR;
  const int my_row = row0 + lane;
  const bool owns_row = MT == 2 || lane < WR;             // (lanes past a 32-row wave tile own no row)
  const bool in_range = owns_row && my_row < n_dst;
  // that offset's neighbour index, fetched while the masks are still on their way: at the
  // start of a launch every workgroup walks this chain of dependent loads at the same time
  // and nothing else covers it (0.4 us of a 46 us launch)
  int g_first = -1;
  if (k_first >= 0 && in_range) g_first = nbr[(size_t)k_first * nbr_stride + my_row];
  if (owns_row) didx[lane] = in_range ? (perm ? perm[my_row] : my_row) : -1;   // my_row is a position in the plan's row order

  // which offsets touch this wave's rows / this workgroup's rows (from the plan)
  unsigned long long wave_mask = row0 < n_dst ? block_masks[row0 / 64] : 0ull;
  // (one value for the whole wave: in scalar registers where vector registers are short)
  if constexpr (sizeof(T) == 2 || RAW == 3 || RAW == 4)
    wave_mask = (unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(wave_mask & 0xffffffffu)) |
              ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(wave_mask >> 32)) << 32);
  if (threadIdx.x == 0) wg_mask = 0;
  __syncthreads();
  if (lane == 0 && wave_mask) atomicOr(&wg_mask, wave_mask);
  __syncthreads();
  unsigned long long todo = wg_mask;
  if (!todo) return;
  // The launch lasts as long as its longest tile, and the tiles with the longest
  // offset lists are few: they get the instruction issue priority, so that they run
  // at their own pace while the many short tiles share what is left.
  {
    const int n_off = __builtin_popcountll(todo);
    if (n_off * 4 > k_vol * 3) __builtin_amdgcn_s_setprio(3);
    else if (n_off * 2 > k_vol) __builtin_amdgcn_s_setprio(1);
  }
  // grid_z > 1: a tile is shared by up to grid_z workgroups, each takes a run
  // of the tile's offsets and adds its partial result with atomics.
  bool shared_tile = pair_view != 0;
  if (grid_z > 1) {
    const int n_off = __builtin_popcountll(todo);
    const int want = (n_off * slabs + part_stages - 1) / part_stages;
    const int parts = min(grid_z, max(want, 1));
    if (block_z >= parts) return;
    if (parts > 1) {
      shared_tile = true;
      const int per = (n_off + parts - 1) / parts;
      for (int i = 0; i < block_z * per; ++i) todo &= todo - 1;      // offsets of earlier parts
      unsigned long long mine = 0, rest = todo;
      for (int i = 0; i < per && rest; ++i) {
        mine |= rest & (0 - rest);
        rest &= rest - 1;
      }
      todo = mine;
      if (!todo) return;
    }
  }

  float16v acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.f;

  // Weights of stage (k, slab), 16-byte chunk e = threadIdx.x + kThreads * i of the stage's tile,
  // through a buffer resource over the weight tensor: the part of a chunk's address that depends
  // on the thread is a per-lane constant (wvoff), the part that depends on the stage is scalar.
  //   RAW = 1: row e / (NT*4) of the slab's 2*S*8 rows of W[k], 16-byte piece e % (NT*4) of the
  //            NT*32 columns from nt0*32 on
  //   RAW = 2, 4: row e / C of the NT*32 rows of W[k] from nt0*32 on (c_dst rows of c_src
  //            elements here), 16-byte piece e % C of the slab
  //   RAW = 3: k-step e / (NT*128) of the stage, then [nt][hi, lo][lane]
  //   RAW = 0: chunks [(slab*S + s) * nts + nt0 + nt] * 64 + lane of the re-laid copy
  const __amdgpu_buffer_rsrc_t wrsrc =
      rows_resource(packed, (unsigned)k_vol * (unsigned)c_src * (unsigned)c_dst * (unsigned)sizeof(T));
  unsigned wvoff[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int e = threadIdx.x + kThreads * i;
    if constexpr (RAW == 1) wvoff[i] = (unsigned)(((e / (NT * 4)) * c_dst + (e % (NT * 4)) * E) * (int)sizeof(T));
    else if constexpr (RAW == 2 || RAW == 4) wvoff[i] = (unsigned)(((e / C) * c_src + (e % C) * E) * (int)sizeof(T));
    else if constexpr (RAW == 3) wvoff[i] = (unsigned)(((e / (NT * 128)) * nts * 128 + e % (NT * 128)) * 16);
    else wvoff[i] = (unsigned)(((e / (NT * 64)) * nts * 64 + e % (NT * 64)) * 16);
  }
  auto weights_issue = [&](int4v (&wreg)[NW], int k, int slab) {
    if constexpr (!kBuf) {
#pragma unroll
      for (int i = 0; i < NW; ++i) {
        const int e = threadIdx.x + kThreads * i;
        if (NW * kThreads == WCH || e < WCH) {
          if constexpr (RAW == 2) {
            const int row = e / C, c = e % C;
            wreg[i] = *reinterpret_cast<const int4v *>(
                packed + ((size_t)k * c_dst + nt0 * 32 + row) * c_src + (size_t)(slab * C + c) * E);
          } else {
            const int q = e / (NT * 64), rem = e % (NT * 64);
            wreg[i] = packed4[packed_per_k * k + ((size_t)(slab * S + q) * nts + nt0) * 64 + rem];
          }
        }
      }
      return;
    }
    unsigned soff;                                       // (wave-uniform: goes to the scalar offset)
    if constexpr (RAW == 1) soff = (unsigned)(((k * c_src + slab * (C * E)) * c_dst + nt0 * 32) * (int)sizeof(T));
    else if constexpr (RAW == 2 || RAW == 4) soff = (unsigned)(((k * c_dst + nt0 * 32) * c_src + slab * (C * E)) * (int)sizeof(T));
    else if constexpr (RAW == 3) soff = (unsigned)(((int)packed_per_k * k + ((slab * 2) * nts + nt0) * 128) * 16);
    else soff = (unsigned)(((int)packed_per_k * k + ((slab * S) * nts + nt0) * 64) * 16);
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int e = threadIdx.x + kThreads * i;
      if (NW * kThreads == WCH || e < WCH)
        wreg[i] = __builtin_bit_cast(int4v, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wvoff[i], soff, 0));
    }
  };
  auto weights_commit = [&](const int4v (&wreg)[NW], int buf) {
#pragma unroll
    for (int i = 0; i < NW; ++i) {
      const int e = threadIdx.x + kThreads * i;
      if (NW * kThreads == WCH || e < WCH) {
        if constexpr (RAW == 1) {
          const int row = e / (NT * 4), c = e % (NT * 4);
          w_lds[buf * WCH + row * (NT * 4) + (c ^ raw_swizzle<NT>(row))] = wreg[i];
        } else if constexpr (RAW == 2) {
          w_lds[buf * WCH + a_slot<S>(e / C, e % C)] = wreg[i];
        } else if constexpr (RAW == 4) {
          split_and_store(w_lds + buf * WCH, __builtin_bit_cast(float4v, wreg[i]), e / C, e % C, lane);
        } else {
          w_lds[buf * WCH + e] = wreg[i];
        }
      }
    }
  };

  int k = __builtin_ctzll(todo);
  todo &= todo - 1;
  int slab = 0;
  int k_nxt = todo ? __builtin_ctzll(todo) : -1;
  if (todo) todo &= todo - 1;
  bool active = (wave_mask >> k) & 1;
  int4v wreg[NW];
  constexpr int NV = MT * S;                              // row chunks per lane and stage
  int4v v[NV];
  int gsel[kBuf ? 1 : NV];
  auto rows_issue = [&](int slab_, int slot_ = 0) {
    if constexpr (kBuf) gather_issue_buf<S>(v, goff + slot_ * WR, rsrc, slab_, lane);
    else gather_issue<T, S>(v, gsel, gidx, src, c_src, slab_, lane);
  };
  auto rows_commit = [&]() {
    if constexpr (RAW == 3 || RAW == 4) gather_commit_bf3_buf(a_lds, v, lane);
    else if constexpr (kBuf) gather_commit_buf<S>(a_lds, v, lane);
    else gather_commit<S>(a_lds, v, gsel, lane);
  };

  // prologue: stage 0 goes straight to LDS
  if (owns_row) goff[lane] = row_offset(k_first >= 0 ? g_first : (in_range ? nbr[(size_t)k * nbr_stride + my_row] : -1));
  int g_nxt = (k_nxt >= 0 && in_range) ? nbr[(size_t)k_nxt * nbr_stride + my_row] : -1;
  wave_lds_fence();
  weights_issue(wreg, k, 0);
  if (active) rows_issue(0);
  weights_commit(wreg, 0);
  if (active) rows_commit();
  __syncthreads();

  int buf = 0;
  if constexpr (kBuf) {
    // Every stage is the same straight run of instructions for every wave: a wave whose rows do
    // not use the next offset still issues its row loads (all its offsets are kAbsentRow, so
    // they fetch nothing and return zeros) and writes the zeros to its tile, and only skips the
    // MFMAs.  With no branch around the loads and their consumers the compiler knows exactly
    // which loads are in flight at every point and waits for none it does not need; in
    // particular the index load below stays in flight across the stage.
    const int safe_row = min(my_row, n_dst - 1);
    auto mma_stage = [&]() {
      if constexpr (RAW == 1) mma_slab_raw<T, NT, S>(acc, a_lds, w_lds + buf * WCH, lane);
      else if constexpr (RAW == 2) mma_slab_rawt<T, NT, S>(acc, a_lds, w_lds + buf * WCH, lane);
      else if constexpr (RAW == 3) mma_slab_bf3<NT>(acc, a_lds, w_lds + buf * WCH, lane);
      else if constexpr (RAW == 4) mma_slab_bf3t<NT>(acc, a_lds, w_lds + buf * WCH, lane);
      else mma_slab<T, NT, S>(acc, a_lds, w_lds + buf * WCH, 0, lane);
    };
    // Offsets are numbered in the order the tile walks them; offset j gathers through the index
    // set j & 1.  While stage (offset j, last slab) runs, set (j + 1) & 1 serves the loads of
    // offset j + 1 and set j & 1, which nothing reads any more, receives the offsets of offset
    // j + 2, whose indices were requested a whole stage earlier; the indices of offset j + 3 are
    // requested then.  So no stage starts by waiting for an index or for its way through LDS.
    int k1 = k_nxt;                                          // the next offset (-1: none)
    int k2 = todo ? __builtin_ctzll(todo) : -1;              // the one after
    if (todo) todo &= todo - 1;
    if (k1 >= 0) {                                           // (requested in the prologue, long landed)
      const bool a1 = (wave_mask >> k1) & 1;
      if (owns_row) goff[WR + lane] = row_offset(in_range && a1 ? g_nxt : -1);
      wave_lds_fence();
    }
    // (nothing of the prologue is in flight any more; said explicitly, because the compiler
    // cannot tell from the prologue's branches and would wait for loads that never were issued)
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
    if (k2 >= 0) g_nxt = nbr[(size_t)k2 * nbr_stride + safe_row];
    int slot = 0;
    // One pass of the loop per stage that has a successor: request the successor's weights and
    // rows, multiply this stage, move the successor to LDS; the last stage's products follow
    // the loop.  (One exit test, at the top: issue and commit always run together.)
    int nk = k, nslab = 1;
    if (nslab == slabs) { nk = k1; nslab = 0; }
    while (nk >= 0) {
      const bool adv = nk != k;
      const int nslot = adv ? slot ^ 1 : slot;
      weights_issue(wreg, nk, nslab);
      rows_issue(nslab, nslot);
      int k3 = -1;
      if (adv) {
        // (a wave that does not use an offset: all absent, also over the pair view, whose list
        // names a row whatever the offset)
        const bool a2 = k2 >= 0 && ((wave_mask >> k2) & 1);
        if (owns_row) goff[slot * WR + lane] = row_offset(in_range && a2 ? g_nxt : -1);
        wave_lds_fence();
        k3 = todo ? __builtin_ctzll(todo) : -1;
        if (todo) todo &= todo - 1;
        if (k3 >= 0) g_nxt = nbr[(size_t)k3 * nbr_stride + safe_row];
      }
      if (active) mma_stage();
      wave_lds_fence();
      rows_commit();
      weights_commit(wreg, buf ^ 1);
      __syncthreads();
      buf ^= 1;
      active = (wave_mask >> nk) & 1;
      k = nk;
      slot = nslot;
      if (adv) { k1 = k2; k2 = k3; }
      nslab += 1;
      if (nslab == slabs) { nk = k1; nslab = 0; }
    }
    if (active) mma_stage();
  } else {
    while (true) {
      int nk = k, nslab = slab + 1;
      if (nslab == slabs) { nk = k_nxt; nslab = 0; }
      const bool has_next = nk >= 0;
      const bool next_active = has_next && ((wave_mask >> nk) & 1);
      if (has_next) {
        if (nk != k) {          // the row loads that used the old indices were issued a stage ago
          if (owns_row) goff[lane] = row_offset(g_nxt);
          wave_lds_fence();
        }
      }
      if (kInterleave && has_next && active && next_active) {
        // The common stage: this stage's MFMAs with the next stage's loads between them,
        // one row load after each (k-step, row tile) group.  A load instruction waits at
        // issue while the CU's memory queue is full; issued in a block before the MFMAs
        // those waits come on top of the MFMA time, issued between them they pass while
        // the matrix pipe works off what it has.  (MFMAs and loads stay on their side of
        // each scheduling barrier, LDS reads and address arithmetic may cross.)
        const int4v *wl = w_lds + buf * WCH;
        const int h = lane / 32, r = lane % 32;
        weights_issue(wreg, nk, nslab);
  #pragma unroll
        for (int s = 0; s < S; ++s) {
          int4v b[NT];
  #pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            if constexpr (RAW == 1) b[nt] = raw_weight_frag<NT, S>(wl, s, nt, lane);
            else if constexpr (RAW == 2) b[nt] = wl[a_slot<S>(nt * 32 + r, h * S + s)];
            else b[nt] = wl[(s * NT + nt) * 64 + lane];
          }
  #pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const int4v a = a_lds[a_slot<S>(mt * 32 + r, h * S + s)];
  #pragma unroll
            for (int nt = 0; nt < NT; ++nt) mma<T>(acc[mt][nt], a, b[nt]);
            const int it = s * MT + mt;                      // one of the MT * S row loads
            gsel[it] = gidx[(it * 64 + lane) / C];
            v[it] = *reinterpret_cast<const int4v *>(src + (size_t)max(gsel[it], 0) * c_src +
                                                     (size_t)(nslab * C + (it * 64 + lane) % C) * E);
            __builtin_amdgcn_sched_barrier(0x386);
          }
        }
      } else {
        if (has_next) {
          weights_issue(wreg, nk, nslab);
          if (next_active) rows_issue(nslab);
        }
        if (active) {
          if constexpr (RAW == 1) mma_slab_raw<T, NT, S>(acc, a_lds, w_lds + buf * WCH, lane);
          else if constexpr (RAW == 2) mma_slab_rawt<T, NT, S>(acc, a_lds, w_lds + buf * WCH, lane);
          else if constexpr (RAW == 3) mma_slab_bf3<NT>(acc, a_lds, w_lds + buf * WCH, lane);
          else if constexpr (RAW == 4) mma_slab_bf3t<NT>(acc, a_lds, w_lds + buf * WCH, lane);
          else mma_slab<T, NT, S>(acc, a_lds, w_lds + buf * WCH, 0, lane);
        }
      }
      if (!has_next) break;
      wave_lds_fence();
      if (next_active) rows_commit();
      weights_commit(wreg, buf ^ 1);
      if (nk != k) {
        k_nxt = todo ? __builtin_ctzll(todo) : -1;
        if (todo) todo &= todo - 1;
        g_nxt = (k_nxt >= 0 && in_range) ? nbr[(size_t)k_nxt * nbr_stride + my_row] : -1;
      }
      __syncthreads();
      buf ^= 1;
      k = nk;
      slab = nslab;
      active = next_active;
    }
  }
  if (wave_mask) {
    wave_lds_fence();
    if (shared_tile)
      add_rows_lds<T, NT, S, true>(acc, dst, didx, reinterpret_cast<float *>(a_lds), c_dst, nt0 * 32, lane);
    else
      add_rows_lds<T, NT, S, false>(acc, dst, didx, reinterpret_cast<float *>(a_lds), c_dst, nt0 * 32, lane);
  }
}

template <typename T, int NT, int S, int RAW, int MT = 2>
__global__ __launch_bounds__(kThreads, MT == 1 ? 4 : (NT == 4 ? 2 : 3)) void gms_rows_kernel(
    const T *__restrict__ src, const T *__restrict__ packed, T *__restrict__ dst,
    const int32_t *__restrict__ nbr, const unsigned long long *__restrict__ block_masks,
    const int32_t *__restrict__ perm, const int32_t *__restrict__ tile_order, int n_dst, int k_vol,
    int c_src, int c_dst, int part_stages, SideJob side, int pair_view, unsigned src_bytes) {
  // the leading workgroups of the grid run the side job, if there is one
  int block_x = blockIdx.x;
  if (side.blocks) {
    if (block_x < side.blocks) {
      if (blockIdx.y == 0 && blockIdx.z == 0) run_side_job(side, block_x);
      return;
    }
    block_x -= side.blocks;
  }
  gms_rows_body<T, NT, S, RAW, MT>(src, packed, dst, nbr, block_masks, perm, tile_order, n_dst, k_vol, c_src,
                                   c_dst, part_stages, block_x, blockIdx.y, blockIdx.z, gridDim.z, src_bytes, pair_view);
}

// ---------------------------------------------------------------------------
struct Shape {
  int c_src, c_dst, S, NT, E;
  int NTR;                // 32-column tiles per wave in the output-stationary kernel
  size_t lds_bytes;       // pair-stationary kernel
  size_t lds_rows_bytes;  // output-stationary kernel
  bool ok;
};

Shape shape_of(const GmsArgs &a) {
  Shape s{};
  s.c_src = a.transpose_w ? a.c_out : a.c_in;
  s.c_dst = a.transpose_w ? a.c_in : a.c_out;
  s.E = a.dtype == FGMS_F16 ? 8 : 4;
  const size_t esz = a.dtype == FGMS_F16 ? 2 : 4;
  s.ok = false;
  if (s.c_dst % 32 != 0 || s.c_src % (2 * s.E) != 0) return s;
  s.S = (s.c_src % (8 * s.E) == 0) ? 4 : (s.c_src % (4 * s.E) == 0) ? 2 : 1;
  s.NT = (s.c_dst % 64 == 0) ? 2 : 1;
  // rows are read with 16-byte loads and fp16 results written as 4-byte pairs
  if (reinterpret_cast<uintptr_t>(a.src) % 16 || reinterpret_cast<uintptr_t>(a.dst) % 4) return s;
  const size_t tiles = (size_t)kWaves * kWaveRows * 2 * s.S * 16  // staging tiles
                       + (size_t)kWaves * 3 * kWaveRows * sizeof(int);
  s.lds_bytes = (size_t)s.c_src * s.NT * 32 * esz + tiles;      // + weights of one offset
  // wide fp16 layers: 128 columns per wave, so that a row is gathered once per 128
  // (not 64) output channels.  Costs 128 accumulator registers (2 waves per SIMD)
  // and halves the number of workgroups, so only when enough of them remain to
  // fill the chip; fp32 has 8x the MFMA time per gathered byte and gains nothing.
  const int64_t wide_wgs = (a.n_dst + kTileRows - 1) / kTileRows * (s.c_dst / 128);
  const bool wide = kernel_policy() == 3 || (a.dtype == FGMS_F16 && wide_wgs * 2 >= 3 * (int64_t)num_cus());
  s.NTR = (s.c_dst % 128 == 0 && wide) ? 4 : s.NT;
  s.lds_rows_bytes = 2 * (size_t)s.S * s.NTR * 64 * 16 + tiles;  // + two stages of weights
  s.ok = s.lds_bytes <= 128 * 1024;
  return s;
}

template <typename T>
int pack_weights(const GmsArgs &a, const Shape &s, const T **packed) {
  void *ws = nullptr;
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  bool fill = true;
  int rc = relaid_weights_buffer(a, (unsigned)s.S << 8 | (a.transpose_w ? 2u : 0u), n * sizeof(T), &ws, &fill);
  if (rc != FGMS_OK) return rc;
  *packed = (const T *)ws;
  if (!fill) return FGMS_OK;
  unsigned blocks = (unsigned)((n + 255) / 256);
  if (blocks > 4096) blocks = 4096;
  pack_weights_kernel<T><<<blocks, 256, 0, a.stream>>>((const T *)a.w, (T *)ws, a.k_vol, a.c_in,
                                                       a.c_out, s.S, a.transpose_w);
  FGMS_HIP_TRY(hipGetLastError());
  relaid_weights_filled(a, ws);
  return FGMS_OK;
}

// The same for the split-bf16 layout of fp32 weights (pack_weights_bf3_kernel).
int pack_weights_bf3(const GmsArgs &a, bool transpose, const void **packed) {
  void *ws = nullptr;
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  bool fill = true;
  int rc = relaid_weights_buffer(a, 1u | (transpose ? 2u : 0u), n * sizeof(float), &ws, &fill);
  if (rc != FGMS_OK) return rc;
  *packed = ws;
  if (!fill) return FGMS_OK;
  size_t blocks = (n / 8 + 255) / 256;
  pack_weights_bf3_kernel<<<(unsigned)(blocks > 4096 ? 4096 : blocks), 256, 0, a.stream>>>(
      (const float *)a.w, (int4v *)ws, a.k_vol, a.c_in, a.c_out, transpose);
  FGMS_HIP_TRY(hipGetLastError());
  relaid_weights_filled(a, ws);
  return FGMS_OK;
}


template <typename T, int NT, int S>
int launch_pairs(const GmsArgs &a, const Shape &s) {
  const T *packed = nullptr;
  // fp32 tensors whose caller allows tf32 precision: products in split bf16
  constexpr bool kCanSplit = sizeof(T) == 4 && S == 4;
  const bool split = kCanSplit && a.reduced && split_bf16_enabled();
  if (split) {
    const void *ws = nullptr;
    int rc = pack_weights_bf3(a, a.transpose_w, &ws);
    if (rc != FGMS_OK) return rc;
    packed = (const T *)ws;
  } else {
    int rc = pack_weights<T>(a, s, &packed);
    if (rc != FGMS_OK) return rc;
  }
  const bool dense = a.dense_k >= 0;
  const int64_t tiles = dense ? (a.n_dense + kTileRows - 1) / kTileRows
                              : (a.n_pairs + kTileRows - 1) / kTileRows + a.k_vol;
  // a few workgroups per CU, each walking a contiguous run of tiles
  const int64_t want_wgs = (int64_t)num_cus() * 8;
  const int tiles_per_wg = (int)((tiles + want_wgs - 1) / want_wgs);
  const unsigned gx = (unsigned)((tiles + tiles_per_wg - 1) / tiles_per_wg);
  auto kern = split ? gms_pairs_kernel<T, NT, S, kCanSplit> : gms_pairs_kernel<T, NT, S, false>;
  { const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)s.lds_bytes); if (rc_lds != FGMS_OK) return rc_lds; }
  {
    ProfileScope prof(split ? (a.transpose_w ? "gms_pairs_kernel(dgrad, bf16x3)" : "gms_pairs_kernel(fwd, bf16x3)")
                            : (a.transpose_w ? "gms_pairs_kernel(dgrad)" : "gms_pairs_kernel(fwd)"),
                      a.stream);
    kern<<<dim3(gx, (unsigned)(s.c_dst / (32 * NT))), kThreads, s.lds_bytes, a.stream>>>(
        (const T *)a.src, packed, (T *)a.dst, a.kpos, a.gmap, a.smap, a.k_vol, s.c_src, s.c_dst,
        tiles_per_wg, a.dense_k, (int)a.n_dense);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

// FGMS_HALF_TILES=0 keeps small launches on 256-row tiles (for comparison).
bool half_tiles_enabled() {
  static const bool on = !(getenv("FGMS_HALF_TILES") && atoi(getenv("FGMS_HALF_TILES")) == 0);
  return on;
}

// Grid of an output-stationary launch over n_dst destination rows: tiles of 256 rows from the
// plan's tile table where there is one (`table_grid` entries), else plain tiles of 256 or --
// where those still fit the chip's workgroup slots in one round -- of 128 rows (32 per wave:
// twice the waves, half the work per wave and stage; such a launch lasts as long as one
// tile's chain of stages).  A launch that then fills less than half of the slots shares every
// tile between two workgroups, each taking half of the tile's stages and adding its part with
// atomics: twice the workgroups, half the critical path.  (Two parts only: the sum of two
// partial results does not depend on their order.  On launches that fill the chip the atomics
// cost more than the split gains.)  The standalone and the one-grid backward launch share this
// choice, so that their input gradients agree bit for bit; an input gradient takes the small
// tiles only where they (times two, for the shared tiles) fill at most half of the slots, since
// in the backward launch its workgroups share the chip with the weight gradient's and more of
// them delay those.  Measured (MI355X, 64 -> 64 fp16 over 10 k / 20 k / 50 k / 60 k voxels of the
// indoor cloud): forward 23.5 -> 16.9, 23.3 -> 18.3, 26.5 -> 22.8, 28.5 -> 25.7 us; backward
// launch 22.5 -> 17.0, 26.1 -> 20.9, 35.6 -> 36.0, 43.2 -> 47.8 us (128 -> 128 over 28 k voxels:
// 53.2 -> 63.0 us), hence the rule; 32 -> 32 fp32 over 20 k voxels, whole step: 64.0 -> 56.6 us.
struct RowsGrid {
  bool half_tiles;
  bool drop_table;      // the launch does better on plain 128-row tiles than on the plan's tile table
  unsigned gx, gz;
  int part_stages;
};
RowsGrid rows_grid(int64_t n_dst, unsigned gy, int stages, bool can_half, bool has_table, int table_grid,
                   bool pair_view, int wgs_per_cu, bool input_gradient) {
  RowsGrid g{};
  const int64_t small_tiles = (int64_t)((n_dst + 127) / 128) * gy;
  // A forward launch too big to share its 256-row tiles between two workgroups (below) and
  // not yet a full round of them is neither short-chained nor busy: 128-row tiles in plain order
  // then beat the table's XCD-aware 256-row tiles (64 -> 64 fp16 over 100 k / 130 k voxels:
  // 40.9 -> 34.4, 41.2 -> 36.9 us; 70 k / 80 k voxels with shared 256-row tiles: 28.1 / 29.1 us).
  g.drop_table = can_half && half_tiles_enabled() && has_table && !pair_view && !input_gradient &&
                 small_tiles <= (int64_t)num_cus() * 4 &&
                 ((int64_t)table_grid * gy * 2 > (int64_t)num_cus() * wgs_per_cu || stages < 8);
  if (g.drop_table) has_table = false;
  g.half_tiles = can_half && half_tiles_enabled() && !has_table && !pair_view &&
                 (input_gradient ? small_tiles * 4 <= (int64_t)num_cus() * 3 : small_tiles <= (int64_t)num_cus() * 4);
  const int tile_rows = g.half_tiles ? kTileRows / 2 : kTileRows;
  g.gx = has_table ? (unsigned)table_grid : (unsigned)((n_dst + tile_rows - 1) / tile_rows);
  // (an input gradient shares its launch with the weight gradient: its 256-row tiles are shared
  // only up to 2.25 workgroups per CU; 64 -> 64 fp16 backward launch over 70 k / 80 k / 90 k voxels
  // shared 50.7 / 58.6 / 60.4 us, not shared 54.7 / 55.8 / 56.4 us)
  const int64_t slots = g.half_tiles ? (int64_t)num_cus() * 4
                        : input_gradient ? (int64_t)num_cus() * 9 / 4 : (int64_t)num_cus() * wgs_per_cu;
  g.gz = 1;
  g.part_stages = 1;
  if (!pair_view && (int64_t)g.gx * gy * 2 <= slots && stages >= 8) {
    g.part_stages = (stages + 1) / 2;
    g.gz = 2;
  }
  return g;
}

// FGMS_RAW_WEIGHTS=0 keeps the forward pass on re-laid weights (for comparison).
bool raw_weights_enabled() {
  static const bool on = !(getenv("FGMS_RAW_WEIGHTS") && atoi(getenv("FGMS_RAW_WEIGHTS")) == 0);
  return on;
}

template <typename T, int NT, int S>
int launch_rows(const GmsArgs &a, const Shape &s, const int32_t *nbr,
                const unsigned long long *masks, const int32_t *perm, const int32_t *tile_order,
                int tile_grid, bool pair_view = false) {
  // With 64-column wave tiles the input gradient and the fp16 forward pass read the weight
  // tensor as it is (16-byte aligned rows of the tile) when the caller brings no re-laid
  // copy; the rest gets one, made here.  Measured: 64 -> 64 over 200k voxels, input gradient
  // 48.3 us raw against 47.3 us + a 4.4 us re-layout launch (the backward call re-lays
  // inside its other launch for free and keeps doing so); with 128-column wave tiles raw
  // weights lose either way (128 -> 128 over 120k voxels: forward 99.7 us against
  // 93.6 + 4.4 us, input gradient 92.9 against 87.7 + 4.4 us).  The fp32 forward pass has no
  // transposing LDS read to use.
  int raw = 0;
  if (NT != 4 && !a.prepacked && reinterpret_cast<uintptr_t>(a.w) % 16 == 0 && raw_weights_enabled())
    raw = a.transpose_w ? 2 : (sizeof(T) == 2 ? 1 : 0);
  // pinned weights: their re-laid copy is made once, and its plain fragment reads beat the
  // transposing ones of the raw tile (64 -> 64 fp16 forward over 200k voxels 41.9 -> 41.3 us)
  if (raw == 1 && weights_pinned(a.w)) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (!(a.stream && hipStreamIsCapturing(a.stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone)) raw = 0;
  }
  // fp32 forward in "tf32" mode: products in split bf16 (three 16-bit MFMAs instead of
  // sixteen fp32 ones per product tile); needs whole 32-channel slabs
  constexpr bool kCanSplit = sizeof(T) == 4 && S == 4 && NT != 4;
  const bool split = kCanSplit && a.reduced && !a.transpose_w && !a.prepacked && split_bf16_enabled();
  if (kCanSplit && a.reduced && raw == 2 && split_bf16_enabled()) raw = 4;   // (the input gradient splits as it reads)
  const T *packed = raw ? (const T *)a.w : (const T *)a.prepacked;
  if (split) {
    const void *ws = nullptr;
    int rc = pack_weights_bf3(a, false, &ws);
    if (rc != FGMS_OK) return rc;
    packed = (const T *)ws;
    raw = 3;
  } else if (!packed) {
    int rc = pack_weights<T>(a, s, &packed);
    if (rc != FGMS_OK) return rc;
  }
  const int slabs = s.c_src / (2 * S * s.E);
  const unsigned gy = (unsigned)(s.c_dst / (32 * NT));
  constexpr bool kCanHalf = NT != 4;
  const RowsGrid rg = rows_grid(a.n_dst, gy, a.k_vol * slabs, kCanHalf, tile_order != nullptr, tile_grid, pair_view,
                                NT == 4 ? 2 : 3, a.transpose_w);
  const bool half_tiles = rg.half_tiles;
  if (rg.drop_table) tile_order = nullptr;
  const size_t lds_rows = half_tiles ? s.lds_rows_bytes - (size_t)kWaves * 32 * (2 * S * 16 + 3 * sizeof(int))
                                     : s.lds_rows_bytes;
  const unsigned gx = rg.gx;
  if (gx == 0) return a.side.kind ? launch_side_job(a.side, a.stream) : FGMS_OK;
  constexpr bool kCanRaw = NT != 4;
  constexpr int kHalfMT = kCanHalf ? 1 : 2;
  auto kern = half_tiles ? (raw == 4   ? gms_rows_kernel<T, NT, S, kCanSplit ? 4 : 0, kHalfMT>
                            : raw == 3 ? gms_rows_kernel<T, NT, S, kCanSplit ? 3 : 0, kHalfMT>
                            : raw == 2 ? gms_rows_kernel<T, NT, S, kCanRaw ? 2 : 0, kHalfMT>
                            : raw == 1 ? gms_rows_kernel<T, NT, S, kCanRaw && sizeof(T) == 2 ? 1 : 0, kHalfMT>
                                       : gms_rows_kernel<T, NT, S, 0, kHalfMT>)
              : raw == 4 ? gms_rows_kernel<T, NT, S, kCanSplit ? 4 : 0>
              : raw == 3 ? gms_rows_kernel<T, NT, S, kCanSplit ? 3 : 0>
              : raw == 2 ? gms_rows_kernel<T, NT, S, kCanRaw ? 2 : 0>
              : raw == 1 ? gms_rows_kernel<T, NT, S, kCanRaw && sizeof(T) == 2 ? 1 : 0>
                         : gms_rows_kernel<T, NT, S, 0>;
  { const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(kern), lds_rows); if (rc_lds != FGMS_OK) return rc_lds; }
  const int part_stages = rg.gz > 1 ? rg.part_stages : 0;
  const unsigned gz = rg.gz;
  {
    ProfileScope prof(pair_view ? (a.transpose_w ? "gms_rows_kernel(dgrad, pair view)" : "gms_rows_kernel(fwd, pair view)") :raw == 4   ? "gms_rows_kernel(dgrad, bf16x3)"
                      : raw == 3 ? "gms_rows_kernel(fwd, bf16x3)"
                      : a.transpose_w ? "gms_rows_kernel(dgrad)" : "gms_rows_kernel(fwd)",
                      a.stream);
    kern<<<dim3(gx + (unsigned)a.side.blocks, gy, gz), kThreads, lds_rows, a.stream>>>(
        (const T *)a.src, packed, (T *)a.dst, nbr, masks, perm, tile_order, (int)a.n_dst, a.k_vol,
        s.c_src, s.c_dst, part_stages > 0 ? part_stages : 1, a.side, pair_view ? 1 : 0,
        (unsigned)((size_t)a.n_src * s.c_src * sizeof(T)));
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

// ---------------------------------------------------------------------------
// Backward in one launch: the output-stationary input gradient (gms_rows_body, weights read
// as they lie) and the per-wave weight gradient (wgrad_wave_body) share a grid.  The two
// do not depend on each other, and workgroups of both kinds resident on the chip at the
// same time finish sooner than the two launches one after the other.
// Measured on 64 -> 64 fp16 over 200k voxels: the two kernels on two streams running
// freely 77 us per (input gradient, weight gradient) pair against 98 us back to back;
// ordering two streams with events costs more than that gain, one grid costs nothing
// (83 us + a 2 us launch that rounds the fp16 weight gradient).  The input gradient's
// workgroups come first in the grid (its longest tiles are the longest jobs of the launch;
// dealing the two kinds alternately or the weight gradient first measured 1-2 us slower).
// Their count is a multiple of 8, so that a workgroup's index mod 8, its XCD, is what the
// plan's XCD-aware orders of either kind assume.
template <typename T, int NT, int S, int BI, int BJ, int RAWD, int MT = 2>
__global__ __launch_bounds__(kThreads, NT == 4 ? 2 : 3) void bwd_fused_kernel(
    const T *__restrict__ gout, const T *__restrict__ w, T *__restrict__ gin,
    const int32_t *__restrict__ nbr, const unsigned long long *__restrict__ block_masks,
    const int32_t *__restrict__ perm, const int32_t *__restrict__ tile_order, int n_in, int k_vol,
    int c_in, int c_out, int part_stages, const T *__restrict__ in, float *__restrict__ gw32,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
    const int32_t *__restrict__ omap, SliceMap smap, int row_x, int row_y, int row_z, int wgrad_x,
    unsigned gout_bytes, unsigned in_bytes, int wgrad_blocks, SideJob check) {
  // grid: row_x * row_y * row_z workgroups of the input gradient (tiles, column tiles,
  // parts of a tile), then wgrad_x * (tiles of dW[k]) of the weight gradient, then those of a
  // side job (the plan's fingerprint check), if there is one
  const int rows_total = row_x * row_y * row_z;
  if ((int)blockIdx.x >= rows_total + wgrad_blocks) {
    run_side_job(check, (int)blockIdx.x - rows_total - wgrad_blocks);
    return;
  }
  if ((int)blockIdx.x < rows_total) {
    const int bx = blockIdx.x % row_x, rest = blockIdx.x / row_x;
    gms_rows_body<T, NT, S, RAWD, MT>(gout, w, gin, nbr, block_masks, perm, tile_order, n_in, k_vol, c_out, c_in,
                                      part_stages, bx, rest % row_y, rest / row_y, row_z, gout_bytes);
  } else {
    const int j = blockIdx.x - rows_total;
    if constexpr (BI <= 2 && BJ <= 2)
      wgrad_wave_body<T, BI, BJ, RAWD == 4>(in, gout, gw32, kpos, imap, omap, k_vol, c_in, c_out, smap,
                                            j % wgrad_x, j / wgrad_x, in_bytes, gout_bytes);
    else
      wgrad_wg_body<T, BI, BJ, RAWD == 4>(in, gout, gw32, kpos, imap, omap, k_vol, c_in, c_out, smap,
                                          j % wgrad_x, j / wgrad_x);
  }
}

// FGMS_FUSED_BWD=0 keeps the backward call on its two launches (for comparison).
bool fused_bwd_enabled() {
  static const bool on = !(getenv("FGMS_FUSED_BWD") && atoi(getenv("FGMS_FUSED_BWD")) == 0);
  return on;
}

template <typename T, int NT, int S, int BI, int BJ>
int launch_fused(const GmsArgs &d, const Shape &s, const Plan *p, const WgradArgs &w, const WgradGeometry &g,
                 float *acc32) {
  // the input gradient's grid, as launch_rows lays it out (tiles padded to a multiple of 8)
  const int slabs = s.c_src / (2 * S * s.E);
  const unsigned row_y = (unsigned)(s.c_dst / (32 * NT));
  constexpr bool kCanHalf = NT != 4;
  const RowsGrid rg = rows_grid(d.n_dst, row_y, d.k_vol * slabs, kCanHalf, p->tile_in != nullptr, p->tile_grid_in,
                                false, NT == 4 ? 2 : 3, true);
  const unsigned row_x = (rg.gx + 7) / 8 * 8;
  const int part_stages = rg.part_stages;
  const unsigned row_z = rg.gz;
  size_t lds = g.lds;
  if (lds < s.lds_rows_bytes) lds = s.lds_rows_bytes;
  // RAWD: how the input gradient reads the weights (2: as they lie; 4: also split into bf16
  // pairs, for fp32 tensors whose caller allows tf32 precision)
  constexpr bool kCanSplit = sizeof(T) == 4 && S == 4 && NT != 4;
  const bool split = kCanSplit && d.reduced && split_bf16_enabled() && g.split;
  constexpr int kHalfMT = kCanHalf ? 1 : 2;
  auto kern = rg.half_tiles ? (split ? bwd_fused_kernel<T, NT, S, BI, BJ, kCanSplit ? 4 : 2, kHalfMT>
                                     : bwd_fused_kernel<T, NT, S, BI, BJ, 2, kHalfMT>)
              : split       ? bwd_fused_kernel<T, NT, S, BI, BJ, kCanSplit ? 4 : 2>
                            : bwd_fused_kernel<T, NT, S, BI, BJ, 2>;
  { const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)lds); if (rc_lds != FGMS_OK) return rc_lds; }
  {
    ProfileScope prof(split ? "bwd_fused_kernel(bf16x3)" : "bwd_fused_kernel", d.stream);
    SideJob check{};
    (void)plan_take_check(p, &check);
    kern<<<row_x * row_y * row_z + (unsigned)(g.tiles * g.ty) + (unsigned)check.blocks, kThreads, lds, d.stream>>>(
        (const T *)d.src, (const T *)d.w, (T *)d.dst, p->nbr_in, p->mask_in, p->perm_in, p->tile_in,
        (int)d.n_dst, d.k_vol, d.c_in, d.c_out, part_stages, (const T *)w.in, acc32, w.kpos, w.imap, w.omap,
        g.smap, (int)row_x, (int)row_y, (int)row_z, (int)g.tiles,
        (unsigned)((size_t)d.n_src * s.c_src * sizeof(T)), (unsigned)((size_t)w.n_in * w.c_in * sizeof(T)),
        (int)(g.tiles * g.ty), check);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

template <typename T, typename F>
int dispatch_shape(const Shape &s, F &&f);

template <typename T, typename F>
int dispatch_rows_shape(const Shape &s, F &&f) {
  if (s.NTR == 4) {
    if (s.S == 4) return f(std::integral_constant<int, 4>{}, std::integral_constant<int, 4>{});
    if (s.S == 2) return f(std::integral_constant<int, 4>{}, std::integral_constant<int, 2>{});
    return f(std::integral_constant<int, 4>{}, std::integral_constant<int, 1>{});
  }
  return dispatch_shape<T>(s, f);
}

template <typename T, typename F>
int dispatch_shape(const Shape &s, F &&f) {
  if (s.NT == 2) {
    if (s.S == 4) return f(std::integral_constant<int, 2>{}, std::integral_constant<int, 4>{});
    if (s.S == 2) return f(std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    return f(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
  }
  if (s.S == 4) return f(std::integral_constant<int, 1>{}, std::integral_constant<int, 4>{});
  if (s.S == 2) return f(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{});
  return f(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
}

}  // namespace

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

int pack_weights_any(const GmsArgs &a, int S, const void **packed) {
  Shape s{};
  s.S = S;
  if (a.dtype == FGMS_F16) {
    const __half *p = nullptr;
    int rc = pack_weights<__half>(a, s, &p);
    *packed = p;
    return rc;
  }
  const float *p = nullptr;
  int rc = pack_weights<float>(a, s, &p);
  *packed = p;
  return rc;
}

// Input gradient `d` (output-stationary, through plan `p`) and weight gradient `w` of one
// layer in one launch where bwd_fused_kernel covers the shape; *done = false (and nothing
// launched) where it does not.
int launch_fused_bwd(const GmsArgs &d, const Plan *p, const WgradArgs &w, bool *done) {
  *done = false;
  if (!fused_bwd_enabled() || !d.transpose_w || d.prepacked || d.side.kind || w.side.kind ||
      d.k_vol != w.k_vol || d.c_in != w.c_in || d.c_out != w.c_out || d.dtype != w.dtype || d.stream != w.stream)
    return FGMS_OK;
  const Shape s = shape_of(d);
  if (!s.ok || reinterpret_cast<uintptr_t>(d.w) % 16 != 0 || !raw_weights_enabled()) return FGMS_OK;
  WgradGeometry g;
  if (!mfma_wgrad_supported(w) || wgrad_geometry(w, &g, true) != FGMS_OK) return FGMS_OK;
  float *acc32 = nullptr;
  int rc = wgrad_accumulator(w, &acc32);
  if (rc != FGMS_OK) return rc;
  bool found = false;
  // (wave tile columns NT of the input gradient, MFMA steps per slab S) follow from c_in and
  // c_out, and so do the block counts (BI, BJ) of the weight gradient's tile
#define FGMS_FB(TT, NTv, Sv, BIv, BJv)                                             \
  if (!found && s.NTR == NTv && s.S == Sv && g.bi == BIv && g.bj == BJv) {          \
    found = true;                                                                    \
    rc = launch_fused<TT, NTv, Sv, BIv, BJv>(d, s, p, w, g, acc32);                 \
  }
  if (d.dtype == FGMS_F16) {
    FGMS_FB(__half, 1, 2, 1, 1) FGMS_FB(__half, 1, 4, 1, 2) FGMS_FB(__half, 1, 4, 1, 4)
    FGMS_FB(__half, 2, 2, 2, 1) FGMS_FB(__half, 2, 4, 2, 2) FGMS_FB(__half, 2, 4, 2, 4)
    FGMS_FB(__half, 2, 2, 4, 1) FGMS_FB(__half, 2, 4, 4, 2) FGMS_FB(__half, 2, 4, 4, 4)
    FGMS_FB(__half, 4, 2, 4, 1) FGMS_FB(__half, 4, 4, 4, 2) FGMS_FB(__half, 4, 4, 4, 4)
  } else {
    FGMS_FB(float, 1, 4, 1, 1) FGMS_FB(float, 1, 4, 1, 2) FGMS_FB(float, 1, 4, 1, 4)
    FGMS_FB(float, 2, 4, 2, 1) FGMS_FB(float, 2, 4, 2, 2) FGMS_FB(float, 2, 4, 2, 4)
    FGMS_FB(float, 2, 4, 4, 1) FGMS_FB(float, 2, 4, 4, 2) FGMS_FB(float, 2, 4, 4, 4)
  }
#undef FGMS_FB
  if (!found) return FGMS_OK;     // (no such kernel: the caller's two launches)
  if (rc != FGMS_OK) return rc;
  *done = true;
  return wgrad_finish(w, acc32);
}

int planned_pack_job(const GmsArgs &a, SideJob *job, const void **packed) {
  const Shape s = shape_of(a);
  if (!s.ok) {
    set_error("planned_pack_job: unsupported shape");
    return FGMS_E_INVALID;
  }
  const size_t esz = a.dtype == FGMS_F16 ? 2 : 4;
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  void *ws = nullptr;
  int rc = workspace_get(a.stream, 0, n * esz, &ws);
  if (rc != FGMS_OK) return rc;
  *job = SideJob{};
  job->kind = 1;
  job->src = a.w;
  job->dst = ws;
  job->n = n;
  job->k_vol = a.k_vol; job->c_in = a.c_in; job->c_out = a.c_out;
  job->S = s.S; job->transpose = a.transpose_w; job->dtype = a.dtype;
  // about 8 elements per thread of 256-thread workgroups
  size_t blocks = ((n + 2047) / 2048 + 7) / 8 * 8;
  job->blocks = (int)(blocks > 1024 ? 1024 : blocks);
  *packed = ws;
  return FGMS_OK;
}

int launch_side_job(const SideJob &job, hipStream_t stream) {
  if (job.kind == 0 || job.blocks <= 0) return FGMS_OK;
  side_job_kernel<<<(unsigned)job.blocks, 256, 0, stream>>>(job);
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

// FGMS_SPLIT_BF16=0 keeps fp32 tensors on fp32 MFMAs in "tf32" mode too (for comparison).
bool split_bf16_enabled() {
  static const bool on = !(getenv("FGMS_SPLIT_BF16") && atoi(getenv("FGMS_SPLIT_BF16")) == 0);
  return on;
}

bool mfma_gms_supported(const GmsArgs &a) { return shape_of(a).ok; }

int launch_mfma_gms(const GmsArgs &a) {
  const Shape s = shape_of(a);
  if (!s.ok) {
    set_error("launch_mfma_gms: unsupported shape");
    return FGMS_E_INVALID;
  }
  if (a.dtype == FGMS_F16)
    return dispatch_shape<__half>(s, [&](auto nt, auto sv) {
      return launch_pairs<__half, decltype(nt)::value, decltype(sv)::value>(a, s);
    });
  return dispatch_shape<float>(s, [&](auto nt, auto sv) {
    return launch_pairs<float, decltype(nt)::value, decltype(sv)::value>(a, s);
  });
}

// The output-stationary kernel gathers through a buffer resource: 32-bit byte offsets, and
// offsets at or above 2^31 stand for "no row" (gather_issue_buf).
static bool rows_fit_buffer(const GmsArgs &a) {
  const size_t c_src = a.transpose_w ? a.c_out : a.c_in;
  return (size_t)a.n_src * c_src * (a.dtype == FGMS_F16 ? 2 : 4) <= kMaxBufferBytes;
}

bool planned_gms_supported(const GmsArgs &a, const Plan *p) {
  if (!p || a.dense_k >= 0 || a.k_vol > 64 || a.k_vol != p->k_vol) return false;
  if (a.transpose_w) {
    if (!p->dgrad_ok || a.n_dst != p->n_in || a.n_src != p->n_out) return false;
  } else {
    if (!p->fwd_ok || a.n_dst != p->n_out || a.n_src != p->n_in) return false;
  }
  // result rows are updated with 8- and 16-byte accesses
  if (reinterpret_cast<uintptr_t>(a.dst) % 16) return false;
  if (!rows_fit_buffer(a)) return false;
  return shape_of(a).ok;
}

int launch_planned_gms(const GmsArgs &a, const Plan *p) {
  const Shape s = shape_of(a);
  if (!s.ok || !planned_gms_supported(a, p)) {
    set_error("launch_planned_gms: unsupported shape or plan");
    return FGMS_E_INVALID;
  }
  const int32_t *nbr = a.transpose_w ? p->nbr_in : p->nbr_out;
  const unsigned long long *masks = a.transpose_w ? p->mask_in : p->mask_out;
  const int32_t *perm = a.transpose_w ? p->perm_in : p->perm_out;
  const int32_t *tile_order = a.transpose_w ? p->tile_in : p->tile_out;
  const int tile_grid = a.transpose_w ? p->tile_grid_in : p->tile_grid_out;
  // (a pending fingerprint check of the plan rides along as the launch's side job)
  GmsArgs with_check = a;
  if (!with_check.side.kind) (void)plan_take_check(p, &with_check.side);
  const GmsArgs &a_ = with_check;
  if (a.dtype == FGMS_F16)
    return dispatch_rows_shape<__half>(s, [&](auto nt, auto sv) {
      return launch_rows<__half, decltype(nt)::value, decltype(sv)::value>(a_, s, nbr, masks, perm, tile_order, tile_grid);
    });
  return dispatch_rows_shape<float>(s, [&](auto nt, auto sv) {
    return launch_rows<float, decltype(nt)::value, decltype(sv)::value>(a_, s, nbr, masks, perm, tile_order, tile_grid);
  });
}

bool pair_view_gms_supported(const GmsArgs &a, const Plan *p) {
  if (!p || !p->pv_in || a.dense_k >= 0 || a.k_vol != p->k_vol) return false;
  if (a.transpose_w ? (a.n_dst != p->n_in || a.n_src != p->n_out) : (a.n_dst != p->n_out || a.n_src != p->n_in))
    return false;
  if (reinterpret_cast<uintptr_t>(a.dst) % 16 || !rows_fit_buffer(a)) return false;
  return shape_of(a).ok;
}

int launch_pair_view_gms(const GmsArgs &a, const Plan *p) {
  if (!pair_view_gms_supported(a, p)) {
    set_error("launch_pair_view_gms: unsupported shape or plan");
    return FGMS_E_INVALID;
  }
  // (the view was built on the stream that first resolved the plan)
  if (p->pv_ready && a.stream != p->pv_stream) FGMS_HIP_TRY(hipStreamWaitEvent(a.stream, p->pv_ready, 0));
  // the virtual rows stand in for the destination rows: tiles, the in-range test and the
  // choice of the wave tile's width go by their number
  GmsArgs v = a;
  v.n_dst = p->pv_rows;
  const Shape s = shape_of(v);
  const int32_t *nbr = a.transpose_w ? p->pv_out : p->pv_in;
  const int32_t *dest = a.transpose_w ? p->pv_in : p->pv_out;
  if (a.dtype == FGMS_F16)
    return dispatch_rows_shape<__half>(s, [&](auto nt, auto sv) {
      return launch_rows<__half, decltype(nt)::value, decltype(sv)::value>(v, s, nbr, p->pv_mask, dest, nullptr, 0, true);
    });
  return dispatch_rows_shape<float>(s, [&](auto nt, auto sv) {
    return launch_rows<float, decltype(nt)::value, decltype(sv)::value>(v, s, nbr, p->pv_mask, dest, nullptr, 0, true);
  });
}

// weight gradient: see fgms_wgrad.hip
}  // namespace fgms
