// Pieces shared by the output-stationary kernels: the swizzled LDS layout of a tile of rows,
// weight fragments read from a raw weight tile, and the update of the destination rows.
#pragma once

#include "fgms_device.h"
#include "fgms_internal.h"
#include "fgms_mma.h"

namespace fgms {

// LDS ordering between lanes of one wave: LDS operations of a wave complete in
// program order; the fence keeps the compiler from moving them across.
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// Slot of 16-byte chunk c of row `row` inside a wave's staging tile (rows of 2*S chunks).
// The LDS serves 16 lanes of a b128 access per clock, 256 bytes across all banks: 16 slots.
// A fragment read has 16 consecutive rows ask for the same chunk; with 128-byte rows (S = 4)
// two rows share a 256-byte span, so the XOR goes by row / 2: rows r and r + 1 sit in the two
// halves of a span, and the eight row pairs of a pass land on eight different slots of their
// half.  (XOR by row % 8 had rows r and r + 8 collide: measured 137 against 255 bytes per
// clock and CU for this read.)  The writes of a staged gather (8 lanes per row, 2 rows per
// pass) are conflict-free either way.
template <int S>
__device__ __forceinline__ int a_slot(int row, int c) {
  constexpr int C = 2 * S;
  if constexpr (C == 8) return row * C + (c ^ ((row >> 1) & 7));
  else return row * C + (c ^ ((row / (8 / C)) % C));
}

// --- forward weights straight from the caller's tensor (fp16) -----------------------
// The forward pass contracts over the ROWS of W[k] (W[k][cs][cd], cd contiguous) while an
// MFMA lane wants 8 consecutive cs of one cd.  Instead of re-laying the weights in a launch
// of their own, a stage's weight tile (2*S*8 rows cs x NT*32 columns cd) goes to LDS as it
// lies in memory, in 16-byte chunks, and the fragments come out through the transposing
// LDS read.  Chunk c of row `row` sits at chunk position c ^ raw_swizzle(row): the four
// consecutive rows one transposing read touches then cover all banks once.
template <int NT>
__device__ __forceinline__ int raw_swizzle(int row) {
  if constexpr (NT == 4) return (row & 3) << 2;          // 256-byte rows
  else if constexpr (NT == 2) return ((row >> 1) & 1) << 2;   // 128-byte rows
  else return 0;                                          // 64-byte rows
}

// B fragment of MFMA step s, 32-column tile nt: the 8 values W[(h*S + s)*8 + 0..7][nt*32 + lane%32].
template <int NT, int S>
__device__ __forceinline__ int4v raw_weight_frag(const int4v *__restrict__ w_lds, int s, int nt, int lane) {
  constexpr int RS = NT * 4;                              // chunks per row
  const int b = lane >> 4, i = lane & 15, h = lane >> 5;
  const int row = (h * S + s) * 8 + (i >> 2);
  const int chunk = nt * 4 + (b & 1) * 2 + ((i & 3) >> 1);
  const __half *base = reinterpret_cast<const __half *>(w_lds) +
                       ((size_t)row * RS + (chunk ^ raw_swizzle<NT>(row))) * 8 + (i & 1) * 4;
  typedef short short4v __attribute__((ext_vector_type(4)));
  typedef short short8v __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) short4v lds_v4;
  const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4 *)(base));
  const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4 *)(base + 4 * RS * 8));   // rows + 4: same swizzle
  const short8v v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(int4v, v);
}

// Writes a wave's accumulators.  Accumulator register r of lane l holds row
// (r / 4) * 8 + (l / 32) * 4 + r % 4 and column l % 32 of its 32x32 tile.  For
// fp16 two lanes swap one value each so that every lane owns two neighbouring
// columns of one row and can issue a packed 4-byte update.
template <typename T, int NT, bool ATOMIC, int MT>
__device__ __forceinline__ void write_tile(const float16v (&acc)[MT][NT], T *__restrict__ dst,
                                           const int *__restrict__ rows, int c_dst, int cd0,
                                           int lane) {
  const int h = lane / 32, col = lane % 32;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = rows[mt * 32 + (r / 4) * 8 + h * 4 + (r % 4)];
          if (row >= 0) {
            float *p = reinterpret_cast<float *>(dst) + (size_t)row * c_dst + cd0 + nt * 32 + col;
            if constexpr (ATOMIC) atomic_add(p, acc[mt][nt][r]);
            else *p += acc[mt][nt][r];
          }
        }
      } else {
        const bool odd = col & 1;
#pragma unroll
        for (int rp = 0; rp < 8; ++rp) {
          const float v0 = acc[mt][nt][2 * rp], v1 = acc[mt][nt][2 * rp + 1];
          const float got = swap_with_neighbour(odd ? v0 : v1);
          const float lo = odd ? got : v0, hi = odd ? v1 : got;
          const int r = 2 * rp + (odd ? 1 : 0);
          const int row = rows[mt * 32 + (r / 4) * 8 + h * 4 + (r % 4)];
          if (row >= 0) {
            __half *p = reinterpret_cast<__half *>(dst) + (size_t)row * c_dst + cd0 + nt * 32 + (col & ~1);
            if constexpr (ATOMIC) {
              atomic_add_pk(p, lo, hi);
            } else {
              __half2 *q = reinterpret_cast<__half2 *>(p);
              const float2 old = __half22float2(*q);
              *q = __floats2half2_rn(old.x + lo, old.y + hi);
            }
          }
        }
      }
    }
  }
}

// dst[rows[r]] += acc for the MT * 32 rows of a wave (rows[] in LDS, -1 = none; no
// atomics: the caller owns these rows).  All reads of the old values are issued
// before the first add so that they overlap.
template <typename T, int NT, int MT>
__device__ __forceinline__ void add_rows(const float16v (&acc)[MT][NT], T *__restrict__ dst,
                                         const int *__restrict__ rows, int c_dst, int cd0,
                                         int lane) {
  const int h = lane / 32, col = lane % 32;
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      int row[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) row[r] = rows[mt * 32 + (r / 4) * 8 + h * 4 + (r % 4)];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        float old[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
          old[r] = dst[(size_t)max(row[r], 0) * c_dst + cd0 + nt * 32 + col];
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (row[r] >= 0) dst[(size_t)row[r] * c_dst + cd0 + nt * 32 + col] = old[r] + acc[mt][nt][r];
      }
    }
  } else {
    const bool odd = col & 1;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      int row[8];
#pragma unroll
      for (int rp = 0; rp < 8; ++rp) {
        const int r = 2 * rp + (odd ? 1 : 0);
        row[rp] = rows[mt * 32 + (r / 4) * 8 + h * 4 + (r % 4)];
      }
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        __half2 old[8];
#pragma unroll
        for (int rp = 0; rp < 8; ++rp)
          old[rp] = *reinterpret_cast<const __half2 *>(
              reinterpret_cast<const __half *>(dst) + (size_t)max(row[rp], 0) * c_dst + cd0 +
              nt * 32 + (col & ~1));
#pragma unroll
        for (int rp = 0; rp < 8; ++rp) {
          const float v0 = acc[mt][nt][2 * rp], v1 = acc[mt][nt][2 * rp + 1];
          const float got = swap_with_neighbour(odd ? v0 : v1);
          const float lo = odd ? got : v0, hi = odd ? v1 : got;
          const float2 o = __half22float2(old[rp]);
          if (row[rp] >= 0)
            *reinterpret_cast<__half2 *>(reinterpret_cast<__half *>(dst) + (size_t)row[rp] * c_dst +
                                         cd0 + nt * 32 + (col & ~1)) =
                __floats2half2_rn(o.x + lo, o.y + hi);
        }
      }
    }
  }
}

// The same update with the tile transposed through the wave's own LDS staging
// region (free once the last MFMAs have read it): accumulators go to LDS as fp32,
// R rows at a time, and come back row-major, so every lane adds 4 consecutive
// columns of one row and a destination row is read and written as whole
// 64..256-byte runs by neighbouring lanes instead of 4 bytes per lane.
// stage: the wave's staging tile, MT * 32 rows of 2*S * 16 bytes.
template <typename T, int NT, int S, bool ATOMIC, int MT>
__device__ __forceinline__ void add_rows_lds(const float16v (&acc)[MT][NT], T *__restrict__ dst,
                                             const int *__restrict__ rows, float *__restrict__ stage,
                                             int c_dst, int cd0, int lane) {
  constexpr int COLS = NT * 32;
  constexpr int WR = MT * 32;             // the wave's rows
  constexpr int R = (WR * 2 * S * 16) / (COLS * 4) >= 32 ? 32 : (WR * 2 * S * 16) / (COLS * 4);
  if constexpr (R < 8) {
    if constexpr (ATOMIC) write_tile<T, NT, true>(acc, dst, rows, c_dst, cd0, lane);
    else add_rows<T, NT>(acc, dst, rows, c_dst, cd0, lane);
  } else {
    constexpr int CH = COLS / 4;            // 16-byte chunks per staged row
    constexpr int IT = R * CH / 64;         // chunks per lane and pass
    constexpr int PASSES = WR / R;
    const int h = lane / 32, col = lane % 32;
    // fp16 with up to 64 columns: the old values of ALL passes are fetched up front (the
    // registers of the gathered rows are free by now), so that the passes do not each wait
    // a memory round trip of their own (0.4 - 0.7 us of a launch)
    constexpr bool kAhead = !ATOMIC && sizeof(T) == 2 && NT <= 2;
    typedef _Float16 half4 __attribute__((ext_vector_type(4)));
    half4 ahead[kAhead ? PASSES : 1][kAhead ? IT : 1];
    if constexpr (kAhead) {
#pragma unroll
      for (int p = 0; p < PASSES; ++p)
#pragma unroll
        for (int it = 0; it < IT; ++it) {
          const int e = it * 64 + lane;
          ahead[p][it] = *reinterpret_cast<const half4 *>(
              reinterpret_cast<const _Float16 *>(dst) + (size_t)max(rows[p * R + e / CH], 0) * c_dst + cd0 +
              (e % CH) * 4);
        }
    }
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int mt = (p * R) / 32, g0 = ((p * R) % 32) / 8;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int g = 0; g < R / 8; ++g)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            stage[(g * 8 + h * 4 + j) * COLS + nt * 32 + col] = acc[mt][nt][(g0 + g) * 4 + j];
      wave_lds_fence();
      if constexpr (ATOMIC) {
        // Other workgroups add to the same rows.  An atomic instruction costs by the cache
        // lines it touches, so neighbouring lanes take neighbouring 4-byte words of a row:
        // one instruction covers 256 contiguous bytes.
        constexpr int WORDS = sizeof(T) == 4 ? COLS : COLS / 2;      // 4-byte words per row
#pragma unroll
        for (int q = 0; q < R * WORDS / 64; ++q) {
          const int e = q * 64 + lane;
          const int r = e / WORDS, c = e % WORDS;
          const int row = rows[p * R + r];
          if constexpr (sizeof(T) == 4) {
            const float v = stage[r * COLS + c];
            if (row >= 0) atomic_add(reinterpret_cast<float *>(dst) + (size_t)row * c_dst + cd0 + c, v);
          } else {
            const float2 v = *reinterpret_cast<const float2 *>(stage + r * COLS + 2 * c);
            if (row >= 0)
              atomic_add_pk(reinterpret_cast<__half *>(dst) + (size_t)row * c_dst + cd0 + 2 * c, v.x, v.y);
          }
        }
        wave_lds_fence();
        continue;
      }
      float4v part[IT];
      int row[IT];
#pragma unroll
      for (int it = 0; it < IT; ++it) {
        const int e = it * 64 + lane;
        part[it] = *reinterpret_cast<const float4v *>(stage + (e / CH) * COLS + (e % CH) * 4);
        row[it] = rows[p * R + e / CH];
      }
      if constexpr (sizeof(T) == 4) {
        float4v old[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it)
          old[it] = *reinterpret_cast<const float4v *>(
              reinterpret_cast<const float *>(dst) + (size_t)max(row[it], 0) * c_dst + cd0 +
              ((it * 64 + lane) % CH) * 4);
#pragma unroll
        for (int it = 0; it < IT; ++it)
          if (row[it] >= 0)
            *reinterpret_cast<float4v *>(reinterpret_cast<float *>(dst) + (size_t)row[it] * c_dst + cd0 +
                                         ((it * 64 + lane) % CH) * 4) = old[it] + part[it];
      } else {
        half4 old[IT];
#pragma unroll
        for (int it = 0; it < IT; ++it) {
          if constexpr (kAhead)
            old[it] = ahead[p][it];
          else
            old[it] = *reinterpret_cast<const half4 *>(
                reinterpret_cast<const _Float16 *>(dst) + (size_t)max(row[it], 0) * c_dst + cd0 +
                ((it * 64 + lane) % CH) * 4);
        }
#pragma unroll
        for (int it = 0; it < IT; ++it) {
          half4 out;
#pragma unroll
          for (int q = 0; q < 4; ++q) out[q] = (_Float16)((float)old[it][q] + part[it][q]);
          if (row[it] >= 0)
            *reinterpret_cast<half4 *>(reinterpret_cast<_Float16 *>(dst) + (size_t)row[it] * c_dst + cd0 +
                                       ((it * 64 + lane) % CH) * 4) = out;
        }
      }
      wave_lds_fence();
    }
  }
}

}  // namespace fgms
