// Skinny-channel gather-GEMM kernel (no MFMA): layers whose narrow side is at
// most 16 channels, e.g. the 4 -> 32 first layer of a voxel network.  Such a
// layer moves ~10x more bytes than it has flops for the matrix cores to matter
// (a 4-channel fp16 row is 8 bytes), so the kernel is organised around memory:
//
//   * output-stationary through the plan's neighbour table: one LANE owns one
//     destination row and keeps its whole output row in registers, so the
//     destination is read and written exactly once, 16 bytes at a time, and
//     there are no atomics;
//   * the neighbour indices of the 64 rows of a wave are one coalesced 256-byte
//     line per offset; the gathered source rows are 8..64-byte vector loads;
//   * the weights of an offset (c_src * c_dst <= 512 values) have one address for
//     the whole wave and arrive through the scalar data path into scalar registers:
//     no LDS, no barrier, one multiply-add instruction per product; offsets that no
//     row of the wave uses are skipped with the plan's 64-row block mask.
//
// The reference handles these shapes with its "_once" kernels
// (backend/spconv.cuh:569-665, 899-992), pair-stationary with scalar atomics.
#include <stdlib.h>

#include "fgms_device.h"
#include "fgms_internal.h"

namespace fgms {
namespace {

constexpr int kSmallThreads = 256;
constexpr int kSmallMaxWeights = 13824;   // values over all offsets: they stay cache-resident

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// N elements starting at p (aligned to min(16, N * sizeof(T)) bytes), widened to fp32.
template <typename T, int N>
__device__ __forceinline__ void load_row(float (&x)[N], const T *__restrict__ p) {
  constexpr int bytes = N * (int)sizeof(T);
  if constexpr (sizeof(T) == 4) {
    if constexpr (bytes % 16 == 0) {
#pragma unroll
      for (int i = 0; i < N / 4; ++i) {
        const f32x4 v = reinterpret_cast<const f32x4 *>(p)[i];
        x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int i = 0; i < N / 2; ++i) {
        const f32x2 v = reinterpret_cast<const f32x2 *>(p)[i];
        x[2 * i] = v.x; x[2 * i + 1] = v.y;
      }
    }
  } else {
    if constexpr (bytes % 16 == 0) {
#pragma unroll
      for (int i = 0; i < N / 8; ++i) {
        const f16x8 v = reinterpret_cast<const f16x8 *>(p)[i];
        x[8 * i] = (float)v.s0; x[8 * i + 1] = (float)v.s1; x[8 * i + 2] = (float)v.s2;
        x[8 * i + 3] = (float)v.s3; x[8 * i + 4] = (float)v.s4; x[8 * i + 5] = (float)v.s5;
        x[8 * i + 6] = (float)v.s6; x[8 * i + 7] = (float)v.s7;
      }
    } else {
#pragma unroll
      for (int i = 0; i < N / 4; ++i) {
        const f16x4 v = reinterpret_cast<const f16x4 *>(p)[i];
        x[4 * i] = (float)v.x; x[4 * i + 1] = (float)v.y; x[4 * i + 2] = (float)v.z;
        x[4 * i + 3] = (float)v.w;
      }
    }
  }
}

template <typename T, int N>
__device__ __forceinline__ void add_store_row(T *__restrict__ p, const float (&acc)[N]) {
  float old[N];
  load_row<T, N>(old, p);
  if constexpr (sizeof(T) == 2) {
    __half2 *q = reinterpret_cast<__half2 *>(p);
#pragma unroll
    for (int i = 0; i < N / 2; ++i) q[i] = __floats2half2_rn(old[2 * i] + acc[2 * i], old[2 * i + 1] + acc[2 * i + 1]);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) p[i] = old[i] + acc[i];
  }
}

// One weight of offset k as fp32, from the 32-bit words `wk` of that offset's matrix.  The
// address is the same for every lane, so the words arrive through the scalar data path.
template <typename T>
__device__ __forceinline__ float weight_at(const uint32_t *__restrict__ wk, int e) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(float, wk[e]);
  } else {
    const uint32_t word = wk[e >> 1];
    const unsigned short bits = (unsigned short)((e & 1) ? (word >> 16) : (word & 0xffffu));
    return (float)__builtin_bit_cast(_Float16, bits);
  }
}

// CS / CD: source / destination channels (compile time: the inner loops unroll
// fully and the accumulators stay in registers).  TR: weights are used transposed.
//
// `parts` (1, 2 or 4) waves share one 64-row block: each takes every parts-th of the
// offsets the block uses and the partial rows meet in LDS before the one update of the
// result.  The kernel's duration is that of its longest wave (a block that uses all 27
// offsets), and a launch of a few thousand blocks leaves the wave slots to spare.
template <typename T, int CS, int CD, bool TR>
__global__ __launch_bounds__(kSmallThreads) void gms_small_kernel(
    const T *__restrict__ src, const uint32_t *__restrict__ w, T *__restrict__ dst,
    const int32_t *__restrict__ nbr, const unsigned long long *__restrict__ block_masks,
    const int32_t *__restrict__ perm, int n_dst, int parts) {
  extern __shared__ __align__(16) float partial[];   // [blocks per WG][parts - 1][CD][64]
  constexpr int kWordsPerOffset = CS * CD * (int)sizeof(T) / 4;
  // (the wave number is the same for the 64 lanes: say so, it steers the offset loop)
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int part = wave & (parts - 1), block_in_wg = wave / parts;
  const int block = blockIdx.x * (kSmallThreads / 64 / parts) + block_in_wg;
  const int row = block * 64 + lane;
  const bool live = row < n_dst;
  // the mask is the same for the 64 lanes: tell the compiler, so that the offset loop and
  // the weight addresses are scalar
  const unsigned long long mask_v = (size_t)block * 64 < (size_t)n_dst ? block_masks[block] : 0ull;
  const unsigned long long mask =
      ((unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)(mask_v >> 32)) << 32) |
      (unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)mask_v);
  // this wave's share: the set bits number part, part + parts, ...
  unsigned long long todo = mask;
  if (parts > 1) {
    todo = 0;
    int i = 0;
    for (unsigned long long m = mask; m; m &= m - 1, ++i)
      if ((i & (parts - 1)) == part) todo |= m & (0 - m);
  }
  float acc[CD];
#pragma unroll
  for (int i = 0; i < CD; ++i) acc[i] = 0.f;

  // Three-deep pipeline over the offsets: the neighbour index of offset t + 2 and the
  // source row of offset t + 1 are in flight while offset t is multiplied.  Every load is
  // unconditional (lanes without a row or a pair read row 0 and drop it): the counter
  // waits then know how many loads are outstanding and let them stay so.
  auto next_k = [&]() {
    if (!todo) return -1;
    const int k = __builtin_ctzll(todo);
    todo &= todo - 1;
    return k;
  };
  // lanes past the last row shadow it and skip the final store; an index asked for past
  // the last offset (k < 0) is read from offset 0 and never used
  const int row_c = live ? row : n_dst - 1;
  auto index_of = [&](int k) { return nbr[(size_t)(k < 0 ? 0 : k) * n_dst + row_c]; };
  auto gather = [&](float (&x)[CS], int g) { load_row<T, CS>(x, src + (size_t)(g < 0 ? 0 : g) * CS); };
  int k0 = next_k();
  if (k0 >= 0) {
    int k1 = next_k(), k2 = next_k();
    int g0 = index_of(k0), g1 = index_of(k1), g2 = index_of(k2);
    float x0[CS], x1[CS];
    gather(x0, g0);
    while (k0 >= 0) {
      gather(x1, g1);                                             // next offset's row
      const int k3 = next_k();
      const int g3 = index_of(k3);                                // index two offsets ahead
      const uint32_t *wk = w + (size_t)k0 * kWordsPerOffset;
      if (g0 >= 0) {                                              // rows without a pair here sit out
#pragma unroll
        for (int cs = 0; cs < CS; ++cs)
#pragma unroll
          for (int cd = 0; cd < CD; ++cd)
            acc[cd] += x0[cs] * weight_at<T>(wk, TR ? cd * CS + cs : cs * CD + cd);
      }
      k0 = k1; g0 = g1;
#pragma unroll
      for (int i = 0; i < CS; ++i) x0[i] = x1[i];
      k1 = k2; g1 = g2;
      k2 = k3; g2 = g3;
    }
  }
  if (parts > 1) {
    float *mine = partial + ((size_t)(block_in_wg * (parts - 1) + part - 1) * CD) * 64 + lane;
    if (part != 0) {
#pragma unroll
      for (int cd = 0; cd < CD; ++cd) mine[cd * 64] = acc[cd];
    }
    __syncthreads();
    if (part != 0) return;
    for (int p = 0; p < parts - 1; ++p) {
      const float *theirs = partial + ((size_t)(block_in_wg * (parts - 1) + p) * CD) * 64 + lane;
#pragma unroll
      for (int cd = 0; cd < CD; ++cd) acc[cd] += theirs[cd * 64];
    }
  }
  // `row` is a position in the plan's row order; a block no pair touches leaves its rows alone
  if (live && mask) add_store_row<T, CD>(dst + (size_t)(perm ? perm[row] : row) * CD, acc);
}

struct Small {
  int cs, cd;
  bool ok;
};

Small small_of(const GmsArgs &a) {
  Small s{};
  s.cs = a.transpose_w ? a.c_out : a.c_in;
  s.cd = a.transpose_w ? a.c_in : a.c_out;
  const size_t esz = a.dtype == FGMS_F16 ? 2 : 4;
  auto allowed = [](int c) { return c == 4 || c == 8 || c == 16 || c == 32 || c == 64; };
  s.ok = allowed(s.cs) && allowed(s.cd) && (s.cs <= 16 || s.cd <= 16) &&
         (size_t)s.cs * esz % 8 == 0 && (size_t)s.cd * esz % 8 == 0 &&
         (size_t)a.k_vol * s.cs * s.cd <= kSmallMaxWeights &&
         reinterpret_cast<uintptr_t>(a.src) % 16 == 0 && reinterpret_cast<uintptr_t>(a.dst) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(a.w) % 4 == 0;
  return s;
}

template <typename T, int CS, int CD>
int launch_small(const GmsArgs &a, const Plan *p) {
  const int32_t *nbr = a.transpose_w ? p->nbr_in : p->nbr_out;
  const unsigned long long *masks = a.transpose_w ? p->mask_in : p->mask_out;
  const int32_t *perm = a.transpose_w ? p->perm_in : p->perm_out;
  if (a.n_dst == 0) return FGMS_OK;
  // waves per 64-row block: four while the launch is a couple of rounds of the chip's wave
  // slots (200k rows: 23 us against 27 us with one wave per block), one when the rounds
  // are many and the longest wave no longer decides
  const size_t blocks = ((size_t)a.n_dst + 63) / 64;
  const size_t slots = (size_t)num_cus() * 4 * 7;
  int parts = blocks <= slots ? 4 : blocks <= 2 * slots ? 2 : 1;
  if (const char *e = getenv("FGMS_SMALL_PARTS")) {   // 1, 2 or 4: overrides the choice
    const int v = atoi(e);
    if (v == 1 || v == 2 || v == 4) parts = v;
  }
  const int blocks_per_wg = kSmallThreads / 64 / parts;
  const unsigned gx = (unsigned)((blocks + blocks_per_wg - 1) / blocks_per_wg);
  const size_t lds = parts > 1 ? (size_t)blocks_per_wg * (parts - 1) * CD * 64 * sizeof(float) : 0;
  {
    ProfileScope prof(a.transpose_w ? "gms_small_kernel(dgrad)" : "gms_small_kernel(fwd)", a.stream);
    if (a.transpose_w)
      gms_small_kernel<T, CS, CD, true><<<gx, kSmallThreads, lds, a.stream>>>(
          (const T *)a.src, (const uint32_t *)a.w, (T *)a.dst, nbr, masks, perm, (int)a.n_dst, parts);
    else
      gms_small_kernel<T, CS, CD, false><<<gx, kSmallThreads, lds, a.stream>>>(
          (const T *)a.src, (const uint32_t *)a.w, (T *)a.dst, nbr, masks, perm, (int)a.n_dst, parts);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

template <typename T>
int dispatch_small(const GmsArgs &a, const Small &s, const Plan *p) {
#define FGMS_SM(S, D) if (s.cs == S && s.cd == D) return launch_small<T, S, D>(a, p);
  FGMS_SM(4, 4) FGMS_SM(4, 8) FGMS_SM(4, 16) FGMS_SM(4, 32) FGMS_SM(4, 64)
  FGMS_SM(8, 4) FGMS_SM(8, 8) FGMS_SM(8, 16) FGMS_SM(8, 32) FGMS_SM(8, 64)
  FGMS_SM(16, 4) FGMS_SM(16, 8) FGMS_SM(16, 16) FGMS_SM(16, 32)
  FGMS_SM(32, 4) FGMS_SM(32, 8) FGMS_SM(32, 16)
  FGMS_SM(64, 4) FGMS_SM(64, 8)
#undef FGMS_SM
  set_error("launch_small_gms: unsupported shape");
  return FGMS_E_INVALID;
}

}  // namespace

bool small_gms_supported(const GmsArgs &a, const Plan *p) {
  if (!p || a.dense_k >= 0 || a.k_vol > 64 || a.k_vol != p->k_vol) return false;
  if (a.transpose_w) {
    if (!p->dgrad_ok || a.n_dst != p->n_in || a.n_src != p->n_out) return false;
  } else {
    if (!p->fwd_ok || a.n_dst != p->n_out || a.n_src != p->n_in) return false;
  }
  const Small s = small_of(a);
  if (!s.ok) return false;
  // shapes listed in dispatch_small
  if (s.cs == 16 && s.cd == 64) return false;
  if (s.cs == 64 && s.cd == 16) return false;
  return true;
}

int launch_small_gms(const GmsArgs &a, const Plan *p) {
  const Small s = small_of(a);
  if (!small_gms_supported(a, p)) {
    set_error("launch_small_gms: unsupported shape or plan");
    return FGMS_E_INVALID;
  }
  if (a.dtype == FGMS_F16) return dispatch_small<__half>(a, s, p);
  return dispatch_small<float>(a, s, p);
}

}  // namespace fgms
