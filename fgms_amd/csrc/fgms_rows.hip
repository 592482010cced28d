// Output-stationary gather-GEMM kernel with register-fed A operands ("rows16").
//
// A wave owns a block of 32 destination rows = two 16-row MFMA tiles and a
// column tile of 16 * NT columns; a workgroup is 8 such waves.  What differs
// from the LDS-staged gms_rows_kernel:
//
//  * v_mfma_f32_16x16x32_f16 / v_mfma_f32_16x16x4_f32: lane (row r = lane % 16,
//    quarter g = lane / 16) holds one 16-byte chunk of its row, so the four
//    lanes of a row read 64 contiguous bytes with one global_load_dwordx4 and
//    the gathered rows go straight into the A-operand registers: no LDS round
//    trip, no intra-wave fences, half the cache accesses of a 32-row layout
//    (where only two lanes share a row).
//  * Weights of a GROUP of offsets sit in LDS at a time, double-buffered and
//    filled by global_load_lds (memory -> LDS without touching VGPRs).  Inside a
//    group the waves do not synchronise: each walks only the offsets its own 32
//    rows use (a 64-bit mask per block from the plan), skips a 16-row tile whose
//    rows have no neighbour at that offset, and prefetches the rows of its next
//    (offset, slab) unit while the MFMAs of the current one run.  One barrier
//    per group instead of one per offset.
//  * Rows may be visited in a permuted order (perm) chosen by the plan.
#include <type_traits>

#include "fgms_device.h"
#include "fgms_internal.h"
#include "fgms_mma.h"

namespace fgms {
namespace {

constexpr int kWavesR = 8;
constexpr int kThreadsR = kWavesR * 64;

typedef float float4v_ __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ void mma16(float4v_ &acc, const int4v &a, const int4v &b) {
  if constexpr (sizeof(T) == 2) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a),
                                                 __builtin_bit_cast(half8, b), acc, 0, 0, 0);
  } else {
    const float4v_ fa = __builtin_bit_cast(float4v_, a), fb = __builtin_bit_cast(float4v_, b);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[0], fb[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[1], fb[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[2], fb[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[3], fb[3], acc, 0, 0, 0);
  }
}

// Weight re-layout for the 16-wide tiles.  packed[k][u][nt][lane][e]:
//   source channel cs = u * 4*E + (lane / 16) * E + e   (u = 64-byte step of the row)
//   dest   channel cd = nt * 16 + lane % 16
//   value = transpose ? W[k][cd][cs] : W[k][cs][cd]
template <typename T>
__global__ void pack_weights16_kernel(const T *__restrict__ w, T *__restrict__ packed, int k_vol,
                                      int c_in, int c_out, bool transpose) {
  constexpr int E = Elem<T>::per_chunk;
  const int c_src = transpose ? c_out : c_in;
  const int c_dst = transpose ? c_in : c_out;
  const size_t per_k = (size_t)c_src * c_dst;
  const size_t total = per_k * k_vol;
  const int nts = c_dst / 16;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (size_t)gridDim.x * blockDim.x) {
    const int k = (int)(i / per_k);
    size_t r = i % per_k;
    const int e = (int)(r % E); r /= E;
    const int lane = (int)(r % 64); r /= 64;
    const int nt = (int)(r % nts); r /= nts;
    const int u = (int)r;
    const int cs = u * 4 * E + (lane / 16) * E + e;
    const int cd = nt * 16 + lane % 16;
    const T *wk = w + (size_t)k * c_in * c_out;
    packed[i] = transpose ? wk[(size_t)cd * c_out + cs] : wk[(size_t)cs * c_out + cd];
  }
}

// NT: 16-column tiles per workgroup (2 or 4); US: 64-byte steps per unit (1 or 2).
template <typename T, int NT, int US>
__global__ __launch_bounds__(kThreadsR) void gms_rows16_kernel(
    const T *__restrict__ src, const T *__restrict__ packed, T *__restrict__ dst,
    const int32_t *__restrict__ nbr, const unsigned long long *__restrict__ mask32,
    const int32_t *__restrict__ perm, int n_rows, int k_vol, int c_src, int c_dst, int G) {
  constexpr int E = Elem<T>::per_chunk;
  extern __shared__ int4v lds[];
  const int steps = c_src / (4 * E);          // 64-byte steps per source row
  const int units = steps / US;
  const int nts = c_dst / 16;
  const int wk = steps * NT * 64;             // 16-byte chunks of one offset's weights (this column tile)
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int r = lane % 16, g4 = lane / 16;
  const int nt0 = blockIdx.y * NT;
  const int block = blockIdx.x * kWavesR + wave;
  const int my_row = block * 32 + (lane % 32);   // lanes 32..63 mirror lanes 0..31
  const unsigned long long mask = (block * 32 < n_rows) ? mask32[block] : 0ull;
  const int4v *packed4 = reinterpret_cast<const int4v *>(packed);
  const size_t packed_per_k = (size_t)c_src * c_dst / E;
  const int ngroups = (k_vol + G - 1) / G;

  auto dma_group = [&](int g, int buf) {
    const int k0 = g * G;
    const int nk = min(G, k_vol - k0);
    const int pieces = nk * steps * NT;       // 1 KiB each: 64 lanes x 16 bytes
    for (int p = wave; p < pieces; p += kWavesR) {
      const int kl = p / (steps * NT), rem = p % (steps * NT);
      const int u = rem / NT, nt = rem % NT;
      const int4v *gsrc = packed4 + packed_per_k * (k0 + kl) + ((size_t)u * nts + nt0 + nt) * 64 + lane;
      int4v *ldst = lds + (size_t)buf * G * wk + (size_t)(kl * steps * NT + rem) * 64;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(gsrc),
                                       (__attribute__((address_space(3))) void *)(ldst), 16, 0, 0);
    }
  };

  float4v_ acc[2][NT];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[m][nt] = float4v_{0.f, 0.f, 0.f, 0.f};

  auto pop = [](unsigned long long &m) {
    if (!m) return -1;
    const int k = __builtin_ctzll(m);
    m &= m - 1;
    return k;
  };
  auto load_idx = [&](int k) {
    return (k >= 0 && my_row < n_rows) ? nbr[(size_t)k * n_rows + my_row] : -1;
  };

  // load cursor: one (offset, unit) ahead of the MFMAs
  unsigned long long rem_load = mask;
  int k_load = pop(rem_load);
  int k_next = pop(rem_load);
  int idx_lane = load_idx(k_load);           // neighbour of row (lane % 32) at k_load
  int idx_next = load_idx(k_next);
  int unit_load = 0;
  int rowsel[2];                              // neighbour of this lane's row in tile m
  int4v a_n[2][US];
  int sel_n[2] = {-1, -1};
  int mt_n = 0;                               // which 16-row tiles of the unit in flight are live
  auto set_rows = [&]() {
    // lane (r, g4) works on rows r and 16 + r of the block
    rowsel[0] = __shfl(idx_lane, r);
    rowsel[1] = __shfl(idx_lane, 16 + r);
    const unsigned long long present = __ballot(idx_lane >= 0);
    mt_n = ((present & 0xffffull) ? 1 : 0) | ((present & 0xffff0000ull) ? 2 : 0);
  };
  auto issue_a = [&]() {
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      if (mt_n & (1 << m)) {
        const T *p = src + (size_t)max(rowsel[m], 0) * c_src + (size_t)(unit_load * US * 4 + g4) * E;
#pragma unroll
        for (int s = 0; s < US; ++s) a_n[m][s] = *reinterpret_cast<const int4v *>(p + s * 4 * E);
      }
      sel_n[m] = rowsel[m];
    }
  };
  if (k_load >= 0) {
    set_rows();
    issue_a();
  }

  dma_group(0, 0);
  for (int g = 0; g < ngroups; ++g) {
    __builtin_amdgcn_s_waitcnt(0);   // this wave's pieces of group g (and its prefetches) landed
    __syncthreads();                 // everyone's pieces landed; group g-1 is no longer read
    if (g + 1 < ngroups) dma_group(g + 1, (g + 1) & 1);
    const int4v *w_lds = lds + (size_t)(g & 1) * G * wk;
    unsigned long long gm = (mask >> (g * G)) & ((G >= 64) ? ~0ull : ((1ull << G) - 1));
    while (gm) {
      const int kl = __builtin_ctzll(gm);
      gm &= gm - 1;
      for (int unit = 0; unit < units; ++unit) {
        int4v a_c[2][US];
        const int mt_c = mt_n;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int s = 0; s < US; ++s) a_c[m][s] = sel_n[m] < 0 ? int4v{0, 0, 0, 0} : a_n[m][s];
        // advance the load cursor and put the next unit in flight
        if (++unit_load == units) {
          unit_load = 0;
          k_load = k_next;
          idx_lane = idx_next;
          k_next = pop(rem_load);
          idx_next = load_idx(k_next);
          if (k_load >= 0) set_rows();
        }
        if (k_load >= 0) issue_a();
#pragma unroll
        for (int s = 0; s < US; ++s) {
          int4v b[NT];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            b[nt] = w_lds[(size_t)((kl * steps + unit * US + s) * NT + nt) * 64 + lane];
#pragma unroll
          for (int m = 0; m < 2; ++m) {
            if (mt_c & (1 << m)) {
#pragma unroll
              for (int nt = 0; nt < NT; ++nt) mma16<T>(acc[m][nt], a_c[m][s], b[nt]);
            }
          }
        }
      }
    }
  }
  if (!mask) return;

  // dst[row] += acc : register i of lane l is row 4 * (l / 16) + i, column l % 16 of its tile
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      int drow[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int p = block * 32 + m * 16 + g4 * 4 + i;
        drow[i] = p < n_rows ? (perm ? perm[p] : p) : -1;
      }
      float old[NT][4];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          old[nt][i] = dst[(size_t)max(drow[i], 0) * c_dst + (nt0 + nt) * 16 + r];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (drow[i] >= 0)
            dst[(size_t)drow[i] * c_dst + (nt0 + nt) * 16 + r] = old[nt][i] + acc[m][nt][i];
    }
  } else {
    // two lanes swap one value each so that a lane owns two neighbouring columns of one row
    const bool odd = r & 1;
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      int drow[2];
#pragma unroll
      for (int ip = 0; ip < 2; ++ip) {
        const int p = block * 32 + m * 16 + g4 * 4 + 2 * ip + (odd ? 1 : 0);
        drow[ip] = p < n_rows ? (perm ? perm[p] : p) : -1;
      }
      __half2 old[NT][2];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int ip = 0; ip < 2; ++ip)
          old[nt][ip] = *reinterpret_cast<const __half2 *>(
              reinterpret_cast<const __half *>(dst) + (size_t)max(drow[ip], 0) * c_dst +
              (nt0 + nt) * 16 + (r & ~1));
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int ip = 0; ip < 2; ++ip) {
          const float v0 = acc[m][nt][2 * ip], v1 = acc[m][nt][2 * ip + 1];
          const float got = swap_with_neighbour(odd ? v0 : v1);
          const float lo = odd ? got : v0, hi = odd ? v1 : got;
          const float2 o = __half22float2(old[nt][ip]);
          if (drow[ip] >= 0)
            *reinterpret_cast<__half2 *>(reinterpret_cast<__half *>(dst) +
                                         (size_t)drow[ip] * c_dst + (nt0 + nt) * 16 + (r & ~1)) =
                __floats2half2_rn(o.x + lo, o.y + hi);
        }
    }
  }
}

struct Shape16 {
  int c_src, c_dst, NT, US, E, G;
  size_t lds_bytes;
  bool ok;
};

Shape16 shape16_of(const GmsArgs &a) {
  Shape16 s{};
  s.c_src = a.transpose_w ? a.c_out : a.c_in;
  s.c_dst = a.transpose_w ? a.c_in : a.c_out;
  s.E = a.dtype == FGMS_F16 ? 8 : 4;
  const size_t esz = a.dtype == FGMS_F16 ? 2 : 4;
  s.ok = false;
  if (s.c_dst % 32 != 0 || s.c_src % (4 * s.E) != 0) return s;
  if (reinterpret_cast<uintptr_t>(a.src) % 16 || reinterpret_cast<uintptr_t>(a.dst) % 4) return s;
  const int steps = s.c_src / (4 * s.E);
  s.US = steps % 2 == 0 ? 2 : 1;
  s.NT = (s.c_dst % 64 == 0) ? 4 : 2;
  size_t wk_bytes = (size_t)s.c_src * s.NT * 16 * esz;   // one offset, this column tile
  if (wk_bytes > 64 * 1024 && s.NT == 4) {
    s.NT = 2;
    wk_bytes /= 2;
  }
  if (wk_bytes > 64 * 1024) return s;
  const size_t per_buf = wk_bytes <= 32 * 1024 ? 32 * 1024 : 64 * 1024;
  s.G = (int)(per_buf / wk_bytes);
  if (s.G > a.k_vol) s.G = a.k_vol;
  if (s.G > 32) s.G = 32;
  s.lds_bytes = 2 * (size_t)s.G * wk_bytes;
  s.ok = true;
  return s;
}

template <typename T, int NT, int US>
int launch16(const GmsArgs &a, const Shape16 &s, const Plan *p) {
  void *ws = nullptr;
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  int rc = workspace_get(a.stream, 0, n * sizeof(T), &ws);
  if (rc != FGMS_OK) return rc;
  unsigned blocks = (unsigned)((n + 255) / 256);
  if (blocks > 4096) blocks = 4096;
  pack_weights16_kernel<T><<<blocks, 256, 0, a.stream>>>((const T *)a.w, (T *)ws, a.k_vol, a.c_in,
                                                         a.c_out, a.transpose_w);
  FGMS_HIP_TRY(hipGetLastError());
  const int32_t *nbr = a.transpose_w ? p->nbr_in : p->nbr_out;
  const unsigned long long *masks = a.transpose_w ? p->mask32_in : p->mask32_out;
  const int n_rows = (int)a.n_dst;
  const unsigned gx = (unsigned)((n_rows + 32 * kWavesR - 1) / (32 * kWavesR));
  if (gx == 0) return FGMS_OK;
  auto kern = gms_rows16_kernel<T, NT, US>;
  FGMS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)s.lds_bytes));
  {
    ProfileScope prof(a.transpose_w ? "gms_rows16_kernel(dgrad)" : "gms_rows16_kernel(fwd)", a.stream);
    kern<<<dim3(gx, (unsigned)(s.c_dst / (16 * NT))), kThreadsR, s.lds_bytes, a.stream>>>(
        (const T *)a.src, (const T *)ws, (T *)a.dst, nbr, masks, nullptr, n_rows, a.k_vol,
        s.c_src, s.c_dst, s.G);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

template <typename T>
int dispatch16(const GmsArgs &a, const Shape16 &s, const Plan *p) {
#define FGMS_R16(N, U) if (s.NT == N && s.US == U) return launch16<T, N, U>(a, s, p);
  FGMS_R16(4, 2) FGMS_R16(4, 1) FGMS_R16(2, 2) FGMS_R16(2, 1)
#undef FGMS_R16
  set_error("launch_rows2: unsupported shape");
  return FGMS_E_INVALID;
}

}  // namespace

bool rows2_supported(const GmsArgs &a, const Plan *p) {
  if (!p || a.dense_k >= 0 || a.k_vol > 64 || a.k_vol != p->k_vol) return false;
  if (a.transpose_w) {
    if (!p->dgrad_ok || a.n_dst != p->n_in || a.n_src != p->n_out) return false;
  } else {
    if (!p->fwd_ok || a.n_dst != p->n_out || a.n_src != p->n_in) return false;
  }
  return shape16_of(a).ok;
}

int launch_rows2(const GmsArgs &a, const Plan *p) {
  const Shape16 s = shape16_of(a);
  if (!s.ok || !rows2_supported(a, p)) {
    set_error("launch_rows2: unsupported shape or plan");
    return FGMS_E_INVALID;
  }
  if (a.dtype == FGMS_F16) return dispatch16<__half>(a, s, p);
  return dispatch16<float>(a, s, p);
}

}  // namespace fgms
