// Shape-agnostic kernels: any channel counts, fp32 or fp16 storage, fp32 math
// on the vector ALUs.  They are the fallback for shapes the MFMA kernels do not
// take (odd / tiny channel counts) and the first correct implementation every
// faster kernel is tested against.  Counterparts in the reference: the
// "_1"/"_2" kernels (backend/spconv.cuh:16-235, 998-1216) for forward and dgrad
// and the "_1x"/"_2x" I_transpose kernels (backend/bwd_kernels.cuh:1119-1368).
#include "fgms_device.h"
#include "fgms_internal.h"

namespace fgms {
namespace {

constexpr int kRows = 32;    // pairs per workgroup tile
constexpr int kSlab = 32;    // contraction slab staged in LDS
constexpr int kCols = 64;    // destination channels per workgroup
constexpr int kThreads = 256;

template <typename T>
__global__ __launch_bounds__(kThreads) void generic_gms_kernel(
    const T *__restrict__ src, const T *__restrict__ w, T *__restrict__ dst,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ gmap,
    const int32_t *__restrict__ smap, int k_vol, int c_in, int c_out, bool transpose_w,
    int dense_k, int dense_rows) {
  __shared__ float As[kRows][kSlab + 1];
  __shared__ float Ws[kSlab][kCols + 1];
  __shared__ int grow[kRows];
  __shared__ int srow[kRows];

  const int c_src = transpose_w ? c_out : c_in;
  const int c_dst = transpose_w ? c_in : c_out;
  int k, first, count;
  if (dense_k >= 0) {
    k = dense_k;
    first = blockIdx.x * kRows;
    if (first >= dense_rows) return;
    count = min(kRows, dense_rows - first);
  } else if (!locate_tile(kpos, k_vol, kRows, blockIdx.x, k, first, count)) {
    return;
  }
  const int tid = threadIdx.x;
  if (tid < kRows) {
    const bool live = tid < count;
    grow[tid] = !live ? -1 : (gmap ? gmap[first + tid] : first + tid);
    srow[tid] = !live ? -1 : (smap ? smap[first + tid] : first + tid);
  }
  __syncthreads();

  const int cd0 = blockIdx.y * kCols;
  const int cd = tid % kCols;
  const int rg = tid / kCols;  // 4 groups of 8 rows
  const T *wk = w + (size_t)k * c_in * c_out;
  float acc[kRows / 4];
#pragma unroll
  for (int r = 0; r < kRows / 4; ++r) acc[r] = 0.f;

  for (int cs0 = 0; cs0 < c_src; cs0 += kSlab) {
    for (int e = tid; e < kRows * kSlab; e += kThreads) {
      const int r = e / kSlab, c = e % kSlab;
      const int g = grow[r];
      As[r][c] = (g >= 0 && cs0 + c < c_src) ? to_float(src[(size_t)g * c_src + cs0 + c]) : 0.f;
    }
    for (int e = tid; e < kSlab * kCols; e += kThreads) {
      const int s = e / kCols, d = e % kCols;
      float v = 0.f;
      if (cs0 + s < c_src && cd0 + d < c_dst) {
        // forward: W[k][cs][cd]; dgrad: W[k][cd][cs] read as its transpose
        v = transpose_w ? to_float(wk[(size_t)(cd0 + d) * c_out + cs0 + s])
                        : to_float(wk[(size_t)(cs0 + s) * c_out + cd0 + d]);
      }
      Ws[s][d] = v;
    }
    __syncthreads();
#pragma unroll 8
    for (int s = 0; s < kSlab; ++s) {
      const float wv = Ws[s][cd];
#pragma unroll
      for (int r = 0; r < kRows / 4; ++r) acc[r] += As[rg * (kRows / 4) + r][s] * wv;
    }
    __syncthreads();
  }
  if (cd0 + cd < c_dst) {
#pragma unroll
    for (int r = 0; r < kRows / 4; ++r) {
      const int s = srow[rg * (kRows / 4) + r];
      if (s >= 0) atomic_add(dst + (size_t)s * c_dst + cd0 + cd, acc[r]);
    }
  }
}

// dW[k][ci][co] += sum over a run of pairs of in[imap[j]][ci] * gout[omap[j]][co].
// One workgroup = up to kWgPairs pairs of one offset x one 32x32 tile of dW[k];
// partial sums go to an fp32 accumulation buffer with atomics.
constexpr int kWgPairs = 512;
constexpr int kStage = 64;
constexpr int kTile = 32;

template <typename T>
__global__ __launch_bounds__(kThreads) void generic_wgrad_kernel(
    const T *__restrict__ in, const T *__restrict__ gout, float *__restrict__ gw32,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
    const int32_t *__restrict__ omap, int k_vol, int c_in, int c_out) {
  __shared__ float As[kStage][kTile + 1];
  __shared__ float Bs[kStage][kTile + 1];
  int k, first, count;
  if (!locate_tile(kpos, k_vol, kWgPairs, blockIdx.x, k, first, count)) return;
  const int tiles_co = (c_out + kTile - 1) / kTile;
  const int ci0 = (blockIdx.y / tiles_co) * kTile;
  const int co0 = (blockIdx.y % tiles_co) * kTile;
  const int tid = threadIdx.x;
  const int ci = tid / 8;          // 0..31
  const int cq = (tid % 8) * 4;    // 4 consecutive co
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int p0 = 0; p0 < count; p0 += kStage) {
    for (int e = tid; e < kStage * kTile; e += kThreads) {
      const int p = e / kTile, c = e % kTile;
      float a = 0.f, b = 0.f;
      if (p0 + p < count) {
        const int j = first + p0 + p;
        if (ci0 + c < c_in) a = to_float(in[(size_t)imap[j] * c_in + ci0 + c]);
        if (co0 + c < c_out) b = to_float(gout[(size_t)omap[j] * c_out + co0 + c]);
      }
      As[p][c] = a;
      Bs[p][c] = b;
    }
    __syncthreads();
#pragma unroll 8
    for (int p = 0; p < kStage; ++p) {
      const float a = As[p][ci];
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[q] += a * Bs[p][cq + q];
    }
    __syncthreads();
  }
  if (ci0 + ci < c_in) {
    float *row = gw32 + ((size_t)k * c_in + ci0 + ci) * c_out + co0;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (co0 + cq + q < c_out) atomic_add(row + cq + q, acc[q]);
  }
}

// dst[i] += src32[i], rounding once to the storage type.
template <typename T>
__global__ void add_from_f32_kernel(T *__restrict__ dst, const float *__restrict__ src, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    if constexpr (sizeof(T) == 4) dst[i] += src[i];
    else dst[i] = __float2half(__half2float(dst[i]) + src[i]);
  }
}

__global__ void fill_zero_kernel(uint32_t *__restrict__ p, size_t words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < words; i += stride) p[i] = 0u;
}
__global__ void fill_zero_bytes_kernel(uint8_t *__restrict__ p, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

}  // namespace

int launch_fill_zero(void *ptr, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return FGMS_OK;
  uintptr_t a = reinterpret_cast<uintptr_t>(ptr);
  // head/tail bytes that are not word aligned (fp16 buffers with odd sizes)
  size_t head = (4 - (a & 3)) & 3;
  if (head > bytes) head = bytes;
  if (head) fill_zero_bytes_kernel<<<1, 64, 0, stream>>>((uint8_t *)ptr, head);
  size_t words = (bytes - head) / 4;
  if (words) {
    size_t blocks = (words + 256 * 4 - 1) / (256 * 4);
    if (blocks > 65535) blocks = 65535;
    fill_zero_kernel<<<(unsigned)blocks, 256, 0, stream>>>((uint32_t *)((uint8_t *)ptr + head), words);
  }
  size_t tail = bytes - head - words * 4;
  if (tail) fill_zero_bytes_kernel<<<1, 64, 0, stream>>>((uint8_t *)ptr + head + words * 4, tail);
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

int launch_generic_gms(const GmsArgs &a) {
  const int c_dst = a.transpose_w ? a.c_in : a.c_out;
  int64_t tiles;
  if (a.dense_k >= 0) tiles = (a.n_dense + kRows - 1) / kRows;
  else tiles = (a.n_pairs + kRows - 1) / kRows + a.k_vol;
  if (tiles <= 0) return FGMS_OK;
  dim3 grid((unsigned)tiles, (unsigned)((c_dst + kCols - 1) / kCols));
  ProfileScope prof(a.transpose_w ? "generic_gms_kernel(dgrad)" : "generic_gms_kernel(fwd)", a.stream);
  if (a.dtype == FGMS_F16) {
    generic_gms_kernel<__half><<<grid, kThreads, 0, a.stream>>>(
        (const __half *)a.src, (const __half *)a.w, (__half *)a.dst, a.kpos, a.gmap, a.smap,
        a.k_vol, a.c_in, a.c_out, a.transpose_w, a.dense_k, (int)a.n_dense);
  } else {
    generic_gms_kernel<float><<<grid, kThreads, 0, a.stream>>>(
        (const float *)a.src, (const float *)a.w, (float *)a.dst, a.kpos, a.gmap, a.smap,
        a.k_vol, a.c_in, a.c_out, a.transpose_w, a.dense_k, (int)a.n_dense);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

int launch_generic_wgrad(const WgradArgs &a) {
  if (a.n_pairs <= 0) return FGMS_OK;
  const size_t n = (size_t)a.k_vol * a.c_in * a.c_out;
  float *acc32 = nullptr;
  if (a.dtype == FGMS_F16) {
    // accumulate in fp32 and round once; fp16 atomics would round per chunk
    void *ws = nullptr;
    int rc = workspace_get(a.stream, 2, n * sizeof(float), &ws);
    if (rc != FGMS_OK) return rc;
    acc32 = (float *)ws;
    rc = launch_fill_zero(acc32, n * sizeof(float), a.stream);
    if (rc != FGMS_OK) return rc;
  } else {
    acc32 = (float *)a.gw;
  }
  const int64_t tiles = (a.n_pairs + kWgPairs - 1) / kWgPairs + a.k_vol;
  const int ty = ((a.c_in + kTile - 1) / kTile) * ((a.c_out + kTile - 1) / kTile);
  dim3 grid((unsigned)tiles, (unsigned)ty);
  if (a.dtype == FGMS_F16) {
    {
      ProfileScope prof("generic_wgrad_kernel", a.stream);
      generic_wgrad_kernel<__half><<<grid, kThreads, 0, a.stream>>>(
          (const __half *)a.in, (const __half *)a.gout, acc32, a.kpos, a.imap, a.omap, a.k_vol,
          a.c_in, a.c_out);
    }
    add_from_f32_kernel<__half><<<(unsigned)((n + 255) / 256), 256, 0, a.stream>>>(
        (__half *)a.gw, acc32, n);
  } else {
    ProfileScope prof("generic_wgrad_kernel", a.stream);
    generic_wgrad_kernel<float><<<grid, kThreads, 0, a.stream>>>(
        (const float *)a.in, (const float *)a.gout, acc32, a.kpos, a.imap, a.omap, a.k_vol,
        a.c_in, a.c_out);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

}  // namespace fgms
