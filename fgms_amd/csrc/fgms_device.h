// Device-side helpers shared by the kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fgms_internal.h"

namespace fgms {

// Offset k is cut into ceil(n_k / rows) tiles; tiles are numbered offset by
// offset.  Finds the offset that owns tile t and the tile's pair range.  The
// reference does this with a bisection over the caller's 256-padded qkpos
// (backend/utils.cuh:6-27, backend/spconv.cuh:484-485); walking kpos instead
// makes the result independent of the padding quantum and skips empty offsets
// the same way.  t is wave-uniform, so the walk runs on the scalar unit.
__device__ __forceinline__ bool locate_tile(const int32_t *__restrict__ kpos, int k_vol,
                                            int rows, int t, int &k, int &first, int &count) {
  int lo = kpos[0];
  for (int i = 0; i < k_vol; ++i) {
    int hi = kpos[i + 1];
    int n = hi - lo;
    int nt = (n + rows - 1) / rows;
    if (t < nt) {
      k = i;
      first = lo + t * rows;
      count = min(rows, hi - first);
      return true;
    }
    t -= nt;
    lo = hi;
  }
  return false;
}

// Row gathers through a buffer resource: a row is addressed by a 32-bit BYTE offset into its
// tensor (row index x row bytes), and the buffer's range check turns every load at or beyond
// the tensor's size into zeros.  kAbsentRow is an offset no tensor reaches: a row that does not
// exist (no neighbour through this offset, a slot past the end of a pair list) is loaded from
// there and arrives as zeros, without a select and without touching memory.  Tensors must stay
// below kMaxBufferBytes (checked by the host), so that kAbsentRow plus any offset inside a row
// does not wrap round.
constexpr unsigned kAbsentRow = 0x80000000u;
constexpr size_t kMaxBufferBytes = 0x7fff0000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_resource(const void *base, unsigned bytes) {
  // raw buffer: stride 0, num_records in bytes, 32-bit data format
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(__half v) { return __half2float(v); }

__device__ __forceinline__ void atomic_add(float *addr, float v) {
  unsafeAtomicAdd(addr, v);
}

// Scalar fp16 accumulate at any 2-byte aligned address: compare-and-swap on the
// enclosing 32-bit word.
__device__ __forceinline__ void atomic_add(__half *addr, float v) {
  uintptr_t a = reinterpret_cast<uintptr_t>(addr);
  unsigned int *word = reinterpret_cast<unsigned int *>(a & ~uintptr_t(3));
  const bool hi = (a & 2) != 0;
  unsigned int old = *word, assumed;
  do {
    assumed = old;
    unsigned short h = hi ? (unsigned short)(assumed >> 16) : (unsigned short)(assumed & 0xffffu);
    float f = __half2float(__ushort_as_half(h)) + v;
    unsigned int nh = __half_as_ushort(__float2half(f));
    unsigned int nw = hi ? ((assumed & 0x0000ffffu) | (nh << 16)) : ((assumed & 0xffff0000u) | nh);
    old = atomicCAS(word, assumed, nw);
  } while (old != assumed);
}

// Packed fp16x2 accumulate (global_atomic_pk_add_f16); addr must be 4-byte aligned.
__device__ __forceinline__ void atomic_add_pk(__half *addr, float lo, float hi) {
  unsafeAtomicAdd(reinterpret_cast<__half2 *>(addr), __floats2half2_rn(lo, hi));
}

// Weight re-layout into per-lane MFMA fragment order.  packed[k][q][nt][lane][e],
// q = slab * S + s, E = elements per 16-byte chunk:
//   source channel  cs = slab * 2*S*E + (lane / 32) * S*E + s * E + e
//   dest   channel  cd = nt * 32 + lane % 32
//   value = transpose ? W[k][cd][cs] : W[k][cs][cd]
// Elements first, first + stride, ... of the packed array.
template <typename T>
__device__ __forceinline__ void pack_weight_elements(const T *__restrict__ w, T *__restrict__ packed,
                                                     int k_vol, int c_in, int c_out, int S,
                                                     bool transpose, size_t first, size_t stride) {
  constexpr int E = 16 / (int)sizeof(T);
  const int c_src = transpose ? c_out : c_in;
  const int c_dst = transpose ? c_in : c_out;
  const size_t per_k = (size_t)c_src * c_dst;
  const size_t total = per_k * k_vol;
  const int nts = c_dst / 32;
  for (size_t i = first; i < total; i += stride) {
    const int k = (int)(i / per_k);
    size_t r = i % per_k;
    const int e = (int)(r % E); r /= E;
    const int lane = (int)(r % 64); r /= 64;
    const int nt = (int)(r % nts); r /= nts;
    const int q = (int)r;
    const int slab = q / S, s = q % S;
    const int cs = slab * 2 * S * E + (lane / 32) * S * E + s * E + e;
    const int cd = nt * 32 + lane % 32;
    const T *wk = w + (size_t)k * c_in * c_out;
    packed[i] = transpose ? wk[(size_t)cd * c_out + cs] : wk[(size_t)cs * c_out + cd];
  }
}

// dst[i] += acc[i] rounded once to fp16, and acc[i] is reset: the accumulator is handed
// back all-zero, which is the state the next weight gradient expects to find it in.
__device__ __forceinline__ void add_and_clear_elements(__half *__restrict__ dst, float *__restrict__ acc,
                                                       size_t n, size_t first, size_t stride) {
  for (size_t i = first; i < n; i += stride) {
    dst[i] = __float2half(__half2float(dst[i]) + acc[i]);
    acc[i] = 0.f;
  }
}

// Fingerprint of the pair lists: the sum, over a fixed sample of positions (every `stride`-th
// pair) and over kpos, of a hash of (position, values).  Taken by the build (inside
// pair_masks_kernel's launch) and again by fgms_plan_check; sums of 64-bit hashes, so the order
// in which threads add does not matter.
__device__ __forceinline__ unsigned long long print_hash(unsigned long long a, unsigned b, unsigned c) {
  unsigned long long x = a * 0x9E3779B97F4A7C15ull + ((unsigned long long)b << 32 | c);
  x ^= x >> 31; x *= 0xBF58476D1CE4E5B9ull; x ^= x >> 29;
  return x;
}
constexpr int kPrintSamples = 4096;
__host__ __device__ inline int print_stride(int n_pairs) { return n_pairs > kPrintSamples ? n_pairs / kPrintSamples : 1; }

// The fingerprint of the lists as they are now, summed by one workgroup (the sample is 4 096
// pairs); valid in thread 0.
__device__ __forceinline__ unsigned long long plan_print_sum(const int32_t *__restrict__ kpos,
                                                             const int32_t *__restrict__ imap,
                                                             const int32_t *__restrict__ omap, int k_vol, int n_pairs) {
  __shared__ unsigned long long part[16];
  const int threads = blockDim.x;
  const int first = kpos[0], total = min(kpos[k_vol], n_pairs);
  const int stride = print_stride(total - first);
  unsigned long long v = 0;
  // (all of a thread's samples are requested before the first is hashed)
  constexpr int kMine = 16;
  for (int s0 = threadIdx.x; first + (long long)s0 * stride < total; s0 += threads * kMine) {
    int a[kMine], b[kMine];
#pragma unroll
    for (int u = 0; u < kMine; ++u) {
      const long long j = first + (long long)(s0 + u * threads) * stride;
      const int jj = (int)(j < total ? j : total - 1);
      a[u] = imap[jj];
      b[u] = omap[jj];
    }
#pragma unroll
    for (int u = 0; u < kMine; ++u) {
      const long long j = first + (long long)(s0 + u * threads) * stride;
      if (j < total) v += print_hash((unsigned long long)(j - first), (unsigned)a[u], (unsigned)b[u]);
    }
  }
  for (int rel = threadIdx.x; rel <= k_vol; rel += threads) v += print_hash(0x100000000ull + rel, (unsigned)kpos[rel], 0u);
  for (int d = 32; d > 0; d >>= 1) v += __shfl_xor(v, d);
  if (threadIdx.x % 64 == 0) part[threadIdx.x / 64] = v;
  __syncthreads();
  unsigned long long sum = 0;
  if (threadIdx.x == 0)
    for (int w = 0; w < threads / 64; ++w) sum += part[w];
  return sum;
}

// Build: the fingerprint goes into the plan's flags.
__device__ __forceinline__ void plan_print_block(const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
                                                 const int32_t *__restrict__ omap, int k_vol, int n_pairs,
                                                 int *__restrict__ flags) {
  const unsigned long long sum = plan_print_sum(kpos, imap, omap, k_vol, n_pairs);
  if (threadIdx.x == 0) *reinterpret_cast<unsigned long long *>(flags + kFlagPrint) = sum;
}

// fgms_plan_check: taken again and compared with the build's; a difference raises the sticky
// flag, in device memory and in the plan's pinned block.
__device__ __forceinline__ void plan_check_block(const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
                                                 const int32_t *__restrict__ omap, int k_vol, int n_pairs,
                                                 int *__restrict__ flags, int *__restrict__ host) {
  const unsigned long long sum = plan_print_sum(kpos, imap, omap, k_vol, n_pairs);
  if (threadIdx.x == 0 && sum != *reinterpret_cast<const unsigned long long *>(flags + kFlagPrint)) {
    flags[kFlagStale] = 1;
    if (host) host[kFlagStale] = 1;
  }
}

// The side job of a launch, run by workgroup `block` of its job.blocks workgroups.
__device__ __forceinline__ void run_side_job(const SideJob &job, int block) {
  const size_t first = (size_t)block * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)job.blocks * blockDim.x;
  if (job.kind == 1) {
    if (job.dtype == FGMS_F16)
      pack_weight_elements<__half>((const __half *)job.src, (__half *)job.dst, job.k_vol, job.c_in,
                                   job.c_out, job.S, job.transpose != 0, first, stride);
    else
      pack_weight_elements<float>((const float *)job.src, (float *)job.dst, job.k_vol, job.c_in,
                                  job.c_out, job.S, job.transpose != 0, first, stride);
  } else if (job.kind == 2) {
    add_and_clear_elements((__half *)job.dst, job.acc, job.n, first, stride);
  } else if (job.kind == 3) {
    if (block == 0)
      plan_check_block((const int32_t *)job.src, (const int32_t *)job.dst, job.omap, job.k_vol, (int)job.n,
                       job.flags, job.host);
  }
}

}  // namespace fgms
