// Device-side helpers shared by the kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

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

}  // namespace fgms
