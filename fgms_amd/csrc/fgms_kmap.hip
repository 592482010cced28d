// Kernel-map builder on the device: from voxel coordinates to the pair lists the
// convolution kernels consume.  The reference has no builder (its scripts load
// in_map / out_map / kernel_nnz / kernel_pos from files, cpu-check.py:89-94,
// spconv-test.py:64-73); this is the step right before the path.
//
// Pairs (i, o) with  in_coords[i] == out_coords[o] * stride + offsets[k],
// grouped by offset k, ascending o inside a group; when several input rows share
// a coordinate the smallest row index wins.  The result is a pure function of
// the inputs (no dependence on thread timing).
//
//   1. insert   every input coordinate, packed into 63 bits, goes into an open-
//               addressing hash table (linear probing, load <= 0.5); the slot
//               keeps the smallest row index (atomicMin)
//   2. lookup   one thread per (offset, output row): probe, write the hit (or
//               -1) into a [k_vol][n_out] table, count hits per 256-row block
//   3. scan     exclusive prefix sum over the (offset, block) counts (one workgroup)
//   4. write    hits are compacted in (offset, row) order: block base from the
//               scan, rank inside the block from wave ballots
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "fgms_device.h"
#include "fgms_internal.h"

namespace fgms {
namespace {

constexpr unsigned long long kEmptyKey = ~0ull;
constexpr int kCoordBits = 21;
constexpr long long kCoordBias = 1ll << (kCoordBits - 1);   // coordinates in [-2^20, 2^20)
constexpr int kBlock = 256;

// Exclusive prefix sum of n ints by one workgroup of 1024 threads, 4096 values a round: every
// thread takes four neighbouring values (the loads of a wave are contiguous), the waves scan
// their threads' sums with lane shuffles, the 16 wave totals go through LDS, and the sum of the
// rounds so far is carried in a register.  The counts are few (offsets x 256-row blocks: 21 k
// for 200 k voxels), so one workgroup is enough.
__global__ __launch_bounds__(1024) void kmap_scan_kernel(const int32_t *__restrict__ in, int32_t *__restrict__ out,
                                                         size_t n) {
  __shared__ int wave_totals[2][16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int carry = 0, round = 0;
  for (size_t base = 0; base < n; base += 4096, round ^= 1) {
    const size_t i = base + (size_t)tid * 4;
    int v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = i + j < n ? in[i + j] : 0;
    const int mine = v[0] + v[1] + v[2] + v[3];
    int incl = mine;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    if (lane == 63) wave_totals[round][wave] = incl;
    __syncthreads();      // the other buffer is written next round, after every wave has passed this barrier
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int t = wave_totals[round][w];
      before += w < wave ? t : 0;
      total += t;
    }
    int run = carry + before + incl - mine;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (i + j < n) out[i + j] = run;
      run += v[j];
    }
    carry += total;
  }
}

__device__ __forceinline__ bool pack_key(long long x, long long y, long long z, unsigned long long &key) {
  x += kCoordBias; y += kCoordBias; z += kCoordBias;
  if ((x | y | z) < 0 || ((x | y | z) >> kCoordBits) != 0) return false;
  key = ((unsigned long long)x << (2 * kCoordBits)) | ((unsigned long long)y << kCoordBits) |
        (unsigned long long)z;
  return true;
}

__device__ __forceinline__ unsigned long long mix(unsigned long long h) {   // splitmix64 finaliser
  h ^= h >> 30; h *= 0xbf58476d1ce4e5b9ull;
  h ^= h >> 27; h *= 0x94d049bb133111ebull;
  return h ^ (h >> 31);
}

__global__ void kmap_fill_kernel(unsigned long long *__restrict__ keys, int32_t *__restrict__ vals,
                                 size_t slots) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < slots) {
    keys[i] = kEmptyKey;
    vals[i] = INT32_MAX;
  }
}

__global__ void kmap_fill_none_kernel(int32_t *__restrict__ p, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = -1;
}

// flags[0]: an input coordinate is outside the packable range; flags[2]: two input rows share
// their coordinates
__global__ void kmap_insert_kernel(const int32_t *__restrict__ coords, int n,
                                   unsigned long long *__restrict__ keys, int32_t *__restrict__ vals,
                                   unsigned long long mask, int *__restrict__ flags) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  unsigned long long key;
  if (!pack_key(coords[3 * i], coords[3 * i + 1], coords[3 * i + 2], key)) {
    flags[0] = 1;
    return;
  }
  unsigned long long slot = mix(key) & mask;
  while (true) {                       // ends: load <= 0.5, a free or equal slot exists
    const unsigned long long prev = atomicCAS(&keys[slot], kEmptyKey, key);
    if (prev == kEmptyKey || prev == key) {
      if (prev == key) flags[2] = 1;
      atomicMin(&vals[slot], i);
      return;
    }
    slot = (slot + 1) & mask;
  }
}

// grid (blocks of 256 output rows, k_vol).  table[k][o] = input row or -1;
// counts[k * n_blocks + block] = hits of the block.
// mirror_k > 0 (= k_vol, odd): the map is its own mirror image -- one coordinate list on
// both sides, unique coordinates, offsets[k_vol - 1 - k] = -offsets[k] -- so a hit (k, o) -> i
// is also the hit (k_vol - 1 - k, i) -> o.  The grid then covers the offsets up to the centre
// only and fills the other half of the table (pre-filled with -1) from its hits: half the
// hash lookups.  kmap_count_kernel then counts that half's hits per block.
__global__ __launch_bounds__(kBlock) void kmap_lookup_kernel(
    const int32_t *__restrict__ out_coords, int n_out, const int32_t *__restrict__ offsets,
    int stride, int skip_offset, const unsigned long long *__restrict__ keys,
    const int32_t *__restrict__ vals, unsigned long long mask, int32_t *__restrict__ table,
    int32_t *__restrict__ counts, int mirror_k) {
  __shared__ int block_hits;
  const int k = blockIdx.y, o = blockIdx.x * kBlock + threadIdx.x;
  if (threadIdx.x == 0) block_hits = 0;
  __syncthreads();
  int hit = -1;
  if (o < n_out && k != skip_offset) {
    unsigned long long key;
    if (pack_key((long long)out_coords[3 * o] * stride + offsets[3 * k],
                 (long long)out_coords[3 * o + 1] * stride + offsets[3 * k + 1],
                 (long long)out_coords[3 * o + 2] * stride + offsets[3 * k + 2], key)) {
      unsigned long long slot = mix(key) & mask;
      while (true) {
        const unsigned long long at = keys[slot];
        if (at == key) { hit = vals[slot]; break; }
        if (at == kEmptyKey) break;
        slot = (slot + 1) & mask;
      }
    }
  }
  if (o < n_out) table[(size_t)k * n_out + o] = hit;
  if (mirror_k > 0 && hit >= 0 && 2 * k + 1 < mirror_k) {
    const int km = mirror_k - 1 - k;
    table[(size_t)km * n_out + hit] = o;      // (counted by kmap_count_kernel afterwards)
  }
  const unsigned long long b = __ballot(hit >= 0);
  if (threadIdx.x % 64 == 0 && b) atomicAdd(&block_hits, __builtin_popcountll(b));
  __syncthreads();
  if (threadIdx.x == 0) counts[(size_t)k * gridDim.x + blockIdx.x] = block_hits;
}

// grid (blocks of 256 output rows, offsets from k_first on): counts[k * n_blocks + block] =
// entries >= 0 of the block.
__global__ __launch_bounds__(kBlock) void kmap_count_kernel(const int32_t *__restrict__ table, int n_out,
                                                            int k_first, int32_t *__restrict__ counts) {
  __shared__ int block_hits;
  const int k = k_first + blockIdx.y, o = blockIdx.x * kBlock + threadIdx.x;
  if (threadIdx.x == 0) block_hits = 0;
  __syncthreads();
  const bool hit = o < n_out && table[(size_t)k * n_out + o] >= 0;
  const unsigned long long b = __ballot(hit);
  if (threadIdx.x % 64 == 0 && b) atomicAdd(&block_hits, __builtin_popcountll(b));
  __syncthreads();
  if (threadIdx.x == 0) counts[(size_t)k * gridDim.x + blockIdx.x] = block_hits;
}

__global__ __launch_bounds__(kBlock) void kmap_write_kernel(
    const int32_t *__restrict__ table, int n_out, const int32_t *__restrict__ bases,
    int32_t *__restrict__ in_map, int32_t *__restrict__ out_map, long long capacity) {
  __shared__ int wave_hits[kBlock / 64];
  const int k = blockIdx.y, o = blockIdx.x * kBlock + threadIdx.x;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int hit = o < n_out ? table[(size_t)k * n_out + o] : -1;
  const unsigned long long b = __ballot(hit >= 0);
  if (lane == 0) wave_hits[wave] = __builtin_popcountll(b);
  __syncthreads();
  if (hit < 0) return;
  long long pos = bases[(size_t)k * gridDim.x + blockIdx.x];
  for (int w = 0; w < wave; ++w) pos += wave_hits[w];
  pos += __builtin_popcountll(b & ((1ull << lane) - 1));
  if (pos < capacity) {
    in_map[pos] = hit;
    out_map[pos] = o;
  }
}

// kpos[k] = first pair of offset k, kernel_nnz[k] = its size; total -> result[0]
__global__ void kmap_finish_kernel(const int32_t *__restrict__ bases, int k_vol, int n_blocks,
                                   int32_t *__restrict__ kernel_nnz, int32_t *__restrict__ kpos,
                                   int32_t *__restrict__ result) {
  const int k = blockIdx.x * blockDim.x + threadIdx.x;
  if (k > k_vol) return;
  const int here = bases[(size_t)k * n_blocks];        // bases has k_vol * n_blocks + 1 entries
  kpos[k] = here;
  if (k < k_vol) kernel_nnz[k] = bases[(size_t)(k + 1) * n_blocks] - here;
  if (k == k_vol) result[0] = here;
}

}  // namespace

namespace {
int build_kernel_map_impl(const int32_t *in_coords, int64_t n_in, const int32_t *out_coords, int64_t n_out,
                          const int32_t *offsets_host, int k_vol, int stride, int skip_offset,
                          int32_t *in_map, int32_t *out_map, int64_t capacity, int32_t *kernel_nnz,
                          int32_t *kpos, int64_t *n_pairs, hipStream_t s, bool allow_mirror, bool *retry) {
  *retry = false;
  // A submanifold map (one coordinate list on both sides, symmetric offsets) is its own
  // mirror image: half of the lookups give the other half (see kmap_lookup_kernel).
  // FGMS_KMAP_MIRROR=0 looks every offset up.
  static const bool mirror_on = !(getenv("FGMS_KMAP_MIRROR") && atoi(getenv("FGMS_KMAP_MIRROR")) == 0);
  bool mirror = allow_mirror && mirror_on && in_coords == out_coords && n_in == n_out && stride == 1 &&
                k_vol >= 3 && k_vol % 2 == 1 && (skip_offset < 0 || skip_offset == k_vol / 2);
  for (int k = 0; mirror && k < k_vol; ++k)
    for (int c = 0; c < 3; ++c)
      if (offsets_host[3 * (k_vol - 1 - k) + c] != -offsets_host[3 * k + c]) mirror = false;
  size_t slots = 64;
  while (slots < 2 * (size_t)n_in) slots <<= 1;
  const int n_blocks = (int)((n_out + kBlock - 1) / kBlock);
  const size_t n_counts = (size_t)k_vol * n_blocks + 1;     // + one zero, so the scan ends with the total

  std::vector<void *> tmp;
  bool synced = false;      // true once the stream has drained
  auto release = [&]() { for (void *q : tmp) pool_free(q, s, synced); tmp.clear(); };
  auto alloc = [&](size_t bytes) -> void * {
    void *q = nullptr;
    if (pool_alloc(&q, bytes, s) != FGMS_OK) return nullptr;
    tmp.push_back(q);
    return q;
  };
  auto *keys = (unsigned long long *)alloc(slots * sizeof(unsigned long long));
  auto *vals = (int32_t *)alloc(slots * sizeof(int32_t));
  auto *table = (int32_t *)alloc((size_t)k_vol * (n_out ? n_out : 1) * sizeof(int32_t));
  auto *counts = (int32_t *)alloc(n_counts * sizeof(int32_t));
  auto *bases = (int32_t *)alloc(n_counts * sizeof(int32_t));
  auto *offs = (int32_t *)alloc((size_t)k_vol * 3 * sizeof(int32_t));
  auto *flags = (int32_t *)alloc(4 * sizeof(int32_t));      // [0] bad coordinate, [1] total
  const bool ok = keys && vals && table && counts && bases && offs && flags;
  if (!ok) {
    release();
    set_error("fgms_build_kernel_map: temporary allocation failed");
    return FGMS_E_NOMEM;
  }
  const unsigned long long mask = slots - 1;
  int rc = FGMS_OK;
  auto fail = [&](const char *what) {
    synced = hipStreamSynchronize(s) == hipSuccess;
    release();
    set_error("fgms_build_kernel_map: %s", what);
    return FGMS_E_HIP;
  };
  if (hipMemcpyAsync(offs, offsets_host, (size_t)k_vol * 3 * sizeof(int32_t), hipMemcpyHostToDevice, s) != hipSuccess)
    return fail("copying the offsets failed");
  if ((rc = launch_fill_zero(flags, 4 * sizeof(int32_t), s)) || (rc = launch_fill_zero(counts, n_counts * sizeof(int32_t), s))) {
    synced = hipStreamSynchronize(s) == hipSuccess;
    release();
    return rc;
  }
  kmap_fill_kernel<<<(unsigned)((slots + 255) / 256), 256, 0, s>>>(keys, vals, slots);
  if (n_in > 0) {
    ProfileScope prof("kmap_insert_kernel", s);
    kmap_insert_kernel<<<(unsigned)((n_in + 255) / 256), 256, 0, s>>>(in_coords, (int)n_in, keys, vals, mask, flags);
  }
  if (n_out > 0) {
    {
      ProfileScope prof("kmap_lookup_kernel", s);
      if (mirror) {
        const size_t half = (size_t)(k_vol / 2) * n_out;     // the offsets after the centre
        size_t blocks = (half + 1023) / 1024;
        kmap_fill_none_kernel<<<(unsigned)(blocks > 65535 ? 65535 : blocks), 256, 0, s>>>(
            table + (size_t)(k_vol / 2 + 1) * n_out, half);
      }
      kmap_lookup_kernel<<<dim3((unsigned)n_blocks, (unsigned)(mirror ? k_vol / 2 + 1 : k_vol)), kBlock, 0, s>>>(
          out_coords, (int)n_out, offs, stride, skip_offset, keys, vals, mask, table, counts, mirror ? k_vol : 0);
      if (mirror)
        kmap_count_kernel<<<dim3((unsigned)n_blocks, (unsigned)(k_vol / 2)), kBlock, 0, s>>>(table, (int)n_out,
                                                                                            k_vol / 2 + 1, counts);
    }
  }
  kmap_scan_kernel<<<1, 1024, 0, s>>>(counts, bases, n_counts);
  if (n_out > 0) {
    ProfileScope prof("kmap_write_kernel", s);
    kmap_write_kernel<<<dim3((unsigned)n_blocks, (unsigned)k_vol), kBlock, 0, s>>>(
        table, (int)n_out, bases, in_map, out_map, (long long)capacity);
  }
  kmap_finish_kernel<<<(unsigned)((k_vol + 1 + 255) / 256), 256, 0, s>>>(bases, k_vol, n_blocks, kernel_nnz, kpos, flags + 1);
  if (hipGetLastError() != hipSuccess) return fail("kernel launch failed");
  int32_t h[3] = {0, 0, 0};
  if (hipMemcpyAsync(h, flags, sizeof(h), hipMemcpyDeviceToHost, s) != hipSuccess ||
      hipStreamSynchronize(s) != hipSuccess)
    return fail("reading the result size failed");
  synced = true;
  release();
  if (mirror && h[2] && !h[0]) {       // rows that share coordinates: every offset has to be looked up
    *retry = true;
    return FGMS_OK;
  }
  if (h[0]) {
    set_error("fgms_build_kernel_map: an input coordinate is outside [-2^20, 2^20)");
    return FGMS_E_INVALID;
  }
  *n_pairs = h[1];
  if (h[1] > capacity) {
    set_error("fgms_build_kernel_map: %d pairs do not fit the capacity of %lld", h[1], (long long)capacity);
    return FGMS_E_INVALID;
  }
  return FGMS_OK;
}
}  // namespace

int build_kernel_map(const int32_t *in_coords, int64_t n_in, const int32_t *out_coords, int64_t n_out,
                     const int32_t *offsets_host, int k_vol, int stride, int skip_offset,
                     int32_t *in_map, int32_t *out_map, int64_t capacity, int32_t *kernel_nnz,
                     int32_t *kpos, int64_t *n_pairs, hipStream_t s) {
  bool retry = false;
  int rc = build_kernel_map_impl(in_coords, n_in, out_coords, n_out, offsets_host, k_vol, stride, skip_offset,
                                 in_map, out_map, capacity, kernel_nnz, kpos, n_pairs, s, true, &retry);
  if (rc == FGMS_OK && retry)
    rc = build_kernel_map_impl(in_coords, n_in, out_coords, n_out, offsets_host, k_vol, stride, skip_offset,
                               in_map, out_map, capacity, kernel_nnz, kpos, n_pairs, s, false, &retry);
  return rc;
}

}  // namespace fgms
