// Kernel-map plan: neighbour tables built on the device from the pair lists.
// nbr_out[k][o] = the input row that reaches output row o through offset k
// (-1 if none); nbr_in[k][i] = the output row that input row i reaches through
// offset k.  Offset-major, so a wave reads the entries of its 64 consecutive
// rows for one offset as one 256-byte line.  The reference keeps only the pair lists and scatters with atomics
// (backend/spconv.cuh:457-563); the tables let a workgroup own a block of
// output rows and sum all offsets in registers.
#include <stdlib.h>
#include <string.h>

#include <map>
#include <mutex>
#include <vector>

#include "fgms_device.h"
#include "fgms_internal.h"

namespace fgms {
namespace {

// p[0 .. n) = v; p is 16-byte aligned (pool blocks are), 16 bytes per store.
__global__ void fill_i32_kernel(int32_t *__restrict__ p, size_t n, int32_t v) {
  typedef int int4v_ __attribute__((ext_vector_type(4)));
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t n4 = n / 4;
  for (size_t q = i; q < n4; q += stride) reinterpret_cast<int4v_ *>(p)[q] = int4v_{v, v, v, v};
  if (i < n % 4) p[n4 * 4 + i] = v;
}

// Two fills in one launch (the build is a chain of small launches, each bound by its latency).
__global__ void fill_two_kernel(int32_t *__restrict__ p1, size_t n1, int32_t v1, int32_t *__restrict__ p2, size_t n2,
                                int32_t v2) {
  typedef int int4v_ __attribute__((ext_vector_type(4)));
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)gridDim.x * blockDim.x;
  for (size_t q = i; q < n1 / 4; q += stride) reinterpret_cast<int4v_ *>(p1)[q] = int4v_{v1, v1, v1, v1};
  if (i < n1 % 4) p1[n1 / 4 * 4 + i] = v1;
  for (size_t q = i; q < n2 / 4; q += stride) reinterpret_cast<int4v_ *>(p2)[q] = int4v_{v2, v2, v2, v2};
  if (i < n2 % 4) p2[n2 / 4 * 4 + i] = v2;
}

// flags[0]: an index is out of range; flags[1]: two pairs of one offset share
// an output row; flags[2]: two pairs of one offset share an input row;
// flags[3]: inside some offset the pairs are not ordered by output row;
// flags[4], flags[5]: (64-position block, offset) combinations in use, output / input side;
// flags[6..9]: unused; flags[10], flags[11]: offset bits
// set over all row masks of the output / input side; flags[12]: pairs in the map.  Two pairs of
// one offset that share a row set one bit between them, so a side whose bits do not add up to
// the pair count has such a pair (what flags[1] / flags[2] used to say).
//
// Step 1 of a plan: per row the set of offsets it has a pair in (bit k of rmask), both
// sides at once, straight from the pair lists.  An offset bit that is already set when a
// pair wants to set it means two pairs of that offset share the row.
__global__ void pair_masks_kernel(const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
                                  const int32_t *__restrict__ omap, int k_vol, int n_pairs, int n_in,
                                  int n_out, unsigned long long *__restrict__ rmask_out,
                                  unsigned long long *__restrict__ rmask_in, int *__restrict__ flags) {
  const int total = kpos[k_vol];
  if (blockIdx.x == 0) {
    // the launch's first workgroup takes the fingerprint of the lists (fgms_plan_check re-takes
    // it); first, so that its chain of loads runs next to the others' work, not behind it
    plan_print_block(kpos, imap, omap, k_vol, n_pairs, flags);
    return;
  }
  const int j = kpos[0] + (blockIdx.x - 1) * blockDim.x + threadIdx.x;      // (kpos[0] > 0: a plan over a slice of the offsets)
  if (j >= total || j >= n_pairs) return;
  int lo = 0, hi = k_vol;          // offset of pair j: the last k with kpos[k] <= j
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (kpos[mid] <= j) lo = mid; else hi = mid;
  }
  const int k = lo;
  const int i = imap[j], o = omap[j];
  if (j == kpos[0]) flags[12] = min(total, n_pairs) - kpos[0];
  if (i < 0 || i >= n_in || o < 0 || o >= n_out) {
    flags[0] = 1;
    return;
  }
  if (j > kpos[k] && omap[j - 1] > o) flags[3] = 1;
  // the 32-bit half of the mask that holds bit k (little-endian words); the old value is not
  // asked for, so the atomics need no reply
  const unsigned bit = 1u << (k & 31);
  (void)__hip_atomic_fetch_or(reinterpret_cast<unsigned *>(rmask_out + o) + (k >> 5), bit, __ATOMIC_RELAXED,
                              __HIP_MEMORY_SCOPE_AGENT);
  (void)__hip_atomic_fetch_or(reinterpret_cast<unsigned *>(rmask_in + i) + (k >> 5), bit, __ATOMIC_RELAXED,
                              __HIP_MEMORY_SCOPE_AGENT);
}

// Step 2: the order in which a side's rows are visited.  Rows are sorted by their offset mask
// (as a number), so that the 64 rows of a wave use nearly the same offsets and whole (block,
// offset) steps can be skipped: on a surface-like cloud of 200 k voxels the number of such
// steps drops from 68.6 k to 37 k (33 k would be perfect).  Numerically close masks share their
// high offsets, which is what makes neighbours in the order similar; so the sort runs most
// significant bits first: a counting sort on the top kBinBits bits of the mask over the whole
// side (histogram per chunk of rows, scan, stable scatter), then a full sort by (mask, row) of
// every window of kWindow positions in LDS.  Inside a bin only rows of one window are ordered
// among themselves; measured on the benchmark clouds that costs 1 % more (block, offset) steps
// than the exact sort, for a third of its time.  Both sides of a plan go through the same
// launches (blockIdx.y = side).
constexpr int kBinBits = 11;
constexpr int kBins = 1 << kBinBits;
constexpr int kChunk = 2048;       // rows per workgroup of the histogram / scatter kernels
constexpr int kWindow = 2048;      // positions per workgroup of the window sort
constexpr int kSortThreads = 1024;

struct SortSide {
  const unsigned long long *rmask;
  int32_t *perm_tmp;     // order after the counting sort
  int32_t *perm;         // final order: position -> row
  int32_t *inv;          // row -> position
  int32_t *hist;         // [chunks][kBins] rows per (chunk, bin)
  int32_t *hist_before;  // [chunks][kBins] rows of the bin in earlier chunks
  int32_t *bin_start;    // [kBins] rows per bin
  int n, chunks;
};
struct SortArgs {
  SortSide side[2];
  int k_vol;
};

__device__ __forceinline__ int top_bits(unsigned long long m, int k_vol) {
  const int shift = k_vol > kBinBits ? k_vol - kBinBits : 0;
  return (int)((m >> shift) & (kBins - 1));
}

__global__ __launch_bounds__(kSortThreads) void sort_hist_kernel(SortArgs a) {
  const SortSide &sd = a.side[blockIdx.y];
  const int chunk = blockIdx.x;
  if (chunk >= sd.chunks) return;
  __shared__ int hist[kBins];
  for (int i = threadIdx.x; i < kBins; i += kSortThreads) hist[i] = 0;
  __syncthreads();
  for (int e = threadIdx.x; e < kChunk; e += kSortThreads) {
    const int row = chunk * kChunk + e;
    if (row < sd.n) atomicAdd(&hist[top_bits(sd.rmask[row], a.k_vol)], 1);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kBins; i += kSortThreads) sd.hist[(size_t)chunk * kBins + i] = hist[i];
}

// hist[chunk][bin] -> hist_before[chunk][bin] = rows of the bin in earlier chunks, and
// bin_total[bin].  Bins are independent: 256 of them per workgroup (one workgroup alone reads
// the 800 KB of counts at 30 GB/s).
constexpr int kScanBins = 256;
__global__ __launch_bounds__(kScanBins) void sort_scan_kernel(SortArgs a) {
  const SortSide &sd = a.side[blockIdx.y];
  if (sd.chunks == 0) return;
  const int bin = blockIdx.x * kScanBins + threadIdx.x;
  const int32_t *__restrict__ h = sd.hist + bin;
  int32_t *__restrict__ hb = sd.hist_before + bin;
  int run = 0, c = 0;
  for (; c + 8 <= sd.chunks; c += 8) {
    int v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = h[(size_t)(c + u) * kBins];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      hb[(size_t)(c + u) * kBins] = run;
      run += v[u];
    }
  }
  for (; c < sd.chunks; ++c) {
    hb[(size_t)c * kBins] = run;
    run += h[(size_t)c * kBins];
  }
  sd.bin_start[bin] = run;        // (the bin's total; the scatter kernel turns totals into starts)
}

// Bitonic sort of n2 (a power of two) (key, value) pairs in LDS, ascending, by the `threads`
// threads of the workgroup.  Wave w owns the elements [w * per, (w + 1) * per), per = n2 / waves:
// a phase whose partner distance j is below `per` stays inside the wave's own elements and needs
// no workgroup barrier (a wave's LDS operations complete in order), the few phases with larger
// j do.
template <typename K, typename V>
__device__ __forceinline__ void bitonic_sort(K *key, V *val, int n2, int threads) {
  const int waves = threads / 64, per = n2 / waves;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  bool wide = true;           // was the previous phase a workgroup-wide one (or the start)?
  for (int k2 = 2; k2 <= n2; k2 <<= 1)
    for (int j = k2 >> 1; j > 0; j >>= 1) {
      const bool local = j < per;
      if (local && wide) __syncthreads();        // the wave's elements as the others left them
      if (!local) __syncthreads();
      for (int c = lane; c < per / 2; c += 64) {
        // comparator c of this wave: elements i and i + j, i without bit j
        const int cc = wave * (per / 2) + c;
        const int i = 2 * cc - (cc & (j - 1));
        const int o = i + j;
        const bool asc = (i & k2) == 0;
        const K a = key[i], b = key[o];
        const V va = val[i], vb = val[o];
        const bool gt = a > b || (a == b && va > vb);
        if (gt == asc) {
          key[i] = b; key[o] = a;
          val[i] = vb; val[o] = va;
        }
      }
      if (local) {
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      wide = !local;
    }
  __syncthreads();
}

// Stable scatter of a chunk's rows into bin order.
__global__ __launch_bounds__(kSortThreads) void sort_scatter_kernel(SortArgs a) {
  const SortSide &sd = a.side[blockIdx.y];
  const int chunk = blockIdx.x;
  if (chunk >= sd.chunks) return;
  __shared__ int key[kChunk];          // bin of the element (kBins: padding)
  __shared__ int val[kChunk];          // its index inside the chunk
  __shared__ int start[kBins + 1];     // first sorted position of each bin inside the chunk
  for (int e = threadIdx.x; e < kChunk; e += kSortThreads) {
    const int row = chunk * kChunk + e;
    key[e] = row < sd.n ? top_bits(sd.rmask[row], a.k_vol) : kBins;
    val[e] = e;
  }
  __syncthreads();
  bitonic_sort(key, val, kChunk, kSortThreads);
  // rows in smaller bins: exclusive scan of the bin totals (2 per thread; thread, wave, workgroup)
  __shared__ int before_bin[kBins];
  __shared__ int part[kSortThreads / 64];
  {
    constexpr int kPer = kBins / kSortThreads;
    int mine[kPer], local = 0;
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
      mine[q] = sd.bin_start[threadIdx.x * kPer + q];
      local += mine[q];
    }
    int incl = local;
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if ((int)(threadIdx.x % 64) >= d) incl += up;
    }
    if (threadIdx.x % 64 == 63) part[threadIdx.x / 64] = incl;
    __syncthreads();
    int before = incl - local;
    for (int wv = 0; wv < (int)threadIdx.x / 64; ++wv) before += part[wv];
#pragma unroll
    for (int q = 0; q < kPer; ++q) {
      before_bin[threadIdx.x * kPer + q] = before;
      before += mine[q];
    }
  }
  for (int e = threadIdx.x; e < kChunk; e += kSortThreads)
    if (e == 0 || key[e - 1] != key[e]) start[key[e]] = e;
  __syncthreads();
  for (int e = threadIdx.x; e < kChunk; e += kSortThreads) {
    const int bin = key[e];
    if (bin < kBins)
      sd.perm_tmp[before_bin[bin] + sd.hist_before[(size_t)chunk * kBins + bin] + (e - start[bin])] =
          chunk * kChunk + val[e];
  }
}

// Full sort by (mask, row) of a window of positions; writes the final order and its inverse.
// perm_tmp == nullptr: the window starts from the identity order (sides of one window).
__global__ __launch_bounds__(kSortThreads) void sort_window_kernel(SortArgs a) {
  const SortSide &sd = a.side[blockIdx.y];
  const int p0 = blockIdx.x * kWindow;
  if (p0 >= sd.n) return;
  extern __shared__ unsigned long long win_key[];                    // [kWindow]
  int *win_val = reinterpret_cast<int *>(win_key + kWindow);        // [kWindow]
  for (int e = threadIdx.x; e < kWindow; e += kSortThreads) {
    const int p = p0 + e;
    const int row = p < sd.n ? (sd.perm_tmp ? sd.perm_tmp[p] : p) : INT32_MAX;
    win_val[e] = row;
    win_key[e] = p < sd.n ? sd.rmask[row] : ~0ull;
  }
  __syncthreads();
  bitonic_sort(win_key, win_val, kWindow, kSortThreads);
  for (int e = threadIdx.x; e < kWindow; e += kSortThreads) {
    const int p = p0 + e;
    if (p < sd.n) {
      sd.perm[p] = win_val[e];
      sd.inv[win_val[e]] = p;
    }
  }
}

// Step 3: the neighbour tables by POSITION, straight from the pair lists (tables pre-filled
// with -1): nbr_out[k][position of o] = i, nbr_in[k][position of i] = o.
__device__ __forceinline__ void tables_body(const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
                                            const int32_t *__restrict__ omap, int k_vol, int n_pairs, int n_in,
                                            int n_out, const int32_t *__restrict__ inv_out,
                                            const int32_t *__restrict__ inv_in, int32_t *__restrict__ nbr_out,
                                            int32_t *__restrict__ nbr_in, int block) {
  const int total = kpos[k_vol];
  const int j = kpos[0] + block * blockDim.x + threadIdx.x;
  if (j >= total || j >= n_pairs) return;
  int lo = 0, hi = k_vol;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (kpos[mid] <= j) lo = mid; else hi = mid;
  }
  const int i = imap[j], o = omap[j];
  if (i < 0 || i >= n_in || o < 0 || o >= n_out) return;
  nbr_out[(size_t)lo * n_out + (inv_out ? inv_out[o] : o)] = i;
  nbr_in[(size_t)lo * n_in + (inv_in ? inv_in[i] : i)] = o;
}

// Step 4: which offsets occur in every block of 64 positions (the OR of its rows' masks), and
// how many (block, offset) combinations that makes in total (flags[4 + side]).
struct MaskSide {
  const unsigned long long *rmask;
  const int32_t *perm;             // nullptr: identity
  unsigned long long *block_mask;
  int n;
};
struct MaskArgs {
  MaskSide side[2];
  int *flags;
};
__global__ __launch_bounds__(1024) void block_masks_kernel(MaskArgs a) {
  const MaskSide &sd = a.side[blockIdx.y];
  __shared__ int partial[16];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int block = blockIdx.x * 16 + wave;
  const int p = block * 64 + lane;
  __shared__ int partial_rows[16];
  int bits = 0, row_bits = 0;
  if (block * 64 < sd.n) {
    unsigned long long m = p < sd.n ? sd.rmask[sd.perm ? sd.perm[p] : p] : 0ull;
    row_bits = __popcll(m);
    for (int d = 32; d > 0; d >>= 1) {
      m |= __shfl_xor(m, d);
      row_bits += __shfl_xor(row_bits, d);
    }
    if (lane == 0) sd.block_mask[block] = m;
    bits = __popcll(m);
  }
  if (lane == 0) {
    partial[wave] = bits;
    partial_rows[wave] = row_bits;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int sum = 0, rows = 0;
    for (int i = 0; i < 16; ++i) {
      sum += partial[i];
      rows += partial_rows[i];
    }
    if (sum) atomicAdd(&a.flags[4 + blockIdx.y], sum);
    if (rows) atomicAdd(&a.flags[10 + blockIdx.y], rows);
  }
}

__global__ void tables_kernel(const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
                              const int32_t *__restrict__ omap, int k_vol, int n_pairs, int n_in, int n_out,
                              const int32_t *__restrict__ inv_out, const int32_t *__restrict__ inv_in,
                              int32_t *__restrict__ nbr_out, int32_t *__restrict__ nbr_in) {
  tables_body(kpos, imap, omap, k_vol, n_pairs, n_in, n_out, inv_out, inv_in, nbr_out, nbr_in, blockIdx.x);
}

// Pair view: the pair lists with every offset's run padded to a multiple of 64 rows
// (pv_in / pv_out pre-filled with -1, pv_mask with 0).  Pair j of offset k goes to row
// vpos[k] + j - kpos[k], vpos = the running sum of the padded run lengths.
__global__ void pair_view_kernel(const int32_t *__restrict__ kpos, const int32_t *__restrict__ imap,
                                 const int32_t *__restrict__ omap, int k_vol, int n_pairs,
                                 long long pv_rows, int32_t *__restrict__ pv_in,
                                 int32_t *__restrict__ pv_out,
                                 unsigned long long *__restrict__ pv_mask) {
  __shared__ int kp[65];
  __shared__ long long vp[65];
  if ((int)threadIdx.x <= k_vol) kp[threadIdx.x] = kpos[threadIdx.x];
  __syncthreads();
  if (threadIdx.x == 0) {
    long long v = 0;
    for (int k = 0; k < k_vol; ++k) {
      vp[k] = v;
      const int n = kp[k + 1] - kp[k];
      if (n > 0) v += (n + 63) / 64 * 64;
    }
    vp[k_vol] = v;
  }
  __syncthreads();
  const int j = kp[0] + blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= kp[k_vol] || j >= n_pairs) return;
  int lo = 0, hi = k_vol;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (kp[mid] <= j) lo = mid; else hi = mid;
  }
  const long long r = vp[lo] + (j - kp[lo]);
  if (j < kp[lo] || r < 0 || r >= pv_rows) return;     // (a kpos that does not ascend)
  pv_in[r] = imap[j];
  pv_out[r] = omap[j];
  if ((r & 63) == 0) pv_mask[r >> 6] = 1ull << lo;
}

// band_start[k][c] = number of pairs of offset k whose output row is below
// c * band_rows (a lower bound over the offset's pairs, which are ordered by
// output row when the result is used); c = band_count gives the offset's size.
__global__ void band_bounds_kernel(const int32_t *__restrict__ kpos, const int32_t *__restrict__ omap,
                                   int n_pairs, int band_count, int band_rows,
                                   int32_t *__restrict__ band_start) {
  const int k = blockIdx.x;
  const int first = min(max(kpos[k], 0), n_pairs);
  const int count = min(max(kpos[k + 1], first), n_pairs) - first;   // never reads past the map
  for (int c = threadIdx.x; c <= band_count; c += blockDim.x) {
    int lo = 0, hi = count;              // first pair with omap >= c * band_rows
    if (c == band_count) lo = count;
    const long long target = (long long)c * band_rows;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (omap[first + mid] < target) lo = mid + 1; else hi = mid;
    }
    band_start[k * (band_count + 1) + c] = lo;
  }
}

// Dispatch order of the 256-position tiles of the output-stationary kernel.
// Workgroup b runs on XCD b % 8 and, inside an XCD, workgroup number q = b / 8
// lands on CU q % cus_per_xcd (the dispatcher goes round the CUs).
//  * A tile's home XCD is the eighth of the cloud its middle row lies in
//    (original row numbers follow the voxel order, i.e. space), so that
//    neighbouring rows meet in one L2.
//  * Inside an XCD the tiles are ranked by the number of offsets they use, most
//    first: the launch lasts as long as its longest tile, so those must start
//    first.  Ranks are laid over the CUs in a snake (first sweep forwards, second
//    backwards, ...), so every CU gets a mix of long and short tiles instead of
//    three long ones competing for the same SIMDs.
//  * Every XCD takes at most cap = ceil(tiles / 8) tiles; the lightest tiles of an
//    overfull XCD go to the XCDs that have room.
// order[q * 8 + xcd] = tile | first offset << 24, -1 where no tile lands.  One workgroup; which of two
// equally heavy tiles comes first depends on timing, the results do not.
struct TileSide {
  const int32_t *perm;
  const unsigned long long *block_masks;
  int32_t *order;
  int n_rows, n_tiles, cap;
};
struct TileArgs {
  TileSide side[2];
  int cus_per_xcd;
  const int *flags;   // the build's findings and where they go on the host (this is the
  int *host;          // build's last launch); nullptr: published by a launch of its own
};
__global__ __launch_bounds__(1024) void tile_order_kernel(TileArgs ta) {
  const int32_t *__restrict__ perm = ta.side[blockIdx.x].perm;
  const unsigned long long *__restrict__ block_masks = ta.side[blockIdx.x].block_masks;
  int32_t *__restrict__ order = ta.side[blockIdx.x].order;
  const int n_rows = ta.side[blockIdx.x].n_rows, n_tiles = ta.side[blockIdx.x].n_tiles;
  const int cap = ta.side[blockIdx.x].cap, cus_per_xcd = ta.cus_per_xcd;
  if (blockIdx.x == 0 && ta.host && threadIdx.x < kPlanFlags) ta.host[threadIdx.x] = ta.flags[threadIdx.x];
  if (!order) return;
  constexpr int kPc = 65;                         // popcount classes 0..64
  __shared__ int hist[8][kPc];                    // tiles per (home, popcount), then start ranks
  __shared__ int cursor[8][kPc];
  __shared__ int total[8];
  __shared__ int spill_count;
  extern __shared__ int32_t spill[];              // [n_tiles]
  const int tid = threadIdx.x;
  const int n_blocks = (n_rows + 63) / 64;
  for (int i = tid; i < 8 * kPc; i += 1024) {
    (&hist[0][0])[i] = 0;
    (&cursor[0][0])[i] = 0;
  }
  if (tid == 0) spill_count = 0;
  for (int i = tid; i < cap * 8; i += 1024) order[i] = -1;     // (slots no tile lands in)
  __syncthreads();
  // entry of tile t in the table: t in the low 24 bits, the first offset the tile uses above
  // them (the kernel starts that offset's index load before it has seen the tile's masks)
  auto classify = [&](int t, int &home, int &pc, int &entry) {
    const int mid = min(t * 256 + 128, n_rows - 1);
    home = (int)((long long)(perm ? perm[mid] : mid) * 8 / n_rows);
    unsigned long long m = 0;
    for (int b = 4 * t; b < min(4 * t + 4, n_blocks); ++b) m |= block_masks[b];
    pc = __builtin_popcountll(m);
    entry = t | ((m ? __builtin_ctzll(m) : 0) << 24);
  };
  for (int t = tid; t < n_tiles; t += 1024) {
    int home, pc, entry;
    classify(t, home, pc, entry);
    atomicAdd(&hist[home][pc], 1);
  }
  __syncthreads();
  if (tid < 8) {                                  // start rank of each class, heaviest first
    int run = 0;
    for (int pc = kPc - 1; pc >= 0; --pc) {
      const int n = hist[tid][pc];
      hist[tid][pc] = run;
      run += n;
    }
    total[tid] = run;
  }
  __syncthreads();
  auto position = [&](int rank) {                 // snake over the CUs
    const int round = rank / cus_per_xcd, j = rank % cus_per_xcd;
    const int in_round = min(cus_per_xcd, cap - round * cus_per_xcd);
    return round * cus_per_xcd + ((round & 1) ? in_round - 1 - j : j);
  };
  for (int t = tid; t < n_tiles; t += 1024) {
    int home, pc, entry;
    classify(t, home, pc, entry);
    const int rank = hist[home][pc] + atomicAdd(&cursor[home][pc], 1);
    if (rank < cap) order[position(rank) * 8 + home] = entry;
    else spill[atomicAdd(&spill_count, 1)] = entry;
  }
  __syncthreads();
  for (int sidx = tid; sidx < spill_count; sidx += 1024) {
    int left = sidx;
    for (int q = 0; q < 8; ++q) {
      const int filled = min(total[q], cap), room = cap - filled;
      if (left < room) {
        order[position(filled + left) * 8 + q] = spill[sidx];
        break;
      }
      left -= room;
    }
  }
}

// Dispatch order of the weight gradient's (offset, band) cells, one table per group
// size g in {1, 2, 4, 8} (blockIdx.z): cells[q * 8 + xcd] is the q-th cell of XCD
// xcd, cell = offset * 65536 + band.  XCD x owns the bands x, x + 8, ...; they are
// taken g at a time (g bands x all offsets are in flight together, so g is chosen
// at launch such that their rows fit the XCD's L2), and inside a group the cells
// are ranked by pair count, most first (the longest workgroups start first), ties
// by cell number.  One thread per cell; a cell's rank is found by comparing with
// the other cells of its XCD (a few hundred).
__global__ void band_cells_kernel(const int32_t *__restrict__ band_start, int k_vol, int bands,
                                  int32_t *__restrict__ cells) {
  // the pair counts of the XCD's cells (and which of its bands a cell lies in) go to LDS
  // once: every thread compares with all of them, and the integer divisions of the cell
  // arithmetic would otherwise dominate the loop
  constexpr int kCached = 2048;
  __shared__ int count[kCached];
  __shared__ short band_of[kCached];
  const int per_xcd = (bands / 8) * k_vol;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;   // cell number inside its XCD: (band / 8) * k_vol + k
  const int x = blockIdx.y, shift = blockIdx.z;           // groups of 1 << shift bands
  auto pairs_of = [&](int cell) {
    const int k = cell % k_vol, band = (cell / k_vol) * 8 + x;
    return band_start[k * (bands + 1) + band + 1] - band_start[k * (bands + 1) + band];
  };
  for (int o = threadIdx.x; o < per_xcd && o < kCached; o += blockDim.x) {
    count[o] = pairs_of(o);
    band_of[o] = (short)(o / k_vol);
  }
  __syncthreads();
  if (c >= per_xcd) return;
  const int mine = pairs_of(c), my_group = (c / k_vol) >> shift;
  int rank = 0;
#pragma unroll 8      // (independent LDS reads in flight: the loop is bound by their latency)
  for (int o = 0; o < per_xcd; ++o) {
    const bool cached = o < kCached;
    const int theirs = cached ? count[o] : pairs_of(o);
    const int their_group = (cached ? (int)band_of[o] : o / k_vol) >> shift;
    const bool before = their_group != my_group ? their_group < my_group
                                                 : (theirs > mine || (theirs == mine && o < c));
    rank += before ? 1 : 0;
  }
  cells[(size_t)blockIdx.z * bands * k_vol + rank * 8 + x] = (c % k_vol) * 65536 + (c / k_vol) * 8 + x;
}

// The two directions of a plan (output side, input side) are chains of a dozen small
// launches each (masks, radix sort, permutation, block masks, tile order) that do not
// depend on each other; at 200 k rows every launch is bound by its latency, so the input
// side's chain runs on a stream of the library's own (default priority, one per device,
// created on first use) next to the caller's.  nullptr: creation failed, one stream is used.
hipStream_t side_stream(int device) {
  static std::mutex m;
  static std::map<int, hipStream_t> streams;
  std::lock_guard<std::mutex> lock(m);
  auto it = streams.find(device);
  if (it != streams.end()) return it->second;
  hipStream_t st = nullptr;
  if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess) st = nullptr;
  streams[device] = st;
  return st;
}

// Pinned blocks for the builds' flag read-backs (hipHostMalloc costs as much as the whole
// build; freed blocks are kept).
std::mutex g_pinned_mutex;
std::vector<int *> g_pinned_free;

int *pinned_flags_get() {
  {
    std::lock_guard<std::mutex> lock(g_pinned_mutex);
    if (!g_pinned_free.empty()) {
      int *q = g_pinned_free.back();
      g_pinned_free.pop_back();
      return q;
    }
  }
  int *q = nullptr;
  note_allocation();
  if (hipHostMalloc((void **)&q, kPlanFlags * sizeof(int), hipHostMallocDefault) != hipSuccess) return nullptr;
  return q;
}

void pinned_flags_put(int *q) {
  std::lock_guard<std::mutex> lock(g_pinned_mutex);
  g_pinned_free.push_back(q);
}

// fgms_plan_check: the fingerprint taken again from the lists as they are now (one workgroup:
// the sample is 4 096 pairs), compared with the build's; a difference raises the sticky flag,
// in device memory and in the plan's pinned block.
__global__ __launch_bounds__(1024) void plan_check_kernel(const int32_t *__restrict__ kpos,
                                                          const int32_t *__restrict__ imap,
                                                          const int32_t *__restrict__ omap, int k_vol, int n_pairs,
                                                          int *__restrict__ flags, int *__restrict__ host) {
  plan_check_block(kpos, imap, omap, k_vol, n_pairs, flags, host);
}

// The build's findings -> pinned host memory (mapped into the device's address space).
__global__ void publish_flags_kernel(const int *__restrict__ flags, int *__restrict__ host) {
  if (threadIdx.x < kPlanFlags) host[threadIdx.x] = flags[threadIdx.x];
}

int fill_i32(int32_t *p, size_t n, int32_t v, hipStream_t s) {
  if (n == 0) return FGMS_OK;
  if (reinterpret_cast<uintptr_t>(p) % 16) {
    set_error("fill_i32: unaligned block");
    return FGMS_E_INVALID;
  }
  size_t blocks = (n / 4 + 255) / 256;          // one 16-byte store per thread, a few for big blocks
  if (blocks > 8192) blocks = 8192;
  if (blocks == 0) blocks = 1;
  fill_i32_kernel<<<(unsigned)blocks, 256, 0, s>>>(p, n, v);
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

}  // namespace
}  // namespace fgms

using namespace fgms;

namespace fgms {

// Builds a plan.  Everything is queued on `stream` (the weight gradient's band tables and the
// table pre-fill on a stream of the library's own next to it); nothing waits for the GPU.  What
// the build finds out about the map (index out of range, rows shared inside an offset, pair
// order, block counts) travels to pinned host memory behind the last kernel and is read by
// plan_resolve when the plan is first used.
int plan_create(fgms_plan_t **plan_out, const int32_t *kpos, const int32_t *in_map,
                const int32_t *out_map, int64_t n_in, int64_t n_out, int k_vol, int64_t n_pairs, void *stream,
                bool want_bands) {
  if (!plan_out) {
    set_error("plan output pointer is null");
    return FGMS_E_INVALID;
  }
  *plan_out = nullptr;
  if (!kpos || k_vol <= 0 || n_in < 0 || n_out < 0 || n_pairs < 0 ||
      (n_pairs > 0 && (!in_map || !out_map)) || n_in > INT32_MAX || n_out > INT32_MAX ||
      n_pairs > INT32_MAX - 65536) {
    set_error("fgms_plan_create: bad argument");
    return FGMS_E_INVALID;
  }
  hipStream_t s = (hipStream_t)stream;
  {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (s && hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone) {
      set_error("fgms_plan_create: the stream is being captured (the build allocates; make the plan before)");
      return FGMS_E_INVALID;
    }
  }
  Plan *p = new Plan();          // (value-initialised: every field starts out zero)
  p->k_vol = k_vol; p->n_in = n_in; p->n_out = n_out; p->n_pairs = n_pairs;
  p->last_stream = s;
  p->create_stream = s;
  p->kpos = kpos; p->in_map = in_map; p->out_map = out_map;
  int rc = FGMS_OK;
  std::vector<void *> tmp;          // temporaries: handed back to the pool behind the last kernel
  hipStream_t side_in_use = nullptr;     // the library's own stream, once work of this build is queued on it
  auto fail = [&](int code) {
    // (blocks are handed back behind `s` alone: the side stream's work must have finished)
    if (side_in_use) (void)hipStreamSynchronize(side_in_use);
    for (void *q : tmp) pool_free(q, s, false);
    fgms_plan_destroy((fgms_plan_t *)p);
    return code;
  };
  auto take = [&](void **q, size_t bytes, bool temporary) {
    if (pool_alloc(q, bytes ? bytes : 256, s) != FGMS_OK) return false;
    if (temporary) tmp.push_back(*q);
    return true;
  };
  if (hipGetDevice(&p->device) != hipSuccess) return fail(FGMS_E_HIP);
  if ((p->host_flags = pinned_flags_get())) p->host_flags[kFlagStale] = 0;     // (a recycled block: the flag is read before the build has run)
  if (!p->host_flags ||
      hipEventCreateWithFlags(&p->ready, hipEventDisableTiming) != hipSuccess) {
    set_error("fgms_plan_create: pinned flag block / event creation failed");
    return fail(FGMS_E_NOMEM);
  }
  // weight-gradient row bands: 8, 16, 32 or 64 (the XCDs take them in groups of 1, 2, 4 or 8;
  // other counts measured worse), the fewest that leave an (offset, band) cell at most ~1 900
  // pairs -- a workgroup's fixed costs (first loads, the four waves' partial tiles summed through
  // LDS, 16 KB of atomic updates) are those of ~600 pairs, and with bigger cells the chip waits
  // for the last ones -- then more while the cells are fewer than 1.5 per CU and keep ~400 pairs.
  // 64 -> 64 fp16 backward launch with 64 bands throughout / with this rule: 50 k voxels 35.5 /
  // 29.8 us, 80 k 55.6 / 45.2, 100 k 59.1 / 46.2, 120 k 61.5 / 55.6, 140 k 67.7 / 65.3 (32 bands
  // each), 170 k and 200 k voxels 64 bands either way.
  {
    constexpr int kMaxBands = 64;
    int bands = 8;
    while (bands < kMaxBands && n_pairs / ((int64_t)k_vol * bands) > 1900) bands *= 2;
    while (bands < kMaxBands && (int64_t)bands * k_vol * 2 < 3 * (int64_t)num_cus() &&
           n_pairs / ((int64_t)k_vol * bands * 2) >= 384)
      bands *= 2;
    p->band_count = bands;
  }
  const int band_rows = (int)((n_out + p->band_count - 1) / p->band_count);
  p->band_rows = band_rows;
  const bool tables = k_vol <= 64;      // (64-bit offset masks; beyond that the plan is bands only)
  const size_t so = tables ? (size_t)n_out * k_vol : 0, si = tables ? (size_t)n_in * k_vol : 0;
  const size_t bo = (size_t)(n_out + 63) / 64, bi = (size_t)(n_in + 63) / 64;
  unsigned long long *rmask = nullptr;          // [n_out] then [n_in]
  if ((want_bands && (!take((void **)&p->band_start, (size_t)k_vol * (p->band_count + 1) * sizeof(int32_t), false) ||
                      !take((void **)&p->band_cells, (size_t)4 * k_vol * p->band_count * sizeof(int32_t), false))) ||
      !take((void **)&p->flags, kPlanFlags * sizeof(int), false) ||
      (tables && (!take((void **)&p->nbr_out, (so + si) * sizeof(int32_t), false) ||
                  !take((void **)&p->mask_out, (bo + bi) * sizeof(unsigned long long), false) ||
                  !take((void **)&rmask, (size_t)(n_out + n_in) * sizeof(unsigned long long), true)))) {
    set_error("fgms_plan_create: table allocation failed");
    return fail(FGMS_E_NOMEM);
  }
  if (tables) {
    p->nbr_in = p->nbr_out + so;
    p->mask_in = p->mask_out + bo;
  }
  unsigned long long *rmask_out = rmask, *rmask_in = rmask ? rmask + n_out : nullptr;
  // (the flags are cleared together with the row masks below; without tables, here)
  if (!tables && (rc = fill_i32(p->flags, kPlanFlags, 0, s))) return fail(rc);
  p->has_tables = tables;
  p->has_bands = want_bands;

  // fork: the band tables and the pre-fill of the neighbour tables do not depend on the rest
  static const bool two_streams = !(getenv("FGMS_PLAN_STREAMS") && atoi(getenv("FGMS_PLAN_STREAMS")) == 1);
  hipStream_t s2 = two_streams ? side_stream(p->device) : nullptr;
  hipEvent_t forked = nullptr, joined = nullptr;
  if (s2) {
    if (hipEventCreateWithFlags(&forked, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&joined, hipEventDisableTiming) != hipSuccess ||
        hipEventRecord(forked, s) != hipSuccess || hipStreamWaitEvent(s2, forked, 0) != hipSuccess) {
      if (forked) (void)hipEventDestroy(forked);
      if (joined) (void)hipEventDestroy(joined);
      forked = joined = nullptr;
      s2 = nullptr;      // (nothing was queued on it)
    }
  }
  auto drop_events = [&]() {
    if (forked) (void)hipEventDestroy(forked);
    if (joined) (void)hipEventDestroy(joined);
    forked = joined = nullptr;
  };
  {
    hipStream_t sb = s2 ? s2 : s;
    side_in_use = s2;
    if (want_bands) {
      band_bounds_kernel<<<(unsigned)k_vol, 128, 0, sb>>>(kpos, out_map, (int)n_pairs, p->band_count,
                                                          band_rows > 0 ? band_rows : 1, p->band_start);
      const int per_xcd = (p->band_count / 8) * k_vol;
      band_cells_kernel<<<dim3((unsigned)((per_xcd + 255) / 256), 8, 4), 256, 0, sb>>>(
          p->band_start, k_vol, p->band_count, p->band_cells);
    }
    if (tables && (rc = fill_i32(p->nbr_out, so + si, -1, sb))) {
      drop_events();
      return fail(rc);
    }
    if (s2 && (hipEventRecord(joined, s2) != hipSuccess)) {
      (void)hipStreamSynchronize(s2);
      drop_events();
      set_error("fgms_plan_create: recording on the side stream failed");
      return fail(FGMS_E_HIP);
    }
  }
  if (tables) {
    const size_t n_mask = (size_t)(n_out + n_in) * 2;
    size_t blocks = (n_mask / 4 + 255) / 256;
    fill_two_kernel<<<(unsigned)(blocks > 8192 ? 8192 : (blocks ? blocks : 1)), 256, 0, s>>>(
        (int32_t *)rmask, n_mask, 0, p->flags, (size_t)kPlanFlags, 0);
    if (hipGetLastError() != hipSuccess) {
      drop_events();
      set_error("fgms_plan_create: a build launch failed");
      return fail(FGMS_E_HIP);
    }
  }
  if (tables && n_pairs > 0) {
    pair_masks_kernel<<<(unsigned)((n_pairs + 255) / 256) + 1, 256, 0, s>>>(
        kpos, in_map, out_map, k_vol, (int)n_pairs, (int)n_in, (int)n_out, rmask_out, rmask_in, p->flags);
  }
  // row orders (both sides in the same launches)
  static const bool sort_rows = !(getenv("FGMS_PLAN_SORT") && atoi(getenv("FGMS_PLAN_SORT")) == 0);
  int32_t *inv[2] = {nullptr, nullptr};
  bool published = false;      // the flags reach the host with the tile-order launch
  if (tables) {
    SortArgs sa{};
    sa.k_vol = k_vol;
    bool any_sort = false, any_count = false;
    int max_chunks = 0, max_windows = 0;
    for (int d = 0; d < 2; ++d) {
      const int64_t n = d ? n_in : n_out;
      SortSide &sd = sa.side[d];
      sd.rmask = d ? rmask_in : rmask_out;
      sd.n = 0;
      sd.chunks = 0;
      if (!sort_rows || n <= 64) continue;
      int32_t *&perm = d ? p->perm_in : p->perm_out;
      if (!take((void **)&perm, (size_t)n * sizeof(int32_t), false) ||
          !take((void **)&inv[d], (size_t)n * sizeof(int32_t), true)) {
        drop_events();
        set_error("fgms_plan_create: reorder allocation failed");
        return fail(FGMS_E_NOMEM);
      }
      sd.perm = perm;
      sd.inv = inv[d];
      sd.n = (int)n;
      any_sort = true;
      const int windows = (int)((n + kWindow - 1) / kWindow);
      if (windows > max_windows) max_windows = windows;
      if (n > kWindow) {            // more than one window: counting sort on the top bits first
        sd.chunks = (int)((n + kChunk - 1) / kChunk);
        if (!take((void **)&sd.perm_tmp, (size_t)n * sizeof(int32_t), true) ||
            !take((void **)&sd.hist, (size_t)kBins * sd.chunks * sizeof(int32_t), true) ||
            !take((void **)&sd.hist_before, (size_t)kBins * sd.chunks * sizeof(int32_t), true) ||
            !take((void **)&sd.bin_start, (size_t)kBins * sizeof(int32_t), true)) {
          drop_events();
          set_error("fgms_plan_create: sort allocation failed");
          return fail(FGMS_E_NOMEM);
        }
        any_count = true;
        if (sd.chunks > max_chunks) max_chunks = sd.chunks;
      }
    }
    if (any_count) {
      sort_hist_kernel<<<dim3((unsigned)max_chunks, 2), kSortThreads, 0, s>>>(sa);
      sort_scan_kernel<<<dim3(kBins / kScanBins, 2), kScanBins, 0, s>>>(sa);
      sort_scatter_kernel<<<dim3((unsigned)max_chunks, 2), kSortThreads, 0, s>>>(sa);
    }
    if (any_sort)
      sort_window_kernel<<<dim3((unsigned)max_windows, 2), kSortThreads,
                           kWindow * (sizeof(unsigned long long) + sizeof(int)), s>>>(sa);
  }
  // join: the tables are pre-filled
  if (s2 && hipStreamWaitEvent(s, joined, 0) != hipSuccess) {
    (void)hipStreamSynchronize(s2);
    drop_events();
    set_error("fgms_plan_create: joining the side stream failed");
    return fail(FGMS_E_HIP);
  }
  drop_events();
  if (tables) {
    MaskArgs ma{};
    ma.flags = p->flags;
    ma.side[0] = MaskSide{rmask_out, p->perm_out, p->mask_out, (int)n_out};
    ma.side[1] = MaskSide{rmask_in, p->perm_in, p->mask_in, (int)n_in};
    const size_t most = bo > bi ? bo : bi;
    if (n_pairs > 0)
      tables_kernel<<<(unsigned)((n_pairs + 255) / 256), 256, 0, s>>>(
          kpos, in_map, out_map, k_vol, (int)n_pairs, (int)n_in, (int)n_out, inv[0], inv[1], p->nbr_out, p->nbr_in);
    if (most > 0) block_masks_kernel<<<dim3((unsigned)((most + 15) / 16), 2), 1024, 0, s>>>(ma);
    // tile -> XCD homes pay off once every XCD has a few dozen tiles of its own
    static const bool xcd_homes = !(getenv("FGMS_XCD_HOME") && atoi(getenv("FGMS_XCD_HOME")) == 0);
    TileArgs ta{};
    ta.cus_per_xcd = num_cus() >= 8 ? num_cus() / 8 : 1;
    int most_tiles = 0;
    for (int d = 0; d < 2; ++d) {
      const int64_t n = d ? n_in : n_out;
      const int n_tiles = (int)((n + 255) / 256);
      if (!xcd_homes || n_tiles < 256 || (size_t)n_tiles * sizeof(int32_t) > 60000) continue;
      int32_t *&order = d ? p->tile_in : p->tile_out;
      const int cap = (n_tiles + 7) / 8;
      if (!take((void **)&order, (size_t)cap * 8 * sizeof(int32_t), false)) {
        order = nullptr;       // (the kernels then take the tiles in plain order)
        continue;
      }
      (d ? p->tile_grid_in : p->tile_grid_out) = cap * 8;
      ta.side[d] = TileSide{d ? p->perm_in : p->perm_out, d ? p->mask_in : p->mask_out, order, (int)n, n_tiles, cap};
      if (n_tiles > most_tiles) most_tiles = n_tiles;
    }
    if (most_tiles > 0) {
      if (hipHostGetDevicePointer((void **)&ta.host, p->host_flags, 0) != hipSuccess) ta.host = nullptr;
      ta.flags = p->flags;
      tile_order_kernel<<<2, 1024, (size_t)most_tiles * sizeof(int32_t), s>>>(ta);
      published = ta.host != nullptr;
    }
  }
  if (hipGetLastError() != hipSuccess) {
    set_error("fgms_plan_create: a build launch failed");
    return fail(FGMS_E_HIP);
  }
  int *host_dev = nullptr;
  if (hipHostGetDevicePointer((void **)&host_dev, p->host_flags, 0) != hipSuccess) host_dev = nullptr;
  if (host_dev && !published) publish_flags_kernel<<<1, 64, 0, s>>>(p->flags, host_dev);
  if ((!host_dev && hipMemcpyAsync(p->host_flags, p->flags, kPlanFlags * sizeof(int), hipMemcpyDeviceToHost, s) != hipSuccess) ||
      hipEventRecord(p->ready, s) != hipSuccess) {
    set_error("fgms_plan_create: queuing the flag read-back failed");
    return fail(FGMS_E_HIP);
  }
  for (void *q : tmp) pool_free(q, s, false);
  tmp.clear();
  // More than 64 offsets: the tables and masks hold 64 offsets each, so the offsets are cut
  // into groups of 64, every group with tables of its own (the pairs of a group are one
  // contiguous run of the lists); the entry points walk the groups, the weight gradient uses
  // this plan's row bands over all offsets.
  if (!tables) {
    for (int k0 = 0; k0 < k_vol; k0 += 64) {
      fgms_plan_t *g = nullptr;
      rc = plan_create(&g, kpos + k0, in_map, out_map, n_in, n_out, k_vol - k0 < 64 ? k_vol - k0 : 64, n_pairs,
                       stream, false);
      if (rc != FGMS_OK) {
        fgms_plan_destroy((fgms_plan_t *)p);
        return rc;
      }
      p->groups.push_back((Plan *)g);
    }
  }
  *plan_out = (fgms_plan_t *)p;
  return FGMS_OK;
}

// What the build found out, once its last kernel has run.  Returns the plan when its flags are
// known (waiting for the build if it has not finished yet), nullptr when they cannot be had
// now (the stream is being captured into a graph: the caller then takes the kernels that need
// no plan) or when the map turned out to be invalid (*rc = FGMS_E_INVALID).
// The plan if its build results are already known to the host, else nullptr: never waits,
// never allocates, never launches (for the entry point that promises that).
const Plan *plan_if_resolved(fgms_plan_t *plan) {
  Plan *p = (Plan *)plan;
  if (!p) return nullptr;
  std::lock_guard<std::mutex> lock(p->mutex);
  return p->resolved && !p->invalid ? p : nullptr;
}

static Plan *check_owner(const Plan *p) { return const_cast<Plan *>(p->base ? p->base : p); }

bool plan_take_check(const Plan *p, SideJob *job) {
  Plan *b = check_owner(p);
  if (!b->check_pending || !b->has_tables || !b->flags || b->n_pairs == 0) return false;
  if (!b->resolved) return false;     // (the build may still be running: the fingerprint is not final)
  int *host_dev = nullptr;
  if (hipHostGetDevicePointer((void **)&host_dev, b->host_flags, 0) != hipSuccess) host_dev = nullptr;
  *job = SideJob{};
  job->kind = 3;
  job->blocks = 8;                 // (a multiple of 8: the workgroups behind keep their XCDs)
  job->src = b->kpos;
  job->dst = const_cast<int32_t *>(b->in_map);
  job->omap = b->out_map;
  job->n = (size_t)b->n_pairs;
  job->k_vol = b->k_vol;
  job->flags = b->flags;
  job->host = host_dev;
  b->check_pending = false;
  b->checked = true;
  return true;
}

int plan_flush_check(const Plan *p, hipStream_t s) {
  Plan *b = check_owner(p);
  for (Plan *g : b->groups) {
    const int rc = plan_flush_check(g, s);
    if (rc != FGMS_OK) return rc;
  }
  if (!b->check_pending) return FGMS_OK;
  b->check_pending = false;
  if (!b->has_tables || !b->flags || b->n_pairs == 0) return FGMS_OK;
  int *host_dev = nullptr;
  if (hipHostGetDevicePointer((void **)&host_dev, b->host_flags, 0) != hipSuccess) host_dev = nullptr;
  // (queued behind the build if that ran on another stream: the fingerprint must be final)
  // (a resolved plan's build has finished; no event is queried then, which a stream under
  // capture would not allow)
  if (!b->resolved && s != b->create_stream) FGMS_HIP_TRY(hipStreamWaitEvent(s, b->ready, 0));
  plan_check_kernel<<<1, 1024, 0, s>>>(b->kpos, b->in_map, b->out_map, b->k_vol, (int)b->n_pairs, b->flags, host_dev);
  FGMS_HIP_TRY(hipGetLastError());
  b->checked = true;
  return FGMS_OK;
}

// Has an earlier fgms_plan_check found the lists changed?  (Reads the pinned block; no wait.)
static bool plan_is_stale(const Plan *p) {
  const Plan *b = p->base ? p->base : p;
  if (b->checked && b->host_flags && b->host_flags[kFlagStale]) return true;
  for (const Plan *g : b->groups)
    if (g->checked && g->host_flags && g->host_flags[kFlagStale]) return true;
  return false;
}

const Plan *plan_resolve(fgms_plan_t *plan, hipStream_t stream, int *rc) {
  *rc = FGMS_OK;
  Plan *p = (Plan *)plan;
  if (!p) return nullptr;
  if (plan_is_stale(p)) {
    set_error("plan: the pair lists were rewritten after the plan was made (make a new plan)");
    *rc = FGMS_E_STALE;
    return nullptr;
  }
  if (p->base && !p->resolved) {
    // a transposed view: the base's tables with the sides swapped
    const Plan *b = plan_resolve((fgms_plan_t *)p->base, stream, rc);
    if (!b) return nullptr;
    std::lock_guard<std::mutex> lock(p->mutex);
    if (!p->resolved) {
      p->nbr_out = b->nbr_in; p->nbr_in = b->nbr_out;
      p->perm_out = b->perm_in; p->perm_in = b->perm_out;
      p->mask_out = b->mask_in; p->mask_in = b->mask_out;
      p->tile_out = b->tile_in; p->tile_in = b->tile_out;
      p->tile_grid_out = b->tile_grid_in; p->tile_grid_in = b->tile_grid_out;
      p->stages_out = b->stages_in; p->stages_in = b->stages_out;
      p->fwd_ok = b->dgrad_ok; p->dgrad_ok = b->fwd_ok;
      p->pv_in = b->pv_out; p->pv_out = b->pv_in; p->pv_mask = b->pv_mask; p->pv_rows = b->pv_rows;
      p->pv_ready = b->pv_ready; p->pv_stream = b->pv_stream;
      p->has_tables = b->has_tables;
      p->pairs_counted = b->pairs_counted;
      p->ordered = false;
      // (the weight gradient's row bands follow the base's output rows: not valid for the swapped lists)
      p->bands_ok = false; p->band_start = nullptr; p->band_cells = nullptr; p->band_count = 0;
      p->invalid = false;
      p->resolved = true;
    }
    return p;
  }
  if (!p->resolved) {
    std::lock_guard<std::mutex> lock(p->mutex);
    if (!p->resolved) {
      if (hipEventQuery(p->ready) != hipSuccess) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (stream && hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone)
          return nullptr;
        if (hipEventSynchronize(p->ready) != hipSuccess) {
          set_error("plan: waiting for the build failed");
          *rc = FGMS_E_HIP;
          return nullptr;
        }
      }
      const int *h = p->host_flags;
      p->invalid = h[0] != 0;
      p->fwd_ok = p->has_tables && !h[0] && !h[1] && h[10] == h[12];
      p->dgrad_ok = p->has_tables && !h[0] && !h[2] && h[11] == h[12];
      p->ordered = !h[0] && !h[3];
      p->bands_ok = p->has_bands && p->ordered;
      p->stages_out = h[4];
      p->stages_in = h[5];
      p->pairs_counted = p->has_tables ? h[12] : p->n_pairs;
      // The pair view, for maps sparse enough that some layer would take it (fp32 layers prefer
      // it from about 1 + 45 / channels row slots per pair on, never below 1.4): built now that
      // the counts are known, so that dense maps pay nothing.
      static const bool pair_view = !(getenv("FGMS_PAIR_VIEW") && atoi(getenv("FGMS_PAIR_VIEW")) == 0);
      const int most = p->stages_out > p->stages_in ? p->stages_out : p->stages_in;
      if (!p->invalid && pair_view && p->has_tables && p->pairs_counted > 0 &&
          (kernel_policy() == 5 || (double)most * 64.0 >= 1.35 * (double)p->pairs_counted)) {
        // (a caller that names no stream -- fgms_plan_usable, fgms_plan_stats -- must not put the
        // view on the legacy null stream, which the streams torch makes do not wait for: the
        // stream the plan itself was built on takes it)
        hipStream_t s = stream ? stream : p->create_stream;
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        const bool capturing = s && hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
        const int64_t rows = (p->pairs_counted + 64 * (int64_t)p->k_vol + 255) / 256 * 256;
        if (!capturing &&
            pool_alloc((void **)&p->pv_in, (size_t)rows * sizeof(int32_t), s) == FGMS_OK &&
            pool_alloc((void **)&p->pv_out, (size_t)rows * sizeof(int32_t), s) == FGMS_OK &&
            pool_alloc((void **)&p->pv_mask, (size_t)(rows / 64) * sizeof(unsigned long long), s) == FGMS_OK &&
            fill_i32(p->pv_in, (size_t)rows, -1, s) == FGMS_OK && fill_i32(p->pv_out, (size_t)rows, -1, s) == FGMS_OK &&
            fill_i32((int32_t *)p->pv_mask, (size_t)(rows / 64) * 2, 0, s) == FGMS_OK) {
          pair_view_kernel<<<(unsigned)((p->n_pairs + 255) / 256), 256, 0, s>>>(
              p->kpos, p->in_map, p->out_map, p->k_vol, (int)p->n_pairs, (long long)rows, p->pv_in, p->pv_out,
              p->pv_mask);
          // launches on other streams wait for this event (launch_pair_view_gms, the destroy path)
          if (hipGetLastError() != hipSuccess ||
              hipEventCreateWithFlags(&p->pv_ready, hipEventDisableTiming) != hipSuccess ||
              hipEventRecord(p->pv_ready, s) != hipSuccess) {
            // without the event nothing else can be ordered behind the build: finish it here
            (void)hipStreamSynchronize(s);
            if (p->pv_ready) (void)hipEventDestroy(p->pv_ready);
            p->pv_ready = nullptr;
          }
          p->pv_rows = rows;
          p->pv_stream = s;
        } else {
          if (p->pv_in) pool_free(p->pv_in, s, false);
          if (p->pv_out) pool_free(p->pv_out, s, false);
          if (p->pv_mask) pool_free(p->pv_mask, s, false);
          p->pv_in = p->pv_out = nullptr;
          p->pv_mask = nullptr;
        }
      }
      // (a plan over more than 64 offsets: its groups)
      for (Plan *g : p->groups) {
        int grc = FGMS_OK;
        const Plan *gr = plan_resolve((fgms_plan_t *)g, stream, &grc);
        if (!gr && grc == FGMS_E_INVALID) p->invalid = true;
        if (!gr && grc != FGMS_E_INVALID) return nullptr;        // (cannot be known now: try again later)
        if (gr) {
          p->fwd_ok = (g == p->groups.front() ? true : p->fwd_ok) && gr->fwd_ok;
          p->dgrad_ok = (g == p->groups.front() ? true : p->dgrad_ok) && gr->dgrad_ok;
          p->stages_out += gr->stages_out;
          p->stages_in += gr->stages_in;
          p->ordered = p->ordered && gr->ordered;
        }
      }
      if (!p->groups.empty()) p->bands_ok = p->has_bands && p->ordered && !p->invalid;
      p->resolved = true;
    }
  }
  if (p->invalid) {
    set_error("plan: a map index is outside [0, n_in) x [0, n_out)");
    *rc = FGMS_E_INVALID;
    return nullptr;
  }
  return p;
}
}  // namespace fgms

extern "C" {

int fgms_plan_create(fgms_plan_t **plan_out, const int32_t *kpos, const int32_t *in_map,
                     const int32_t *out_map, int64_t n_in, int64_t n_out, int k_vol,
                     int64_t n_pairs, void *stream) {
  return plan_create(plan_out, kpos, in_map, out_map, n_in, n_out, k_vol, n_pairs, stream, true);
}

int fgms_plan_transposed(fgms_plan_t **view_out, fgms_plan_t *base_plan) {
  Plan *b = (Plan *)base_plan;
  if (!view_out || !b || b->base || !b->groups.empty()) {
    set_error("fgms_plan_transposed: needs a plan made by fgms_plan_create over at most 64 offsets");
    return FGMS_E_INVALID;
  }
  Plan *v = new Plan();
  v->device = b->device;
  v->k_vol = b->k_vol; v->n_in = b->n_out; v->n_out = b->n_in; v->n_pairs = b->n_pairs;
  v->kpos = b->kpos; v->in_map = b->out_map; v->out_map = b->in_map;
  v->last_stream = b->last_stream;
  v->base = b;
  {
    std::lock_guard<std::mutex> lock(b->mutex);
    b->views += 1;
  }
  *view_out = (fgms_plan_t *)v;
  return FGMS_OK;
}

void fgms_plan_destroy(fgms_plan_t *plan) {
  Plan *p = (Plan *)plan;
  if (!p) return;
  if (p->base) {
    // a view owns nothing; the base goes with its last view if it was destroyed before
    Plan *b = p->base;
    bool free_base = false;
    {
      std::lock_guard<std::mutex> lock(b->mutex);
      if (p->last_stream != b->last_stream || p->many_streams) b->many_streams = true;
      b->views -= 1;
      free_base = b->views == 0 && b->destroyed;
    }
    delete p;
    if (free_base) fgms_plan_destroy((fgms_plan_t *)b);
    return;
  }
  {
    std::lock_guard<std::mutex> lock(p->mutex);
    p->destroyed = true;
    if (p->views > 0) return;       // (still shared: freed with the last view)
  }
  for (Plan *g : p->groups) {
    if (p->many_streams) g->many_streams = true;
    g->last_stream = p->last_stream;
    fgms_plan_destroy((fgms_plan_t *)g);
  }
  p->groups.clear();
  if (p->many_streams) (void)hipDeviceSynchronize();     // (blocks are handed back behind ONE stream's work)
  if (p->nbr_out) pool_free(p->nbr_out, p->last_stream, false);      // (nbr_in is the same block)
  if (p->mask_out) pool_free(p->mask_out, p->last_stream, false);    // (mask_in likewise)
  if (p->perm_out) pool_free(p->perm_out, p->last_stream, false);
  if (p->perm_in) pool_free(p->perm_in, p->last_stream, false);
  if (p->band_start) pool_free(p->band_start, p->last_stream, false);
  if (p->band_cells) pool_free(p->band_cells, p->last_stream, false);
  if (p->tile_out) pool_free(p->tile_out, p->last_stream, false);
  if (p->tile_in) pool_free(p->tile_in, p->last_stream, false);
  if (p->pv_ready) {
    // the view may have been built on another stream than the one the blocks are handed back behind
    if (p->pv_stream != p->last_stream) (void)hipStreamWaitEvent(p->last_stream, p->pv_ready, 0);
    (void)hipEventDestroy(p->pv_ready);
  }
  if (p->pv_in) pool_free(p->pv_in, p->last_stream, false);
  if (p->pv_out) pool_free(p->pv_out, p->last_stream, false);
  if (p->pv_mask) pool_free(p->pv_mask, p->last_stream, false);
  if (p->ready) {
    // the flag read-back must not land in freed host memory
    (void)hipEventSynchronize(p->ready);
    (void)hipEventDestroy(p->ready);
  }
  if (p->flags) pool_free(p->flags, p->last_stream, false);
  if (p->host_flags) pinned_flags_put(p->host_flags);
  delete p;
}

int fgms_plan_check(fgms_plan_t *plan, void *stream, int with_next_launch) {
  Plan *p = (Plan *)plan;
  if (!p) return FGMS_OK;
  Plan *b = p->base ? p->base : p;           // (a view shares its base's lists and flags)
  if (plan_is_stale(p)) {
    set_error("plan: the pair lists were rewritten after the plan was made (make a new plan)");
    return FGMS_E_STALE;
  }
  b->check_pending = true;
  for (Plan *g : b->groups) g->check_pending = true;
  if (with_next_launch) return FGMS_OK;
  return plan_flush_check(p, (hipStream_t)stream);
}

int fgms_plan_usable(const fgms_plan_t *plan, int for_dgrad) {
  int rc = FGMS_OK;
  const Plan *p = plan_resolve(const_cast<fgms_plan_t *>(plan), nullptr, &rc);
  if (!p) return 0;
  return for_dgrad ? (p->dgrad_ok ? 1 : 0) : (p->fwd_ok ? 1 : 0);
}

int fgms_plan_stats(const fgms_plan_t *plan, int64_t stats[4]) {
  if (!plan || !stats) {
    set_error("fgms_plan_stats: null argument");
    return FGMS_E_INVALID;
  }
  int rc = FGMS_OK;
  const Plan *p = plan_resolve(const_cast<fgms_plan_t *>(plan), nullptr, &rc);
  if (!p) return rc ? rc : FGMS_E_INVALID;
  stats[0] = p->groups.empty() ? p->pairs_counted : p->n_pairs;
  stats[1] = p->stages_out;
  stats[2] = p->stages_in;
  stats[3] = p->pv_in ? p->pv_rows : 0;
  return FGMS_OK;
}

}  // extern "C"
