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

#include <rocprim/device/device_radix_sort.hpp>

#include "fgms_device.h"
#include "fgms_internal.h"

namespace fgms {
namespace {

__global__ void fill_i32_kernel(int32_t *__restrict__ p, size_t n, int32_t v) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = v;
}

// flags[0]: an index is out of range; flags[1]: two pairs of one offset share
// an output row; flags[2]: two pairs of one offset share an input row;
// flags[3]: inside some offset the pairs are not ordered by output row.
__global__ void build_tables_kernel(const int32_t *__restrict__ kpos,
                                    const int32_t *__restrict__ imap,
                                    const int32_t *__restrict__ omap, int k_vol, int n_pairs,
                                    int n_in, int n_out, int32_t *__restrict__ nbr_out,
                                    int32_t *__restrict__ nbr_in, int *__restrict__ flags) {
  const int total = kpos[k_vol];
  int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= total || j >= n_pairs) return;
  // offset of pair j: the last k with kpos[k] <= j
  int lo = 0, hi = k_vol;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (kpos[mid] <= j) lo = mid; else hi = mid;
  }
  const int k = lo;
  const int i = imap[j], o = omap[j];
  if (i < 0 || i >= n_in || o < 0 || o >= n_out) {
    flags[0] = 1;
    return;
  }
  if (j > kpos[k] && omap[j - 1] > o) flags[3] = 1;
  if (atomicCAS(&nbr_out[(size_t)k * n_out + o], -1, i) != -1) flags[1] = 1;
  if (atomicCAS(&nbr_in[(size_t)k * n_in + i], -1, o) != -1) flags[2] = 1;
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
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
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

// One wave per block of 64 consecutive rows: which offsets have a neighbour there.
__global__ void block_masks_kernel(const int32_t *__restrict__ nbr, int n_rows, int k_vol,
                                   unsigned long long *__restrict__ masks64) {
  const int block = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  const int row = block * 64 + (int)(threadIdx.x % 64);
  if (block * 64 >= n_rows) return;
  unsigned long long m = 0;
  for (int k0 = 0; k0 < k_vol; k0 += 8) {
    int g[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      g[i] = (k0 + i < k_vol && row < n_rows) ? nbr[(size_t)(k0 + i) * n_rows + row] : -1;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (__ballot(g[i] >= 0)) m |= 1ull << (k0 + i);
  }
  if (threadIdx.x % 64 == 0) masks64[block] = m;
}

// *stages = the number of (block, offset) combinations in use: the set bits of all block
// masks.  One workgroup (a few thousand masks; thousands of same-address atomics from the
// mask kernel itself cost 25 us).
__global__ __launch_bounds__(1024) void count_stages_kernel(const unsigned long long *__restrict__ masks64,
                                                            int n_blocks, int *__restrict__ stages) {
  __shared__ int partial[16];
  int sum = 0;
  for (int b = threadIdx.x; b < n_blocks; b += blockDim.x) sum += __popcll(masks64[b]);
  for (int d = 32; d > 0; d >>= 1) sum += __shfl_down(sum, d);
  if (threadIdx.x % 64 == 0) partial[threadIdx.x / 64] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
    for (int i = 0; i < (int)blockDim.x / 64; ++i) total += partial[i];
    *stages = total;
  }
}

// rmask[row] = bit k set iff row has a neighbour through offset k.
// Also rows[row] = row, the values the sort permutes.
__global__ void row_masks_kernel(const int32_t *__restrict__ nbr, int n_rows, int k_vol,
                                 unsigned long long *__restrict__ rmask, int32_t *__restrict__ rows) {
  const int row = blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= n_rows) return;
  rows[row] = row;
  unsigned long long m = 0;
  for (int k = 0; k < k_vol; ++k)
    if (nbr[(size_t)k * n_rows + row] >= 0) m |= 1ull << k;
  rmask[row] = m;
}

// Row order: rows are sorted by their offset mask (stable, so rows with equal
// masks keep their relative order and with it most of their spatial locality).
// The 64 rows a wave works on then use nearly the same offsets and whole
// (block, offset) steps can be skipped: on a surface-like cloud of 200 k voxels
// the number of such steps drops from 68.6 k to 36.7 k (33 k would be perfect).
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
__global__ __launch_bounds__(1024) void tile_order_kernel(const int32_t *__restrict__ perm,
                                                          const unsigned long long *__restrict__ block_masks,
                                                          int n_rows, int n_tiles, int cap,
                                                          int cus_per_xcd, int32_t *__restrict__ order) {
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

// out[k][pos] = in[k][perm[pos]]
__global__ void permute_table_kernel(const int32_t *__restrict__ in, const int32_t *__restrict__ perm,
                                     int n_rows, int k_vol, int32_t *__restrict__ out) {
  const int pos = blockIdx.x * blockDim.x + threadIdx.x;
  if (pos >= n_rows) return;
  const int row = perm[pos];
  // (one offset per blockIdx.y: 27 independent loads per row in flight instead of a loop)
  for (int k = blockIdx.y; k < k_vol; k += gridDim.y) out[(size_t)k * n_rows + pos] = in[(size_t)k * n_rows + row];
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

int fill_i32(int32_t *p, size_t n, int32_t v, hipStream_t s) {
  if (n == 0) return FGMS_OK;
  size_t blocks = (n + 1023) / 1024;
  if (blocks > 65535) blocks = 65535;
  fill_i32_kernel<<<(unsigned)blocks, 256, 0, s>>>(p, n, v);
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

}  // namespace
}  // namespace fgms

using namespace fgms;

namespace fgms {
int plan_create(fgms_plan_t **plan_out, const int32_t *kpos, const int32_t *in_map,
                const int32_t *out_map, int64_t n_in, int64_t n_out, int k_vol, int64_t n_pairs,
                const int32_t *in_coords, const int32_t *out_coords, int coord_bits, void *stream) {
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
  Plan *p = new Plan();
  p->k_vol = k_vol; p->n_in = n_in; p->n_out = n_out; p->n_pairs = n_pairs;
  p->nbr_out = p->nbr_in = nullptr; p->mask_out = p->mask_in = nullptr;
  p->perm_out = p->perm_in = nullptr;
  p->band_count = 0; p->band_start = nullptr; p->band_cells = nullptr; p->bands_ok = false;
  p->tile_out = p->tile_in = nullptr; p->tile_grid_out = p->tile_grid_in = 0;
  p->fwd_ok = p->dgrad_ok = false;
  p->pv_in = p->pv_out = nullptr; p->pv_mask = nullptr; p->pv_rows = 0;
  p->halo[0] = p->halo[1] = HaloSide{};
  p->last_stream = s;
  int *flags = nullptr;
  int rc = FGMS_OK;
  bool synced = false;      // true once the stream has drained: freed blocks are idle then
  auto fail = [&](int code) {
    if (flags) pool_free(flags, s, synced);
    fgms_plan_destroy((fgms_plan_t *)p);
    return code;
  };
  if (hipGetDevice(&p->device) != hipSuccess) return fail(FGMS_E_HIP);
  // weight-gradient row bands: about 2048 output rows each but enough bands to
  // fill the chip (bands x offsets >= ~1536 workgroups) and no more than leaves a
  // workgroup ~400 pairs on average; a multiple of 8 (one per XCD), 8..kMaxBands
  {
    int64_t want = n_out / 2048;
    const int64_t fill = (1536 + k_vol - 1) / k_vol;
    if (want < fill) want = fill;
    const int64_t by_work = n_pairs / ((int64_t)k_vol * 384);
    if (want > by_work) want = by_work;
    want = (want + 7) / 8 * 8;
    constexpr int kMaxBands = 64;
    p->band_count = (int)(want < 8 ? 8 : (want > kMaxBands ? kMaxBands : want));
  }
  const int band_rows = (int)((n_out + p->band_count - 1) / p->band_count);
  p->band_rows = band_rows;
  const size_t so = (size_t)n_out * k_vol, si = (size_t)n_in * k_vol;
  const size_t bo = (size_t)(n_out + 63) / 64, bi = (size_t)(n_in + 63) / 64;
  if (pool_alloc((void **)&p->nbr_out, (so ? so : 1) * sizeof(int32_t), s) != FGMS_OK ||
      pool_alloc((void **)&p->nbr_in, (si ? si : 1) * sizeof(int32_t), s) != FGMS_OK ||
      pool_alloc((void **)&p->mask_out, (bo ? bo : 1) * sizeof(unsigned long long), s) != FGMS_OK ||
      pool_alloc((void **)&p->mask_in, (bi ? bi : 1) * sizeof(unsigned long long), s) != FGMS_OK ||
      pool_alloc((void **)&p->band_start, (size_t)k_vol * (p->band_count + 1) * sizeof(int32_t), s) != FGMS_OK ||
      pool_alloc((void **)&p->band_cells, (size_t)4 * k_vol * p->band_count * sizeof(int32_t), s) != FGMS_OK ||
      pool_alloc((void **)&flags, 10 * sizeof(int), s) != FGMS_OK) {
    set_error("fgms_plan_create: table allocation failed");
    return fail(FGMS_E_NOMEM);
  }
  if ((rc = fill_i32(p->nbr_out, so, -1, s))) return fail(rc);
  if ((rc = fill_i32(p->nbr_in, si, -1, s))) return fail(rc);
  if ((rc = fill_i32(flags, 10, 0, s))) return fail(rc);
  if (n_pairs > 0) {
    build_tables_kernel<<<(unsigned)((n_pairs + 255) / 256), 256, 0, s>>>(
        kpos, in_map, out_map, k_vol, (int)n_pairs, (int)n_in, (int)n_out, p->nbr_out, p->nbr_in, flags);
    if (hipGetLastError() != hipSuccess) {
      set_error("fgms_plan_create: table build launch failed");
      return fail(FGMS_E_HIP);
    }
  }
  // Row orders for the LDS-neighbourhood kernels: Morton order of the voxel coordinates where
  // the caller supplies them (one order serves both sides of a submanifold map).
  std::vector<void *> tmp_more;
  int32_t *ord[2] = {nullptr, nullptr}, *inv[2] = {nullptr, nullptr};   // [0] output side, [1] input side
  if (k_vol <= 64 && out_coords && in_coords) {
    if ((rc = halo_morton_order(out_coords, n_out, coord_bits, &ord[0], &inv[0], &tmp_more, s)) == FGMS_OK) {
      if (in_coords == out_coords && n_in == n_out) {
        ord[1] = ord[0];
        inv[1] = inv[0];
      } else {
        rc = halo_morton_order(in_coords, n_in, coord_bits, &ord[1], &inv[1], &tmp_more, s);
      }
    }
    if (rc != FGMS_OK) {
      for (void *q : tmp_more) pool_free(q, s, false);
      return fail(rc);
    }
  }
  // fork: the input side's chain waits for the tables only
  static const bool two_streams = !(getenv("FGMS_PLAN_STREAMS") && atoi(getenv("FGMS_PLAN_STREAMS")) == 1);
  hipStream_t s2 = (two_streams && k_vol <= 64 && n_in > 0 && n_out > 0) ? side_stream(p->device) : nullptr;
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
  band_bounds_kernel<<<(unsigned)k_vol, 128, 0, s>>>(kpos, out_map, (int)n_pairs, p->band_count,
                                                     band_rows > 0 ? band_rows : 1, p->band_start);
  {
    const int per_xcd = (p->band_count / 8) * k_vol;
    band_cells_kernel<<<dim3((unsigned)((per_xcd + 255) / 256), 8, 4), 256, 0, s>>>(
        p->band_start, k_vol, p->band_count, p->band_cells);
  }
  // Reorder the rows (stable sort by offset mask), then derive the block masks
  // from the tables in their final order.  Temporaries are freed after the
  // stream synchronisation below.
  int32_t *tmp_tab[2] = {nullptr, nullptr};
  unsigned long long *tmp_mask[2] = {nullptr, nullptr};
  auto free_tmp = [&]() {
    if (s2 && !synced) {
      // work of the side stream may still use the temporaries: drain both streams first
      (void)hipStreamSynchronize(s2);
      (void)hipStreamSynchronize(s);
      synced = true;
    }
    if (forked) (void)hipEventDestroy(forked);
    if (joined) (void)hipEventDestroy(joined);
    forked = joined = nullptr;
    for (int d = 0; d < 2; ++d) {
      if (tmp_tab[d]) pool_free(tmp_tab[d], s, synced);
      if (tmp_mask[d]) pool_free(tmp_mask[d], s, synced);
      tmp_tab[d] = nullptr; tmp_mask[d] = nullptr;
    }
    for (void *q : tmp_more) pool_free(q, s, synced);
    tmp_more.clear();
  };
  static const bool sort_rows = !(getenv("FGMS_PLAN_SORT") && atoi(getenv("FGMS_PLAN_SORT")) == 0);
  if (k_vol <= 64) {
    for (int d = 0; d < 2; ++d) {
      const int64_t n = d ? n_in : n_out;
      hipStream_t sd = (d == 1 && s2) ? s2 : s;   // the stream of this direction's chain
      const size_t blocks = d ? bi : bo;
      int32_t *&tab = d ? p->nbr_in : p->nbr_out;
      int32_t *&perm = d ? p->perm_in : p->perm_out;
      unsigned long long *mask = d ? p->mask_in : p->mask_out;
      if (n == 0) continue;
      if (sort_rows && n > 64) {
        int32_t *sorted = nullptr;
        if (pool_alloc((void **)&tmp_mask[d], (size_t)n * sizeof(unsigned long long), sd) != FGMS_OK ||
            pool_alloc((void **)&perm, (size_t)n * sizeof(int32_t), sd) != FGMS_OK ||
            pool_alloc((void **)&sorted, (size_t)n * k_vol * sizeof(int32_t), sd) != FGMS_OK) {
          if (sorted) pool_free(sorted, s, synced);
          free_tmp();
          set_error("fgms_plan_create: reorder allocation failed");
          return fail(FGMS_E_NOMEM);
        }
        // stable LSD radix sort over the k_vol significant bits of the masks
        unsigned long long *keys_out = nullptr;
        int32_t *rows_in = nullptr;
        void *sort_tmp = nullptr;
        size_t sort_bytes = 0;
        bool ok = pool_alloc((void **)&keys_out, (size_t)n * sizeof(unsigned long long), sd) == FGMS_OK;
        if (ok) tmp_more.push_back(keys_out);
        ok = ok && pool_alloc((void **)&rows_in, (size_t)n * sizeof(int32_t), sd) == FGMS_OK;
        if (ok) tmp_more.push_back(rows_in);
        ok = ok && rocprim::radix_sort_pairs(nullptr, sort_bytes, tmp_mask[d], keys_out, rows_in, perm,
                                             (size_t)n, 0u, (unsigned)k_vol, sd) == hipSuccess;
        ok = ok && pool_alloc(&sort_tmp, sort_bytes, sd) == FGMS_OK;
        if (ok) tmp_more.push_back(sort_tmp);
        if (ok) {
          row_masks_kernel<<<(unsigned)((n + 255) / 256), 256, 0, sd>>>(tab, (int)n, k_vol, tmp_mask[d], rows_in);
          ok = rocprim::radix_sort_pairs(sort_tmp, sort_bytes, tmp_mask[d], keys_out, rows_in, perm,
                                         (size_t)n, 0u, (unsigned)k_vol, sd) == hipSuccess;
        }
        if (!ok) {
          pool_free(sorted, s, synced);
          free_tmp();
          set_error("fgms_plan_create: row sort failed");
          return fail(FGMS_E_HIP);
        }
        permute_table_kernel<<<dim3((unsigned)((n + 255) / 256), (unsigned)k_vol), 256, 0, sd>>>(tab, perm, (int)n, k_vol, sorted);
        tmp_tab[d] = tab;      // the unsorted table, freed after the sync
        tab = sorted;
      }
      block_masks_kernel<<<(unsigned)((blocks + 3) / 4), 256, 0, sd>>>(tab, (int)n, k_vol, mask);
      count_stages_kernel<<<1, 1024, 0, sd>>>(mask, (int)blocks, flags + 4 + d);
      // tile -> XCD homes pay off once every XCD has a few dozen tiles of its own
      static const bool xcd_homes = !(getenv("FGMS_XCD_HOME") && atoi(getenv("FGMS_XCD_HOME")) == 0);
      const int n_tiles = (int)((n + 255) / 256);
      if (xcd_homes && n_tiles >= 256 && (size_t)n_tiles * sizeof(int32_t) <= 60000) {
        int32_t *&order = d ? p->tile_in : p->tile_out;
        const int cap = (n_tiles + 7) / 8;
        if (pool_alloc((void **)&order, (size_t)cap * 8 * sizeof(int32_t), sd) != FGMS_OK) {
          free_tmp();
          return fail(FGMS_E_NOMEM);
        }
        (d ? p->tile_grid_in : p->tile_grid_out) = cap * 8;
        tile_order_kernel<<<1, 1024, (size_t)n_tiles * sizeof(int32_t), sd>>>(
            perm, mask, (int)n, n_tiles, cap, num_cus() >= 8 ? num_cus() / 8 : 1, order);
      }
      // tile tables of the LDS-neighbourhood kernels, from the table by destination row
      if ((rc = halo_build(p, d, tmp_tab[d] ? tmp_tab[d] : tab, ord[d], inv[1 - d], ord[1 - d], flags + 6 + 2 * d, sd))) {
        free_tmp();
        return fail(rc);
      }
    }
    if (s2 && (hipEventRecord(joined, s2) != hipSuccess || hipStreamWaitEvent(s, joined, 0) != hipSuccess)) {
      free_tmp();
      set_error("fgms_plan_create: joining the side stream failed");
      return fail(FGMS_E_HIP);
    }
    if (hipGetLastError() != hipSuccess) {
      free_tmp();
      set_error("fgms_plan_create: reorder / mask build launch failed");
      return fail(FGMS_E_HIP);
    }
  }
  int h[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  if (hipMemcpyAsync(h, flags, sizeof(h), hipMemcpyDeviceToHost, s) != hipSuccess ||
      hipStreamSynchronize(s) != hipSuccess) {
    free_tmp();
    set_error("fgms_plan_create: reading the build flags failed");
    return fail(FGMS_E_HIP);
  }
  synced = true;
  free_tmp();
  pool_free(flags, s, synced);
  flags = nullptr;
  if (h[0]) {
    set_error("fgms_plan_create: a map index is outside [0, n_in) x [0, n_out)");
    return fail(FGMS_E_INVALID);
  }
  p->fwd_ok = !h[1];
  p->dgrad_ok = !h[2];
  p->bands_ok = !h[3];
  p->stages_out = h[4];
  p->stages_in = h[5];
  for (int d = 0; d < 2; ++d) {
    p->halo[d].ok = p->halo[d].order != nullptr && !h[6 + 2 * d];
    p->halo[d].extra_rounds = h[7 + 2 * d];
  }
  // The pair view, for maps sparse enough that some layer would take it (fp32 layers prefer
  // it from about 1 + 45 / channels row slots per pair on, never below 1.4): built after the
  // counts are known, with a synchronisation of its own, so that dense maps pay nothing.
  static const bool pair_view = !(getenv("FGMS_PAIR_VIEW") && atoi(getenv("FGMS_PAIR_VIEW")) == 0);
  const int most = p->stages_out > p->stages_in ? p->stages_out : p->stages_in;
  if (pair_view && k_vol <= 64 && n_pairs > 0 &&
      (kernel_policy() == 5 || (double)most * 64.0 >= 1.35 * (double)n_pairs)) {
    p->pv_rows = (n_pairs + 64 * (int64_t)k_vol + 255) / 256 * 256;
    if (pool_alloc((void **)&p->pv_in, (size_t)p->pv_rows * sizeof(int32_t), s) != FGMS_OK ||
        pool_alloc((void **)&p->pv_out, (size_t)p->pv_rows * sizeof(int32_t), s) != FGMS_OK ||
        pool_alloc((void **)&p->pv_mask, (size_t)(p->pv_rows / 64) * sizeof(unsigned long long), s) != FGMS_OK) {
      set_error("fgms_plan_create: pair view allocation failed");
      return fail(FGMS_E_NOMEM);
    }
    if ((rc = fill_i32(p->pv_in, (size_t)p->pv_rows, -1, s)) || (rc = fill_i32(p->pv_out, (size_t)p->pv_rows, -1, s)) ||
        (rc = fill_i32((int32_t *)p->pv_mask, (size_t)(p->pv_rows / 64) * 2, 0, s)))
      return fail(rc);
    pair_view_kernel<<<(unsigned)((n_pairs + 255) / 256), 256, 0, s>>>(kpos, in_map, out_map, k_vol, (int)n_pairs,
                                                                      (long long)p->pv_rows, p->pv_in, p->pv_out,
                                                                      p->pv_mask);
    if (hipGetLastError() != hipSuccess || hipStreamSynchronize(s) != hipSuccess) {
      set_error("fgms_plan_create: pair view build failed");
      return fail(FGMS_E_HIP);
    }
  }
  *plan_out = (fgms_plan_t *)p;
  return FGMS_OK;
}
}  // namespace fgms

extern "C" {

int fgms_plan_create(fgms_plan_t **plan_out, const int32_t *kpos, const int32_t *in_map,
                     const int32_t *out_map, int64_t n_in, int64_t n_out, int k_vol,
                     int64_t n_pairs, void *stream) {
  return plan_create(plan_out, kpos, in_map, out_map, n_in, n_out, k_vol, n_pairs, nullptr, nullptr, 0, stream);
}

int fgms_plan_create_coords(fgms_plan_t **plan_out, const int32_t *kpos, const int32_t *in_map,
                            const int32_t *out_map, int64_t n_in, int64_t n_out, int k_vol,
                            int64_t n_pairs, const int32_t *in_coords, const int32_t *out_coords,
                            int coord_bits, void *stream) {
  if ((n_in > 0 && !in_coords) || (n_out > 0 && !out_coords) || coord_bits < 0 || coord_bits > 21) {
    set_error("fgms_plan_create_coords: null coordinates or coord_bits outside 0..21");
    return FGMS_E_INVALID;
  }
  return plan_create(plan_out, kpos, in_map, out_map, n_in, n_out, k_vol, n_pairs, in_coords, out_coords,
                     coord_bits, stream);
}

void fgms_plan_destroy(fgms_plan_t *plan) {
  Plan *p = (Plan *)plan;
  if (!p) return;
  halo_release(p);
  if (p->nbr_out) pool_free(p->nbr_out, p->last_stream, false);
  if (p->nbr_in) pool_free(p->nbr_in, p->last_stream, false);
  if (p->mask_out) pool_free(p->mask_out, p->last_stream, false);
  if (p->mask_in) pool_free(p->mask_in, p->last_stream, false);
  if (p->perm_out) pool_free(p->perm_out, p->last_stream, false);
  if (p->perm_in) pool_free(p->perm_in, p->last_stream, false);
  if (p->band_start) pool_free(p->band_start, p->last_stream, false);
  if (p->band_cells) pool_free(p->band_cells, p->last_stream, false);
  if (p->tile_out) pool_free(p->tile_out, p->last_stream, false);
  if (p->tile_in) pool_free(p->tile_in, p->last_stream, false);
  if (p->pv_in) pool_free(p->pv_in, p->last_stream, false);
  if (p->pv_out) pool_free(p->pv_out, p->last_stream, false);
  if (p->pv_mask) pool_free(p->pv_mask, p->last_stream, false);
  delete p;
}

int fgms_plan_usable(const fgms_plan_t *plan, int for_dgrad) {
  const Plan *p = (const Plan *)plan;
  if (!p) return 0;
  return for_dgrad ? (p->dgrad_ok ? 1 : 0) : (p->fwd_ok ? 1 : 0);
}

int fgms_plan_stats(const fgms_plan_t *plan, int64_t stats[4]) {
  const Plan *p = (const Plan *)plan;
  if (!p || !stats) {
    set_error("fgms_plan_stats: null argument");
    return FGMS_E_INVALID;
  }
  stats[0] = p->n_pairs;
  stats[1] = p->stages_out;
  stats[2] = p->stages_in;
  stats[3] = p->pv_in ? p->pv_rows : 0;
  return FGMS_OK;
}

}  // extern "C"
