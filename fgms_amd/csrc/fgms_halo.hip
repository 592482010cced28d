// Output-stationary gather-GEMM-scatter with the tile's neighbourhood resident in LDS.
//
// On voxel clouds the rows gathered for a tile of neighbouring destination rows overlap
// heavily: 128 spatially compact rows of a surface-like cloud issue ~1 350 row gathers over
// their 27 offsets but touch only ~210 distinct source rows.  The reference re-gathers a
// row for every offset and every column tile that uses it (backend/spconv.cuh:1397-1449,
// backend/fwd_kernels.cuh:95-97); the kernel here brings every distinct row of a tile into
// LDS once and serves all offsets from there:
//
//   * plan side (halo_build_kernel): destination rows are taken in a spatially compact
//     order (Morton order of the voxel coordinates the caller supplies), cut into tiles of
//     128, and every tile gets the sorted list of the distinct source rows its pairs read
//     ("neighbourhood") plus, per (offset, row), the 16-bit position of the neighbour in
//     that list;
//   * kernel side (gms_halo_kernel): a workgroup streams its tile's neighbourhood into LDS
//     with direct global -> LDS loads (128-byte rows, XOR-swizzled by row); its waves then
//     split the tile's offsets among themselves (see the kernel).
//
// A neighbourhood larger than the LDS window is worked off in rounds of kHaloCap rows (the
// accumulators persist, lanes whose neighbour is not resident read a row of zeros).
//
// Measured on MI355X, 64 -> 64 fp16 over 200 k voxels (2.1 M pairs): 57 us per pass against
// 50 us for the kernel that gathers per pair (gms_rows_kernel).  It brings a sixth of the row
// bytes into the CU (42 MB of neighbourhood rows against 270 MB of gathers) and reads half as
// much from HBM (FETCH_SIZE 64 MB against 138 MB, L2 hit rate 85 % against 69 %), but with tiles
// of 128 rows an offset's 8 KB of weights serve only 128 rows, 225 MB of weight reads per
// pass against 84 MB, so the L1 asks the L2 for about as much as before (TCP_TCC_READ_REQ
// 2.8 M against 3.1 M), and with 128 accumulator registers a CU holds 8 waves: a tile's 14 us
// are mostly memory round trips those few waves cannot cover (neighbourhood load 2.9 us, the
// offsets' weight fetches 8 us for 1.9 us of MFMA work, reduction and row update 3.5 us).
// Tiles of 256 rows halve the weight reads but need 256 accumulator registers per wave or
// rows split over more waves, which was measured too (64 - 66 us: waves own rows, an offset's
// weights pass through LDS behind a workgroup barrier per offset).
// Weight-stationary variants (one persistent workgroup per CU that keeps every offset's B
// fragments in registers for the whole launch, so that a tile brings in nothing but its
// neighbourhood rows; next tile's rows streamed into a second LDS buffer meanwhile; the waves
// split the offsets, k mod 4, and their partial tiles meet in LDS) were measured too:
//   * 8 waves (offset group x column half, 112 fragment registers each): 60 - 78 us.  Both
//     column halves read the same A fragments, and with 16 waves' worth of 16-byte row reads
//     per 128 MFMA clocks the LDS is the limit, not the matrix pipe.
//   * 4 waves with 512 registers each (224 fragment registers, held in the accumulation
//     register file through register constraints and hand-written MFMAs, since the compiler
//     spills MFMA B operands rather than place them there; A fragments read from inline
//     assembly one 32-row block ahead of their products): parity-exact, 71 us.  Without the
//     products 41 us, without the reduction and row update 55 us: a (offset, block) step takes
//     about 600 clocks against 256 of MFMA issue with a single wave per SIMD to cover LDS
//     latency, the four partial tiles cost 128 four-byte LDS writes per wave and three barriers
//     per tile (2.7 us), and with 6.1 tiles per workgroup and 2 x different tile lengths the
//     static tile runs end 25 % apart.
//   * the first attempt combined the partial tiles with ds_add_f32 (about a lane per clock):
//     620 us.
// 27 offsets x 64 x 64 weights fill the registers of a CU; nothing is left to hide latency with.
// So this path is opt-in: the tables are built by fgms_plan_create_coords only, and the
// kernel runs under kernel policy 6 only.
#include <stdlib.h>

#include <type_traits>

#include <rocprim/device/device_radix_sort.hpp>

#include "fgms_device.h"
#include "fgms_internal.h"
#include "fgms_mma.h"
#include "fgms_tile_ops.h"

namespace fgms {
namespace {

constexpr int kHaloTile = 128;    // destination rows per tile (4 blocks of 32)
constexpr int kHaloCap = 352;     // neighbourhood rows resident in LDS per round
constexpr int kHaloThreads = 256; // the kernel's workgroup
constexpr int kBuildThreads = kHaloTile;   // the plan kernel's: one thread per position of a tile
constexpr int kHashSlots = 8192;  // >= 64 offsets x 128 rows; 27 x 256 = 6 912 keys fit too
constexpr unsigned short kNoNbr = 0xFFFF;

// Where the neighbour-list position of (tile, offset k, position t of the tile) sits in the
// table: the four 32-row blocks' entries of one row-of-block next to each other, so that an
// MFMA lane (row t % 32 of every block) fetches its four entries of an offset in one 8-byte load.
__host__ __device__ __forceinline__ size_t lnbr_slot(int tile, int k_vol, int k, int t) {
  return (((size_t)tile * k_vol + k) * 32 + t % 32) * 4 + t / 32;
}

// ---------------------------------------------------------------------------------------
// Row orders.

// Morton key of a voxel: the low `bits` bits of each (biased) coordinate interleaved.
__device__ __forceinline__ unsigned long long spread3(unsigned long long v) {
  v &= 0x1FFFFFull;
  v = (v | (v << 32)) & 0x1F00000000FFFFull;
  v = (v | (v << 16)) & 0x1F0000FF0000FFull;
  v = (v | (v << 8)) & 0x100F00F00F00F00Full;
  v = (v | (v << 4)) & 0x10C30C30C30C30C3ull;
  v = (v | (v << 2)) & 0x1249249249249249ull;
  return v;
}

__global__ void morton_keys_kernel(const int32_t *__restrict__ coords, int n, int bias,
                                   unsigned long long *__restrict__ keys, int32_t *__restrict__ rows) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const unsigned long long x = (unsigned)(coords[3 * i] + bias), y = (unsigned)(coords[3 * i + 1] + bias),
                           z = (unsigned)(coords[3 * i + 2] + bias);
  keys[i] = (spread3(x) << 2) | (spread3(y) << 1) | spread3(z);
  rows[i] = i;
}

__global__ void invert_order_kernel(const int32_t *__restrict__ order, int n, int32_t *__restrict__ inv) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p < n) inv[order[p]] = p;
}

// ---------------------------------------------------------------------------------------
// One workgroup per tile of kHaloTile positions: (optionally) sorts the tile's rows by offset
// mask, lists the distinct source rows of the tile in source-position order and renumbers
// the neighbour table in positions of that list.
//   nbr       [k_vol][n_dst]  by the plan's POSITION of the destination row: source row or -1
//   plan_pos  [n_dst]         destination row -> that position (nullptr: identity)
//   order_dst [n_dst]         position -> destination row (nullptr: identity)
//   inv_src   [n_src]         source row -> source position (nullptr: identity)
//   order_src [n_src]         source position -> source row (nullptr: identity)
// out: order_pad [n_tiles * kHaloTile], rows [n_tiles][list_cap], count [n_tiles],
//      lnbr [n_tiles][k_vol][32][4] (see lnbr_slot), mask32 [n_tiles * kHaloTile / 32];
//      flags[0] = 1 if some list did not fit, flags[1] += rounds beyond the first.
__global__ __launch_bounds__(kBuildThreads) void halo_build_kernel(
    const int32_t *__restrict__ nbr, const int32_t *__restrict__ plan_pos, const int32_t *__restrict__ order_dst,
    const int32_t *__restrict__ inv_src, const int32_t *__restrict__ order_src, int n_dst, int k_vol,
    int sort_by_mask, int list_cap, int32_t *__restrict__ order_pad, int32_t *__restrict__ rows,
    int32_t *__restrict__ count, unsigned short *__restrict__ lnbr,
    unsigned long long *__restrict__ mask32, int *__restrict__ flags) {
  __shared__ int table[kHashSlots];
  __shared__ int list[1024];
  __shared__ unsigned long long skey[kHaloTile];
  __shared__ int sval[kHaloTile];
  __shared__ int n_list;
  const int tid = threadIdx.x, tile = blockIdx.x;
  const int n_pad = gridDim.x * kHaloTile;
  const int p = tile * kHaloTile + tid;
  int row = p < n_dst ? (order_dst ? order_dst[p] : p) : -1;
  int col = row >= 0 ? (plan_pos ? plan_pos[row] : row) : 0;      // the row's column of the table
  for (int i = tid; i < kHashSlots; i += kBuildThreads) table[i] = -1;
  for (int i = tid; i < 1024; i += kBuildThreads) list[i] = INT32_MAX;
  if (tid == 0) n_list = 0;
  if (sort_by_mask) {
    // rows with the same set of offsets next to each other: a 32-row block then skips the
    // offsets none of its rows uses.  Ties keep their order (the key carries the position).
    unsigned long long m = 0;
    for (int k = 0; k < k_vol; ++k)
      if (row >= 0 && nbr[(size_t)k * n_dst + col] >= 0) m |= 1ull << k;
    skey[tid] = row >= 0 ? m : ~0ull;
    sval[tid] = row;
    __syncthreads();
    // bitonic sort of (mask, original position): one element per thread
    __shared__ int spos[kHaloTile];
    spos[tid] = tid;
    __syncthreads();
    for (int k2 = 2; k2 <= kHaloTile; k2 <<= 1)
      for (int j = k2 >> 1; j > 0; j >>= 1) {
        const int o = tid ^ j;
        if (o > tid) {
          const bool asc = (tid & k2) == 0;
          const unsigned long long a = skey[tid], b = skey[o];
          const int pa = spos[tid], pb = spos[o];
          const bool gt = a > b || (a == b && pa > pb);
          if (gt == asc) {
            skey[tid] = b; skey[o] = a;
            spos[tid] = pb; spos[o] = pa;
            const int va = sval[tid];
            sval[tid] = sval[o]; sval[o] = va;
          }
        }
        __syncthreads();
      }
    row = sval[tid];
    col = row >= 0 ? (plan_pos ? plan_pos[row] : row) : 0;
  }
  order_pad[p] = row;
  __syncthreads();
  // distinct source positions of the tile
  for (int k = 0; k < k_vol; ++k) {
    const int g = row >= 0 ? nbr[(size_t)k * n_dst + col] : -1;
    if (g < 0) continue;
    const int key = inv_src ? inv_src[g] : g;
    unsigned slot = ((unsigned)key * 2654435761u) >> 19;       // 13 bits
    while (true) {
      const int old = atomicCAS(&table[slot], -1, key);
      if (old == -1 || old == key) break;
      slot = (slot + 1) & (kHashSlots - 1);
    }
  }
  __syncthreads();
  for (int i = tid; i < kHashSlots; i += kBuildThreads) {
    const int key = table[i];
    if (key >= 0) {
      const int j = atomicAdd(&n_list, 1);
      if (j < 1024) list[j] = key;
    }
  }
  __syncthreads();
  const int u = n_list;
  if (u > list_cap || u > 1024) {
    if (tid == 0) {
      flags[0] = 1;
      count[tile] = 0;
    }
    for (int k = 0; k < k_vol; ++k) lnbr[lnbr_slot(tile, k_vol, k, tid)] = kNoNbr;
    if (tid % 32 == 0) mask32[p / 32] = 0;
    return;
  }
  // sort the list (bitonic over the next power of two, >= 256)
  int n2 = 256;
  while (n2 < u) n2 <<= 1;
  for (int k2 = 2; k2 <= n2; k2 <<= 1)
    for (int j = k2 >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < n2; i += kBuildThreads) {
        const int o = i ^ j;
        if (o > i) {
          const bool asc = (i & k2) == 0;
          const int a = list[i], b = list[o];
          if ((a > b) == asc) {
            list[i] = b;
            list[o] = a;
          }
        }
      }
      __syncthreads();
    }
  // (padded to a multiple of 8 with the last row: the kernels fetch row numbers in groups of 8)
  for (int i = tid; i < min((u + 7) / 8 * 8, list_cap); i += kBuildThreads) {
    const int key = list[min(i, u - 1)];
    rows[(size_t)tile * list_cap + i] = order_src ? order_src[key] : key;
  }
  if (tid == 0) {
    count[tile] = u;
    const int extra = (u + kHaloCap - 1) / kHaloCap - 1;
    if (extra > 0) atomicAdd(&flags[1], extra);
  }
  // neighbour table in list positions, and the 32-row blocks' offset masks
  unsigned long long mine = 0;
  for (int k = 0; k < k_vol; ++k) {
    const int g = row >= 0 ? nbr[(size_t)k * n_dst + col] : -1;
    unsigned short lid = kNoNbr;
    if (g >= 0) {
      const int key = inv_src ? inv_src[g] : g;
      int lo = 0, hi = u - 1;
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (list[mid] < key) lo = mid + 1; else hi = mid;
      }
      lid = (unsigned short)lo;
    }
    lnbr[lnbr_slot(tile, k_vol, k, tid)] = lid;
    const unsigned long long b = __ballot(g >= 0);
    const unsigned half = (tid & 32) ? (unsigned)(b >> 32) : (unsigned)b;
    if (half) mine |= 1ull << k;
  }
  if (tid % 32 == 0) mask32[p / 32] = mine;
}

// ---------------------------------------------------------------------------------------
// The kernel.  fp16, 64 source channels (one 128-byte row per voxel), 64 destination
// channels per workgroup (blockIdx.y walks wider layers).  A workgroup (4 waves) owns a tile
// of 128 destination rows = 4 blocks of 32.
//
// The waves split the tile's OFFSETS, not its rows: a wave draws an offset from the
// workgroup's queue, brings that offset's 64 x 64 weights into registers as MFMA B fragments
// (through 8 KB of LDS of its own, which does the transposition the forward pass needs) and
// applies them to every 32-row block of the tile that uses the offset; the A operand of a
// block is a gather of 16-byte chunks out of the LDS-resident neighbourhood.  So the weights
// of an offset are read once per tile, an offset's fragments serve up to four blocks from
// registers, and between the barrier that closes the neighbourhood load and the one that opens
// the reduction no wave waits for another.  Each wave ends up with a partial sum of the whole
// 128 x 64 result tile (128 accumulator registers); the four partial tiles are added through
// LDS (which the neighbourhood no longer needs) and every destination row is updated once.
//
// RAW = 1: forward, weights W[k][cs][cd] contracted over their rows (transposing LDS reads);
// RAW = 2: input gradient, contracted over their columns (a fragment is one 16-byte piece).
constexpr int kBlocks = kHaloTile / 32;
constexpr int kRedStride = 68;       // floats per row of a partial tile in LDS (64 + padding)

template <int RAW>
__global__ __launch_bounds__(kHaloThreads, 2) void gms_halo_kernel(
    const __half *__restrict__ src, const __half *__restrict__ w, __half *__restrict__ dst,
    const int32_t *__restrict__ order, const int32_t *__restrict__ hrows,
    const int32_t *__restrict__ hcount, const unsigned short *__restrict__ lnbr,
    const unsigned long long *__restrict__ mask32, int n_tiles, int list_cap, int k_vol, int c_dst,
    int w_rows, int w_cols) {
  constexpr int S = 4, NT = 2, C = 8;
  constexpr int WCH = 512;                    // 16-byte chunks of one offset's 64 x 64 weights
  extern __shared__ int4v lds[];
  __shared__ int next_offset;
  int4v *halo = lds;                                  // [kHaloCap + 1][8], the last row is zeros
  int4v *stage_all = lds + (kHaloCap + 1) * C;        // [4 waves][WCH]
  int *didx = reinterpret_cast<int *>(stage_all + 4 * WCH);   // [128]
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);     // (wave-uniform, and the compiler knows it)
  const int r = lane % 32, h = lane / 32;
  // consecutive tiles share neighbourhood rows: an XCD (workgroup index mod 8) takes a
  // contiguous eighth of the tiles, so that those rows meet in one L2
  const int per_xcd = (n_tiles + 7) / 8;
  const int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if ((int)(blockIdx.x / 8) >= per_xcd || tile >= n_tiles) return;
  const int p0 = tile * kHaloTile;
  const int cd0 = blockIdx.y * 64;
  const int count = hcount[tile];
  unsigned long long m[kBlocks];
#pragma unroll
  for (int b = 0; b < kBlocks; ++b) m[b] = mask32[p0 / 32 + b];
  unsigned long long all = 0;
#pragma unroll
  for (int b = 0; b < kBlocks; ++b) all |= m[b];
  if (!all) return;
  if (tid < kHaloTile) didx[tid] = order[p0 + tid];
  if (tid < C) halo[kHaloCap * C + tid] = int4v{0, 0, 0, 0};
  // The tile's offsets in the order the waves draw them: those that touch most blocks first
  // (the longest jobs start first).  Lane k of every wave ranks offset k; the i-th offset of
  // the order is then the lane whose rank is i.
  const int n_offsets = __builtin_popcountll(all);
  int my_blocks = 0;
#pragma unroll
  for (int b = 0; b < kBlocks; ++b) my_blocks += (int)((m[b] >> lane) & 1);
  int my_rank = 0;
#pragma unroll
  for (int want = kBlocks; want >= 1; --want) {
    const unsigned long long same = __ballot(my_blocks == want);
    if (want > my_blocks) my_rank += __builtin_popcountll(same);
    else if (want == my_blocks) my_rank += __builtin_popcountll(same & ((1ull << lane) - 1));
  }
  auto offset_at = [&](int i) {
    const unsigned long long hit = __ballot(my_blocks > 0 && my_rank == i);
    return i < n_offsets ? (int)__builtin_ctzll(hit) : -1;
  };

  float16v acc[kBlocks][NT];
#pragma unroll
  for (int b = 0; b < kBlocks; ++b)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[b][nt][i] = 0.f;

  // an offset's weights: 512 chunks, eight per lane (chunk e = lane + 64 i: row e / 8, piece e % 8)
  int4v *stage = stage_all + wave * WCH;
  const int w_row0 = lane / C, w_c = lane % C;
  // RAW = 1: rows cs of W[k], the 64 columns from cd0 on; RAW = 2: rows ci = cd0 + row, all 64 columns co
  const int w_off0 = RAW == 1 ? w_row0 * w_cols + cd0 + w_c * 8 : (cd0 + w_row0) * w_cols + w_c * 8;
  const size_t w_per_k = (size_t)w_rows * w_cols;
  auto weights_issue = [&](int4v (&wraw)[8], int k) {
    const __half *wk = w + (size_t)k * w_per_k + w_off0;
#pragma unroll
    for (int i = 0; i < 8; ++i) wraw[i] = *reinterpret_cast<const int4v *>(wk + (size_t)i * 8 * w_cols);
  };
  // registers -> this wave's LDS tile -> B fragments bf[s][nt]
  auto weights_fragments = [&](const int4v (&wraw)[8], int4v (&bf)[S][NT]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = w_row0 + 8 * i;
      if constexpr (RAW == 1) stage[row * C + (w_c ^ raw_swizzle<NT>(row))] = wraw[i];
      else stage[a_slot<S>(row, w_c)] = wraw[i];
    }
    wave_lds_fence();
#pragma unroll
    for (int s = 0; s < S; ++s)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        if constexpr (RAW == 1) bf[s][nt] = raw_weight_frag<NT, S>(stage, s, nt, lane);
        else bf[s][nt] = stage[a_slot<S>(nt * 32 + r, h * S + s)];
      }
    wave_lds_fence();
  };
  auto idx_issue = [&](int (&ix)[kBlocks], int k) {
    typedef unsigned short ushort4v __attribute__((ext_vector_type(4)));
    const ushort4v e = *reinterpret_cast<const ushort4v *>(lnbr + lnbr_slot(tile, k_vol, k, r));
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) ix[b] = e[b];
  };
  auto grab = [&]() {
    int i = 0;
    if (lane == 0) i = atomicAdd(&next_offset, 1);
    i = __builtin_amdgcn_readfirstlane(i);
    return offset_at(i);
  };

  const int32_t *my_rows = hrows + (size_t)tile * list_cap;
  for (int base = 0; base < count; base += kHaloCap) {
    const int nrows = min(kHaloCap, count - base);
    if (base > 0) __syncthreads();        // everybody is done with the previous round's rows
    if (tid == 0) next_offset = 4;          // (the waves' first offsets are numbers 0 .. 3 of the order)
    // the round's rows -> LDS, 8 rows (64 lanes x 16 bytes) per instruction; chunk c of row l
    // lands at slot l * 8 + (c ^ (l & 7)).  The row numbers of all of this wave's instructions
    // (j = wave + 4 i) come in two loads (lane L holds the row of instruction i = L / 8 (+ 8),
    // sub-row L % 8); each instruction picks its eight numbers out of those registers with a
    // lane permute, so that no load waits on another.
    const int n_inst = (nrows + 7) / 8;
    constexpr int kPerWave = (kHaloCap / 8 + 3) / 4;
    static_assert(kPerWave <= 16, "two index loads per lane cover a wave's rows");
    const int ia = my_rows[base + min((wave + 4 * (lane / 8)) * 8 + lane % 8, nrows - 1)];
    const int ib = my_rows[base + min((wave + 4 * (8 + lane / 8)) * 8 + lane % 8, nrows - 1)];
    // this wave's first offset: its weights and indices are requested before the rows
    int k = offset_at(wave);
    int4v wraw[8];
    int ix[kBlocks];
    {
      const int kf = k >= 0 ? k : __builtin_ctzll(all);
      weights_issue(wraw, kf);
      idx_issue(ix, kf);
    }
    {
      int g[kPerWave];
#pragma unroll
      for (int i = 0; i < kPerWave; ++i) g[i] = __shfl(i < 8 ? ia : ib, (i % 8) * 8 + lane / 8);
#pragma unroll
      for (int i = 0; i < kPerWave; ++i) {
        const int j = wave + 4 * i;
        if (j < n_inst) {
          const int lrow = j * 8 + lane / 8;
          const int c = (lane % 8) ^ (lrow & 7);
          const __half *gsrc = src + (size_t)g[i] * 64 + c * 8;
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gsrc,
                                           (__attribute__((address_space(3))) void *)(halo + j * 64), 16, 0, 0);
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);    // vmcnt(0): this wave's direct-to-LDS loads have landed
    __syncthreads();

    // this wave's offsets
    if (k >= 0) {
      int4v bf[S][NT];
      int al[kBlocks];
      auto resolve = [&]() {
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
          const int l = ix[b] - base;
          al[b] = (unsigned)l < (unsigned)nrows ? l : kHaloCap;    // not resident (or no neighbour): zeros
        }
      };
      weights_fragments(wraw, bf);
      resolve();
      while (true) {
        const int kn = grab();
        {
          // (unconditional, past the last offset a repeat of the current one: a load under a
          // branch would make every later use wait for all loads in flight)
          const int kf = kn >= 0 ? kn : k;
          weights_issue(wraw, kf);
          idx_issue(ix, kf);
        }
        {
#pragma unroll
          for (int b = 0; b < kBlocks; ++b) {
            if ((m[b] >> k) & 1) {
              const int4v *ra = halo + al[b] * C;
              const int x = al[b] & 7;
              int4v fa[S];
#pragma unroll
              for (int s = 0; s < S; ++s) fa[s] = ra[(h * S + s) ^ x];
#pragma unroll
              for (int s = 0; s < S; ++s)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) mma<__half>(acc[b][nt], fa[s], bf[s][nt]);
            }
          }
        }
        if (kn < 0) break;
        weights_fragments(wraw, bf);
        resolve();
        k = kn;
      }
    }
  }
  // The four partial tiles meet in LDS, 64 rows at a time; wave w then owns rows 16 w .. 16 w + 15
  // of those 64: four 16-byte pieces per lane, 16 lanes to a 128-byte destination row.
  float *red = reinterpret_cast<float *>(lds);
  float *mine = red + wave * 64 * kRedStride;
  typedef _Float16 half4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    __syncthreads();          // the neighbourhood rows (or the previous half's tiles) are dead
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          mine[(j * 32 + (i / 4) * 8 + h * 4 + i % 4) * kRedStride + nt * 32 + r] = acc[2 * half + j][nt][i];
    // the old values of this wave's destination rows, requested before the barrier
    int drow[4];
    half4 old[4];
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int e = it * 64 + lane;
      drow[it] = didx[half * 64 + wave * 16 + e / 16];
      old[it] = *reinterpret_cast<const half4 *>(reinterpret_cast<const _Float16 *>(dst) +
                                                 (size_t)max(drow[it], 0) * c_dst + cd0 + (e % 16) * 4);
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int e = it * 64 + lane;
      const float *p = red + (wave * 16 + e / 16) * kRedStride + (e % 16) * 4;
      float4v sum = *reinterpret_cast<const float4v *>(p);
#pragma unroll
      for (int q = 1; q < 4; ++q) sum += *reinterpret_cast<const float4v *>(p + q * 64 * kRedStride);
      half4 out;
#pragma unroll
      for (int q = 0; q < 4; ++q) out[q] = (_Float16)((float)old[it][q] + sum[q]);
      if (drow[it] >= 0)
        *reinterpret_cast<half4 *>(reinterpret_cast<_Float16 *>(dst) + (size_t)drow[it] * c_dst + cd0 + (e % 16) * 4) = out;
    }
  }
}

constexpr size_t kHaloLds = (size_t)((kHaloCap + 1) * 8 + 4 * 512) * 16 + kHaloTile * sizeof(int);
static_assert(4 * 64 * kRedStride * sizeof(float) <= (size_t)((kHaloCap + 1) * 8 + 4 * 512) * 16,
              "the four partial tiles fit the LDS of the neighbourhood and the weight tiles");

bool halo_enabled() {
  static const bool on = !(getenv("FGMS_HALO") && atoi(getenv("FGMS_HALO")) == 0);
  return on;
}

}  // namespace

void halo_release(Plan *p) {
  for (int d = 0; d < 2; ++d) {
    HaloSide &hs = p->halo[d];
    if (hs.order) pool_free(hs.order, p->last_stream, false);
    if (hs.rows) pool_free(hs.rows, p->last_stream, false);
    if (hs.count) pool_free(hs.count, p->last_stream, false);
    if (hs.lnbr) pool_free(hs.lnbr, p->last_stream, false);
    if (hs.mask32) pool_free(hs.mask32, p->last_stream, false);
    hs = HaloSide{};
  }
}

// Morton order of `n` voxels: order[position] = row, inv[row] = position (pooled blocks the
// caller frees; `tmp` collects the sort's temporaries, freed by the caller once the stream
// has passed them).
int halo_morton_order(const int32_t *coords, int64_t n, int coord_bits, int32_t **order, int32_t **inv,
                      std::vector<void *> *tmp, hipStream_t s) {
  *order = *inv = nullptr;
  if (n == 0) return FGMS_OK;
  unsigned long long *keys = nullptr, *keys_out = nullptr;
  int32_t *rows_in = nullptr;
  void *sort_tmp = nullptr;
  size_t sort_bytes = 0;
  const int bits = coord_bits > 0 && coord_bits <= 21 ? coord_bits : 21;
  const int bias = coord_bits > 0 && coord_bits <= 21 ? 0 : 1 << 20;
  auto take = [&](void **q, size_t bytes) {
    if (pool_alloc(q, bytes, s) != FGMS_OK) return false;
    tmp->push_back(*q);
    return true;
  };
  if (!take((void **)&keys, (size_t)n * 8) || !take((void **)&keys_out, (size_t)n * 8) ||
      !take((void **)&rows_in, (size_t)n * 4) || !take((void **)order, (size_t)n * 4) ||
      !take((void **)inv, (size_t)n * 4)) {
    set_error("halo_morton_order: allocation failed");
    return FGMS_E_NOMEM;
  }
  if (rocprim::radix_sort_pairs(nullptr, sort_bytes, keys, keys_out, rows_in, *order, (size_t)n, 0u,
                                (unsigned)(3 * bits), s) != hipSuccess ||
      !take(&sort_tmp, sort_bytes ? sort_bytes : 256)) {
    set_error("halo_morton_order: sort set-up failed");
    return FGMS_E_NOMEM;
  }
  morton_keys_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(coords, (int)n, bias, keys, rows_in);
  if (rocprim::radix_sort_pairs(sort_tmp, sort_bytes, keys, keys_out, rows_in, *order, (size_t)n, 0u,
                                (unsigned)(3 * bits), s) != hipSuccess) {
    set_error("halo_morton_order: sort failed");
    return FGMS_E_HIP;
  }
  invert_order_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(*order, (int)n, *inv);
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

// Builds direction d of the plan's tile tables (0: forward, destination = output rows;
// 1: input gradient, destination = input rows) from the plan's neighbour table.
// flags: two device ints, zeroed by the caller (see halo_build_kernel).
int halo_build(Plan *p, int d, const int32_t *nbr_by_pos, const int32_t *plan_pos, const int32_t *order_dst,
               const int32_t *inv_src, const int32_t *order_src, int *flags, hipStream_t s) {
  HaloSide &hs = p->halo[d];
  hs = HaloSide{};
  const int64_t n_dst = d ? p->n_in : p->n_out;
  if (!halo_enabled() || !order_dst || p->k_vol > 64 || n_dst == 0) return FGMS_OK;
  static const int sort_by_mask = getenv("FGMS_HALO_SORT") ? atoi(getenv("FGMS_HALO_SORT")) : 1;
  hs.n_tiles = (int)((n_dst + kHaloTile - 1) / kHaloTile);
  hs.list_cap = 1024;
  const size_t n_pad = (size_t)hs.n_tiles * kHaloTile;
  if (pool_alloc((void **)&hs.order, n_pad * sizeof(int32_t), s) != FGMS_OK ||
      pool_alloc((void **)&hs.rows, (size_t)hs.n_tiles * hs.list_cap * sizeof(int32_t), s) != FGMS_OK ||
      pool_alloc((void **)&hs.count, (size_t)hs.n_tiles * sizeof(int32_t), s) != FGMS_OK ||
      pool_alloc((void **)&hs.lnbr, (size_t)p->k_vol * n_pad * sizeof(unsigned short), s) != FGMS_OK ||
      pool_alloc((void **)&hs.mask32, n_pad / 32 * sizeof(unsigned long long), s) != FGMS_OK) {
    set_error("halo_build: table allocation failed");
    return FGMS_E_NOMEM;
  }
  halo_build_kernel<<<(unsigned)hs.n_tiles, kBuildThreads, 0, s>>>(
      nbr_by_pos, plan_pos, order_dst, inv_src, order_src, (int)n_dst, p->k_vol, sort_by_mask, hs.list_cap, hs.order,
      hs.rows, hs.count, hs.lnbr, hs.mask32, flags);
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

bool halo_gms_supported(const GmsArgs &a, const Plan *p) {
  if (!p || !halo_enabled() || a.dense_k >= 0 || a.k_vol != p->k_vol || a.dtype != FGMS_F16) return false;
  const HaloSide &hs = p->halo[a.transpose_w ? 1 : 0];
  if (!hs.ok || a.prepacked || a.side.kind) return false;
  if (a.transpose_w ? (!p->dgrad_ok || a.n_dst != p->n_in || a.n_src != p->n_out)
                    : (!p->fwd_ok || a.n_dst != p->n_out || a.n_src != p->n_in))
    return false;
  const int c_src = a.transpose_w ? a.c_out : a.c_in, c_dst = a.transpose_w ? a.c_in : a.c_out;
  if (c_src != 64 || c_dst % 64 != 0) return false;
  if (reinterpret_cast<uintptr_t>(a.src) % 16 || reinterpret_cast<uintptr_t>(a.dst) % 16 ||
      reinterpret_cast<uintptr_t>(a.w) % 16)
    return false;
  return true;
}

int launch_halo_gms(const GmsArgs &a, const Plan *p) {
  if (!halo_gms_supported(a, p)) {
    set_error("launch_halo_gms: unsupported shape or plan");
    return FGMS_E_INVALID;
  }
  const HaloSide &hs = p->halo[a.transpose_w ? 1 : 0];
  const int c_dst = a.transpose_w ? a.c_in : a.c_out;
  auto kern = a.transpose_w ? gms_halo_kernel<2> : gms_halo_kernel<1>;
  { const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(kern), (size_t)kHaloLds); if (rc_lds != FGMS_OK) return rc_lds; }
  const unsigned gx = (unsigned)((hs.n_tiles + 7) / 8 * 8);
  {
    ProfileScope prof(a.transpose_w ? "gms_halo_kernel(dgrad)" : "gms_halo_kernel(fwd)", a.stream);
    kern<<<dim3(gx, (unsigned)(c_dst / 64)), kHaloThreads, kHaloLds, a.stream>>>(
        (const __half *)a.src, (const __half *)a.w, (__half *)a.dst, hs.order, hs.rows, hs.count, hs.lnbr,
        hs.mask32, hs.n_tiles, hs.list_cap, a.k_vol, c_dst, a.c_in, a.c_out);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

}  // namespace fgms
