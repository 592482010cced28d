// Pair-stationary gather-GEMM-scatter for wide fp16 layers (256 destination channels per
// workgroup), every source row gathered once.
//
// The pair-stationary kernel of fgms_mfma.hip gives a workgroup 256 pairs x 64 destination
// columns, so a 256-column layer gathers every source row four times, and with the column
// block's weights of a whole offset resident in LDS a CU holds two workgroups of four waves:
// each of them waits out its weight load, its row gathers and its atomic updates with little
// to cover them.  Here a workgroup of 16 waves owns 256 pairs x 256 columns: wave (i, j)
// multiplies rows 64 i .. 64 i + 63 by columns 64 j .. 64 j + 63.  Source channels go through
// LDS in slabs of 64: the slab of the 256 gathered rows (32 KB, each row fetched once, by
// eight neighbouring lanes) and the slab of the offset's weights (32 KB, in MFMA fragment
// order), both double-buffered, one barrier per slab; the loads of the next slab, of the
// next tile if need be, are in flight while the current one is multiplied.  The reference
// re-gathers per column tile as well (backend/spconv.cuh:1397-1449 walks its 64- or
// 128-column blocks in blockIdx.y).
#include "fgms_device.h"
#include "fgms_internal.h"
#include "fgms_mma.h"
#include "fgms_tile_ops.h"

namespace fgms {
namespace {

constexpr int kWideRows = 256;       // pairs per tile
constexpr int kWideCols = 256;       // destination channels per workgroup
constexpr int kWideThreads = 1024;   // 16 waves
constexpr int kSlabChunks = kWideRows * 8;   // 16-byte chunks of a slab of rows, and of a slab of weights

__global__ __launch_bounds__(kWideThreads) void gms_wide_kernel(
    const __half *__restrict__ src, const int4v *__restrict__ packed, __half *__restrict__ dst,
    const int32_t *__restrict__ kpos, const int32_t *__restrict__ gmap,
    const int32_t *__restrict__ smap, int k_vol, int c_src, int c_dst, int tiles_per_wg,
    int dense_k, int dense_rows) {
  constexpr int S = 4;
  extern __shared__ int4v lds[];
  int4v *a_buf = lds;                              // [2][4 row groups][512]
  int4v *w_buf = lds + 2 * kSlabChunks;            // [2][4 k-steps][8 column tiles][64]
  int *gidx = reinterpret_cast<int *>(lds + 4 * kSlabChunks);   // [2][256]
  int *sidx = gidx + 2 * kWideRows;                               // [2][256]
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
  const int rg = wave / 4, cg = wave % 4;
  const int r = lane % 32, h = lane / 32;
  const int slabs = c_src / 64;
  const int nts = c_dst / 32;
  const int nt0 = blockIdx.y * (kWideCols / 32);
  const size_t packed_per_k = (size_t)c_src * c_dst / 8;   // chunks

  auto tile_at = [&](int t, int &k, int &first, int &count) {
    if (dense_k >= 0) {
      k = dense_k;
      first = t * kWideRows;
      count = min(kWideRows, dense_rows - first);
      return first < dense_rows;
    }
    return locate_tile(kpos, k_vol, kWideRows, t, k, first, count);
  };
  // the indices of a tile's pairs -> LDS (buffer `par`)
  auto load_indices = [&](int par, int first, int count) {
    if (tid < kWideRows) {
      const bool live = tid < count;
      const int j = first + tid;
      gidx[par * kWideRows + tid] = !live ? -1 : (gmap ? gmap[j] : j);
      sidx[par * kWideRows + tid] = !live ? -1 : (smap ? smap[j] : j);
    }
  };
  int4v av[2], wv[2];
  int ag[2];
  auto issue = [&](int par, int k, int slab) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int e = tid + kWideThreads * i;
      ag[i] = gidx[par * kWideRows + e / 8];
      av[i] = *reinterpret_cast<const int4v *>(src + (size_t)max(ag[i], 0) * c_src + slab * 64 + (e % 8) * 8);
      wv[i] = packed[packed_per_k * k + ((size_t)(slab * S + e / 512) * nts + nt0) * 64 + e % 512];
    }
  };
  auto commit = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int e = tid + kWideThreads * i;
      const int row = e / 8;
      a_buf[buf * kSlabChunks + (row / 64) * 512 + a_slot<S>(row % 64, e % 8)] =
          ag[i] < 0 ? int4v{0, 0, 0, 0} : av[i];
      w_buf[buf * kSlabChunks + e] = wv[i];
    }
  };

  float16v acc[2][2];
  auto clear = [&]() {
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;
  };
  clear();

  int t = blockIdx.x * tiles_per_wg;
  const int t_end = t + tiles_per_wg;
  int k, first, count;
  if (!tile_at(t, k, first, count)) return;
  load_indices(0, first, count);
  __syncthreads();
  issue(0, k, 0);
  commit(0);
  // the next tile, if this workgroup has one
  int kn = 0, firstn = 0, countn = 0;
  bool more = t + 1 < t_end && tile_at(t + 1, kn, firstn, countn);
  if (more) load_indices(1, firstn, countn);
  __syncthreads();

  int buf = 0, par = 0, slab = 0;
  while (true) {
    const bool last_slab = slab + 1 == slabs;
    const bool has_next = !last_slab || more;
    if (has_next) {
      if (last_slab) issue(par ^ 1, kn, 0);
      else issue(par, k, slab + 1);
    }
    {
      const int4v *al = a_buf + buf * kSlabChunks + rg * 512;
      const int4v *wl = w_buf + buf * kSlabChunks + cg * 128 + lane;
#pragma unroll
      for (int s = 0; s < S; ++s) {
        const int4v b0 = wl[s * 512], b1 = wl[s * 512 + 64];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const int4v a = al[a_slot<S>(mt * 32 + r, h * S + s)];
          mma<__half>(acc[mt][0], a, b0);
          mma<__half>(acc[mt][1], a, b1);
        }
      }
    }
    if (has_next) commit(buf ^ 1);
    if (last_slab) {
      write_tile<__half, 2, true>(acc, dst, sidx + par * kWideRows + rg * 64, c_dst, nt0 * 32 + cg * 64, lane);
      clear();
    }
    if (!has_next) break;
    __syncthreads();
    buf ^= 1;
    if (last_slab) {
      // on to the next tile; the indices of the one after it go to the buffer just released
      par ^= 1;
      slab = 0;
      k = kn;
      ++t;
      more = t + 1 < t_end && tile_at(t + 1, kn, firstn, countn);
      if (more) load_indices(par ^ 1, firstn, countn);
    } else {
      ++slab;
    }
  }
}

}  // namespace

bool wide_gms_supported(const GmsArgs &a) {
  const int c_src = a.transpose_w ? a.c_out : a.c_in;
  const int c_dst = a.transpose_w ? a.c_in : a.c_out;
  if (a.dtype != FGMS_F16 || c_src % 64 != 0 || c_src < 128 || c_dst % kWideCols != 0) return false;
  // rows are read with 16-byte loads and results added as 4-byte pairs
  return reinterpret_cast<uintptr_t>(a.src) % 16 == 0 && reinterpret_cast<uintptr_t>(a.dst) % 4 == 0;
}

int launch_wide_gms(const GmsArgs &a) {
  if (!wide_gms_supported(a)) {
    set_error("launch_wide_gms: unsupported shape");
    return FGMS_E_INVALID;
  }
  const int c_src = a.transpose_w ? a.c_out : a.c_in;
  const int c_dst = a.transpose_w ? a.c_in : a.c_out;
  const void *packed = a.prepacked;
  if (!packed) {
    int rc = pack_weights_any(a, 4, &packed);
    if (rc != FGMS_OK) return rc;
  }
  const bool dense = a.dense_k >= 0;
  const int64_t tiles = dense ? (a.n_dense + kWideRows - 1) / kWideRows
                              : (a.n_pairs + kWideRows - 1) / kWideRows + a.k_vol;
  if (tiles <= 0) return FGMS_OK;
  // one workgroup per CU at a time: each takes a contiguous run of tiles (mostly one offset,
  // whose weights then stay in the L2 between its tiles)
  const int64_t want_wgs = (int64_t)num_cus() / (c_dst / kWideCols > 1 ? c_dst / kWideCols : 1);
  const int tiles_per_wg = (int)((tiles + want_wgs - 1) / (want_wgs > 0 ? want_wgs : 1));
  const unsigned gx = (unsigned)((tiles + tiles_per_wg - 1) / tiles_per_wg);
  const size_t lds_bytes = 4 * (size_t)kSlabChunks * 16 + 4 * kWideRows * sizeof(int);
  const int rc_lds = allow_dynamic_lds(reinterpret_cast<const void *>(gms_wide_kernel), lds_bytes);
  if (rc_lds != FGMS_OK) return rc_lds;
  {
    ProfileScope prof(a.transpose_w ? "gms_wide_kernel(dgrad)" : "gms_wide_kernel(fwd)", a.stream);
    gms_wide_kernel<<<dim3(gx, (unsigned)(c_dst / kWideCols)), kWideThreads, lds_bytes, a.stream>>>(
        (const __half *)a.src, (const int4v *)packed, (__half *)a.dst, a.kpos, a.gmap, a.smap, a.k_vol, c_src,
        c_dst, tiles_per_wg, a.dense_k, (int)a.n_dense);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

}  // namespace fgms
