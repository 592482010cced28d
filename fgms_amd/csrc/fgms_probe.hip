// Gather-only probe: reads exactly the source rows the output-stationary kernel
// reads for a plan (per 64-row block and per offset the block uses: one line of
// neighbour indices, then the rows in 16-byte pieces) and
// throws the data away.  No LDS, no MFMA, no weights, no result rows; 32
// registers, so the wave slots are full.  Its duration is what the memory system
// alone needs for the kernel's gathers: the floor a gather-GEMM-scatter kernel
// with this dataflow can approach, and the yardstick for how much of a kernel's
// time is the gathers and how much is everything else.
#include "fgms_device.h"
#include "fgms_internal.h"

namespace fgms {
namespace {

typedef int int4v __attribute__((ext_vector_type(4)));

// CR: 16-byte pieces per row (compile time, so the loads of a step are issued
// back to back).  Like the real kernel, a row without a neighbour through the
// offset reads row 0 instead (a cache hit) and the value is dropped.
template <int CR>
__global__ __launch_bounds__(256) void gather_probe_kernel(
    const int4v *__restrict__ src, const int32_t *__restrict__ nbr,
    const unsigned long long *__restrict__ block_masks, int n_dst, int *__restrict__ sink) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int row0 = (blockIdx.x * 4 + wave) * 64;
  if (row0 >= n_dst) return;
  unsigned long long todo = block_masks[row0 / 64];
  const int my = min(row0 + lane, n_dst - 1);
  const bool live = row0 + lane < n_dst;
  int4v acc = {0, 0, 0, 0};
  int g_next = -1;
  if (todo) g_next = nbr[(size_t)__builtin_ctzll(todo) * n_dst + my];
  while (todo) {
    todo &= todo - 1;
    const int g = live ? g_next : -1;
    if (todo) g_next = nbr[(size_t)__builtin_ctzll(todo) * n_dst + my];   // next offset's line in flight
    // 64 rows x CR pieces, 64 pieces per load instruction, consecutive lanes on one row
    constexpr int kBatch = CR < 8 ? CR : 8;
#pragma unroll 1
    for (int it0 = 0; it0 < CR; it0 += kBatch) {
      int4v v[kBatch];
      int gi[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        const int s = (it0 + i) * 64 + lane;
        gi[i] = __shfl(g, s / CR);
        v[i] = src[(size_t)max(gi[i], 0) * CR + s % CR];
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i)
        if (gi[i] >= 0) acc ^= v[i];
    }
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5eed5eed) sink[0] = 1;   // keeps the loads alive
}

}  // namespace

int launch_gather_probe(const Plan *p, const void *src, int c_src, int dtype, bool for_dgrad,
                        void *sink, hipStream_t stream) {
  const int64_t n_dst = for_dgrad ? p->n_in : p->n_out;
  const size_t row_bytes = (size_t)c_src * (dtype == FGMS_F16 ? 2 : 4);
  if (row_bytes % 16 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0 || p->k_vol > 64) {
    set_error("fgms_probe_gather: rows must be a multiple of 16 bytes, 16-byte aligned, k_vol <= 64");
    return FGMS_E_INVALID;
  }
  if (n_dst == 0) return FGMS_OK;
  const unsigned gx = (unsigned)((n_dst + 255) / 256);
  const int cr = (int)(row_bytes / 16);
  void (*kern)(const int4v *, const int32_t *, const unsigned long long *, int, int *) = nullptr;
  switch (cr) {
    case 1: kern = gather_probe_kernel<1>; break;
    case 2: kern = gather_probe_kernel<2>; break;
    case 4: kern = gather_probe_kernel<4>; break;
    case 8: kern = gather_probe_kernel<8>; break;
    case 16: kern = gather_probe_kernel<16>; break;
    case 32: kern = gather_probe_kernel<32>; break;
    case 64: kern = gather_probe_kernel<64>; break;
    default:
      set_error("fgms_probe_gather: row size must be 16 * 2^j bytes, j = 0..6");
      return FGMS_E_INVALID;
  }
  {
    ProfileScope prof(for_dgrad ? "gather_probe_kernel(dgrad)" : "gather_probe_kernel(fwd)", stream);
    kern<<<gx, 256, 0, stream>>>((const int4v *)src, for_dgrad ? p->nbr_in : p->nbr_out,
                                 for_dgrad ? p->mask_in : p->mask_out, (int)n_dst, (int *)sink);
  }
  FGMS_HIP_TRY(hipGetLastError());
  return FGMS_OK;
}

}  // namespace fgms
