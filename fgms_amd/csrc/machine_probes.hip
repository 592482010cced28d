// Stand-alone micro-benchmarks of the machine limits the gather-GEMM-scatter kernels run into.
// Not part of the library: a small program (build.py links it as fgms_amd/lib/machine_probes)
// that prints, for the GPU it runs on,
//   1. the payload rate of scattered global atomics, stores and read-modify-writes
//      (what the pair-stationary kernels' result updates cost),
//   2. the rate of random 128-byte row gathers against the size of the table they draw from
//      (local L2 hits against Infinity Cache / HBM),
//   3. the same gathers with 4 instead of 8 lanes per row (the operand layout of
//      v_mfma_f32_16x16x32_f16: why rows are not gathered straight into MFMA registers),
//   4. direct global -> LDS loads against loads through registers,
//   5. LDS throughput of the access patterns of the output-stationary kernel.
// Rates per CU and clock assume 256 CUs at 2.1 GHz.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>

typedef int int4v __attribute__((ext_vector_type(4)));

#define CK(x)                                                            \
  do {                                                                   \
    hipError_t e_ = (x);                                                 \
    if (e_ != hipSuccess) {                                              \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      exit(1);                                                           \
    }                                                                    \
  } while (0)

static hipEvent_t g_e0, g_e1;
template <typename F>
static float time_ms(F &&launch, int reps = 3) {
  float ms = 0;
  for (int r = 0; r < reps; ++r) {
    CK(hipEventRecord(g_e0));
    launch();
    CK(hipEventRecord(g_e1));
    CK(hipEventSynchronize(g_e1));
    CK(hipEventElapsedTime(&ms, g_e0, g_e1));
  }
  return ms;
}

__device__ __forceinline__ unsigned mix(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

// ---- 1. scattered updates: piece p = 256 bytes of row rows[p / pieces_per_row] ----------------
template <int MODE>
__global__ void update_kernel(const int *__restrict__ rows, unsigned *__restrict__ dst, int n_pieces, int row_words) {
  const int ppr = row_words / 64;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / 64, lane = threadIdx.x % 64;
  const int nw = gridDim.x * blockDim.x / 64;
  for (int p = wave; p < n_pieces; p += nw) {
    unsigned *a = dst + (size_t)rows[p / ppr] * row_words + (p % ppr) * 64 + lane;
    if (MODE == 0) unsafeAtomicAdd(reinterpret_cast<__half2 *>(a), __floats2half2_rn(1.f, 2.f));
    else if (MODE == 1) unsafeAtomicAdd(reinterpret_cast<float *>(a), 1.f);
    else if (MODE == 2) *a = 0x3c003c00u;
    else *a = *a + 1;
  }
}

static void probe_updates() {
  const int n_rows = 50000, row_words = 128, n_src = 170000;   // 512-byte rows, 170 k updates of a whole row
  std::vector<int> rows(n_src);
  srand(1);
  for (auto &r : rows) r = rand() % n_rows;
  int *d_rows;
  unsigned *dst;
  CK(hipMalloc(&d_rows, n_src * 4));
  CK(hipMalloc(&dst, (size_t)n_rows * row_words * 4));
  CK(hipMemcpy(d_rows, rows.data(), n_src * 4, hipMemcpyHostToDevice));
  CK(hipMemset(dst, 0, (size_t)n_rows * row_words * 4));
  const int n_pieces = n_src * (row_words / 64);
  const char *names[] = {"global_atomic_pk_add_f16", "global_atomic_add_f32", "store", "load + store"};
  printf("1. scattered updates of 256-byte row pieces (%.1f MB of payload over %d rows of 512 bytes)\n",
         n_pieces * 256.0 / 1e6, n_rows);
  for (int mode = 0; mode < 4; ++mode) {
    const float ms = time_ms([&] {
      for (int i = 0; i < 20; ++i) {
        if (mode == 0) update_kernel<0><<<2048, 256>>>(d_rows, dst, n_pieces, row_words);
        if (mode == 1) update_kernel<1><<<2048, 256>>>(d_rows, dst, n_pieces, row_words);
        if (mode == 2) update_kernel<2><<<2048, 256>>>(d_rows, dst, n_pieces, row_words);
        if (mode == 3) update_kernel<3><<<2048, 256>>>(d_rows, dst, n_pieces, row_words);
      }
    }) / 20;
    printf("   %-26s %7.1f us per launch, %.2f TB/s of payload\n", names[mode], ms * 1e3, n_pieces * 256.0 / (ms * 1e-3) / 1e12);
  }
  CK(hipFree(d_rows));
  CK(hipFree(dst));
}

// ---- 2. / 3. random row gathers --------------------------------------------------------------
// LANES = 8: one instruction reads 8 whole rows; LANES = 4: 16 half rows, a second instruction
// 64 bytes further on reads the other halves.
template <int LANES>
__global__ __launch_bounds__(256, 3) void gather_kernel(const int4v *__restrict__ src, int n_rows, int iters,
                                                        int *__restrict__ out) {
  const int lane = threadIdx.x % 64;
  const unsigned wid = (blockIdx.x * 256 + threadIdx.x) / 64;
  int4v acc = {0, 0, 0, 0};
  for (int it = 0; it < iters; ++it) {
    int4v v[8];
    if (LANES == 8) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const unsigned row = mix((wid * 64 + j * 8 + lane / 8) * 2654435761u + it * 40503u) % (unsigned)n_rows;
        v[j] = src[(size_t)row * 8 + lane % 8];
      }
    } else {
#pragma unroll
      for (int rb = 0; rb < 4; ++rb) {
        const unsigned row = mix((wid * 64 + rb * 16 + lane % 16) * 2654435761u + it * 40503u) % (unsigned)n_rows;
        v[rb * 2] = src[(size_t)row * 8 + lane / 16];
        v[rb * 2 + 1] = src[(size_t)row * 8 + 4 + lane / 16];
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) acc ^= v[j];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) out[0] = 1;
}

static void probe_gathers() {
  const size_t total_rows = 1 << 21;     // 256 MB
  int4v *src;
  int *out;
  CK(hipMalloc(&src, total_rows * 128));
  CK(hipMalloc(&out, 4));
  CK(hipMemset(src, 1, total_rows * 128));
  const int iters = 64, grid = 768 * 4;
  const double bytes = (double)grid * 256 * iters * 8 * 16;
  printf("2. random 128-byte row gathers, 8 lanes x 16 bytes per row, 12 waves per CU, by table size\n");
  for (int kb : {256, 1024, 4096, 8192, 32768, 262144}) {
    const int n_rows = kb * 1024 / 128;
    const float ms = time_ms([&] { gather_kernel<8><<<grid, 256>>>(src, n_rows, iters, out); });
    printf("   table %7d KB: %.2f TB/s (%.1f bytes per clock and CU)\n", kb, bytes / (ms * 1e-3) / 1e12,
           bytes / (ms * 1e-3) / 256 / 2.1e9);
  }
  printf("3. the same with 4 lanes per row and two instructions per 16 rows (half rows of 64 bytes)\n");
  for (int kb : {2048, 25600}) {
    const int n_rows = kb * 1024 / 128;
    const float a = time_ms([&] { gather_kernel<8><<<grid, 256>>>(src, n_rows, iters, out); });
    const float b = time_ms([&] { gather_kernel<4><<<grid, 256>>>(src, n_rows, iters, out); });
    printf("   table %7d KB: whole rows %.2f TB/s, half rows %.2f TB/s\n", kb, bytes / (a * 1e-3) / 1e12,
           bytes / (b * 1e-3) / 1e12);
  }
  CK(hipFree(src));
  CK(hipFree(out));
}

// ---- 4. direct global -> LDS loads -------------------------------------------------------------
__device__ __forceinline__ void dma16(const void *gptr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory");
}
template <int MODE>
__global__ __launch_bounds__(256) void stage_kernel(const int4v *__restrict__ src, int n_chunks, int iters, int *out) {
  extern __shared__ int4v lds[];
  const int lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) void *)(lds + wave * 1024);
  unsigned x = blockIdx.x * 977 + wave * 131;
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        x = x * 1664525u + 1013904223u;
        const unsigned row = (x >> 8) % (unsigned)(n_chunks / 8 - 8);
        dma16(src + (size_t)(row + lane / 8) * 8 + lane % 8, base + j * 1024);
      }
      __builtin_amdgcn_s_waitcnt(0x0F70);     // vmcnt(0)
    } else {
      int4v v[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        x = x * 1664525u + 1013904223u;
        const unsigned row = (x >> 8) % (unsigned)(n_chunks / 8 - 8);
        v[j] = src[(size_t)(row + lane / 8) * 8 + lane % 8];
      }
#pragma unroll
      for (int j = 0; j < 16; ++j) lds[wave * 1024 + j * 64 + lane] = v[j];
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    }
  }
  __syncthreads();
  const int4v a = lds[threadIdx.x];
  if ((a[0] ^ a[1]) == 0x12345678) out[0] = 1;
}

static void probe_staging() {
  const int n_chunks = (2 << 20) / 16;   // a 2 MB source: L2-resident
  int4v *src;
  int *out;
  CK(hipMalloc(&src, (size_t)n_chunks * 16));
  CK(hipMalloc(&out, 4));
  CK(hipMemset(src, 1, (size_t)n_chunks * 16));
  const int iters = 200;
  printf("4. 8-row gathers from a 2 MB table into LDS, 16 KB in flight per wave\n");
  for (int wgs = 1; wgs <= 2; ++wgs)
    for (int mode = 0; mode < 2; ++mode) {
      const int grid = 256 * wgs;
      const float ms = time_ms([&] {
        if (mode == 0) stage_kernel<0><<<grid, 256, 65536>>>(src, n_chunks, iters, out);
        else stage_kernel<1><<<grid, 256, 65536>>>(src, n_chunks, iters, out);
      });
      const double bytes = (double)grid * 4 * iters * 16 * 1024;
      printf("   %d waves per CU, %-30s %.1f bytes per clock and CU\n", 4 * wgs,
             mode == 0 ? "global_load_lds_dwordx4:" : "global_load_dwordx4 + ds_write:", bytes / (ms * 1e-3) / 256 / 2.1e9);
    }
  CK(hipFree(src));
  CK(hipFree(out));
}

// ---- 5. LDS access patterns ----------------------------------------------------------------------
// slot of 16-byte chunk c of a 128-byte row: XOR by row pairs (the library's a_slot<4>) or by row
template <int PAIRS>
__device__ __forceinline__ int slot_of(int row, int c) {
  return row * 8 + (c ^ (PAIRS ? ((row >> 1) & 7) : (row & 7)));
}
template <int MODE>
__global__ __launch_bounds__(256) void lds_kernel(int iters, int *out) {
  extern __shared__ int4v lds[];
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  int4v *mine = lds + wave * 1024;        // 16 KB per wave
  const int h = lane / 32, r = lane % 32;
  int4v acc = {0, 0, 0, 0}, v = {lane, 1, 2, 3};
  for (int i = threadIdx.x; i < 4096; i += 256) lds[i] = v;
  __syncthreads();
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {            // a staged gather's writes: chunk slot of (row, piece) = (e / 8, e % 8)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int e = j * 64 + lane;
        mine[slot_of<1>(e / 8, e % 8)] = v;
      }
    } else if (MODE == 1 || MODE == 2) {     // A fragments of v_mfma_f32_32x32x16_f16: lane = row, piece h * 4 + s
#pragma unroll
      for (int j = 0; j < 8; ++j) acc ^= mine[slot_of<MODE == 1>((j / 4) * 32 + r, h * 4 + j % 4)];
    } else if (MODE == 3) {     // contiguous
#pragma unroll
      for (int j = 0; j < 8; ++j) acc ^= mine[j * 64 + lane];
    } else {                    // transposing reads of a forward weight tile (64 rows x 128 bytes)
      typedef short short4v __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) short4v lds_v4;
      const int b = lane >> 4, i = lane & 15;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int s = j / 4, nt = (j / 2) % 2, hi = j % 2;
        const int row = (h * 4 + s) * 8 + (i >> 2) + hi * 4;
        const int chunk = nt * 4 + (b & 1) * 2 + ((i & 3) >> 1);
        const __half *base = reinterpret_cast<const __half *>(lds) +
                             ((size_t)row * 8 + (chunk ^ (((row >> 1) & 1) << 2))) * 8 + (i & 1) * 4;
        const short4v x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4 *)(base));
        acc[0] ^= x[0]; acc[1] ^= x[1]; acc[2] ^= x[2]; acc[3] ^= x[3];
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    v[1] += acc[0];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3] ^ v[1]) == 0x12345678) out[0] = 1;
}

static void probe_lds() {
  int *out;
  CK(hipMalloc(&out, 4));
  const int iters = 2000;
  const char *names[] = {"ds_write_b128, staged gather", "ds_read_b128, A fragments, XOR by row / 2",
                         "ds_read_b128, A fragments, XOR by row", "ds_read_b128, contiguous",
                         "ds_read_b64_tr_b16, weight fragments"};
  printf("5. LDS throughput, 8 waves per CU\n");
  for (int mode = 0; mode < 5; ++mode) {
    const float ms = time_ms([&] {
      if (mode == 0) lds_kernel<0><<<512, 256, 65536>>>(iters, out);
      if (mode == 1) lds_kernel<1><<<512, 256, 65536>>>(iters, out);
      if (mode == 2) lds_kernel<2><<<512, 256, 65536>>>(iters, out);
      if (mode == 3) lds_kernel<3><<<512, 256, 65536>>>(iters, out);
      if (mode == 4) lds_kernel<4><<<512, 256, 65536>>>(iters, out);
    });
    const double bytes = 512.0 * 4 * iters * (mode == 4 ? 16 * 512 : 8 * 1024);
    printf("   %-44s %6.1f bytes per clock and CU\n", names[mode], bytes / (ms * 1e-3) / 256 / 2.1e9);
  }
  CK(hipFree(out));
}

int main() {
  CK(hipEventCreate(&g_e0));
  CK(hipEventCreate(&g_e1));
  hipDeviceProp_t p;
  CK(hipGetDeviceProperties(&p, 0));
  printf("%s (%s), %d CUs\n", p.name, p.gcnArchName, p.multiProcessorCount);
  probe_updates();
  probe_gathers();
  probe_staging();
  probe_lds();
  return 0;
}
