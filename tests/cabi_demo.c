/*
 * cabi_demo.c -- the C ABI of libfgms_hip.so driven from plain C, no Python and no torch:
 * what a caller of hkeee21/FGMS that is not a PyTorch program would write.
 *
 * A line of n voxels with three offsets (left neighbour, itself, right neighbour), one-hot
 * features and weights W[k] = (k + 1) * I: the forward result has the closed form
 *   out[i][c] = sum over the neighbours j = i-1, i, i+1 inside the line of (k + 1) * x[j][c]
 * and the weight gradient of an all-ones output gradient is diagonal with the pair counts
 * on it.  The map is built on the device (fgms_build_kernel_map), a plan is made, forward
 * and backward run on a stream of the program's own, and every number is checked.
 *
 * Build (fgms_amd/build.py does it, with the host C compiler):
 *   gcc -std=c11 -D__HIP_PLATFORM_AMD__=1 -I/opt/rocm/include -I../include cabi_demo.c \
 *       -L../fgms_amd/lib -lfgms_hip -L/opt/rocm/lib -lamdhip64 -o cabi_demo
 * Exit status 0 and a line "cabi demo ok" on success.
 */
#include <hip/hip_runtime_api.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fgms.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { \
  fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); return 2; } } while (0)
#define CHECK_FGMS(x) do { int r_ = (x); if (r_ != FGMS_OK) { \
  fprintf(stderr, "%s:%d: fgms error %d: %s\n", __FILE__, __LINE__, r_, fgms_last_error()); return 3; } } while (0)

int main(void) {
  enum { N = 1000, C = 32, K = 3 };
  printf("%s\n", fgms_version());
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));

  /* coordinates (i, 0, 0) and the three offsets */
  int32_t *h_coords = (int32_t *)calloc((size_t)N * 3, sizeof(int32_t));
  for (int i = 0; i < N; ++i) h_coords[3 * i] = i;
  const int32_t offsets[K * 3] = {-1, 0, 0, 0, 0, 0, 1, 0, 0};
  int32_t *d_coords, *d_imap, *d_omap, *d_knnz, *d_kpos;
  const int64_t cap = (int64_t)N * K;
  CHECK_HIP(hipMalloc((void **)&d_coords, (size_t)N * 3 * sizeof(int32_t)));
  CHECK_HIP(hipMalloc((void **)&d_imap, (size_t)cap * sizeof(int32_t)));
  CHECK_HIP(hipMalloc((void **)&d_omap, (size_t)cap * sizeof(int32_t)));
  CHECK_HIP(hipMalloc((void **)&d_knnz, K * sizeof(int32_t)));
  CHECK_HIP(hipMalloc((void **)&d_kpos, (K + 1) * sizeof(int32_t)));
  CHECK_HIP(hipMemcpyAsync(d_coords, h_coords, (size_t)N * 3 * sizeof(int32_t), hipMemcpyHostToDevice, stream));
  int64_t n_pairs = 0;
  CHECK_FGMS(fgms_build_kernel_map(d_coords, N, d_coords, N, offsets, K, 1, -1, d_imap, d_omap, cap,
                                   d_knnz, d_kpos, &n_pairs, stream));
  if (n_pairs != 3 * (int64_t)N - 2) { fprintf(stderr, "pairs %lld\n", (long long)n_pairs); return 4; }

  /* x[i] = unit vector i mod C; W[k] = (k + 1) * I; dOut = 1 */
  float *h_x = (float *)calloc((size_t)N * C, sizeof(float));
  float *h_w = (float *)calloc((size_t)K * C * C, sizeof(float));
  float *h_g = (float *)malloc((size_t)N * C * sizeof(float));
  for (int i = 0; i < N; ++i) h_x[(size_t)i * C + i % C] = 1.f;
  for (int k = 0; k < K; ++k)
    for (int c = 0; c < C; ++c) h_w[((size_t)k * C + c) * C + c] = (float)(k + 1);
  for (size_t i = 0; i < (size_t)N * C; ++i) h_g[i] = 1.f;
  float *d_x, *d_w, *d_out, *d_g, *d_gi, *d_gw;
  CHECK_HIP(hipMalloc((void **)&d_x, (size_t)N * C * sizeof(float)));
  CHECK_HIP(hipMalloc((void **)&d_w, (size_t)K * C * C * sizeof(float)));
  CHECK_HIP(hipMalloc((void **)&d_out, (size_t)N * C * sizeof(float)));
  CHECK_HIP(hipMalloc((void **)&d_g, (size_t)N * C * sizeof(float)));
  CHECK_HIP(hipMalloc((void **)&d_gi, (size_t)N * C * sizeof(float)));
  CHECK_HIP(hipMalloc((void **)&d_gw, (size_t)K * C * C * sizeof(float)));
  CHECK_HIP(hipMemcpyAsync(d_x, h_x, (size_t)N * C * sizeof(float), hipMemcpyHostToDevice, stream));
  CHECK_HIP(hipMemcpyAsync(d_w, h_w, (size_t)K * C * C * sizeof(float), hipMemcpyHostToDevice, stream));
  CHECK_HIP(hipMemcpyAsync(d_g, h_g, (size_t)N * C * sizeof(float), hipMemcpyHostToDevice, stream));
  CHECK_HIP(hipMemsetAsync(d_out, 0, (size_t)N * C * sizeof(float), stream));   /* outputs are caller-zeroed */
  CHECK_HIP(hipMemsetAsync(d_gi, 0, (size_t)N * C * sizeof(float), stream));
  CHECK_HIP(hipMemsetAsync(d_gw, 0, (size_t)K * C * C * sizeof(float), stream));

  fgms_plan_t *plan = NULL;
  CHECK_FGMS(fgms_plan_create(&plan, d_kpos, d_imap, d_omap, N, N, K, n_pairs, stream));
  CHECK_FGMS(fgms_fusion_fwd(d_x, d_w, 0, d_out, d_kpos, NULL, d_imap, d_omap, 0, 0, N, N, C, C, K, n_pairs,
                             FGMS_F32, plan, stream));
  CHECK_FGMS(fgms_bwd(d_g, d_x, d_w, 0, d_gi, d_gw, d_kpos, NULL, d_imap, d_omap, 0, 0, N, N, C, C, K, n_pairs,
                      FGMS_F32, plan, stream));
  float *h_out = (float *)malloc((size_t)N * C * sizeof(float));
  float *h_gi = (float *)malloc((size_t)N * C * sizeof(float));
  float *h_gw = (float *)malloc((size_t)K * C * C * sizeof(float));
  CHECK_HIP(hipMemcpyAsync(h_out, d_out, (size_t)N * C * sizeof(float), hipMemcpyDeviceToHost, stream));
  CHECK_HIP(hipMemcpyAsync(h_gi, d_gi, (size_t)N * C * sizeof(float), hipMemcpyDeviceToHost, stream));
  CHECK_HIP(hipMemcpyAsync(h_gw, d_gw, (size_t)K * C * C * sizeof(float), hipMemcpyDeviceToHost, stream));
  CHECK_HIP(hipStreamSynchronize(stream));

  /* offset k pairs input i + (k - 1) with output i */
  int bad = 0;
  for (int i = 0; i < N && !bad; ++i)
    for (int c = 0; c < C; ++c) {
      float want = 0.f, want_gi = 0.f;
      for (int k = 0; k < K; ++k) {
        const int j = i + k - 1;                 /* the input that reaches output i through offset k */
        if (j >= 0 && j < N && j % C == c) want += (float)(k + 1);
        const int o = i - (k - 1);               /* the output that input i reaches through offset k */
        if (o >= 0 && o < N) want_gi += (float)(k + 1);   /* dOut = 1, W[k]^T = (k + 1) I */
      }
      if (h_out[(size_t)i * C + c] != want || h_gi[(size_t)i * C + c] != want_gi) {
        fprintf(stderr, "row %d channel %d: out %g (want %g), gi %g (want %g)\n", i, c,
                h_out[(size_t)i * C + c], want, h_gi[(size_t)i * C + c], want_gi);
        bad = 1;
        break;
      }
    }
  /* dW[k][a][b] = number of pairs of offset k whose input row is a mod C (dOut = 1) */
  for (int k = 0; k < K && !bad; ++k)
    for (int a = 0; a < C && !bad; ++a) {
      float want = 0.f;
      for (int i = 0; i < N; ++i) {
        const int j = i + k - 1;
        if (j >= 0 && j < N && j % C == a) want += 1.f;
      }
      for (int b = 0; b < C; ++b)
        if (h_gw[((size_t)k * C + a) * C + b] != want) {
          fprintf(stderr, "dW[%d][%d][%d] = %g, want %g\n", k, a, b, h_gw[((size_t)k * C + a) * C + b], want);
          bad = 1;
          break;
        }
    }
  fgms_plan_destroy(plan);
  if (bad) return 5;
  printf("cabi demo ok: %d voxels, %lld pairs, forward + backward through the C ABI\n", N, (long long)n_pairs);
  return 0;
}
