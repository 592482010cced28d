/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the gather-GEMM-scatter sparse
 * convolution that hkeee21/FGMS computes.  Nothing in the shipped library links,
 * loads or calls this file; only tests, the smoke check and the benchmark's
 * cpu_baseline leg do, as the checker.
 *
 * Every loop nest below follows the reference's own CPU check scripts:
 *   forward            cpu-check.py:16-44        (cpu_compute)
 *   dgrad / wgrad      cpu-check-back.py:16-44   (cpu_compute)
 *   qkpos              cpu-check.py:6-14         (kpos_quantized)
 *   offset lookup      backend/utils.cuh:6-27    (binary_search)
 *   mid offset index   cpu-check.py:26, backend/spconv.cu:52
 *
 * Arithmetic: inputs are widened to fp32, every sum is kept in fp32 and the
 * result is rounded once to the storage type at the end (the reference's python
 * loops round to the tensor dtype after every += ; the parity contract is the
 * math, with the tolerances of cpu-check.py:127).
 *
 * Parity pins (tests/test_oracle_*.py): dense-grid equivalence with
 * torch.nn.functional.conv3d / conv_transpose3d, autograd of an independent
 * float64 index_add formulation, adjoint identities, brute-force python loops
 * on tiny inputs, exhaustive bisect comparison for the offset lookup.
 *
 * dtype: 0 = IEEE binary32, 1 = IEEE binary16 (stored as uint16_t).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define FGMS_ORACLE_F32 0
#define FGMS_ORACLE_F16 1

/* ---- binary16 <-> binary32, round-to-nearest-even ---------------------- */
static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0));
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) return sign; /* below half of the smallest subnormal */
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u;
  uint32_t shift;
  uint32_t base;
  if (e < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - e));
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
  return (uint16_t)(sign | (base + q)); /* mantissa carry bumps the exponent */
}

/* exported for the conversion tests */
float fgms_oracle_half_to_float(uint16_t h) { return half_to_float(h); }
uint16_t fgms_oracle_float_to_half(float f) { return float_to_half(f); }

static float *widen(const void *src, int64_t n, int dtype) {
  float *dst = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
  if (!dst) return NULL;
  if (dtype == FGMS_ORACLE_F32) {
    memcpy(dst, src, sizeof(float) * (size_t)n);
  } else {
    const uint16_t *s = (const uint16_t *)src;
    for (int64_t i = 0; i < n; ++i) dst[i] = half_to_float(s[i]);
  }
  return dst;
}

static void narrow(void *dst, const float *src, int64_t n, int dtype) {
  if (dtype == FGMS_ORACLE_F32) {
    memcpy(dst, src, sizeof(float) * (size_t)n);
  } else {
    uint16_t *d = (uint16_t *)dst;
    for (int64_t i = 0; i < n; ++i) d[i] = float_to_half(src[i]);
  }
}

static int pick_threads(int threads) {
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
  return threads < 1 ? 1 : threads;
#else
  (void)threads;
  return 1;
#endif
}

/* kpos_quantized, cpu-check.py:6-14.  Returns qkpos[K]. */
int64_t fgms_oracle_qkpos(const int32_t *knnz, int k_vol, int q, int32_t *qkpos) {
  qkpos[0] = 0;
  for (int k = 0; k < k_vol; ++k)
    qkpos[k + 1] = qkpos[k] + (knnz[k] + q - 1) / q * q;
  return qkpos[k_vol];
}

/* binary_search, backend/utils.cuh:6-27: the last i in [start,end] with
 * pos[i] <= eid among the entries the bisection visits. */
int fgms_oracle_offset_of(const int32_t *pos, int eid, int start, int end) {
  int lo = start, hi = end;
  if (lo == hi) return lo;
  while (lo < hi) {
    int mid = (lo + hi) >> 1;
    if (pos[mid] <= eid) lo = mid + 1; else hi = mid;
  }
  return pos[hi] <= eid ? hi : hi - 1;
}

/* Forward, cpu-check.py:16-44.
 *   out[omap[j], :] += in[imap[j], :] @ W[k]   for j in the k-th run of knnz[k] pairs
 *   if precompute:  out[i, :] += in[i, :] @ W[mid]  for every i < n_out
 * `out` is read as the starting value (the script starts from zeros, :27) and
 * overwritten with the rounded result.  Pairs of one offset are spread over
 * threads by output row, so duplicate output rows inside an offset stay
 * race-free and the per-row summation order is the pair order. */
int fgms_oracle_fwd(const void *in_feats, const void *kernel, void *out_feats,
                    const int32_t *knnz, const int32_t *imap, const int32_t *omap,
                    int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
                    int dtype, int precompute, int threads) {
  float *in = widen(in_feats, n_in * c_in, dtype);
  float *w = widen(kernel, (int64_t)k_vol * c_in * c_out, dtype);
  float *out = widen(out_feats, n_out * c_out, dtype);
  if (!in || !w || !out) return -1;
  int mid_k = (k_vol % 2 == 1) ? k_vol / 2 : 0;
  int nt = pick_threads(threads);
  int64_t nbaddr = 0;
  for (int k = 0; k < k_vol; ++k) {
    int64_t nbsize = knnz[k];
    if (nbsize == 0) continue;
    const float *wk = w + (int64_t)k * c_in * c_out;
#pragma omp parallel num_threads(nt)
    {
#ifdef _OPENMP
      int tid = omp_get_thread_num(), np = omp_get_num_threads();
#else
      int tid = 0, np = 1;
#endif
      for (int64_t i = 0; i < nbsize; ++i) {
        int64_t o = omap[nbaddr + i];
        if ((int)(o % np) != tid) continue;
        const float *x = in + (int64_t)imap[nbaddr + i] * c_in;
        float *y = out + o * c_out;
        for (int ci = 0; ci < c_in; ++ci) {
          float xv = x[ci];
          const float *wr = wk + (int64_t)ci * c_out;
          for (int co = 0; co < c_out; ++co) y[co] += xv * wr[co];
        }
      }
    }
    nbaddr += nbsize;
  }
  if (precompute) {
    const float *wk = w + (int64_t)mid_k * c_in * c_out;
#pragma omp parallel for num_threads(nt) schedule(static)
    for (int64_t i = 0; i < n_out; ++i) {
      const float *x = in + i * c_in;
      float *y = out + i * c_out;
      for (int ci = 0; ci < c_in; ++ci) {
        float xv = x[ci];
        const float *wr = wk + (int64_t)ci * c_out;
        for (int co = 0; co < c_out; ++co) y[co] += xv * wr[co];
      }
    }
  }
  narrow(out_feats, out, n_out * c_out, dtype);
  free(in); free(w); free(out);
  return 0;
}

/* Input gradient, cpu-check-back.py:28-41 (first statement of the body):
 *   in_grad[imap[j], ci] += sum_co out_grad[omap[j], co] * W[k, ci, co] */
int fgms_oracle_dgrad(const void *out_grad, const void *kernel, void *in_grad,
                      const int32_t *knnz, const int32_t *imap, const int32_t *omap,
                      int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
                      int dtype, int threads) {
  float *go = widen(out_grad, n_out * c_out, dtype);
  float *w = widen(kernel, (int64_t)k_vol * c_in * c_out, dtype);
  float *gi = widen(in_grad, n_in * c_in, dtype);
  if (!go || !w || !gi) return -1;
  int nt = pick_threads(threads);
  int64_t nbaddr = 0;
  for (int k = 0; k < k_vol; ++k) {
    int64_t nbsize = knnz[k];
    if (nbsize == 0) continue;
    const float *wk = w + (int64_t)k * c_in * c_out;
#pragma omp parallel num_threads(nt)
    {
#ifdef _OPENMP
      int tid = omp_get_thread_num(), np = omp_get_num_threads();
#else
      int tid = 0, np = 1;
#endif
      for (int64_t i = 0; i < nbsize; ++i) {
        int64_t r = imap[nbaddr + i];
        if ((int)(r % np) != tid) continue;
        const float *g = go + (int64_t)omap[nbaddr + i] * c_out;
        float *y = gi + r * c_in;
        for (int ci = 0; ci < c_in; ++ci) {
          const float *wr = wk + (int64_t)ci * c_out;
          float acc = 0.f;
          for (int co = 0; co < c_out; ++co) acc += g[co] * wr[co];
          y[ci] += acc;
        }
      }
    }
    nbaddr += nbsize;
  }
  narrow(in_grad, gi, n_in * c_in, dtype);
  free(go); free(w); free(gi);
  return 0;
}

/* Weight gradient, cpu-check-back.py:28-41 (second statement of the body):
 *   weight_grad[k, ci, co] += in[imap[j], ci] * out_grad[omap[j], co]
 * Threads split the rows ci of each dW[k], so the summation order over pairs
 * is the pair order whatever the thread count. */
int fgms_oracle_wgrad(const void *in_feats, const void *out_grad, void *kernel_grad,
                      const int32_t *knnz, const int32_t *imap, const int32_t *omap,
                      int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
                      int dtype, int threads) {
  float *in = widen(in_feats, n_in * c_in, dtype);
  float *go = widen(out_grad, n_out * c_out, dtype);
  float *gw = widen(kernel_grad, (int64_t)k_vol * c_in * c_out, dtype);
  if (!in || !go || !gw) return -1;
  int nt = pick_threads(threads);
  int64_t nbaddr = 0;
  for (int k = 0; k < k_vol; ++k) {
    int64_t nbsize = knnz[k];
    if (nbsize == 0) continue;
    float *gk = gw + (int64_t)k * c_in * c_out;
#pragma omp parallel for num_threads(nt) schedule(static)
    for (int ci = 0; ci < c_in; ++ci) {
      float *row = gk + (int64_t)ci * c_out;
      for (int64_t i = 0; i < nbsize; ++i) {
        float xv = in[(int64_t)imap[nbaddr + i] * c_in + ci];
        const float *g = go + (int64_t)omap[nbaddr + i] * c_out;
        for (int co = 0; co < c_out; ++co) row[co] += xv * g[co];
      }
    }
    nbaddr += nbsize;
  }
  narrow(kernel_grad, gw, (int64_t)k_vol * c_in * c_out, dtype);
  free(in); free(go); free(gw);
  return 0;
}

int fgms_oracle_max_threads(void) { return pick_threads(0); }
