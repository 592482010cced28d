/*
 * fgms.h -- C ABI of the MI355X (gfx950) fused gather-GEMM-scatter library.
 *
 * One entry point per function that hkeee21/FGMS exports through pybind
 * (backend/pybind_cuda.cpp:8-10, declared in backend/spconv.h:10-49).  Tensors
 * become raw device pointers plus the sizes the reference reads off the
 * at::Tensor arguments (backend/spconv.cu:36-48); everything else keeps the
 * reference's name, order and meaning.
 *
 * Conventions shared by all entry points
 *   - in_feats  [n_in,  c_in ]  row-major, device
 *   - kernel    [k_vol, c_in, c_out] row-major, device
 *   - out_feats [n_out, c_out]  row-major, device, caller-zeroed, accumulated
 *   - in_map / out_map: int32[n_pairs], device; the pairs of offset k occupy
 *     [kpos[k], kpos[k+1]); pair j adds in_feats[in_map[j]] @ kernel[k] to
 *     out_feats[out_map[j]].
 *   - kpos: int32[k_vol+1] device, exclusive prefix sum of the per-offset pair
 *     counts.  qkpos / sum_nnz (the 256-padded prefix sum and its total,
 *     cpu-check.py:6-14) are accepted for signature compatibility; tile
 *     scheduling is derived from kpos, so any padding quantum works.
 *   - dtype: FGMS_F32 or FGMS_F16 for features, weights and gradients alike
 *     (the reference keys on in_feats.scalar_type(), backend/spconv.cu:47-48).
 *   - arch80: for FGMS_F32, non-zero = "tf32 mode" in the reference
 *     (backend/spconv.cu:67-68,213): the products may be rounded to tf32
 *     precision, the sums are fp32.  gfx950 has no tf32 matrix instruction;
 *     the forward pass, the input gradient and the weight gradient (the MFMA
 *     kernels: channel counts that are multiples of 32) then multiply in split
 *     bf16 (every value
 *     as hi + lo, three 16-bit MFMAs per product: about 2^-16 relative error,
 *     finer than tf32, at about twice the speed of the fp32 kernels).
 *     Everything else, and arch80 = 0, runs the fp32 MFMA kernels.
 *   - stream: a hipStream_t (NULL = the null stream).  All work is enqueued on
 *     it; calls return without waiting for the GPU, as the reference's do.
 *   - plan: optional (NULL allowed) handle from fgms_plan_create for the same
 *     maps; with a plan the output-stationary kernels run (no atomics,
 *     deterministic), without one the pair-stationary atomic kernels run.
 *   - return value: 0 on success, a negative FGMS_E_* code otherwise;
 *     fgms_last_error() describes the last failure on the calling thread.
 */
#ifndef FGMS_H_
#define FGMS_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FGMS_F32 0
#define FGMS_F16 1

#define FGMS_OK 0
#define FGMS_E_INVALID (-1)   /* bad argument (shape, dtype, null pointer)   */
#define FGMS_E_HIP (-2)       /* a HIP runtime call failed                    */
#define FGMS_E_NOMEM (-3)     /* workspace / plan allocation failed           */
#define FGMS_E_STALE (-4)     /* the pair lists changed after the plan was made */

typedef struct fgms_plan fgms_plan_t;

/* Library identification; also proves the shared object loads. */
const char *fgms_version(void);
const char *fgms_last_error(void);

/*
 * Kernel-map plan.  Built once per (in_map, out_map, kpos) on the device and
 * reusable by every layer and every pass that shares the map: a neighbour
 * table "output row x offset -> input row" (and its transpose for dgrad), the rows
 * of each side ordered by the set of offsets they use.  The reference has no
 * counterpart: it re-reads the pair lists on every call (backend/spconv.cuh:457-563).
 * The build is QUEUED on `stream` and the call returns without waiting for it, like every
 * other entry point.  What the build finds out about the map -- an index outside
 * [0, n_in) x [0, n_out), an offset that maps two pairs onto one row (the plan is then
 * not usable for that direction and the entry points silently use the atomic
 * kernels), pair order, block counts -- is read when the plan is first used or asked
 * about: that call waits for the build if it has not finished, and an entry point
 * given a plan whose map has an out-of-range index returns FGMS_E_INVALID.  Exception:
 * a first use recorded into a HIP graph (stream capture) cannot wait and records the
 * kernels that need no plan.  The map arrays must stay valid and unchanged while the plan
 * lives.  Not to be called on a stream that is being captured.
 */
int fgms_plan_create(fgms_plan_t **plan, const int32_t *kpos,
                     const int32_t *in_map, const int32_t *out_map,
                     int64_t n_in, int64_t n_out, int k_vol, int64_t n_pairs,
                     void *stream);
/*
 * A plan for the same pairs with the roles of the two sides swapped (in_map and out_map
 * exchanged: the map of the transposed convolution, backend/spconv.cu:460 swaps them the
 * same way for the input gradient).  It shares the tables of `base`, which already hold both
 * directions, and costs nothing to make; destroy it like any plan (the shared tables go with
 * the last of base and its views).  No counterpart in the reference.
 */
int fgms_plan_transposed(fgms_plan_t **view, fgms_plan_t *base);
void fgms_plan_destroy(fgms_plan_t *plan);
/*
 * Guards against a plan that outlived its map (no counterpart in the reference, which reads
 * the pair lists on every call, backend/spconv.cuh:484-485, and so cannot compute with last
 * iteration's neighbours).  The build keeps a fingerprint of the lists: kpos and a fixed
 * sample of about 4 096 (in_map, out_map) entries.  fgms_plan_check has the fingerprint taken
 * again from the lists as they are then: by one small kernel queued on `stream` right away
 * (with_next_launch = 0), or by one extra workgroup of the next forward / backward launch
 * that reads the plan (with_next_launch = 1: no launch of its own, `stream` is not used).  A
 * difference raises a flag in the plan, and every later call that is handed the plan (this
 * one included) returns FGMS_E_STALE once the flag has reached the host.  The check does not
 * wait for the GPU, so the call that carried it may still have computed with the old tables:
 * a caller that rewrites its lists in place must make a new plan; this only makes the
 * omission loud.  A sample is not a proof: rewrites that leave kpos and every sampled entry
 * as they were go unnoticed.
 */
int fgms_plan_check(fgms_plan_t *plan, void *stream, int with_next_launch);
/* 1 if the output-stationary kernels can use it for forward / for dgrad. */
int fgms_plan_usable(const fgms_plan_t *plan, int for_dgrad);
/* What the build counted (no counterpart in the reference): stats[0] = pairs in the map,
 * stats[1] / stats[2] = (64-row block, offset) combinations with at least one pair in the
 * forward / input-gradient direction (the output-stationary kernels run 64 row slots for
 * each, so stats[1] * 64 / stats[0] is their row slots per pair), stats[3] = rows of the
 * pair view (0: the plan keeps none).  Returns FGMS_OK or FGMS_E_INVALID. */
int fgms_plan_stats(const fgms_plan_t *plan, int64_t stats[4]);

/*
 * Replaces ConvolutionForwardFused  (backend/spconv.cu:23-246; pybind name
 * fgms_fusion_fwd_cuda, backend/pybind_cuda.cpp:8).
 * separate_mid != 0: the centre offset (k_vol/2 for odd k_vol, else 0,
 * backend/spconv.cu:52) is not in the map; out_feats is first OVERWRITTEN with
 * in_feats @ kernel[mid] (GEMM with beta = 0, backend/spconv.cu:56,76-106), so
 * n_in must equal n_out, and the map's pairs are accumulated on top.
 */
int fgms_fusion_fwd(const void *in_feats, const void *kernel, int sum_nnz,
                    void *out_feats, const int32_t *kpos, const int32_t *qkpos,
                    const int32_t *in_map, const int32_t *out_map,
                    int separate_mid, int arch80,
                    int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
                    int64_t n_pairs, int dtype, fgms_plan_t *plan, void *stream);

/*
 * Replaces ConvolutionForward  (backend/spconv.cu:249-411; pybind name
 * fgms_fwd_cuda, backend/pybind_cuda.cpp:9): the per-offset "sequential" form.
 * kernel_nnz is a HOST array int32[k_vol] (backend/spconv.cu:308); kernel_pos
 * is the device kpos.  With separate_mid the centre product is ADDED after the
 * map's pairs (beta = 1, backend/spconv.cu:377-410).
 */
int fgms_fwd(const void *in_feats, const void *kernel, int sum_nnz,
             void *out_feats, const int32_t *kernel_nnz, const int32_t *kernel_pos,
             const int32_t *in_map, const int32_t *out_map,
             int separate_mid, int arch80,
             int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
             int64_t n_pairs, int dtype, fgms_plan_t *plan, void *stream);

/*
 * Replaces ConvolutionBackward  (backend/spconv.cu:414-571; pybind name
 * fgms_bwd_cuda, backend/pybind_cuda.cpp:10): input gradient and weight
 * gradient, both accumulated into caller-zeroed buffers.  separate_mid is
 * accepted and ignored, as in the reference; arch80 is ignored there because its
 * backward pass of fp32 tensors is always tf32 (backend/spconv.cu:551-569), here
 * it allows that precision as in the forward pass (see above).  (The reference launches
 * the input gradient, then the weight gradient; the two do not depend on each
 * other, and with a plan this library runs the workgroups of both in one launch,
 * followed for fp16 by a small one that rounds the weight gradient's fp32 sums.)
 *   in_feats_grad[in_map[j]]  += out_feats_grad[out_map[j]] @ kernel[k]^T
 *   kernel_grad[k]            += in_feats[in_map[j]]^T (x) out_feats_grad[out_map[j]]
 */
int fgms_bwd(const void *out_feats_grad, const void *in_feats, const void *kernel,
             int sum_nnz, void *in_feats_grad, void *kernel_grad,
             const int32_t *kpos, const int32_t *qkpos,
             const int32_t *in_map, const int32_t *out_map,
             int separate_mid, int arch80,
             int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
             int64_t n_pairs, int dtype, fgms_plan_t *plan, void *stream);

/* The two halves of fgms_bwd on their own (the reference launches them back to
 * back, backend/spconv.cu:454-461 + 495-548 / 553-569); exposed so each can be
 * timed and tested separately. */
int fgms_dgrad(const void *out_feats_grad, const void *kernel, void *in_feats_grad,
               const int32_t *kpos, const int32_t *in_map, const int32_t *out_map,
               int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
               int64_t n_pairs, int dtype, fgms_plan_t *plan, void *stream);
int fgms_wgrad(const void *in_feats, const void *out_feats_grad, void *kernel_grad,
               const int32_t *kpos, const int32_t *in_map, const int32_t *out_map,
               int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
               int64_t n_pairs, int dtype, fgms_plan_t *plan, void *stream);

/*
 * fgms_wgrad for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * Same arguments and results as fgms_wgrad, but the fp32 accumulator that the fp16 weight
 * gradient sums in lives in a static device array inside the library (8 MiB per GPU, held
 * until the process ends) instead of a workspace grown on demand, and the call makes no
 * hipMalloc / hipFree or any other allocating call.  Limits: fp16 needs
 * k_vol * c_in * c_out <= 2 097 152 (27 offsets of 256 x 256 fit); only the shapes of the
 * MFMA and skinny kernels (channel counts that are multiples of 32, or 4/8/16 -> 16/32/64,
 * 16-byte aligned rows) -- anything else returns FGMS_E_INVALID instead of falling back to a
 * kernel that would need a workspace.  A plan is used only if an earlier call has already
 * taken its build results (the first use of a plan waits for the build and may allocate);
 * otherwise the call runs without the plan's row bands.  All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (two streams, two threads) race; calls
 * on one stream do not.
 */
int fgms_wgrad_static(const void *in_feats, const void *out_feats_grad, void *kernel_grad,
                      const int32_t *kpos, const int32_t *in_map, const int32_t *out_map,
                      int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol,
                      int64_t n_pairs, int dtype, fgms_plan_t *plan, void *stream);

/*
 * Weights that do not change between calls.  No counterpart in the reference, which hands its
 * kernels the weight tensor as it is (backend/spconv.cu:112-238).  Some kernels here read the
 * weights from a re-laid copy that a small launch makes in front of the main one (wide fp16
 * layers, fp32 forward passes: 4-9 us per call).  fgms_weights_pin(kernel) is the caller's
 * promise that the bytes at `kernel` stay as they are until the next fgms_weights_pin or
 * fgms_weights_unpin of that address: the library then makes each such copy once and keeps it
 * (device memory of the tensor's size per layout used, on the current device).  After writing
 * to the tensor (an optimizer step, loading a checkpoint) call fgms_weights_pin again, which
 * drops the copies; before freeing it call fgms_weights_unpin (NULL: every pinned address on
 * the current device).  A call on a pinned tensor whose bytes were changed without this reads
 * the old weights.  Calls under stream capture and the backward calls do not use the copies.
 */
int fgms_weights_pin(const void *kernel);
int fgms_weights_unpin(const void *kernel);

/*
 * Kernel-map builder.  No counterpart in the reference, whose scripts load the
 * maps from files (cpu-check.py:89-94, spconv-test.py:64-73); this is the step
 * right before the path.  Finds every pair (i, o) with
 *     in_coords[i] == out_coords[o] * stride + offsets[k]
 * and writes them grouped by offset k, ascending o inside an offset (if input
 * rows share a coordinate the smallest row index is taken):
 * in_map / out_map (device, room for `capacity` pairs; k_vol * n_out always
 * suffices), kernel_nnz[k_vol] and kpos[k_vol + 1] (device), *n_pairs (host).
 * in_coords / out_coords: device int32 [n][3], every component in
 * [-2^20, 2^20); offsets: HOST int32 [k_vol][3]; skip_offset: an offset to
 * leave empty (the centre, for callers that use separate_mid), or -1.
 * Synchronises the stream once.  FGMS_E_INVALID if a coordinate is out of
 * range or the pairs do not fit `capacity` (*n_pairs is set, the lists hold
 * the first `capacity` pairs).
 */
int fgms_build_kernel_map(const int32_t *in_coords, int64_t n_in,
                          const int32_t *out_coords, int64_t n_out,
                          const int32_t *offsets, int k_vol, int stride, int skip_offset,
                          int32_t *in_map, int32_t *out_map, int64_t capacity,
                          int32_t *kernel_nnz, int32_t *kpos, int64_t *n_pairs, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FGMS_H_ */
