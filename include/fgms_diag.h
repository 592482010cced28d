/*
 * fgms_diag.h -- test and measurement surface of libfgms_hip.so.
 *
 * Nothing here has a counterpart in hkeee21/FGMS and no caller of the drop-in entry points
 * (fgms.h) needs it: kernel selection by hand for the parity tests, per-kernel timing with
 * HIP events for the benchmark, and a gather-only pass that measures the memory side of the
 * output-stationary kernels.
 */
#ifndef FGMS_DIAG_H_
#define FGMS_DIAG_H_

#include "fgms.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Selects kernels by hand for tests and profiling: 0 = automatic dispatch,
 * 1 = force the generic (non-MFMA) kernels, 2 = force the pair-stationary MFMA
 * kernels even when a usable plan is passed, 3 = automatic dispatch but the
 * output-stationary kernel uses its 128-column wave tiles whenever the layer
 * has a multiple of 128 output channels (normally only large fp16 layers),
 * 4 = automatic dispatch but never the pair-stationary kernel where the
 * output-stationary one can run: forward and input-gradient results are then the
 * same bit for bit from run to run (automatic dispatch gives wide layers over
 * scattered clouds, with few pairs per 64-row block and offset, to the
 * pair-stationary kernel, whose atomic sums depend on their order; fp32 layers of
 * that kind run the output-stationary kernel's body over the plan's pair view, also
 * with atomic sums),
 * 5 = forward and input gradient over the plan's pair view whenever the plan has
 * one (plans created under this policy keep it for dense maps too),
 * 7 = forward and input gradient of fp16 layers with a multiple of 256 destination channels
 * through the pair-stationary kernel with 256-column workgroups even when a usable plan is
 * passed (automatic dispatch takes it where it would otherwise take the pair-stationary kernel).
 * Process-wide. */
void fgms_set_kernel_policy(int policy);

/*
 * Diagnostic, no counterpart in the reference: reads exactly the feature rows
 * the output-stationary forward (for_dgrad = 0: feats = in_feats, c_src = c_in)
 * or input-gradient kernel (for_dgrad != 0: feats = out_feats_grad,
 * c_src = c_out) gathers for this plan, and nothing else: no weights, no
 * matrix cores, no result.  Timed through fgms_profile_* it gives the time the
 * memory system alone needs for the gathers of one pass, the floor that the
 * real kernel's duration is compared with.  Rows must be 16 * 2^j bytes
 * (j = 0..6); k_vol <= 64.
 */
int fgms_probe_gather(const void *feats, int c_src, int dtype, int for_dgrad,
                      fgms_plan_t *plan, void *stream);

/*
 * Per-kernel timing with HIP events on the stream the kernels are launched on
 * (no counterpart in the reference, which times whole calls from python,
 * spconv-test.py:95-122).  While enabled, every main kernel launch (not the
 * small weight re-layout or zero-fill launches) is bracketed by two events.
 * fgms_profile_read synchronises with the recorded events and returns the
 * index-th record: kernel name and milliseconds; it returns FGMS_E_INVALID
 * once index runs past the records.  fgms_profile_reset drops all records.
 */
/* How many device or pinned-host allocations (hipMalloc, hipHostMalloc) the library has made
 * since it was loaded: a test can assert that a call made none. */
long long fgms_allocation_count(void);
/* How many launches found the re-laid copy of a pinned weight tensor (fgms_weights_pin)
 * already made, since the library was loaded. */
long long fgms_relaid_weights_hits(void);
void fgms_profile_enable(int on);
int fgms_profile_read(int index, char *name, int name_len, float *ms);
void fgms_profile_reset(void);

#ifdef __cplusplus
}
#endif
#endif /* FGMS_DIAG_H_ */
