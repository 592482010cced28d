// Internal declarations shared by the translation units of libfgms_hip.so.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <vector>

#include "../../include/fgms.h"
#include "../../include/fgms_diag.h"

namespace fgms {

void set_error(const char *fmt, ...);

#define FGMS_HIP_TRY(expr)                                                     \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess) {                                                    \
      ::fgms::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                        __FILE__, __LINE__);                                   \
      return FGMS_E_HIP;                                                       \
    }                                                                          \
  } while (0)

// One gather-GEMM-scatter pass over a pair list.
//   dst[smap[j], :] += src[gmap[j], :] @ op(W[k])      for j in [kpos[k], kpos[k+1])
// forward: src = in_feats, dst = out_feats, gmap = in_map, smap = out_map,
//          op(W) = W            (c_src = c_in,  c_dst = c_out)
// dgrad:   src = out_grad, dst = in_grad, gmap = out_map, smap = in_map,
//          op(W) = W^T          (c_src = c_out, c_dst = c_in)
// A small job that rides along with a big launch instead of costing a launch of its own:
// the first `blocks` workgroups (x) of the grid run it and exit, the rest see their index
// lowered by `blocks`.  A multiple of 8, so that a workgroup keeps its XCD (index mod 8).
//   kind 1: re-lay the weights `src` into MFMA fragment order at `dst` (what
//           pack_weights_kernel does), for the launch that follows on the stream;
//   kind 2: dst[i] += acc[i] rounded once to fp16 and acc[i] = 0 (what add_and_clear_kernel
//           does) for the fp32 accumulator the previous launch on the stream filled;
//   kind 3: the plan's fingerprint check (fgms_plan_check): src = kpos, dst = in_map, omap,
//           n = the pair bound, k_vol; one workgroup works, the others of the job leave.
struct SideJob {
  int kind;      // 0: none
  int blocks;
  const void *src;
  void *dst;
  float *acc;
  size_t n;      // elements
  int k_vol, c_in, c_out, S, transpose, dtype;
  const int32_t *omap;
  int *flags, *host;
};

// dense:   gmap == smap == nullptr means the identity map over n_dense rows of
//          the single offset `dense_k` (the separately handled centre offset).
struct GmsArgs {
  const void *src;
  const void *w;      // [k_vol, c_in, c_out]
  void *dst;
  const int32_t *kpos;
  const int32_t *gmap;
  const int32_t *smap;
  int64_t n_src, n_dst;
  int c_in, c_out;    // the weight's own shape, whatever the direction
  int k_vol;
  int64_t n_pairs;    // upper bound on kpos[k_vol]
  bool transpose_w;   // dgrad
  int dense_k;        // >= 0: identity map over n_dense rows with W[dense_k]
  int64_t n_dense;
  int dtype;
  hipStream_t stream;
  // fp32 tensors in the reference's "tf32" mode: products may be rounded to tf32 precision
  // (10 mantissa bits) or better, sums stay fp32
  bool reduced;
  const void *prepacked;   // output-stationary kernel only: the weights are already re-laid here
  SideJob side;            // ... and this rides along with its launch
};

struct WgradArgs {
  const void *in;     // [n_in, c_in]
  const void *gout;   // [n_out, c_out]
  void *gw;           // [k_vol, c_in, c_out]
  const int32_t *kpos;
  const int32_t *imap;
  const int32_t *omap;
  int64_t n_in, n_out;
  int c_in, c_out, k_vol;
  int64_t n_pairs;
  int dtype;
  hipStream_t stream;
  const struct Plan *plan;   // optional
  bool reduced;              // fp32 tensors: products may be rounded to tf32 precision or better
  SideJob side;              // MFMA kernels only: rides along with the launch
  // MFMA kernels, fp16: do not launch the fp32 -> fp16 flush of the accumulator; describe
  // it in *deferred_flush instead, for the caller to attach to its next launch
  SideJob *deferred_flush;
  // MFMA kernels, fp16: use this fp32 accumulator (k_vol * c_in * c_out floats, all zero)
  // instead of the stream's workspace; nothing is allocated then
  float *acc_override;
};

constexpr int kPlanFlags = 16;      // ints the plan build reports back (see fgms_plan.hip)
constexpr int kFlagStale = 13;      // flags[13]: a later check found another fingerprint (fgms_plan_check)
constexpr int kFlagPrint = 14;      // flags[14], flags[15]: fingerprint of the pair lists (one 64-bit word)

// Plan: neighbour tables built from the pair lists.
struct Plan {
  int device;
  // the build is asynchronous: `flags` (device) is copied to `host_flags` (pinned) behind the
  // build's last kernel, `ready` fires after that copy; plan_resolve reads them on first use
  int *flags;
  int *host_flags;
  hipEvent_t ready;
  std::mutex mutex;
  bool resolved, invalid;
  bool has_bands;         // the weight gradient's row-band tables were built
  bool ordered;           // every offset's pairs are ordered by output row (what the bands need)
  int64_t pairs_counted;  // pairs the build saw (kpos[k_vol] - kpos[0]); n_pairs is the caller's bound
  std::vector<Plan *> groups;   // k_vol > 64: one plan per 64 offsets (owned)
  bool has_tables;        // k_vol <= 64: neighbour tables and masks exist (else the plan is the weight gradient's bands only)
  const int32_t *kpos, *in_map, *out_map;    // the caller's lists (for the pair view, built on first use)
  hipStream_t pv_stream;        // the stream the pair view was built on
  hipEvent_t pv_ready;          // fires behind its last kernel (launches on other streams wait for it)
  hipStream_t create_stream;    // the stream the build was queued on
  mutable bool checked;         // a fingerprint check has been queued at least once (host_flags[kFlagStale] means something)
  mutable bool check_pending;   // fgms_plan_check was called: the next launch through the plan carries the check
  int k_vol;
  int64_t n_in, n_out, n_pairs;
  // Destination rows are visited in a plan-chosen order (rows with the same set
  // of offsets next to each other: a stable sort by offset mask): position p of
  // the order is row perm[p] (perm == nullptr: identity).  The tables and masks
  // below are indexed by POSITION.
  int32_t *perm_out;  // [n_out]
  int32_t *perm_in;   // [n_in]
  int32_t *nbr_out;   // [k_vol, n_out]: input row feeding the output row at position p through offset k, or -1
  int32_t *nbr_in;    // [k_vol, n_in]:  output row fed by the input row at position p through offset k, or -1
  // bit k of mask_out[b] : some row of the 64-row block b has a neighbour through
  // offset k (only built when k_vol <= 64; the output-stationary kernels need it)
  unsigned long long *mask_out;  // [ceil(n_out / 64)]
  unsigned long long *mask_in;   // [ceil(n_in / 64)]
  // Row bands for the weight gradient: the output rows are cut into band_count
  // equal bands and band_start[k * (band_count + 1) + c] is the first pair of
  // offset k whose output row lies in band c or later (relative to kpos[k]).
  // Only valid when every offset's pairs are ordered by output row (bands_ok).
  int band_count;
  int32_t *band_start;   // [k_vol, band_count + 1]
  // Dispatch order of the (offset, band) cells, one table per group size 1, 2, 4, 8:
  // workgroup b of the weight gradient (XCD b % 8) takes cell
  // band_cells[t][b] = offset * 65536 + band; an XCD owns the bands congruent to it
  // mod 8, takes them 2^t at a time and, inside such a group, biggest cell first.
  int32_t *band_cells;   // [4][k_vol * band_count]
  int band_rows;         // output rows per band
  bool bands_ok;
  // Workgroup -> tile of 256 positions for the output-stationary kernel:
  // workgroup b runs on XCD b % 8 and takes tile tile_out[b] & 0xFFFFFF (or -1: none; the
  // bits above hold the first offset the tile uses), chosen
  // so that a tile runs on the XCD that owns the eighth of the cloud most of its
  // rows lie in (their neighbours then meet in that XCD's L2).  nullptr: tile = b.
  int32_t *tile_out, *tile_in;
  int tile_grid_out, tile_grid_in;   // entries of the tables (a multiple of 8)
  mutable hipStream_t last_stream;   // the stream of the latest launch that read the plan
  mutable bool many_streams;         // launches on more than one stream have read it (destroy then drains the device)
  // a transposed view (fgms_plan_transposed) shares the tables of `base` with the sides swapped
  // and owns nothing; `views` counts the views alive on a base, which is freed after the last one
  Plan *base;
  int views;
  bool destroyed;
  // (64-row block, offset) combinations with at least one pair: the output-stationary
  // kernels run stages * 64 row slots for n_pairs pairs
  int stages_out, stages_in;
  // Pair view, kept for maps that leave most row slots of the output-stationary kernels
  // empty (scattered clouds): the pair lists with every offset's run padded to a multiple
  // of 64 (padding = -1), so that a 64-row block of pv_in / pv_out belongs to one offset,
  // bit k of pv_mask[b] says which.  The output-stationary kernel walks these "virtual
  // rows" like a plan whose rows have one neighbour each and adds its results with
  // atomics.  nullptr: not built.
  int32_t *pv_in, *pv_out;        // [pv_rows]
  unsigned long long *pv_mask;    // [pv_rows / 64]
  int64_t pv_rows;                // a multiple of 256
  bool fwd_ok;        // no offset maps two pairs onto one output row
  bool dgrad_ok;      // no offset maps two pairs from one input row
};

// Fp32 scratch that outlives a call (per device and stream, grown on demand).
// slot 0: packed weights, slot 1: fp32 weight-gradient accumulator of the MFMA kernels (kept
// all-zero between calls), slot 2: the generic kernel's accumulator, slot 3: the gather probe's sink.
// *fresh (optional) is set when the buffer was (re)allocated by this call.
int workspace_get(hipStream_t stream, int slot, size_t bytes, void **ptr, bool *fresh = nullptr);
// Buffer for a re-laid copy of a.w in `layout` (any number that tells the layouts of one weight
// tensor apart): the stream's workspace, to be filled (*fill = true), or -- for weights under
// fgms_weights_pin -- a kept copy that a first call fills (relaid_weights_filled once its fill
// is queued) and later calls find filled (*fill = false).
int relaid_weights_buffer(const GmsArgs &a, unsigned layout, size_t bytes, void **ptr, bool *fill);
void relaid_weights_filled(const GmsArgs &a, void *ptr);
bool weights_pinned(const void *w);   // under fgms_weights_pin on the current device
size_t workspace_bytes(hipStream_t stream, int slot);

// Brackets a main-kernel launch with events when profiling is enabled.
struct ProfileScope {
  ProfileScope(const char *name, hipStream_t stream);
  ~ProfileScope();
  int slot;
  hipStream_t stream;
};

// ---- launchers (each returns an FGMS_* code) ----
int launch_fill_zero(void *ptr, size_t bytes, hipStream_t stream);
int launch_generic_gms(const GmsArgs &a);
int launch_generic_wgrad(const WgradArgs &a);
bool mfma_gms_supported(const GmsArgs &a);
// Pooled device blocks (plans, map-builder temporaries).  `user`: the stream the
// block will be used on; `last_user` / `idle`: the stream that used it last, or
// idle = true when no queued work can still touch it.
int pool_alloc(void **ptr, size_t bytes, hipStream_t user);
void pool_free(void *ptr, hipStream_t last_user, bool idle);
void pool_trim(size_t keep_bytes);
// Raises a kernel's dynamic-LDS limit to `bytes` (hipFuncSetAttribute) unless an earlier call
// on this device already allowed as much: the attribute call costs a microsecond per launch.
int allow_dynamic_lds(const void *kernel, size_t bytes);
int kernel_policy();   // fgms_set_kernel_policy's value
int num_cus();         // compute units of the current device
int launch_mfma_gms(const GmsArgs &a);
// Pair-stationary kernel for wide fp16 layers: 256 destination channels per workgroup, every
// source row gathered once (fgms_wide.hip).
bool wide_gms_supported(const GmsArgs &a);
int launch_wide_gms(const GmsArgs &a);
bool mfma_wgrad_supported(const WgradArgs &a);
int launch_mfma_wgrad(const WgradArgs &a);
// The MFMA / skinny weight gradient with its fp32 accumulator in a static device array: no
// allocation of any kind.
int wgrad_static(WgradArgs a);
// Describes the weight re-layout the output-stationary kernel needs for `a` as a side job
// (nothing is launched) and returns where the packed weights will be.
int planned_pack_job(const GmsArgs &a, SideJob *job, const void **packed);
// Both gradients of a layer in one launch where that is supported (*done says whether).
int launch_fused_bwd(const GmsArgs &d, const struct Plan *p, const WgradArgs &w, bool *done);
// Runs a side job in a launch of its own.
int launch_side_job(const SideJob &job, hipStream_t stream);
bool split_bf16_enabled();   // products of fp32 tensors in split bf16 where the caller allows tf32 precision
bool small_gms_supported(const GmsArgs &a, const Plan *p);
int launch_small_gms(const GmsArgs &a, const Plan *p);
bool planned_gms_supported(const GmsArgs &a, const Plan *p);
int launch_planned_gms(const GmsArgs &a, const Plan *p);
// The same kernel over the plan's pair view (no wasted row slots, atomic adds).
bool pair_view_gms_supported(const GmsArgs &a, const Plan *p);
int launch_pair_view_gms(const GmsArgs &a, const Plan *p);
// Notes that a launch on `stream` reads the plan.
inline void plan_touch(const Plan *p, hipStream_t stream) {
  if (p->last_stream != stream && p->resolved) p->many_streams = true;
  p->last_stream = stream;
}
// The plan with its build results known, or nullptr (see fgms_plan.hip).
const Plan *plan_resolve(fgms_plan_t *plan, hipStream_t stream, int *rc);
const Plan *plan_if_resolved(fgms_plan_t *plan);
// fgms_plan_check only marks the plan; the check itself rides along with the next launch that
// reads the plan and can carry a side job (plan_take_check fills one in and returns true), or
// goes out as a small launch of its own behind the call (plan_flush_check).
bool plan_take_check(const Plan *p, SideJob *job);
int plan_flush_check(const Plan *p, hipStream_t stream);
void note_allocation();      // counts a hipMalloc / hipHostMalloc of the library (fgms_allocation_count)
int build_kernel_map(const int32_t *in_coords, int64_t n_in, const int32_t *out_coords, int64_t n_out,
                     const int32_t *offsets_host, int k_vol, int stride, int skip_offset,
                     int32_t *in_map, int32_t *out_map, int64_t capacity, int32_t *kernel_nnz,
                     int32_t *kpos, int64_t *n_pairs, hipStream_t stream);
int launch_gather_probe(const Plan *p, const void *src, int c_src, int dtype, bool for_dgrad,
                        void *sink, hipStream_t stream);

}  // namespace fgms
