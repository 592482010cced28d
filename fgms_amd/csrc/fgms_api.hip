// extern "C" entry points of libfgms_hip.so: argument checks, kernel selection,
// workspace bookkeeping.  The host-side counterpart of backend/spconv.cu:23-571.
#include <stdarg.h>
#include <stdio.h>

#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <utility>
#include <vector>
#include <string.h>

#include "fgms_internal.h"

namespace fgms {

static thread_local char g_error[512] = "";
static int g_policy = 0;
int kernel_policy() { return g_policy; }

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// ---- workspace: one growable buffer per (device, stream, slot) --------------
namespace {
struct WsKey {
  int device;
  hipStream_t stream;
  int slot;
  bool operator<(const WsKey &o) const {
    if (device != o.device) return device < o.device;
    if (stream != o.stream) return stream < o.stream;
    return slot < o.slot;
  }
};
struct WsBuf {
  void *ptr = nullptr;
  size_t bytes = 0;
};
std::mutex g_ws_mutex;
std::map<WsKey, WsBuf> g_ws;
}  // namespace

size_t workspace_bytes(hipStream_t stream, int slot) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_ws.find(WsKey{dev, stream, slot});
  return it == g_ws.end() ? 0 : it->second.bytes;
}

// Device / pinned allocations the library has made since it was loaded (fgms_allocation_count).
std::atomic<long long> g_allocations{0};
void note_allocation() { g_allocations.fetch_add(1, std::memory_order_relaxed); }

int workspace_get(hipStream_t stream, int slot, size_t bytes, void **ptr, bool *fresh) {
  if (fresh) *fresh = false;
  int dev = 0;
  FGMS_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  WsBuf &b = g_ws[WsKey{dev, stream, slot}];
  if (b.bytes < bytes) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (stream && hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone) {
      // growing would free a buffer that recorded kernels point at, and allocate under capture
      set_error("a workspace of %zu bytes is needed while the stream is being captured: run the call once "
                "outside the capture first", bytes);
      return FGMS_E_INVALID;
    }
    if (b.ptr) {
      // the old buffer may still be in use by work queued on this stream
      FGMS_HIP_TRY(hipStreamSynchronize(stream));
      FGMS_HIP_TRY(hipFree(b.ptr));
      b.ptr = nullptr;
      b.bytes = 0;
    }
    size_t want = bytes + bytes / 4 + 4096;
    note_allocation();
    if (hipMalloc(&b.ptr, want) != hipSuccess) {
      b.ptr = nullptr;
      set_error("workspace allocation of %zu bytes failed", want);
      return FGMS_E_NOMEM;
    }
    b.bytes = want;
    if (fresh) *fresh = true;
  }
  *ptr = b.ptr;
  return FGMS_OK;
}

// ---- re-laid copies of pinned weights -----------------------------------------
// Some kernels read the weights from a re-laid copy, made by a small launch in front of the
// main one (4-9 us where the main launch takes 90).  A caller that promises that a weight
// tensor's bytes stay as they are (fgms_weights_pin: inference, or between two optimizer
// steps) lets the library keep those copies, per (address, layout), until fgms_weights_unpin
// or the next fgms_weights_pin of the address.
namespace {
struct RelaidCopy {
  const void *w;
  int device;
  unsigned layout;
  int k_vol, c_in, c_out;
  size_t bytes;
  void *ptr;
  hipStream_t made_on;
  hipEvent_t ready;                  // nullptr: the fill has not been queued (yet)
  std::vector<hipStream_t> users;    // streams other than made_on that wait for `ready` already
};
std::mutex g_pin_mutex;
std::vector<std::pair<int, const void *>> g_pinned;
std::vector<RelaidCopy> g_relaid;
std::atomic<int> g_pinned_count{0};
std::atomic<long long> g_relaid_hits{0};

bool is_pinned_locked(int dev, const void *w) {
  for (const auto &e : g_pinned)
    if (e.first == dev && e.second == w) return true;
  return false;
}

// Hands a copy's block back to the pool once every stream that read it has passed this point.
void retire_locked(RelaidCopy &c) {
  for (hipStream_t s : c.users) {
    hipEvent_t ev = nullptr;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) continue;
    if (hipEventRecord(ev, s) == hipSuccess) (void)hipStreamWaitEvent(c.made_on, ev, 0);
    (void)hipEventDestroy(ev);
  }
  if (c.ready) (void)hipEventDestroy(c.ready);
  pool_free(c.ptr, c.made_on, false);
}

void drop_copies_locked(int dev, const void *w) {
  for (size_t i = 0; i < g_relaid.size();) {
    if (g_relaid[i].device == dev && g_relaid[i].w == w) {
      retire_locked(g_relaid[i]);
      g_relaid.erase(g_relaid.begin() + i);
    } else {
      ++i;
    }
  }
}
}  // namespace

bool weights_pinned(const void *w) {
  if (g_pinned_count.load(std::memory_order_relaxed) == 0) return false;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  std::lock_guard<std::mutex> lock(g_pin_mutex);
  return is_pinned_locked(dev, w);
}

int relaid_weights_buffer(const GmsArgs &a, unsigned layout, size_t bytes, void **ptr, bool *fill) {
  *fill = true;
  if (g_pinned_count.load(std::memory_order_relaxed) > 0) {
    int dev = 0;
    FGMS_HIP_TRY(hipGetDevice(&dev));
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const bool capturing = a.stream && hipStreamIsCapturing(a.stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    if (!capturing && is_pinned_locked(dev, a.w)) {
      for (RelaidCopy &c : g_relaid) {
        if (c.w != a.w || c.device != dev || c.layout != layout || c.k_vol != a.k_vol || c.c_in != a.c_in ||
            c.c_out != a.c_out || c.bytes != bytes)
          continue;
        *ptr = c.ptr;
        if (!c.ready) {           // an earlier call failed between the buffer and its fill
          c.made_on = a.stream;
          c.users.clear();
          return FGMS_OK;
        }
        if (a.stream != c.made_on && std::find(c.users.begin(), c.users.end(), a.stream) == c.users.end()) {
          FGMS_HIP_TRY(hipStreamWaitEvent(a.stream, c.ready, 0));
          c.users.push_back(a.stream);
        }
        *fill = false;
        g_relaid_hits.fetch_add(1, std::memory_order_relaxed);
        return FGMS_OK;
      }
      void *p = nullptr;
      int rc = pool_alloc(&p, bytes, a.stream);
      if (rc != FGMS_OK) return rc;
      g_relaid.push_back(RelaidCopy{a.w, dev, layout, a.k_vol, a.c_in, a.c_out, bytes, p, a.stream, nullptr, {}});
      *ptr = p;
      return FGMS_OK;
    }
  }
  return workspace_get(a.stream, 0, bytes, ptr);
}

void relaid_weights_filled(const GmsArgs &a, void *ptr) {
  if (g_pinned_count.load(std::memory_order_relaxed) == 0) return;
  std::lock_guard<std::mutex> lock(g_pin_mutex);
  for (RelaidCopy &c : g_relaid) {
    if (c.ptr != ptr || c.ready) continue;
    hipEvent_t ev = nullptr;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) return;
    if (hipEventRecord(ev, a.stream) != hipSuccess) {
      (void)hipEventDestroy(ev);
      return;
    }
    c.ready = ev;
    return;
  }
}

extern "C" int fgms_weights_pin(const void *kernel) {
  if (!kernel) {
    set_error("fgms_weights_pin: null pointer");
    return FGMS_E_INVALID;
  }
  int dev = 0;
  FGMS_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_pin_mutex);
  if (is_pinned_locked(dev, kernel)) {
    drop_copies_locked(dev, kernel);       // pinned again: the bytes have changed since
  } else {
    g_pinned.emplace_back(dev, kernel);
    g_pinned_count.store((int)g_pinned.size(), std::memory_order_relaxed);
  }
  return FGMS_OK;
}

extern "C" int fgms_weights_unpin(const void *kernel) {
  int dev = 0;
  FGMS_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_pin_mutex);
  for (size_t i = 0; i < g_pinned.size();) {
    if (g_pinned[i].first == dev && (!kernel || g_pinned[i].second == kernel)) {
      drop_copies_locked(dev, g_pinned[i].second);
      g_pinned.erase(g_pinned.begin() + i);
    } else {
      ++i;
    }
  }
  g_pinned_count.store((int)g_pinned.size(), std::memory_order_relaxed);
  return FGMS_OK;
}

extern "C" long long fgms_relaid_weights_hits(void) { return g_relaid_hits.load(std::memory_order_relaxed); }

// ---- dynamic-LDS limits already granted, per (device, kernel) ------------------
namespace {
std::mutex g_lds_mutex;
std::map<std::pair<int, const void *>, size_t> g_lds_granted;
}  // namespace

int allow_dynamic_lds(const void *kernel, size_t bytes) {
  int dev = 0;
  FGMS_HIP_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_lds_mutex);
  size_t &granted = g_lds_granted[{dev, kernel}];
  if (granted >= bytes) return FGMS_OK;
  FGMS_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  granted = bytes;
  return FGMS_OK;
}

// ---- block pool: device memory of plans and of the map builder's temporaries --
// hipMalloc / hipFree cost 50-100 us each and a plan needs a dozen blocks, which
// made building a plan (once per kernel map, i.e. several times per training
// step) three times as expensive as its kernels.  Freed blocks are kept per
// device and handed out again to requests of similar size.  A block that may
// still be read by queued work carries an event recorded on the stream that used
// it last; whoever gets the block next makes its own stream wait for that event.
namespace {
struct PoolBlock {
  void *ptr;
  size_t bytes;
  int device;
  hipEvent_t ready;    // nullptr: idle
};
std::mutex g_pool_mutex;
std::vector<PoolBlock> g_pool_free;
std::map<void *, std::pair<size_t, int>> g_pool_live;   // ptr -> (bytes, device)
size_t g_pool_cached = 0;
constexpr size_t kPoolMaxCached = (size_t)2 << 30;
}  // namespace

int pool_alloc(void **ptr, size_t bytes, hipStream_t user) {
  *ptr = nullptr;
  if (bytes == 0) bytes = 256;
  bytes = (bytes + 255) & ~(size_t)255;
  int dev = 0;
  FGMS_HIP_TRY(hipGetDevice(&dev));
  PoolBlock got{};
  {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    int best = -1;
    for (int i = 0; i < (int)g_pool_free.size(); ++i) {
      const PoolBlock &b = g_pool_free[i];
      if (b.device != dev || b.bytes < bytes || b.bytes > 2 * bytes + 4096) continue;
      if (best < 0 || b.bytes < g_pool_free[best].bytes) best = i;
    }
    if (best >= 0) {
      got = g_pool_free[best];
      g_pool_free.erase(g_pool_free.begin() + best);
      g_pool_cached -= got.bytes;
      g_pool_live[got.ptr] = {got.bytes, dev};
    }
  }
  if (got.ptr) {
    if (got.ready) {
      hipError_t e = hipStreamWaitEvent(user, got.ready, 0);
      (void)hipEventDestroy(got.ready);
      if (e != hipSuccess) {
        set_error("pool_alloc: hipStreamWaitEvent: %s", hipGetErrorString(e));
        return FGMS_E_HIP;
      }
    }
    *ptr = got.ptr;
    return FGMS_OK;
  }
  void *q = nullptr;
  note_allocation();
  if (hipMalloc(&q, bytes) != hipSuccess) {
    // give cached blocks back to the driver and try once more
    pool_trim(0);
    if (hipMalloc(&q, bytes) != hipSuccess) {
      set_error("device allocation of %zu bytes failed", bytes);
      return FGMS_E_NOMEM;
    }
  }
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  g_pool_live[q] = {bytes, dev};
  *ptr = q;
  return FGMS_OK;
}

void pool_free(void *ptr, hipStream_t last_user, bool idle) {
  if (!ptr) return;
  PoolBlock b{};
  {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    auto it = g_pool_live.find(ptr);
    if (it == g_pool_live.end()) return;
    b = PoolBlock{ptr, it->second.first, it->second.second, nullptr};
    g_pool_live.erase(it);
  }
  if (!idle) {
    // queued work may still read the block: mark the point after which it is free
    hipEvent_t ev = nullptr;
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess ||
        hipEventRecord(ev, last_user) != hipSuccess) {
      if (ev) (void)hipEventDestroy(ev);
      (void)hipFree(ptr);     // synchronises; also the path taken while the runtime shuts down
      return;
    }
    b.ready = ev;
  }
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  g_pool_free.push_back(b);
  g_pool_cached += b.bytes;
  while (g_pool_cached > kPoolMaxCached && !g_pool_free.empty()) {
    PoolBlock old = g_pool_free.front();
    g_pool_free.erase(g_pool_free.begin());
    g_pool_cached -= old.bytes;
    if (old.ready) (void)hipEventDestroy(old.ready);
    (void)hipFree(old.ptr);
  }
}

void pool_trim(size_t keep_bytes) {
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  while (g_pool_cached > keep_bytes && !g_pool_free.empty()) {
    PoolBlock old = g_pool_free.front();
    g_pool_free.erase(g_pool_free.begin());
    g_pool_cached -= old.bytes;
    if (old.ready) (void)hipEventDestroy(old.ready);
    (void)hipFree(old.ptr);
  }
}

// ---- profiling records -------------------------------------------------------
namespace {
struct ProfRec {
  const char *name;
  hipEvent_t start, stop;
};
std::mutex g_prof_mutex;
std::vector<ProfRec> g_prof;
bool g_prof_on = false;
}  // namespace

ProfileScope::ProfileScope(const char *name, hipStream_t s) : slot(-1), stream(s) {
  if (!g_prof_on) return;
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  ProfRec r{name, nullptr, nullptr};
  if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) return;
  (void)hipEventRecord(r.start, stream);
  g_prof.push_back(r);
  slot = (int)g_prof.size() - 1;
}

ProfileScope::~ProfileScope() {
  if (slot < 0) return;
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  if (slot < (int)g_prof.size()) (void)hipEventRecord(g_prof[slot].stop, stream);
}

namespace {

int check_common(const void *a, const void *b, const void *c, const int32_t *kpos,
                 const int32_t *imap, const int32_t *omap, int64_t n_in, int64_t n_out, int c_in,
                 int c_out, int k_vol, int64_t n_pairs, int dtype) {
  if (dtype != FGMS_F32 && dtype != FGMS_F16) {
    set_error("dtype must be FGMS_F32 (0) or FGMS_F16 (1), got %d", dtype);
    return FGMS_E_INVALID;
  }
  if (n_in < 0 || n_out < 0 || c_in <= 0 || c_out <= 0 || k_vol <= 0 || n_pairs < 0) {
    set_error("bad sizes: n_in=%lld n_out=%lld c_in=%d c_out=%d k_vol=%d n_pairs=%lld",
              (long long)n_in, (long long)n_out, c_in, c_out, k_vol, (long long)n_pairs);
    return FGMS_E_INVALID;
  }
  if (n_in > INT32_MAX || n_out > INT32_MAX || n_pairs > INT32_MAX - 65536) {
    set_error("row and pair counts must fit int32 (the maps are int32)");
    return FGMS_E_INVALID;
  }
  if (!kpos || (n_pairs > 0 && (!imap || !omap)) ||
      ((n_in > 0 || n_out > 0) && (!a || !b || !c))) {
    set_error("null pointer argument");
    return FGMS_E_INVALID;
  }
  return FGMS_OK;
}

// The output-stationary kernel multiplies every (64-row block, offset) combination in
// use, 64 row slots each, whether or not a row has a pair there; the pair-stationary
// kernels multiply pairs only and pay with an atomic per result element.  Which one wins
// depends on the row slots per pair of the map (1.0 .. 1.2 for surface-like clouds at full
// density, 2 .. 3 for random subsamples of them) and on the channel count.  Measured on
// MI355X over subsamples of a 200 k-voxel indoor-like cloud (35 k .. 200 k voxels, 32 .. 256
// channels), the slots per pair at which both take the same time:
//   fp32: 2.35 / 1.76 / 1.3 at 32 / 64 / 128 channels, i.e. about 1 + 45 / c (the MFMA time
//         of the empty slots against a fixed cost per atomic);
//   fp16: 2.25 .. 2.5 at every channel count (2.2 + 16 / c).
// The kernel without atomics, whose results do not depend on the run, gets 5 % on top.
bool sparse_rows(const GmsArgs &a, const Plan *plan) {
  const int stages = a.transpose_w ? plan->stages_in : plan->stages_out;
  if (stages <= 0 || plan->pairs_counted <= 0) return false;   // (the plan's own pair count: a.n_pairs is a bound)
  const double slots_per_pair = (double)stages * 64.0 / (double)plan->pairs_counted;
  const double c_src = a.transpose_w ? a.c_out : a.c_in;
  const double even = a.dtype == FGMS_F16 ? 2.2 + 16.0 / c_src : 1.0 + 45.0 / c_src;
  // (no break-even point was measured below 1.3: denser maps stay output-stationary)
  const double need = 1.05 * even;
  return slots_per_pair > (need > 1.4 ? need : 1.4);
}

enum class Route { kSkinny, kRows, kPairView, kWide, kPairs, kGeneric };

// Which kernel a forward / input-gradient pass takes.
Route route_of(const GmsArgs &a, const Plan *plan) {
  const bool dense = a.dense_k >= 0;
  if (g_policy == 1) return Route::kGeneric;
  const bool pair_view = !dense && pair_view_gms_supported(a, plan);
  if (g_policy == 5 && pair_view) return Route::kPairView;
  if (!dense && (g_policy == 0 || g_policy == 4) && small_gms_supported(a, plan)) return Route::kSkinny;
  if (g_policy == 7 && wide_gms_supported(a)) return Route::kWide;
  if (!dense && g_policy != 2 && planned_gms_supported(a, plan) &&
      !(g_policy != 4 && sparse_rows(a, plan) && mfma_gms_supported(a)))
    return Route::kRows;
  // Which pair-stationary kernel: the output-stationary kernel's body over the plan's pair
  // view streams the weights of a stage through LDS where gms_pairs_kernel holds a column
  // block's weights of one offset.  Measured (same clouds): fp32 a tie up to 128 channels,
  // 245 against 341 us at 256 -> 256 over 50 k voxels; fp16 14.2 against 18.3 us at 64
  // channels over 35 k voxels, a tie from 128 channels on (96.6 against 96.3 us at 256).
  if (g_policy == 0 && pair_view && (a.dtype == FGMS_F32 || (a.transpose_w ? a.c_out : a.c_in) <= 64))
    return Route::kPairView;
  if (g_policy == 0 && wide_gms_supported(a)) return Route::kWide;
  return mfma_gms_supported(a) ? Route::kPairs : Route::kGeneric;
}

int run_gms_one(GmsArgs a, const Plan *plan);

// A pass over all offsets: one walk for plans of up to 64 offsets (or none), one per group of 64
// offsets for larger kernels (the groups' results add up in the destination rows).
int run_gms(GmsArgs a, const Plan *plan) {
  if (!plan || plan->groups.empty() || a.dense_k >= 0) return run_gms_one(a, plan);
  plan_touch(plan, a.stream);
  const size_t esz = a.dtype == FGMS_F16 ? 2 : 4;
  int k0 = 0;
  for (const Plan *g : plan->groups) {
    GmsArgs ga = a;
    ga.w = (const char *)a.w + (size_t)k0 * a.c_in * a.c_out * esz;
    ga.kpos = a.kpos + k0;
    ga.k_vol = g->k_vol;
    int rc = run_gms_one(ga, g);
    if (rc != FGMS_OK) return rc;
    k0 += g->k_vol;
  }
  return FGMS_OK;
}

int run_gms_one(GmsArgs a, const Plan *plan) {
  if (plan) plan_touch(plan, a.stream);
  const bool dense = a.dense_k >= 0;
  if ((!dense && a.n_pairs == 0) || (dense && a.n_dense == 0)) return FGMS_OK;
  switch (route_of(a, plan)) {
    case Route::kSkinny: return launch_small_gms(a, plan);
    case Route::kRows: return launch_planned_gms(a, plan);
    case Route::kPairView: return launch_pair_view_gms(a, plan);
    case Route::kWide: return launch_wide_gms(a);
    case Route::kPairs: return launch_mfma_gms(a);
    default: return launch_generic_gms(a);
  }
}

int run_wgrad(const WgradArgs &a) {
  if (a.n_pairs == 0) return FGMS_OK;
  if (a.plan) plan_touch(a.plan, a.stream);
  if (g_policy != 1 && mfma_wgrad_supported(a)) return launch_mfma_wgrad(a);
  return launch_generic_wgrad(a);
}

int mid_of(int k_vol) { return (k_vol % 2 == 1) ? k_vol / 2 : 0; }

GmsArgs fwd_args(const void *in, const void *w, void *out, const int32_t *kpos,
                 const int32_t *imap, const int32_t *omap, int64_t n_in, int64_t n_out, int c_in,
                 int c_out, int k_vol, int64_t n_pairs, int dtype, hipStream_t s) {
  GmsArgs a{};
  a.src = in; a.w = w; a.dst = out; a.kpos = kpos; a.gmap = imap; a.smap = omap;
  a.n_src = n_in; a.n_dst = n_out; a.c_in = c_in; a.c_out = c_out; a.k_vol = k_vol;
  a.n_pairs = n_pairs; a.transpose_w = false; a.dense_k = -1; a.n_dense = 0; a.dtype = dtype;
  a.stream = s;
  return a;
}

int check_mid(int separate_mid, int64_t n_in, int64_t n_out) {
  if (separate_mid && n_in != n_out) {
    set_error("separate_mid needs n_in == n_out (got %lld, %lld)", (long long)n_in, (long long)n_out);
    return FGMS_E_INVALID;
  }
  return FGMS_OK;
}

}  // namespace
}  // namespace fgms

using namespace fgms;

// A fingerprint check of the plan that none of the call's launches carried as a side job goes
// out as a launch of its own when the entry point returns.
namespace {
struct CheckFlush {
  const Plan *p;
  hipStream_t s;
  ~CheckFlush() { if (p) (void)plan_flush_check(p, s); }
};
}  // namespace

extern "C" {

const char *fgms_version(void) { return "fgms-hip 0.1 (gfx950)"; }
const char *fgms_last_error(void) { return g_error; }
void fgms_set_kernel_policy(int policy) { g_policy = policy; }

void fgms_profile_enable(int on) { g_prof_on = on != 0; }
long long fgms_allocation_count(void) { return g_allocations.load(std::memory_order_relaxed); }

void fgms_profile_reset(void) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  for (auto &r : g_prof) {
    (void)hipEventSynchronize(r.stop);
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_prof.clear();
}

int fgms_profile_read(int index, char *name, int name_len, float *ms) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  if (index < 0 || index >= (int)g_prof.size() || !ms) return FGMS_E_INVALID;
  FGMS_HIP_TRY(hipEventSynchronize(g_prof[index].stop));
  FGMS_HIP_TRY(hipEventElapsedTime(ms, g_prof[index].start, g_prof[index].stop));
  if (name && name_len > 0) {
    strncpy(name, g_prof[index].name, (size_t)name_len - 1);
    name[name_len - 1] = 0;
  }
  return FGMS_OK;
}

int fgms_fusion_fwd(const void *in_feats, const void *kernel, int sum_nnz, void *out_feats,
                    const int32_t *kpos, const int32_t *qkpos, const int32_t *in_map,
                    const int32_t *out_map, int separate_mid, int arch80, int64_t n_in,
                    int64_t n_out, int c_in, int c_out, int k_vol, int64_t n_pairs, int dtype,
                    fgms_plan_t *plan, void *stream) {
  (void)sum_nnz; (void)qkpos;
  int rc = check_common(in_feats, kernel, out_feats, kpos, in_map, out_map, n_in, n_out, c_in,
                        c_out, k_vol, n_pairs, dtype);
  if (rc) return rc;
  if ((rc = check_mid(separate_mid, n_in, n_out))) return rc;
  hipStream_t s = (hipStream_t)stream;
  GmsArgs a = fwd_args(in_feats, kernel, out_feats, kpos, in_map, out_map, n_in, n_out, c_in,
                       c_out, k_vol, n_pairs, dtype, s);
  a.reduced = arch80 != 0 && dtype == FGMS_F32;
  if (separate_mid) {
    // centre product first and overwriting, as the beta = 0 GEMM of the reference
    const size_t esz = dtype == FGMS_F16 ? 2 : 4;
    if ((rc = launch_fill_zero(out_feats, (size_t)n_out * c_out * esz, s))) return rc;
    GmsArgs d = a;
    d.gmap = d.smap = nullptr;
    d.dense_k = mid_of(k_vol);
    d.n_dense = n_out;
    if ((rc = run_gms(d, nullptr))) return rc;
  }
  const Plan *p = plan_resolve(plan, s, &rc);
  CheckFlush flush{p, s};
  if (rc) return rc;
  return run_gms(a, p);
}

int fgms_fwd(const void *in_feats, const void *kernel, int sum_nnz, void *out_feats,
             const int32_t *kernel_nnz, const int32_t *kernel_pos, const int32_t *in_map,
             const int32_t *out_map, int separate_mid, int arch80, int64_t n_in, int64_t n_out,
             int c_in, int c_out, int k_vol, int64_t n_pairs, int dtype, fgms_plan_t *plan,
             void *stream) {
  (void)sum_nnz;
  int rc = check_common(in_feats, kernel, out_feats, kernel_pos, in_map, out_map, n_in, n_out,
                        c_in, c_out, k_vol, n_pairs, dtype);
  if (rc) return rc;
  if ((rc = check_mid(separate_mid, n_in, n_out))) return rc;
  if (!kernel_nnz) {
    set_error("kernel_nnz (host int32[k_vol]) is null");
    return FGMS_E_INVALID;
  }
  // The host-side counts bound the pair range exactly (the reference walks them
  // to slice the maps, backend/spconv.cu:307-324).
  int64_t total = 0;
  for (int k = 0; k < k_vol; ++k) {
    if (kernel_nnz[k] < 0) {
      set_error("kernel_nnz[%d] is negative", k);
      return FGMS_E_INVALID;
    }
    total += kernel_nnz[k];
  }
  if (total > n_pairs) {
    set_error("kernel_nnz sums to %lld but the maps hold %lld pairs", (long long)total,
              (long long)n_pairs);
    return FGMS_E_INVALID;
  }
  hipStream_t s = (hipStream_t)stream;
  GmsArgs a = fwd_args(in_feats, kernel, out_feats, kernel_pos, in_map, out_map, n_in, n_out,
                       c_in, c_out, k_vol, total, dtype, s);
  a.reduced = arch80 != 0 && dtype == FGMS_F32;
  const Plan *p = plan_resolve(plan, s, &rc);
  CheckFlush flush{p, s};
  if (rc) return rc;
  if ((rc = run_gms(a, p))) return rc;
  if (separate_mid) {
    GmsArgs d = a;
    d.gmap = d.smap = nullptr;
    d.dense_k = mid_of(k_vol);
    d.n_dense = n_out;
    if ((rc = run_gms(d, nullptr))) return rc;
  }
  return FGMS_OK;
}

int fgms_dgrad(const void *out_feats_grad, const void *kernel, void *in_feats_grad,
               const int32_t *kpos, const int32_t *in_map, const int32_t *out_map, int64_t n_in,
               int64_t n_out, int c_in, int c_out, int k_vol, int64_t n_pairs, int dtype,
               fgms_plan_t *plan, void *stream) {
  int rc = check_common(out_feats_grad, kernel, in_feats_grad, kpos, in_map, out_map, n_in, n_out,
                        c_in, c_out, k_vol, n_pairs, dtype);
  if (rc) return rc;
  GmsArgs a{};
  a.src = out_feats_grad; a.w = kernel; a.dst = in_feats_grad; a.kpos = kpos;
  a.gmap = out_map; a.smap = in_map;   // roles swap, as at backend/spconv.cu:460,559
  a.n_src = n_out; a.n_dst = n_in; a.c_in = c_in; a.c_out = c_out; a.k_vol = k_vol;
  a.n_pairs = n_pairs; a.transpose_w = true; a.dense_k = -1; a.n_dense = 0; a.dtype = dtype;
  a.stream = (hipStream_t)stream;
  const Plan *p = plan_resolve(plan, a.stream, &rc);
  CheckFlush flush{p, a.stream};
  if (rc) return rc;
  return run_gms(a, p);
}

int fgms_wgrad(const void *in_feats, const void *out_feats_grad, void *kernel_grad,
               const int32_t *kpos, const int32_t *in_map, const int32_t *out_map, int64_t n_in,
               int64_t n_out, int c_in, int c_out, int k_vol, int64_t n_pairs, int dtype,
               fgms_plan_t *plan, void *stream) {
  int rc = check_common(in_feats, out_feats_grad, kernel_grad, kpos, in_map, out_map, n_in, n_out,
                        c_in, c_out, k_vol, n_pairs, dtype);
  if (rc) return rc;
  WgradArgs a{};
  a.in = in_feats; a.gout = out_feats_grad; a.gw = kernel_grad; a.kpos = kpos;
  a.imap = in_map; a.omap = out_map; a.n_in = n_in; a.n_out = n_out; a.c_in = c_in;
  a.c_out = c_out; a.k_vol = k_vol; a.n_pairs = n_pairs; a.dtype = dtype;
  a.stream = (hipStream_t)stream;
  a.plan = plan_resolve(plan, a.stream, &rc);
  CheckFlush flush{a.plan, a.stream};
  if (rc) return rc;
  return run_wgrad(a);
}

int fgms_wgrad_static(const void *in_feats, const void *out_feats_grad, void *kernel_grad,
                      const int32_t *kpos, const int32_t *in_map, const int32_t *out_map, int64_t n_in,
                      int64_t n_out, int c_in, int c_out, int k_vol, int64_t n_pairs, int dtype,
                      fgms_plan_t *plan, void *stream) {
  int rc = check_common(in_feats, out_feats_grad, kernel_grad, kpos, in_map, out_map, n_in, n_out,
                        c_in, c_out, k_vol, n_pairs, dtype);
  if (rc) return rc;
  WgradArgs a{};
  a.in = in_feats; a.gout = out_feats_grad; a.gw = kernel_grad; a.kpos = kpos;
  a.imap = in_map; a.omap = out_map; a.n_in = n_in; a.n_out = n_out; a.c_in = c_in;
  a.c_out = c_out; a.k_vol = k_vol; a.n_pairs = n_pairs; a.dtype = dtype;
  a.stream = (hipStream_t)stream;
  // (resolving a plan on its first use waits for the build and may allocate the pair view: this
  // entry point does neither, it takes the plan's row bands only if they are known already)
  a.plan = plan_if_resolved(plan);
  return wgrad_static(a);
}

int fgms_bwd(const void *out_feats_grad, const void *in_feats, const void *kernel, int sum_nnz,
             void *in_feats_grad, void *kernel_grad, const int32_t *kpos, const int32_t *qkpos,
             const int32_t *in_map, const int32_t *out_map, int separate_mid, int arch80,
             int64_t n_in, int64_t n_out, int c_in, int c_out, int k_vol, int64_t n_pairs,
             int dtype, fgms_plan_t *plan, void *stream) {
  (void)sum_nnz; (void)qkpos; (void)separate_mid;
  int rc = check_common(out_feats_grad, kernel, in_feats_grad, kpos, in_map, out_map, n_in, n_out,
                        c_in, c_out, k_vol, n_pairs, dtype);
  if (rc) return rc;
  if ((rc = check_common(in_feats, out_feats_grad, kernel_grad, kpos, in_map, out_map, n_in, n_out,
                         c_in, c_out, k_vol, n_pairs, dtype)))
    return rc;
  const Plan *p = plan_resolve(plan, (hipStream_t)stream, &rc);
  CheckFlush flush{p, (hipStream_t)stream};
  if (rc) return rc;
  GmsArgs d{};
  d.src = out_feats_grad; d.w = kernel; d.dst = in_feats_grad; d.kpos = kpos;
  d.gmap = out_map; d.smap = in_map;   // roles swap, as at backend/spconv.cu:460,559
  d.n_src = n_out; d.n_dst = n_in; d.c_in = c_in; d.c_out = c_out; d.k_vol = k_vol;
  d.n_pairs = n_pairs; d.transpose_w = true; d.dense_k = -1; d.n_dense = 0; d.dtype = dtype;
  d.stream = (hipStream_t)stream;
  d.reduced = arch80 != 0 && dtype == FGMS_F32;     // (the reference's backward is tf32 whenever the tensors are fp32)
  WgradArgs w{};
  w.in = in_feats; w.gout = out_feats_grad; w.gw = kernel_grad; w.kpos = kpos;
  w.imap = in_map; w.omap = out_map; w.n_in = n_in; w.n_out = n_out; w.c_in = c_in;
  w.c_out = c_out; w.k_vol = k_vol; w.n_pairs = n_pairs; w.dtype = dtype;
  w.stream = (hipStream_t)stream;
  w.plan = p;
  w.reduced = d.reduced;
  // Both gradients through their main kernels: two launches instead of four.  The weight
  // gradient goes first and its launch also re-lays the weights for the input gradient,
  // whose launch in turn also rounds the weight gradient's fp32 sums into the caller's
  // fp16 tensor.  (The two gradients do not depend on each other.)
  if (n_pairs > 0 && (!p || p->groups.empty()) && route_of(d, p) == Route::kRows && g_policy != 1 && mfma_wgrad_supported(w)) {
    plan_touch(p, d.stream);
    // one launch for both where the shapes allow (and a small one that rounds an fp16
    // weight gradient), else two
    bool fused = false;
    if ((rc = launch_fused_bwd(d, p, w, &fused))) return rc;
    if (fused) return FGMS_OK;
    SideJob pack{}, flush{};
    const void *packed = nullptr;
    if ((rc = planned_pack_job(d, &pack, &packed))) return rc;
    w.side = pack;
    w.deferred_flush = &flush;
    if ((rc = launch_mfma_wgrad(w))) return rc;
    d.prepacked = packed;
    d.side = flush;
    if ((rc = launch_planned_gms(d, p))) {
      (void)launch_side_job(flush, d.stream);   // the accumulator must not stay filled
      return rc;
    }
    return FGMS_OK;
  }
  if ((rc = run_gms(d, p))) return rc;
  return run_wgrad(w);
}

int fgms_build_kernel_map(const int32_t *in_coords, int64_t n_in, const int32_t *out_coords,
                          int64_t n_out, const int32_t *offsets, int k_vol, int stride,
                          int skip_offset, int32_t *in_map, int32_t *out_map, int64_t capacity,
                          int32_t *kernel_nnz, int32_t *kpos, int64_t *n_pairs, void *stream) {
  if (n_in < 0 || n_out < 0 || k_vol <= 0 || stride <= 0 || capacity < 0 || !offsets || !kernel_nnz ||
      !kpos || !n_pairs || (n_in > 0 && !in_coords) || (n_out > 0 && !out_coords) ||
      (capacity > 0 && (!in_map || !out_map)) || n_in > INT32_MAX ||
      (int64_t)k_vol * n_out > INT32_MAX - 65536) {
    set_error("fgms_build_kernel_map: bad argument");
    return FGMS_E_INVALID;
  }
  return build_kernel_map(in_coords, n_in, out_coords, n_out, offsets, k_vol, stride, skip_offset,
                          in_map, out_map, capacity, kernel_nnz, kpos, n_pairs, (hipStream_t)stream);
}

int fgms_probe_gather(const void *feats, int c_src, int dtype, int for_dgrad, fgms_plan_t *plan,
                      void *stream) {
  int prc = FGMS_OK;
  const Plan *p = plan_resolve(plan, (hipStream_t)stream, &prc);
  if (!p || !feats || c_src <= 0 || (dtype != FGMS_F16 && dtype != FGMS_F32)) {
    if (!prc) set_error("fgms_probe_gather: bad argument");
    return FGMS_E_INVALID;
  }
  plan_touch(p, (hipStream_t)stream);
  void *sink = nullptr;
  int rc = workspace_get((hipStream_t)stream, 3, 256, &sink);
  if (rc) return rc;
  return launch_gather_probe(p, feats, c_src, dtype, for_dgrad != 0, sink, (hipStream_t)stream);
}

}  // extern "C"
