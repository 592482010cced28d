// Python module FGMS.backend: the three functions hkeee21/FGMS exports
// (backend/pybind_cuda.cpp:7-11) with the same names and positional arguments
// (backend/spconv.h:10-49), over the C ABI of libfgms_hip.so.
//
// Differences a caller can observe, all deliberate:
//  * work is queued on torch's current HIP stream, not on stream 0
//    (the reference uses bare <<<>>> launches, backend/spconv.cu:112);
//  * a kernel-map plan is built on first use of a (kpos, in_map, out_map)
//    triple (asynchronously: the call queues the build and goes on) and kept in a
//    small cache; an entry holds references to the three tensors, so their storage
//    cannot be recycled while it is cached, and is dropped when one of them is
//    modified in place (version counter).  Writes through raw pointers do not bump
//    it, and tensors made under inference mode have none: every cache hit therefore
//    queues a fingerprint check of the lists (fgms_plan_check), and the call after
//    a rewrite raises RuntimeError and drops the plan.  A call with in_map and out_map exchanged (the
//    transposed convolution over the same pairs) shares the cached plan's tables;
//  * fgms_weights_pin(kernel) lets the library keep the re-laid copies of a weight tensor that
//    some kernels read (inference); a forward call that finds the tensor's version counter
//    moved drops them;
//  * HIP errors raise RuntimeError instead of passing silently.
#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <cstdlib>
#include <list>
#include <mutex>
#include <stdexcept>
#include <vector>

#include "fgms.h"
#include "fgms_diag.h"

namespace {

struct CacheEntry {
  at::Tensor kpos, in_map, out_map;       // keeps the storage alive
  int64_t v_kpos, v_in, v_out;            // version counters at build time
  int64_t n_in, n_out;
  int device;
  fgms_plan_t *plan;
  bool view;                              // a transposed view of another entry's plan
};

// Inference tensors track no version.
int64_t version_of(const at::Tensor &t) { return t.is_inference() ? 0 : (int64_t)t._version(); }

size_t g_views_made = 0;

std::mutex g_mutex;
std::list<CacheEntry> g_cache;            // most recently used first
size_t g_cache_cap = 8;
bool g_cache_enabled = true;

void drop(std::list<CacheEntry>::iterator it) {
  fgms_plan_destroy(it->plan);
  g_cache.erase(it);
}

void clear_cache() {
  std::lock_guard<std::mutex> lock(g_mutex);
  while (!g_cache.empty()) drop(g_cache.begin());
}

void set_cache(bool enabled, int64_t capacity) {
  clear_cache();
  std::lock_guard<std::mutex> lock(g_mutex);
  g_cache_enabled = enabled;
  if (capacity > 0) g_cache_cap = (size_t)capacity;
}

size_t cache_size() {
  std::lock_guard<std::mutex> lock(g_mutex);
  return g_cache.size();
}

void check(int rc) {
  if (rc == FGMS_OK) return;
  if (rc == FGMS_E_INVALID) throw std::invalid_argument(fgms_last_error());
  throw std::runtime_error(fgms_last_error());
}

const int32_t *i32(const at::Tensor &t) { return t.numel() ? t.data_ptr<int>() : nullptr; }

int dtype_of(const at::Tensor &t) {
  if (t.scalar_type() == at::ScalarType::Half) return FGMS_F16;
  if (t.scalar_type() == at::ScalarType::Float) return FGMS_F32;
  throw std::invalid_argument("FGMS handles float32 and float16 tensors");
}

void same_dtype(const at::Tensor &a, const at::Tensor &b, const char *what) {
  if (a.scalar_type() != b.scalar_type())
    throw std::invalid_argument(std::string(what) + " must have the dtype of the features");
}

void need_contiguous_cuda(const at::Tensor &t, const char *name) {
  if (!t.is_cuda()) throw std::invalid_argument(std::string(name) + " must be a GPU tensor");
  if (!t.is_contiguous()) throw std::invalid_argument(std::string(name) + " must be contiguous");
}

// Finds or builds the plan for this map.  Returns nullptr when caching is off.
fgms_plan_t *plan_for(const at::Tensor &kpos, const at::Tensor &in_map, const at::Tensor &out_map,
                      int64_t n_in, int64_t n_out, int k_vol, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_cache_enabled) return nullptr;
  const int dev = in_map.get_device();
  for (auto it = g_cache.begin(); it != g_cache.end(); ++it) {
    if (it->in_map.is_same(in_map) && it->out_map.is_same(out_map) && it->kpos.is_same(kpos) &&
        it->n_in == n_in && it->n_out == n_out && it->device == dev) {
      if (it->v_in == version_of(in_map) && it->v_out == version_of(out_map) &&
          it->v_kpos == version_of(kpos)) {
        // The version counters do not see writes through raw pointers (a map builder filling a
        // pre-allocated tensor, this library's own included).  Every hit queues a check of the
        // lists against the fingerprint the plan was built with; what it finds reaches the host
        // a call later: that call drops the plan and raises.
        const int rc = fgms_plan_check(it->plan, stream, 1);      // (rides along with this call's launch)
        if (rc == FGMS_E_STALE) {
          drop(it);
          throw std::runtime_error(
              "FGMS: the kernel map tensors were rewritten in place after their plan was cached "
              "(a write through data_ptr() does not bump the version counter); the previous call on this "
              "map used the old neighbour tables.  Call fgms_plan_cache_clear() after rewriting a map.");
        }
        check(rc);
        g_cache.splice(g_cache.begin(), g_cache, it);
        return g_cache.front().plan;
      }
      drop(it);  // modified in place since the plan was built
      break;
    }
  }
  // a map first seen while the stream is being captured into a graph: no plan is built (the build
  // allocates, and its kernels would be recorded); the call records the kernels that need none
  {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone) return nullptr;
  }
  fgms_plan_t *plan = nullptr;
  bool view = false;
  // the same pairs with the sides exchanged: share that plan's tables
  for (auto it = g_cache.begin(); it != g_cache.end(); ++it) {
    if (!it->view && it->in_map.is_same(out_map) && it->out_map.is_same(in_map) && it->kpos.is_same(kpos) &&
        it->n_in == n_out && it->n_out == n_in && it->device == dev && it->v_in == version_of(out_map) &&
        it->v_out == version_of(in_map) && it->v_kpos == version_of(kpos)) {
      check(fgms_plan_transposed(&plan, it->plan));
      view = true;
      ++g_views_made;
      break;
    }
  }
  if (!plan)
    check(fgms_plan_create(&plan, i32(kpos), i32(in_map), i32(out_map), n_in, n_out, k_vol,
                           in_map.numel(), stream));
  g_cache.push_front(CacheEntry{kpos, in_map, out_map, version_of(kpos), version_of(in_map),
                                version_of(out_map), n_in, n_out, dev, plan, view});
  while (g_cache.size() > g_cache_cap) drop(std::prev(g_cache.end()));
  return plan;
}

// Weight tensors whose re-laid copies the library may keep (fgms_weights_pin): the entry holds
// the tensor, so that its address cannot go to another tensor meanwhile, and its version counter;
// a forward call that finds the counter moved pins the address again, which drops the copies.
struct PinnedWeights {
  at::Tensor kernel;
  int64_t version;
};
std::vector<PinnedWeights> g_pins;

void pin_weights(const at::Tensor &kernel) {
  need_contiguous_cuda(kernel, "kernel");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(kernel.device());
  std::lock_guard<std::mutex> lock(g_mutex);
  for (auto &p : g_pins)
    if (p.kernel.is_same(kernel)) {
      p.version = version_of(kernel);
      check(fgms_weights_pin(kernel.data_ptr()));
      return;
    }
  check(fgms_weights_pin(kernel.data_ptr()));
  g_pins.push_back(PinnedWeights{kernel, version_of(kernel)});
}

void unpin_weights(const at::Tensor &kernel) {
  c10::hip::HIPGuardMasqueradingAsCUDA guard(kernel.device());
  std::lock_guard<std::mutex> lock(g_mutex);
  for (size_t i = 0; i < g_pins.size(); ++i)
    if (g_pins[i].kernel.is_same(kernel)) {
      check(fgms_weights_unpin(kernel.data_ptr()));
      g_pins.erase(g_pins.begin() + i);
      return;
    }
}

// (with the device guard of the call in place)
void refresh_pin(const at::Tensor &kernel) {
  if (g_pins.empty()) return;
  std::lock_guard<std::mutex> lock(g_mutex);
  for (auto &p : g_pins)
    if (p.kernel.is_same(kernel)) {
      const int64_t v = version_of(kernel);
      if (v != p.version) {
        check(fgms_weights_pin(kernel.data_ptr()));
        p.version = v;
      }
      return;
    }
}

void check_channels(const at::Tensor &in_feats, const at::Tensor &kernel) {
  // the reference's one argument check, backend/spconv.cu:39-43
  if (in_feats.size(1) != kernel.size(1))
    throw std::invalid_argument("Input feature size and kernel size mismatch");
}

}  // namespace

void ConvolutionForwardFused(const at::Tensor in_feats, const at::Tensor kernel, const int sum_nnz,
                             at::Tensor out_feats, const at::Tensor kpos, const at::Tensor qkpos,
                             const at::Tensor in_map, const at::Tensor out_map,
                             const bool separate_mid, const bool arch80) {
  check_channels(in_feats, kernel);
  need_contiguous_cuda(in_feats, "in_feats"); need_contiguous_cuda(kernel, "kernel");
  need_contiguous_cuda(out_feats, "out_feats"); need_contiguous_cuda(kpos, "kpos");
  need_contiguous_cuda(in_map, "in_map"); need_contiguous_cuda(out_map, "out_map");
  same_dtype(in_feats, kernel, "kernel"); same_dtype(in_feats, out_feats, "out_feats");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(in_feats.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  const int k_vol = (int)kernel.size(0);
  refresh_pin(kernel);
  fgms_plan_t *plan = plan_for(kpos, in_map, out_map, in_feats.size(0), out_feats.size(0), k_vol, stream);
  check(fgms_fusion_fwd(in_feats.data_ptr(), kernel.data_ptr(), sum_nnz, out_feats.data_ptr(),
                        i32(kpos), qkpos.defined() && qkpos.numel() ? i32(qkpos) : nullptr,
                        i32(in_map), i32(out_map), separate_mid, arch80, in_feats.size(0),
                        out_feats.size(0), (int)kernel.size(1), (int)kernel.size(2), k_vol,
                        in_map.numel(), dtype_of(in_feats), plan, stream));
}

void ConvolutionForward(const at::Tensor in_feats, const at::Tensor kernel, const int sum_nnz,
                        at::Tensor out_feats, const at::Tensor kernel_nnz,
                        const at::Tensor kernel_pos, const at::Tensor in_map,
                        const at::Tensor out_map, const bool separate_mid, const bool arch80) {
  check_channels(in_feats, kernel);
  need_contiguous_cuda(in_feats, "in_feats"); need_contiguous_cuda(kernel, "kernel");
  need_contiguous_cuda(out_feats, "out_feats"); need_contiguous_cuda(kernel_pos, "kernel_pos");
  need_contiguous_cuda(in_map, "in_map"); need_contiguous_cuda(out_map, "out_map");
  same_dtype(in_feats, kernel, "kernel"); same_dtype(in_feats, out_feats, "out_feats");
  if (kernel_nnz.is_cuda())
    throw std::invalid_argument("kernel_nnz must be a CPU int32 tensor (it is read on the host)");
  const int k_vol = (int)kernel.size(0);
  if (kernel_nnz.numel() < k_vol) throw std::invalid_argument("kernel_nnz is shorter than k_vol");
  at::Tensor knnz = kernel_nnz.contiguous();
  c10::hip::HIPGuardMasqueradingAsCUDA guard(in_feats.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  refresh_pin(kernel);
  fgms_plan_t *plan = plan_for(kernel_pos, in_map, out_map, in_feats.size(0), out_feats.size(0), k_vol, stream);
  check(fgms_fwd(in_feats.data_ptr(), kernel.data_ptr(), sum_nnz, out_feats.data_ptr(),
                 knnz.data_ptr<int>(), i32(kernel_pos), i32(in_map), i32(out_map), separate_mid,
                 arch80, in_feats.size(0), out_feats.size(0), (int)kernel.size(1),
                 (int)kernel.size(2), k_vol, in_map.numel(), dtype_of(in_feats), plan, stream));
}

void ConvolutionBackward(const at::Tensor out_feats_grad, const at::Tensor in_feats,
                         const at::Tensor kernel, const int sum_nnz, at::Tensor in_feats_grad,
                         at::Tensor kernel_grad, const at::Tensor kpos, const at::Tensor qkpos,
                         const at::Tensor in_map, const at::Tensor out_map,
                         const bool separate_mid, const bool arch80) {
  check_channels(in_feats, kernel);
  need_contiguous_cuda(out_feats_grad, "out_feats_grad"); need_contiguous_cuda(in_feats, "in_feats");
  need_contiguous_cuda(kernel, "kernel"); need_contiguous_cuda(in_feats_grad, "in_feats_grad");
  need_contiguous_cuda(kernel_grad, "kernel_grad"); need_contiguous_cuda(kpos, "kpos");
  need_contiguous_cuda(in_map, "in_map"); need_contiguous_cuda(out_map, "out_map");
  same_dtype(in_feats, kernel, "kernel"); same_dtype(in_feats, out_feats_grad, "out_feats_grad");
  same_dtype(in_feats, in_feats_grad, "in_feats_grad"); same_dtype(in_feats, kernel_grad, "kernel_grad");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(in_feats.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
  const int k_vol = (int)kernel.size(0);
  fgms_plan_t *plan = plan_for(kpos, in_map, out_map, in_feats.size(0), out_feats_grad.size(0), k_vol, stream);
  check(fgms_bwd(out_feats_grad.data_ptr(), in_feats.data_ptr(), kernel.data_ptr(), sum_nnz,
                 in_feats_grad.data_ptr(), kernel_grad.data_ptr(), i32(kpos),
                 qkpos.defined() && qkpos.numel() ? i32(qkpos) : nullptr, i32(in_map),
                 i32(out_map), separate_mid, arch80, in_feats.size(0), out_feats_grad.size(0),
                 (int)kernel.size(1), (int)kernel.size(2), k_vol, in_map.numel(),
                 dtype_of(in_feats), plan, stream));
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("fgms_fusion_fwd_cuda", &ConvolutionForwardFused);
  m.def("fgms_fwd_cuda", &ConvolutionForward);
  m.def("fgms_bwd_cuda", &ConvolutionBackward);
  // additions (not in the reference): plan-cache control and library identity
  m.def("fgms_plan_cache", &set_cache, pybind11::arg("enabled"), pybind11::arg("capacity") = 8);
  m.def("fgms_plan_cache_clear", &clear_cache);
  m.def("fgms_plan_cache_size", &cache_size);
  m.def("fgms_plan_cache_views", []() { std::lock_guard<std::mutex> lock(g_mutex); return g_views_made; });
  m.def("fgms_weights_pin", &pin_weights, pybind11::arg("kernel"));
  m.def("fgms_weights_unpin", &unpin_weights, pybind11::arg("kernel"));
  m.def("fgms_version", []() { return std::string(fgms_version()); });
  m.def("fgms_set_kernel_policy", &fgms_set_kernel_policy);
}
