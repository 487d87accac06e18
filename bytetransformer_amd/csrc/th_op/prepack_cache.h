// Process-wide cache of pre-packed ([N, K], k-contiguous) copies of weight
// tensors for the PyTorch operator.  The operator is called once per layer with
// the same weight tensors on every forward, so the transposes are made once and
// reused for as long as the very same tensor object still holds the very same
// data: an entry is keyed on the TensorImpl address and is valid only while
//   - that TensorImpl is still alive (weak reference lock succeeds),
//   - its version counter is unchanged (any in-place write, also through a
//     view, bumps it),
//   - its data pointer, shape and device are unchanged, and
//   - the calling stream is the one the copy was made on.
// Anything else re-packs.  Inference tensors carry no version counter and are
// never cached.  BT_PREPACK_CACHE=0 in the environment disables the cache.
#pragma once
#include <c10/util/intrusive_ptr.h>
#include <torch/all.h>

#include <cstdlib>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "bt_hip.h"

namespace bytetransformer {
namespace torch_ext {

class PrepackCache {
 public:
  static PrepackCache &instance() {
    static PrepackCache c;
    return c;
  }

  bool enabled() const { return enabled_; }

  // Returns the [N, K] copy of the 2-D weight `w` ([K, N]); `hit` reports whether
  // the copy came from the cache.  A miss leaves `packed` undefined.
  bool lookup(const torch::Tensor &w, void *stream, torch::Tensor *packed) {
    if (!enabled_ || w.is_inference()) return false;
    std::lock_guard<std::mutex> g(mu_);
    auto it = map_.find(w.unsafeGetTensorImpl());
    if (it == map_.end()) return false;
    Entry &e = it->second;
    auto alive = e.owner.lock();
    if (!alive || alive.get() != w.unsafeGetTensorImpl() || e.version != w._version() ||
        e.data != w.data_ptr() || e.stream != stream || e.k != w.size(0) || e.n != w.size(1) ||
        e.device != w.device()) {
      map_.erase(it);
      return false;
    }
    *packed = e.packed;
    return true;
  }

  void store(const torch::Tensor &w, void *stream, const torch::Tensor &packed) {
    if (!enabled_ || w.is_inference()) return;
    std::lock_guard<std::mutex> g(mu_);
    if (map_.size() >= kMaxEntries) sweep();
    Entry e;
    e.owner = c10::weak_intrusive_ptr<c10::TensorImpl>(w.getIntrusivePtr());
    e.version = w._version();
    e.data = w.data_ptr();
    e.stream = stream;
    e.k = w.size(0);
    e.n = w.size(1);
    e.device = w.device();
    e.packed = packed;
    map_[w.unsafeGetTensorImpl()] = std::move(e);
  }

  void clear() {
    std::lock_guard<std::mutex> g(mu_);
    map_.clear();
  }

  size_t size() {
    std::lock_guard<std::mutex> g(mu_);
    return map_.size();
  }

 private:
  struct Entry {
    c10::weak_intrusive_ptr<c10::TensorImpl> owner{c10::intrusive_ptr<c10::TensorImpl>()};
    int64_t version = 0;
    void *data = nullptr;
    void *stream = nullptr;
    int64_t k = 0, n = 0;
    c10::Device device{c10::kCPU};
    torch::Tensor packed;
  };
  static constexpr size_t kMaxEntries = 1024;

  PrepackCache() {
    const char *e = std::getenv("BT_PREPACK_CACHE");
    enabled_ = !(e && e[0] == '0');
  }

  // drop entries whose weight tensor has died; if everything is alive, start over
  void sweep() {
    for (auto it = map_.begin(); it != map_.end();)
      it = it->second.owner.expired() ? map_.erase(it) : std::next(it);
    if (map_.size() >= kMaxEntries) map_.clear();
  }

  bool enabled_ = true;
  std::mutex mu_;
  std::unordered_map<const c10::TensorImpl *, Entry> map_;
};

// Offsets of an attention mask (batch_idx, word_idx, valid-token count), cached
// per mask tensor under the same validity rules as the weight copies.  A model
// calls the operator once per layer with one mask, so the prefix sum - and the
// one host synchronisation that fetches the token count used to pick GEMM tile
// shapes - happens once per mask instead of once per layer.
class MaskPlanCache {
 public:
  struct Plan {
    torch::Tensor batch_idx, word_idx, seq_order;
    int valid_word_num = 0;
    int prefix_state = -1;   // is the mask the plain prefix mask of these lengths? -1 = not checked
  };

  static MaskPlanCache &instance() {
    static MaskPlanCache c;
    return c;
  }

  bool lookup(const torch::Tensor &mask, void *stream, Plan *plan) {
    std::lock_guard<std::mutex> g(mu_);
    auto it = map_.find(mask.unsafeGetTensorImpl());
    if (it == map_.end()) return false;
    Entry &e = it->second;
    auto alive = e.owner.lock();
    if (!alive || alive.get() != mask.unsafeGetTensorImpl() || e.version != mask._version() ||
        e.data != mask.data_ptr() || e.stream != stream || e.sizes != mask.sizes().vec() ||
        e.device != mask.device()) {
      map_.erase(it);
      return false;
    }
    *plan = e.plan;
    return true;
  }

  void store(const torch::Tensor &mask, void *stream, const Plan &plan) {
    std::lock_guard<std::mutex> g(mu_);
    if (map_.size() >= kMaxEntries) {
      for (auto it = map_.begin(); it != map_.end();)
        it = it->second.owner.expired() ? map_.erase(it) : std::next(it);
      if (map_.size() >= kMaxEntries) map_.clear();
    }
    Entry e;
    e.owner = c10::weak_intrusive_ptr<c10::TensorImpl>(mask.getIntrusivePtr());
    e.version = mask._version();
    e.data = mask.data_ptr();
    e.stream = stream;
    e.sizes = mask.sizes().vec();
    e.device = mask.device();
    e.plan = plan;
    map_[mask.unsafeGetTensorImpl()] = std::move(e);
  }

 private:
  struct Entry {
    c10::weak_intrusive_ptr<c10::TensorImpl> owner{c10::intrusive_ptr<c10::TensorImpl>()};
    int64_t version = 0;
    void *data = nullptr;
    void *stream = nullptr;
    std::vector<int64_t> sizes;
    c10::Device device{c10::kCPU};
    Plan plan;
  };
  static constexpr size_t kMaxEntries = 64;
  std::mutex mu_;
  std::unordered_map<const c10::TensorImpl *, Entry> map_;
};

}  // namespace torch_ext
}  // namespace bytetransformer
