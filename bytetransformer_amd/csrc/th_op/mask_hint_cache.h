// The one thing the PyTorch operator keeps between calls: the number of valid tokens of a
// mask tensor, read back once per mask (one host synchronisation).  It is a HINT: it picks
// tile shapes and weight layouts, never a launch size; the offsets themselves are rebuilt
// from the mask on the device in every call, and the weights are read as they are at the
// call.  A stale count costs time and nothing else.  An entry is found through the
// tensor's identity (TensorImpl alive, version counter, data pointer, shape, device, stream
// unchanged); inference tensors carry no version counter and are never cached.
// BT_PREPACK_CACHE=0 in the environment, or set_caches_enabled(false), turns it off;
// clear_caches() drops every entry.
#pragma once
#include <c10/util/intrusive_ptr.h>
#include <torch/all.h>

#include <atomic>
#include <cstdlib>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "bt_hip.h"

namespace bytetransformer {
namespace torch_ext {

// Identity of one tensor as the host can see it.
struct TensorStamp {
  c10::weak_intrusive_ptr<c10::TensorImpl> owner{c10::intrusive_ptr<c10::TensorImpl>()};
  const c10::TensorImpl *impl = nullptr;
  int64_t version = 0;
  void *data = nullptr;
  std::vector<int64_t> sizes;
  c10::Device device{c10::kCPU};

  static TensorStamp of(const torch::Tensor &t) {
    TensorStamp s;
    s.owner = c10::weak_intrusive_ptr<c10::TensorImpl>(t.getIntrusivePtr());
    s.impl = t.unsafeGetTensorImpl();
    s.version = t._version();
    s.data = t.data_ptr();
    s.sizes = t.sizes().vec();
    s.device = t.device();
    return s;
  }
  bool expired() const { return owner.expired(); }
  bool matches(const torch::Tensor &t) const {
    auto alive = owner.lock();
    return alive && alive.get() == t.unsafeGetTensorImpl() && version == t._version() &&
           data == t.data_ptr() && sizes == t.sizes().vec() && device == t.device();
  }
};

inline std::atomic<bool> &caches_enabled() {
  static std::atomic<bool> on{[] {
    const char *e = std::getenv("BT_PREPACK_CACHE");
    return !(e && e[0] == '0');
  }()};
  return on;
}

class MaskHintCache {
 public:
  static MaskHintCache &instance() {
    static MaskHintCache c;
    return c;
  }

  bool lookup(const torch::Tensor &mask, void *stream, int *valid_word_num) {
    if (!caches_enabled().load(std::memory_order_relaxed)) return false;
    std::lock_guard<std::mutex> g(mu_);
    auto it = map_.find(mask.unsafeGetTensorImpl());
    if (it == map_.end()) return false;
    if (it->second.stream != stream || !it->second.stamp.matches(mask)) {
      map_.erase(it);
      return false;
    }
    *valid_word_num = it->second.valid_word_num;
    return true;
  }

  void store(const torch::Tensor &mask, void *stream, int valid_word_num) {
    std::lock_guard<std::mutex> g(mu_);
    for (auto it = map_.begin(); it != map_.end();)
      it = it->second.stamp.expired() ? map_.erase(it) : std::next(it);
    if (map_.size() >= kMaxEntries) map_.clear();
    Entry e;
    e.stamp = TensorStamp::of(mask);
    e.stream = stream;
    e.valid_word_num = valid_word_num;
    map_[mask.unsafeGetTensorImpl()] = std::move(e);
  }

  void clear() {
    std::lock_guard<std::mutex> g(mu_);
    map_.clear();
  }

 private:
  struct Entry {
    TensorStamp stamp;
    void *stream = nullptr;
    int valid_word_num = 0;
  };
  static constexpr size_t kMaxEntries = 64;
  std::mutex mu_;
  std::unordered_map<const c10::TensorImpl *, Entry> map_;
};

}  // namespace torch_ext
}  // namespace bytetransformer
