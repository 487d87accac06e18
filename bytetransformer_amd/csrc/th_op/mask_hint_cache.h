// The one thing the PyTorch operator keeps between calls: the number of valid tokens of a
// mask tensor.  It is a HINT: it picks tile shapes and weight layouts, never a launch size;
// the offsets themselves are rebuilt from the mask on the device in every call, and the
// weights are read as they are at the call.  A stale count costs time and nothing else.
//
// The host never waits for it (the reference blocks on this very count in every call,
// remove_padding.h:99-100): the first layer call that meets a mask tensor hands the layer a
// slot of pinned host memory, the layer's first launch is followed by a one-wave launch that
// stores the count there, and whichever later call finds the slot filled uses it - in a
// 12-layer forward that is the second or third layer.  Until then the layer runs on its own
// estimate (60 % of the padded rows).
//
// An entry is found through the tensor's identity (TensorImpl alive, version counter, data
// pointer, shape, device, stream unchanged); inference tensors carry no version counter and
// are matched by data pointer and shape alone.  BT_PREPACK_CACHE=0 in the environment, or
// set_caches_enabled(false), turns the hint off; clear_caches() drops every entry.
#pragma once
#include <c10/util/intrusive_ptr.h>
#include <hip/hip_runtime_api.h>
#include <torch/all.h>

#include <atomic>
#include <cstdlib>
#include <mutex>
#include <vector>

#include "bt_hip.h"

namespace bytetransformer {
namespace torch_ext {

// Identity of one tensor as the host can see it.
struct TensorStamp {
  c10::weak_intrusive_ptr<c10::TensorImpl> owner{c10::intrusive_ptr<c10::TensorImpl>()};
  bool versioned = false;
  int64_t version = 0;
  void *data = nullptr;
  std::vector<int64_t> sizes;
  c10::Device device{c10::kCPU};

  static TensorStamp of(const torch::Tensor &t) {
    TensorStamp s;
    s.versioned = !t.is_inference();
    if (s.versioned) {
      s.owner = c10::weak_intrusive_ptr<c10::TensorImpl>(t.getIntrusivePtr());
      s.version = t._version();
    }
    s.data = t.data_ptr();
    s.sizes = t.sizes().vec();
    s.device = t.device();
    return s;
  }
  bool matches(const torch::Tensor &t) const {
    if (data != t.data_ptr() || sizes != t.sizes().vec() || device != t.device()) return false;
    if (versioned != !t.is_inference()) return false;
    if (!versioned) return true;
    auto alive = owner.lock();
    return alive && alive.get() == t.unsafeGetTensorImpl() && version == t._version();
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

  // The count for this mask on this stream if a layer call has published it by now (then
  // *count > 0 and the return value is null), else 0; for a mask not met before also a
  // slot for the layer to publish the count into (null when none is free: the pool is a
  // ring, and a slot whose count is still on its way is not handed out again).
  int *lookup_or_reserve(const torch::Tensor &mask, void *stream, int *count) {
    *count = 0;
    if (!caches_enabled().load(std::memory_order_relaxed)) return nullptr;
    std::lock_guard<std::mutex> g(mu_);
    if (!pool_ && !allocate()) return nullptr;
    for (Entry &e : entries_) {
      if (!e.used || e.stream != stream || !e.stamp.matches(mask)) continue;
      const int v = *(volatile int *)(pool_ + (&e - entries_.data()));
      if (v > 0) *count = v;
      return nullptr;       // published, or still on its way
    }
    Entry &e = entries_[next_];
    int *slot = pool_ + next_;
    if (e.used && *(volatile int *)slot == kPending) return nullptr;
    next_ = (next_ + 1) % kSlots;
    *(volatile int *)slot = kPending;
    e.used = true;
    e.stamp = TensorStamp::of(mask);
    e.stream = stream;
    return slot;
  }

  void clear() {
    std::lock_guard<std::mutex> g(mu_);
    for (size_t i = 0; i < entries_.size(); ++i)
      // (a slot whose count is still on its way stays reserved until it has arrived)
      if (!pool_ || *(volatile int *)(pool_ + i) != kPending) entries_[i].used = false;
      else entries_[i].stamp = TensorStamp();
  }

 private:
  struct Entry {
    bool used = false;
    TensorStamp stamp;
    void *stream = nullptr;
  };
  static constexpr int kSlots = 64;
  static constexpr int kPending = -1;

  bool allocate() {
    // pinned host memory that the device can write; kept until the process ends
    void *p = nullptr;
    if (hipHostMalloc(&p, kSlots * sizeof(int), hipHostMallocPortable | hipHostMallocMapped) != hipSuccess || !p) {
      (void)hipGetLastError();
      return false;
    }
    pool_ = (int *)p;
    for (int i = 0; i < kSlots; ++i) pool_[i] = 0;
    entries_.resize(kSlots);
    return true;
  }

  std::mutex mu_;
  int *pool_ = nullptr;
  std::vector<Entry> entries_;
  int next_ = 0;
};

}  // namespace torch_ext
}  // namespace bytetransformer
