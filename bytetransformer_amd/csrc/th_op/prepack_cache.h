// Process-wide caches of the PyTorch operator.  The operator is called once per layer
// with the same weight tensors on every forward and with one mask per forward, so two
// things are worth keeping between calls - and neither may ever change a result:
//
//   PrepackCache   the pre-packed ([N, K], k-contiguous) copies of a layer's four weight
//                  matrices.  An entry is found through the tensors' identity (TensorImpl
//                  alive, version counter, data pointer, shape, device, stream unchanged);
//                  that bookkeeping cannot see a write that goes around the version counter
//                  (`w.data.copy_()`, DLPack, a raw-pointer kernel), so every reuse is also
//                  CHECKED ON THE DEVICE: the layer's prologue launch fingerprints the four
//                  weight tensors and re-packs inside that launch when the fingerprint is
//                  not the one the copies were made from (bt_layer_prologue).  A hit is
//                  therefore only ever a saving of time.
//   MaskHintCache  the number of valid tokens of a mask tensor, read back once per mask
//                  (one host synchronisation).  It is a HINT: it picks tile shapes, never a
//                  launch size; the offsets themselves are rebuilt from the mask on the
//                  device in every call.  A stale count costs time and nothing else.
//
// Inference tensors carry no version counter and are never cached.  BT_PREPACK_CACHE=0 in
// the environment, or set_enabled(false), turns both off; clear() drops every entry.
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

class PrepackCache {
 public:
  struct Packed {
    torch::Tensor block;       // the four copies back to back (QKV, projection, FFN1, FFN2)
    torch::Tensor packed[4];   // views into block, [N, K] each
    torch::Tensor state;       // int64[BT_PREPACK_STATE_WORDS]: fingerprint record of bt_layer_prologue
  };

  static PrepackCache &instance() {
    static PrepackCache c;
    return c;
  }

  bool enabled() const { return caches_enabled().load(std::memory_order_relaxed); }

  // The copies made from exactly these four tensor objects on this stream, if any.
  bool lookup(const torch::Tensor *const (&w)[4], void *stream, Packed *out) {
    if (!enabled()) return false;
    for (const torch::Tensor *t : w)
      if (t->is_inference()) return false;
    std::lock_guard<std::mutex> g(mu_);
    auto it = map_.find(w[0]->unsafeGetTensorImpl());
    if (it == map_.end()) return false;
    Entry &e = it->second;
    bool ok = e.stream == stream;
    for (int i = 0; ok && i < 4; ++i) ok = e.stamp[i].matches(*w[i]);
    if (!ok) {
      map_.erase(it);
      sweep();
      return false;
    }
    *out = e.value;
    return true;
  }

  void store(const torch::Tensor *const (&w)[4], void *stream, const Packed &value) {
    if (!enabled()) return;
    for (const torch::Tensor *t : w)
      if (t->is_inference()) return;
    std::lock_guard<std::mutex> g(mu_);
    sweep();
    if (map_.size() >= kMaxEntries) map_.clear();
    Entry e;
    for (int i = 0; i < 4; ++i) e.stamp[i] = TensorStamp::of(*w[i]);
    e.stream = stream;
    e.value = value;
    map_[w[0]->unsafeGetTensorImpl()] = std::move(e);
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
    TensorStamp stamp[4];
    void *stream = nullptr;
    Packed value;
  };
  static constexpr size_t kMaxEntries = 1024;

  // Entries whose weights have died hold a layer's worth of device memory each: they go
  // at every miss and store (a scan of at most kMaxEntries weak pointers).
  void sweep() {
    for (auto it = map_.begin(); it != map_.end();) {
      bool dead = false;
      for (const TensorStamp &s : it->second.stamp) dead = dead || s.expired();
      it = dead ? map_.erase(it) : std::next(it);
    }
  }

  std::mutex mu_;
  std::unordered_map<const c10::TensorImpl *, Entry> map_;
};

class MaskHintCache {
 public:
  static MaskHintCache &instance() {
    static MaskHintCache c;
    return c;
  }

  bool lookup(const torch::Tensor &mask, void *stream, int *valid_word_num) {
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
