// Argument checks shared by the PyTorch operator and the TorchScript class.  The
// messages are those of the reference's bytetransformer/th_op/util.h:30-40, so that
// callers matching on them keep working ("CUDA tensor" is PyTorch-ROCm's own name for
// a GPU tensor).
#pragma once
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/all.h>

#include <vector>

namespace bytetransformer {
namespace torch_ext {

constexpr int64_t kMaxSeqLen = 1024;   // the reference's limit (util.h:40)

// Placement, layout and dtype of one named tensor.
inline void check_tensor(const torch::Tensor &t, const char *name, at::ScalarType st,
                         bool any_dtype) {
  TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(any_dtype || t.scalar_type() == st, "Inconsistency of Tensor type: ", name);
}

inline void check_seq_len(int64_t seq_len) {
  TORCH_CHECK(seq_len <= kMaxSeqLen, "Input seq_len too long");
}

template <typename T>
inline T *get_ptr(const torch::Tensor &t) {
  return reinterpret_cast<T *>(t.data_ptr());
}
}  // namespace torch_ext
}  // namespace bytetransformer
