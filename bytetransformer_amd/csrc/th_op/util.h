// Argument checks shared by the PyTorch operator and the TorchScript class.
// Same messages as the reference's bytetransformer/th_op/util.h:30-40 so that
// callers matching on them keep working ("CUDA tensor" is PyTorch-ROCm's own
// name for a GPU tensor).
#pragma once
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/all.h>

#include <vector>

#define CHECK_TYPE(x, st) TORCH_CHECK(x.scalar_type() == st, "Inconsistency of Tensor type: " #x)
#define CHECK_CUDA(x) TORCH_CHECK(x.is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x, st) \
  CHECK_CUDA(x);           \
  CHECK_CONTIGUOUS(x);     \
  CHECK_TYPE(x, st)
#define CHECK_INPUT_LOOSE(x) \
  CHECK_CUDA(x);             \
  CHECK_CONTIGUOUS(x)
#define CHECK_SEQ_LEN(x) TORCH_CHECK(x <= 1024, "Input seq_len too long")

namespace bytetransformer {
namespace torch_ext {
template <typename T>
inline T *get_ptr(const torch::Tensor &t) {
  return reinterpret_cast<T *>(t.data_ptr());
}
}  // namespace torch_ext
}  // namespace bytetransformer
