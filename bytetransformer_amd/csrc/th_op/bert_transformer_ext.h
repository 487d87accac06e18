// BTEncoder<T>: binds twelve weight tensors to a BertTransformerParam and runs
// one layer on the caller's current HIP stream.  Role of the reference's
// bytetransformer/th_op/bert_transformer_ext.h:30-117.
#pragma once
#include "bytetransformer/bert_transformer.h"
#include "mask_hint_cache.h"
#include "util.h"

#include <hip/hip_runtime_api.h>

#include <memory>

namespace bytetransformer {
namespace torch_ext {
using torch::Tensor;

template <typename T>
struct THTraits;
template <>
struct THTraits<float> {
  static const OperationType OpType = OperationType::FP32;
};
template <>
struct THTraits<__half> {
  static const OperationType OpType = OperationType::HALF;
};

class IBTEncoder {
 public:
  virtual ~IBTEncoder() {}
  virtual void forward(int batch_size, int seq_len, Tensor &input, Tensor &attr_mask,
                       Tensor &output, bool is_remove_padding, bool use_fused_attention,
                       const ModelType model_type = ModelType::Bert,
                       const Tensor attention_bias = Tensor()) = 0;
};

template <typename T>
class BTEncoder : public IBTEncoder {
  static const OperationType kOp = THTraits<T>::OpType;

 public:
  BTEncoder(int head_num, int head_size, const std::vector<Tensor> &w)
      : head_num_(head_num), head_size_(head_size), weights_(w) {
    TORCH_CHECK(w.size() == 12, "expected 12 weight tensors");
    param_.attr_kernel_QKV = get_ptr<T>(weights_[0]);
    param_.attention_param.attr_bias_QKV = get_ptr<T>(weights_[1]);
    param_.attr_output_kernel = get_ptr<T>(weights_[2]);
    param_.attr_output_bias = get_ptr<T>(weights_[3]);
    param_.attr_output_layernorm_gamma = get_ptr<void>(weights_[4]);
    param_.attr_output_layernorm_beta = get_ptr<void>(weights_[5]);
    param_.inter_kernel = get_ptr<T>(weights_[6]);
    param_.inter_bias = get_ptr<T>(weights_[7]);
    param_.output_kernel = get_ptr<T>(weights_[8]);
    param_.output_bias = get_ptr<T>(weights_[9]);
    param_.output_layernorm_gamma = get_ptr<void>(weights_[10]);
    param_.output_layernorm_beta = get_ptr<void>(weights_[11]);
    // fp32 gamma/beta next to fp16 weights, detected from the last LayerNorm
    // gamma like the reference does (bert_transformer_ext.h:60-63)
    use_fp32_ = kOp == OperationType::HALF && weights_[10].scalar_type() == at::ScalarType::Float;
    // FFN width from the weight itself (the reference leaves it at 4)
    const int64_t hidden = (int64_t)head_num * head_size;
    if (weights_[6].dim() == 2 && hidden > 0 && weights_[6].size(1) % hidden == 0)
      param_.intermediate_size = (int)(weights_[6].size(1) / hidden);
  }

  void forward(int batch_size, int seq_len, Tensor &input, Tensor &attr_mask, Tensor &output,
               bool is_remove_padding = true, bool use_fused_attention = true,
               const ModelType model_type = ModelType::Bert,
               const Tensor attention_bias = Tensor()) override {
    check_seq_len(seq_len);
    if (attention_bias.defined()) {
      check_tensor(attention_bias, "attention_bias", input.scalar_type(), false);
      TORCH_CHECK(attention_bias.dim() == 3 && attention_bias.size(0) == head_num_ &&
                      attention_bias.size(1) == seq_len && attention_bias.size(2) == seq_len,
                  "attention_bias must be [head_num, seq_len, seq_len]");
    }
    c10::DeviceGuard device_guard(input.device());

    hipStream_t stream = c10::hip::getCurrentHIPStream(input.device().index()).stream();
    // While the stream is being captured into a graph the host may not wait for a count:
    // the layer then goes without the row-count hint.
    hipStreamCaptureStatus capture_status = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(stream, &capture_status) != hipSuccess ||
                           capture_status != hipStreamCaptureStatusNone;
    const BertTransformerParam<kOp> &param = param_;

    BertTransformer<kOp> encoder(batch_size, head_num_, head_size_, seq_len, use_fused_attention,
                                 is_remove_padding, use_fp32_, model_type);
    encoder.initialize(param);
    const unsigned long long buf_size = encoder.cal_bufsize();
    auto buf_tensor = torch::empty({(int64_t)buf_size},
                                   torch::dtype(torch::kInt8).device(input.device()));
    struct BertTransformerInferParam<T> infer_param {
      get_ptr<T>(input), get_ptr<T>(attr_mask), get_ptr<T>(output), get_ptr<void>(buf_tensor),
          batch_size, seq_len, nullptr, stream
    };
    infer_param.attention_bias = attention_bias.defined() ? get_ptr<T>(attention_bias) : NULL;
    // The layer reads the weights as they are and rebuilds the offsets from the mask on the
    // device, in every call; all the host keeps between calls is the valid-token count per
    // mask tensor, as a hint for tile shapes (the packed rows only: on the padded rows
    // every row is live).  It never waits for that count: the first call that meets a mask
    // asks the layer to publish it into pinned memory, later calls use it once it is there.
    if (!capturing && encoder.is_remove_padding()) {
      // (what is published is the count of THIS device: the slot is per mask and stream)
      int count = 0;
      infer_param.valid_word_num_out =
          MaskHintCache::instance().lookup_or_reserve(attr_mask, stream, &count);
      infer_param.valid_rows_hint = count;
    }
    encoder.infer(infer_param);
  }

 private:
  const int head_num_, head_size_;
  bool use_fp32_ = false;
  std::vector<Tensor> weights_;
  BertTransformerParam<kOp> param_;
};

// Names of the twelve per-layer tensors in operator-argument order; gamma / beta
// (positions 4, 5, 10, 11) may be float next to fp16 weights.
static const char *const kWeightNames[12] = {
    "qkv_kernel",     "qkv_bias",    "attr_output_kernel",
    "attr_output_bias", "attr_output_layernorm_gamma", "attr_output_layernorm_beta",
    "inter_kernel",   "inter_bias",  "output_kernel",
    "output_bias",    "output_layernorm_gamma",      "output_layernorm_beta"};

inline bool is_affine_slot(int i) { return i == 4 || i == 5 || i == 10 || i == 11; }

inline void check_weights(const std::vector<Tensor> &w) {
  TORCH_CHECK(w.size() == 12, "expected 12 weight tensors");
  const at::ScalarType st = w[0].scalar_type();
  for (int i = 0; i < 12; ++i) check_tensor(w[i], kWeightNames[i], st, is_affine_slot(i));
}

// The encoder for the weights' dtype; anything but float / half is refused with the
// reference's text (ths_op_f.cc:62-64).
inline std::unique_ptr<IBTEncoder> make_encoder(int64_t head_num, int64_t head_size,
                                                const std::vector<Tensor> &w) {
  switch (w[0].scalar_type()) {
    case at::ScalarType::Float:
      return std::unique_ptr<IBTEncoder>(new BTEncoder<float>((int)head_num, (int)head_size, w));
    case at::ScalarType::Half:
      return std::unique_ptr<IBTEncoder>(new BTEncoder<__half>((int)head_num, (int)head_size, w));
    default:
      throw std::runtime_error("Wrong Tensor type.");
  }
}

inline void check_layer_shapes(int64_t head_num, int64_t head_size, const std::vector<Tensor> &w) {
  const int64_t H = head_num * head_size;
  TORCH_CHECK(head_num > 0 && head_size > 0, "head_num and head_size must be positive");
  TORCH_CHECK(w[0].scalar_type() != at::ScalarType::Half || H % 64 == 0,
              "fp16 layers need head_num * head_size to be a multiple of 64, got ", H,
              " (float tensors have no such rule)");
  TORCH_CHECK(w[0].dim() == 2 && w[0].size(0) == H && w[0].size(1) == 3 * H,
              "qkv_kernel must be [hidden_dim, 3 * hidden_dim]");
  TORCH_CHECK(w[1].numel() == 3 * H, "qkv_bias must have 3 * hidden_dim elements");
  TORCH_CHECK(w[2].dim() == 2 && w[2].size(0) == H && w[2].size(1) == H,
              "attr_output_kernel must be [hidden_dim, hidden_dim]");
  TORCH_CHECK(w[6].dim() == 2 && w[6].size(0) == H && w[6].size(1) % H == 0,
              "inter_kernel must be [hidden_dim, k * hidden_dim]");
  const int64_t F = w[6].size(1);
  TORCH_CHECK(w[7].numel() == F, "inter_bias must match inter_kernel");
  TORCH_CHECK(w[8].dim() == 2 && w[8].size(0) == F && w[8].size(1) == H,
              "output_kernel must be [k * hidden_dim, hidden_dim]");
  for (int i : {3, 4, 5, 9, 10, 11})
    TORCH_CHECK(w[i].numel() == H, "bias / gamma / beta tensors must have hidden_dim elements");
  TORCH_CHECK(w[4].scalar_type() == w[5].scalar_type() &&
                  w[4].scalar_type() == w[10].scalar_type() &&
                  w[4].scalar_type() == w[11].scalar_type(),
              "LayerNorm gamma / beta must share one dtype");
}
}  // namespace torch_ext
}  // namespace bytetransformer
