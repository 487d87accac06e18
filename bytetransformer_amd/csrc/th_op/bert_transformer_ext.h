// BTEncoder<T>: binds twelve weight tensors to a BertTransformerParam and runs
// one layer on the caller's current HIP stream.  Role of the reference's
// bytetransformer/th_op/bert_transformer_ext.h:30-117.
#pragma once
#include "bytetransformer/bert_transformer.h"
#include "prepack_cache.h"
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
    BertTransformerParam<kOp> param = param_;
    std::vector<Tensor> packed = prepacked_weights(stream);   // keeps the copies alive
    if (packed.size() == 4)
      for (int i = 0; i < 4; ++i) param.prepacked_kernels[i] = get_ptr<T>(packed[i]);

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
    // offsets of this mask: cached per mask tensor (never while the stream is being
    // captured into a graph, where the host may not wait for the token count)
    MaskPlanCache::Plan plan;
    ET_Param offsets{nullptr, nullptr, 0};
    // (batches of one and two run on the padded rows whatever the flag says; the float
    // attention applies the mask tensor on both row layouts)
    const bool mask_tensor_in_use =
        !is_remove_padding || batch_size <= 2 || kOp == OperationType::FP32;
    if (mask_plan(attr_mask, batch_size, seq_len, stream, mask_tensor_in_use, &plan)) {
      offsets.batch_idx = plan.batch_idx.data_ptr<int>();
      offsets.word_idx = plan.word_idx.data_ptr<int>();
      offsets.valid_word_num = plan.valid_word_num;
      infer_param.offsets = &offsets;
      infer_param.seq_order = plan.seq_order.data_ptr<int>();
      infer_param.mask_prefix = plan.prefix_state;
    }
    encoder.infer(infer_param);
  }

 private:
  // The four [N, K] weight copies, from the process-wide cache when the same
  // tensors were seen before, else packed now (one launch) and remembered.
  // Empty for float, whose kernels read the weights as stored.
  std::vector<Tensor> prepacked_weights(hipStream_t stream) {
    std::vector<Tensor> out;
    if (kOp != OperationType::HALF) return out;
    auto &cache = PrepackCache::instance();
    if (!cache.enabled()) return out;
    static const int kIdx[4] = {0, 2, 6, 8};
    for (int i = 0; i < 4; ++i)
      if (weights_[kIdx[i]].dim() != 2) return out;
    out.resize(4);
    bool all_hit = true;
    for (int i = 0; i < 4; ++i) all_hit = cache.lookup(weights_[kIdx[i]], stream, &out[i]) && all_hit;
    if (all_hit) return out;
    const void *src[4];
    void *dst[4];
    int ks[4], ns[4];
    // one allocation for the four copies: the layer hands the last three to the
    // attention kernel as one range to warm the cache with
    int64_t total = 0;
    for (int i = 0; i < 4; ++i) total += weights_[kIdx[i]].numel();
    Tensor block = torch::empty({total}, weights_[kIdx[0]].options());
    int64_t at = 0;
    for (int i = 0; i < 4; ++i) {
      const Tensor &w = weights_[kIdx[i]];
      out[i] = block.narrow(0, at, w.numel()).view({w.size(1), w.size(0)});
      at += w.numel();
      src[i] = w.data_ptr();
      dst[i] = out[i].data_ptr();
      ks[i] = (int)w.size(0);
      ns[i] = (int)w.size(1);
    }
    check_bt_error(bt_transpose_weights(4, src, dst, ks, ns, stream));
    for (int i = 0; i < 4; ++i) cache.store(weights_[kIdx[i]], stream, out[i]);
    return out;
  }

  // want_prefix: the attention of this layer would read the mask tensor, so it pays to know
  // whether that is the plain prefix mask of its lengths (one pass over it, once per mask).
  bool mask_plan(const Tensor &mask, int batch_size, int seq_len, hipStream_t stream,
                 bool want_prefix, MaskPlanCache::Plan *plan) {
    if (!PrepackCache::instance().enabled() || mask.is_inference()) return false;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess ||
        capturing != hipStreamCaptureStatusNone)
      return false;
    auto &cache = MaskPlanCache::instance();
    auto opts = torch::dtype(torch::kInt32).device(mask.device());
    auto check_prefix = [&]() {
      auto scratch = torch::empty({256}, opts);
      int verdict = 0;
      check_bt_error(bt_mask_is_prefix(mask.data_ptr(), Traits<kOp>::dtype, batch_size, seq_len,
                                       plan->batch_idx.data_ptr<int>(), scratch.data_ptr<int>(),
                                       &verdict, stream));
      plan->prefix_state = verdict;
    };
    if (cache.lookup(mask, stream, plan)) {
      if (want_prefix && plan->prefix_state < 0) {
        check_prefix();
        cache.store(mask, stream, *plan);
      }
      return true;
    }
    plan->batch_idx = torch::empty({(int64_t)batch_size + 1}, opts);
    plan->word_idx = torch::empty({(int64_t)batch_size * seq_len}, opts);
    plan->seq_order = torch::empty({(int64_t)batch_size}, opts);
    check_bt_error(bt_build_offsets(mask.data_ptr(), Traits<kOp>::dtype, batch_size, seq_len,
                                    plan->batch_idx.data_ptr<int>(), plan->word_idx.data_ptr<int>(),
                                    plan->seq_order.data_ptr<int>(), &plan->valid_word_num,
                                    stream));
    if (want_prefix) check_prefix();
    cache.store(mask, stream, *plan);
    return true;
  }

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
