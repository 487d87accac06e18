// torch.ops.ByteTransformer.BertTransformer - the functional PyTorch operator,
// rebuilt against PyTorch-ROCm.  Schema, argument order, defaults and error
// messages follow the reference's bytetransformer/th_op/ths_op_f.cc:28-95.
#include <torch/library.h>
#include <torch/script.h>

#include "bert_transformer_ext.h"

namespace bytetransformer {
namespace torch_ths {

using torch::Tensor;

namespace {

// One encoder layer on the caller's current stream: the twelve weights, the padded
// hidden states [batch, seq, hidden] and the mask [batch, seq, seq] in, a fresh
// tensor of the input's shape out.
Tensor bert_transformer_layer(int64_t head_num, int64_t head_size, Tensor qkv_kernel,
                              Tensor qkv_bias, Tensor attr_output_kernel, Tensor attr_output_bias,
                              Tensor attr_output_layernorm_gamma,
                              Tensor attr_output_layernorm_beta, Tensor inter_kernel,
                              Tensor inter_bias, Tensor output_kernel, Tensor output_bias,
                              Tensor output_layernorm_gamma, Tensor output_layernorm_beta,
                              Tensor input, Tensor attr_mask, bool is_remove_padding,
                              bool use_fused_attention) {
  const std::vector<Tensor> weights{
      qkv_kernel,   qkv_bias,   attr_output_kernel, attr_output_bias, attr_output_layernorm_gamma,
      attr_output_layernorm_beta, inter_kernel,     inter_bias,       output_kernel,
      output_bias,  output_layernorm_gamma,         output_layernorm_beta};
  torch_ext::check_weights(weights);
  const at::ScalarType st = qkv_kernel.scalar_type();
  torch_ext::check_tensor(input, "input", st, false);
  torch_ext::check_tensor(attr_mask, "attr_mask", st, false);

  TORCH_CHECK(input.dim() == 3, "input must be [batch_size, seq_len, hidden_dim]");
  const int64_t batch = input.size(0), seq = input.size(1);
  TORCH_CHECK(input.size(2) == head_num * head_size, "input hidden_dim != head_num * head_size");
  TORCH_CHECK(attr_mask.dim() == 3 && attr_mask.size(0) == batch && attr_mask.size(1) == seq &&
                  attr_mask.size(2) == seq,
              "attr_mask must be [batch_size, seq_len, seq_len]");

  auto layer = torch_ext::make_encoder(head_num, head_size, weights);
  torch_ext::check_layer_shapes(head_num, head_size, weights);
  Tensor output = torch::empty_like(input);
  if (batch > 0 && seq > 0)
    layer->forward((int)batch, (int)seq, input, attr_mask, output, is_remove_padding,
                   use_fused_attention);
  return output;
}

// The operator's cache (valid-token counts of mask tensors, a hint for tile shapes): dropped /
// switched on and off.  It never changes a result, so these are for timing experiments.
void clear_caches() { torch_ext::MaskHintCache::instance().clear(); }

void set_caches_enabled(bool enabled) {
  torch_ext::caches_enabled().store(enabled);
  if (!enabled) clear_caches();
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(ByteTransformer, m) {
  m.def("clear_caches() -> ()", &clear_caches);
  m.def("set_caches_enabled(bool enabled) -> ()", &set_caches_enabled);
  m.def(
      "BertTransformer(int head_num, int head_size, Tensor qkv_kernel, Tensor qkv_bias, "
      "Tensor attr_output_kernel, Tensor attr_output_bias, Tensor attr_output_layernorm_gamma, "
      "Tensor attr_output_layernorm_beta, Tensor inter_kernel, Tensor inter_bias, "
      "Tensor output_kernel, Tensor output_bias, Tensor output_layernorm_gamma, "
      "Tensor output_layernorm_beta, Tensor input, Tensor attr_mask, "
      "bool is_remove_padding=True, bool use_fused_attention=True) -> Tensor",
      &bert_transformer_layer);
}

}  // namespace torch_ths
}  // namespace bytetransformer
