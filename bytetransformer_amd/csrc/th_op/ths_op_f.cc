// torch.ops.ByteTransformer.BertTransformer - the functional PyTorch operator,
// rebuilt against PyTorch-ROCm.  Schema, argument order, defaults and error
// messages follow the reference's bytetransformer/th_op/ths_op_f.cc:28-95.
#include <torch/script.h>

#include "bert_transformer_ext.h"

namespace bytetransformer {
namespace torch_ths {

using torch::Tensor;

Tensor TransformerEncoder(int64_t head_num, int64_t head_size, Tensor qkv_kernel, Tensor qkv_bias,
                          Tensor attr_output_kernel, Tensor attr_output_bias,
                          Tensor attr_output_layernorm_gamma, Tensor attr_output_layernorm_beta,
                          Tensor inter_kernel, Tensor inter_bias, Tensor output_kernel,
                          Tensor output_bias, Tensor output_layernorm_gamma,
                          Tensor output_layernorm_beta, Tensor input, Tensor attr_mask,
                          bool is_remove_padding, bool use_fused_attention) {
  const at::ScalarType _st = qkv_kernel.scalar_type();
  CHECK_INPUT(qkv_kernel, _st);
  CHECK_INPUT(qkv_bias, _st);
  CHECK_INPUT(attr_output_kernel, _st);
  CHECK_INPUT(attr_output_bias, _st);
  CHECK_INPUT_LOOSE(attr_output_layernorm_gamma);
  CHECK_INPUT_LOOSE(attr_output_layernorm_beta);
  CHECK_INPUT(inter_kernel, _st);
  CHECK_INPUT(inter_bias, _st);
  CHECK_INPUT(output_kernel, _st);
  CHECK_INPUT(output_bias, _st);
  CHECK_INPUT_LOOSE(output_layernorm_gamma);
  CHECK_INPUT_LOOSE(output_layernorm_beta);
  CHECK_INPUT(input, _st);
  CHECK_INPUT(attr_mask, _st);
  TORCH_CHECK(input.dim() == 3, "input must be [batch_size, seq_len, hidden_dim]");
  const int batch_size = (int)input.size(0);
  const int seq_len = (int)input.size(1);
  TORCH_CHECK(input.size(2) == head_num * head_size, "input hidden_dim != head_num * head_size");
  TORCH_CHECK(attr_mask.dim() == 3 && attr_mask.size(0) == batch_size &&
                  attr_mask.size(1) == seq_len && attr_mask.size(2) == seq_len,
              "attr_mask must be [batch_size, seq_len, seq_len]");
  std::vector<Tensor> weights{qkv_kernel,
                              qkv_bias,
                              attr_output_kernel,
                              attr_output_bias,
                              attr_output_layernorm_gamma,
                              attr_output_layernorm_beta,
                              inter_kernel,
                              inter_bias,
                              output_kernel,
                              output_bias,
                              output_layernorm_gamma,
                              output_layernorm_beta};
  std::unique_ptr<torch_ext::IBTEncoder> btencoder;
  switch (_st) {
    case at::ScalarType::Float:
      btencoder.reset(new torch_ext::BTEncoder<float>(head_num, head_size, weights));
      break;
    case at::ScalarType::Half:
      btencoder.reset(new torch_ext::BTEncoder<__half>(head_num, head_size, weights));
      break;
    default:
      throw std::runtime_error("Wrong Tensor type.");
  }
  torch_ext::check_layer_shapes(head_num, head_size, weights);
  auto output = torch::empty_like(input);
  if (batch_size == 0 || seq_len == 0) return output;
  btencoder->forward(batch_size, seq_len, input, attr_mask, output, is_remove_padding,
                     use_fused_attention);
  return output;
}

static auto registry = torch::RegisterOperators(
    "ByteTransformer::BertTransformer("
    "int head_num, int head_size,"
    "Tensor qkv_kernel, Tensor qkv_bias,"
    "Tensor attr_output_kernel, Tensor attr_output_bias,"
    "Tensor attr_output_layernorm_gamma, Tensor attr_output_layernorm_beta,"
    "Tensor inter_kernel, Tensor inter_bias, Tensor output_kernel, Tensor output_bias,"
    "Tensor output_layernorm_gamma, Tensor output_layernorm_beta, Tensor input, Tensor attr_mask,"
    "bool is_remove_padding = True, bool use_fused_attention = True) -> "
    "Tensor",
    &TransformerEncoder);

}  // namespace torch_ths
}  // namespace bytetransformer
