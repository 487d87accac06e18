// torch.classes.ByteTransformer.BertTransformer - the TorchScript custom class:
// twelve weights bound at construction, forward(input, mask) /
// forwardv2(input, mask, is_remove_padding, use_fused_attention), pickled as the
// twelve tensors plus an int64[2] {head_num, head_size}.  Interface of the
// reference's bytetransformer/th_op/ths_op.{h,cc} (ths_op.h:29-110, ths_op.cc:27-43).
#include <torch/custom_class.h>
#include <torch/script.h>

#include <memory>

#include "bert_transformer_ext.h"

namespace bytetransformer {
namespace torch_ths {
using torch::Tensor;

class BertTransformer : public torch::jit::CustomClassHolder {
 public:
  BertTransformer(int64_t head_num, int64_t head_size, Tensor qkv_kernel, Tensor qkv_bias,
                  Tensor attr_output_kernel, Tensor attr_output_bias,
                  Tensor attr_output_layernorm_gamma, Tensor attr_output_layernorm_beta,
                  Tensor inter_kernel, Tensor inter_bias, Tensor output_kernel, Tensor output_bias,
                  Tensor output_layernorm_gamma, Tensor output_layernorm_beta)
      : st_(qkv_kernel.scalar_type()),
        weights_{qkv_kernel,     qkv_bias,    attr_output_kernel,
                 attr_output_bias, attr_output_layernorm_gamma, attr_output_layernorm_beta,
                 inter_kernel,   inter_bias,  output_kernel,
                 output_bias,    output_layernorm_gamma,      output_layernorm_beta} {
    torch_ext::check_weights(weights_);
    encoder_ = torch_ext::make_encoder(head_num, head_size, weights_);
    torch_ext::check_layer_shapes(head_num, head_size, weights_);
    head_info_ = torch::empty({2}, torch::dtype(torch::kInt64));
    head_info_[0] = head_num;
    head_info_[1] = head_size;
    hidden_ = head_num * head_size;
  }

  Tensor forward(Tensor input, Tensor attr_mask) { return forwardv2(input, attr_mask, true, true); }

  Tensor forwardv2(Tensor input, Tensor attr_mask, bool is_remove_padding,
                   bool use_fused_attention) {
    torch_ext::check_tensor(input, "input", st_, false);
    torch_ext::check_tensor(attr_mask, "attr_mask", st_, false);
    TORCH_CHECK(input.dim() == 3 && input.size(2) == hidden_,
                "input must be [batch_size, seq_len, head_num * head_size]");
    const int batch_size = (int)input.size(0), seq_len = (int)input.size(1);
    TORCH_CHECK(attr_mask.dim() == 3 && attr_mask.size(0) == batch_size &&
                    attr_mask.size(1) == seq_len && attr_mask.size(2) == seq_len,
                "attr_mask must be [batch_size, seq_len, seq_len]");
    auto output = torch::empty_like(input);
    if (batch_size == 0 || seq_len == 0) return output;
    encoder_->forward(batch_size, seq_len, input, attr_mask, output, is_remove_padding,
                      use_fused_attention);
    return output;
  }

  std::vector<Tensor> get_pickle_info() const {
    std::vector<Tensor> state(weights_);
    state.push_back(head_info_);
    return state;
  }

 private:
  const at::ScalarType st_;
  std::unique_ptr<torch_ext::IBTEncoder> encoder_;
  Tensor head_info_;
  int64_t hidden_ = 0;
  std::vector<Tensor> weights_;
};

static auto bertTransformerEncoderTHS =
    torch::jit::class_<BertTransformer>("ByteTransformer", "BertTransformer")
        .def(torch::jit::init<int64_t, int64_t, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor,
                              Tensor, Tensor, Tensor, Tensor, Tensor, Tensor>())
        .def("forward", &BertTransformer::forward)
        .def("forwardv2", &BertTransformer::forwardv2)
        .def_pickle(
            [](const c10::intrusive_ptr<BertTransformer> &self) -> std::vector<Tensor> {
              return self->get_pickle_info();
            },
            [](std::vector<Tensor> state) -> c10::intrusive_ptr<BertTransformer> {
              TORCH_CHECK(state.size() == 13, "expected 12 weight tensors and head_info");
              const int64_t head_num = state[12][0].item().to<int64_t>();
              const int64_t head_size = state[12][1].item().to<int64_t>();
              return c10::make_intrusive<BertTransformer>(
                  head_num, head_size, state[0], state[1], state[2], state[3], state[4], state[5],
                  state[6], state[7], state[8], state[9], state[10], state[11]);
            });

}  // namespace torch_ths
}  // namespace bytetransformer
