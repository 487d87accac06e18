// C entry points over BertTransformer<OpType> for FFI callers.
#include "bt_encoder.h"

#include <memory>
#include <string>
#include <vector>

#include "bytetransformer/bert_encoder.h"
#include "bytetransformer/bert_transformer.h"

namespace {
thread_local std::string g_error;

using bytetransformer::BertTransformer;
using bytetransformer::BertTransformerInferParam;
using bytetransformer::BertTransformerParam;
using bytetransformer::OperationType;

int validate(const bt_encoder_config *cfg) {
  if (!cfg) {
    g_error = "[BT][ERROR] null config";
    return BT_ERR_INVALID_ARGUMENT;
  }
  if (cfg->dtype != BT_F16) {
    g_error = "[BT][ERROR] only BT_F16 is implemented";
    return BT_ERR_UNSUPPORTED;
  }
  if (cfg->max_batch_size <= 0 || cfg->max_seq_len <= 0 || cfg->head_num <= 0 ||
      cfg->size_per_head <= 0 || cfg->intermediate_size <= 0) {
    g_error = "[BT][ERROR] non-positive size in config";
    return BT_ERR_INVALID_ARGUMENT;
  }
  return BT_OK;
}

BertTransformerParam<OperationType::HALF> make_param(const bt_encoder_config *cfg,
                                                     const bt_layer_weights *w) {
  BertTransformerParam<OperationType::HALF> p;
  p.attr_kernel_QKV = (const __half *)w->qkv_kernel;
  p.attention_param.attr_bias_QKV = (const __half *)w->qkv_bias;
  p.attention_param.tao = cfg->tao > 0.f ? cfg->tao : 1.0f;
  p.attr_output_kernel = (const __half *)w->attr_output_kernel;
  p.attr_output_bias = (const __half *)w->attr_output_bias;
  p.attr_output_layernorm_gamma = w->attr_output_layernorm_gamma;
  p.attr_output_layernorm_beta = w->attr_output_layernorm_beta;
  p.inter_kernel = (const __half *)w->inter_kernel;
  p.inter_bias = (const __half *)w->inter_bias;
  p.output_kernel = (const __half *)w->output_kernel;
  p.output_bias = (const __half *)w->output_bias;
  p.output_layernorm_gamma = w->output_layernorm_gamma;
  p.output_layernorm_beta = w->output_layernorm_beta;
  p.intermediate_size = cfg->intermediate_size;
  return p;
}
}  // namespace

extern "C" unsigned long long bt_encoder_bufsize(const bt_encoder_config *cfg) {
  if (validate(cfg) != BT_OK) return 0;
  BertTransformer<OperationType::HALF> enc(cfg->max_batch_size, cfg->head_num, cfg->size_per_head,
                                           cfg->max_seq_len, cfg->use_fused_attention != 0,
                                           cfg->is_remove_padding != 0, cfg->gamma_beta_fp32 != 0);
  BertTransformerParam<OperationType::HALF> p;
  p.intermediate_size = cfg->intermediate_size;
  enc.initialize(p);
  return enc.cal_bufsize();
}

extern "C" int bt_encoder_layer_forward(const bt_encoder_config *cfg,
                                        const bt_layer_weights *weights, const void *input,
                                        const void *atten_mask, void *output, void *buf,
                                        int batch_size, int seq_len, void *stream) {
  return bt_encoder_layer_forward_bias(cfg, weights, input, atten_mask, nullptr, output, buf,
                                       batch_size, seq_len, stream);
}

extern "C" int bt_encoder_layer_forward_bias(const bt_encoder_config *cfg,
                                             const bt_layer_weights *weights, const void *input,
                                             const void *atten_mask, const void *attention_bias,
                                             void *output, void *buf, int batch_size,
                                             int seq_len, void *stream) {
  int rc = validate(cfg);
  if (rc != BT_OK) return rc;
  if (!weights) {
    g_error = "[BT][ERROR] null weights";
    return BT_ERR_INVALID_ARGUMENT;
  }
  const void *const *wp = (const void *const *)weights;
  for (int i = 0; i < 12; ++i)
    if (!wp[i]) {
      g_error = "[BT][ERROR] null weight pointer #" + std::to_string(i);
      return BT_ERR_INVALID_ARGUMENT;
    }
  try {
    BertTransformer<OperationType::HALF> enc(
        cfg->max_batch_size, cfg->head_num, cfg->size_per_head, cfg->max_seq_len,
        cfg->use_fused_attention != 0, cfg->is_remove_padding != 0, cfg->gamma_beta_fp32 != 0);
    if (cfg->layernorm_eps > 0.f) enc.layernorm_eps = cfg->layernorm_eps;
    enc.initialize(make_param(cfg, weights));
    enc.cal_bufsize();
    BertTransformerInferParam<__half> ip{(const __half *)input,
                                         (const __half *)atten_mask,
                                         (__half *)output,
                                         buf,
                                         batch_size,
                                         seq_len,
                                         nullptr,
                                         (hipStream_t)stream};
    ip.attention_bias = (const __half *)attention_bias;
    enc.infer(ip);
  } catch (const std::exception &e) {
    g_error = e.what();
    return BT_ERR_INVALID_ARGUMENT;
  }
  return BT_OK;
}

// ---- whole encoder -----------------------------------------------------------
namespace {
using bytetransformer::BertEncoder;
using bytetransformer::BertEncoderInferParam;

int make_encoder(const bt_encoder_config *cfg, int num_layers, const bt_layer_weights *weights,
                 std::unique_ptr<BertEncoder<OperationType::HALF>> *out) {
  int rc = validate(cfg);
  if (rc != BT_OK) return rc;
  if (num_layers <= 0) {
    g_error = "[BT][ERROR] num_layers must be positive";
    return BT_ERR_INVALID_ARGUMENT;
  }
  out->reset(new BertEncoder<OperationType::HALF>(
      cfg->max_batch_size, cfg->head_num, cfg->size_per_head, cfg->max_seq_len,
      cfg->use_fused_attention != 0, cfg->is_remove_padding != 0, cfg->gamma_beta_fp32 != 0));
  if (cfg->layernorm_eps > 0.f) (*out)->layernorm_eps = cfg->layernorm_eps;
  std::vector<BertTransformerParam<OperationType::HALF>> layers((size_t)num_layers);
  for (int l = 0; l < num_layers; ++l) {
    if (weights) {
      const void *const *wp = (const void *const *)(weights + l);
      for (int i = 0; i < 12; ++i)
        if (!wp[i]) {
          g_error = "[BT][ERROR] null weight pointer #" + std::to_string(i) + " of layer " +
                    std::to_string(l);
          return BT_ERR_INVALID_ARGUMENT;
        }
      layers[(size_t)l] = make_param(cfg, weights + l);
    } else {
      layers[(size_t)l].intermediate_size = cfg->intermediate_size;
    }
  }
  (*out)->initialize(layers);
  return BT_OK;
}
}  // namespace

extern "C" unsigned long long bt_encoder_forward_bufsize(const bt_encoder_config *cfg) {
  std::unique_ptr<BertEncoder<OperationType::HALF>> enc;
  if (make_encoder(cfg, 1, nullptr, &enc) != BT_OK) return 0;
  return enc->cal_bufsize();
}

extern "C" unsigned long long bt_encoder_prepack_bytes(const bt_encoder_config *cfg,
                                                       int num_layers) {
  std::unique_ptr<BertEncoder<OperationType::HALF>> enc;
  if (make_encoder(cfg, num_layers, nullptr, &enc) != BT_OK) return 0;
  return enc->prepack_bytes();
}

extern "C" int bt_encoder_prepack(const bt_encoder_config *cfg, int num_layers,
                                  const bt_layer_weights *weights, void *prepacked,
                                  void *stream) {
  if (!weights) {
    g_error = "[BT][ERROR] null weights";
    return BT_ERR_INVALID_ARGUMENT;
  }
  std::unique_ptr<BertEncoder<OperationType::HALF>> enc;
  int rc = make_encoder(cfg, num_layers, weights, &enc);
  if (rc != BT_OK) return rc;
  try {
    enc->prepack(prepacked, (hipStream_t)stream);
  } catch (const std::exception &e) {
    g_error = e.what();
    return BT_ERR_INVALID_ARGUMENT;
  }
  return BT_OK;
}

extern "C" int bt_encoder_forward(const bt_encoder_config *cfg, int num_layers,
                                  const bt_layer_weights *weights, const void *prepacked,
                                  const void *input, const void *atten_mask,
                                  const void *attention_bias, void *output, void *buf,
                                  int batch_size, int seq_len, int valid_rows_hint,
                                  void *stream) {
  if (!weights) {
    g_error = "[BT][ERROR] null weights";
    return BT_ERR_INVALID_ARGUMENT;
  }
  std::unique_ptr<BertEncoder<OperationType::HALF>> enc;
  int rc = make_encoder(cfg, num_layers, weights, &enc);
  if (rc != BT_OK) return rc;
  try {
    BertEncoderInferParam<__half> ip{(const __half *)input, (const __half *)atten_mask,
                                     (__half *)output,      buf,
                                     batch_size,            seq_len,
                                     (hipStream_t)stream};
    ip.attention_bias = (const __half *)attention_bias;
    ip.prepacked = prepacked;
    ip.valid_rows_hint = valid_rows_hint;
    enc->infer(ip);
  } catch (const std::exception &e) {
    g_error = e.what();
    return BT_ERR_INVALID_ARGUMENT;
  }
  return BT_OK;
}

extern "C" const char *bt_encoder_last_error(void) { return g_error.c_str(); }
