// C entry points over BertTransformer<OpType> for FFI callers.
#include "bt_encoder.h"

#include <memory>
#include <string>
#include <vector>

#include "bytetransformer/bert_encoder.h"
#include "bytetransformer/bert_transformer.h"
#include "host_error.h"

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
  if (cfg->dtype != BT_F16 && cfg->dtype != BT_F32) {
    g_error = "[BT][ERROR] dtype must be BT_F16 or BT_F32";
    return BT_ERR_UNSUPPORTED;
  }
  if (cfg->max_batch_size <= 0 || cfg->max_seq_len <= 0 || cfg->head_num <= 0 ||
      cfg->size_per_head <= 0 || cfg->intermediate_size <= 0) {
    g_error = "[BT][ERROR] non-positive size in config";
    return BT_ERR_INVALID_ARGUMENT;
  }
  return BT_OK;
}

template <OperationType Op>
BertTransformerParam<Op> make_param(const bt_encoder_config *cfg, const bt_layer_weights *w) {
  using T = typename bytetransformer::Traits<Op>::DataType;
  BertTransformerParam<Op> p;
  p.attr_kernel_QKV = (const T *)w->qkv_kernel;
  p.attention_param.attr_bias_QKV = (const T *)w->qkv_bias;
  p.attention_param.tao = cfg->tao > 0.f ? cfg->tao : 1.0f;
  p.attr_output_kernel = (const T *)w->attr_output_kernel;
  p.attr_output_bias = (const T *)w->attr_output_bias;
  p.attr_output_layernorm_gamma = w->attr_output_layernorm_gamma;
  p.attr_output_layernorm_beta = w->attr_output_layernorm_beta;
  p.inter_kernel = (const T *)w->inter_kernel;
  p.inter_bias = (const T *)w->inter_bias;
  p.output_kernel = (const T *)w->output_kernel;
  p.output_bias = (const T *)w->output_bias;
  p.output_layernorm_gamma = w->output_layernorm_gamma;
  p.output_layernorm_beta = w->output_layernorm_beta;
  p.intermediate_size = cfg->intermediate_size;
  return p;
}

template <OperationType Op>
unsigned long long layer_bufsize(const bt_encoder_config *cfg) {
  BertTransformer<Op> enc(cfg->max_batch_size, cfg->head_num, cfg->size_per_head,
                          cfg->max_seq_len, cfg->use_fused_attention != 0,
                          cfg->is_remove_padding != 0, cfg->gamma_beta_fp32 != 0);
  BertTransformerParam<Op> p;
  p.intermediate_size = cfg->intermediate_size;
  enc.initialize(p);
  return enc.cal_bufsize();
}

template <OperationType Op>
void layer_forward(const bt_encoder_config *cfg, const bt_layer_weights *weights,
                   const void *input, const void *atten_mask, const void *attention_bias,
                   void *output, void *buf, int batch_size, int seq_len, void *stream) {
  using T = typename bytetransformer::Traits<Op>::DataType;
  BertTransformer<Op> enc(cfg->max_batch_size, cfg->head_num, cfg->size_per_head,
                          cfg->max_seq_len, cfg->use_fused_attention != 0,
                          cfg->is_remove_padding != 0, cfg->gamma_beta_fp32 != 0);
  if (cfg->layernorm_eps > 0.f) enc.layernorm_eps = cfg->layernorm_eps;
  enc.initialize(make_param<Op>(cfg, weights));
  enc.cal_bufsize();
  BertTransformerInferParam<T> ip{(const T *)input, (const T *)atten_mask, (T *)output, buf,
                                  batch_size,       seq_len,               nullptr,
                                  (hipStream_t)stream};
  ip.attention_bias = (const T *)attention_bias;
  enc.infer(ip);
}
}  // namespace

namespace {
template <OperationType Op>
void layer_plan(const bt_encoder_config *cfg, int batch_size, int seq_len, int rows_hint,
                int *plan) {
  BertTransformer<Op> enc(cfg->max_batch_size, cfg->head_num, cfg->size_per_head,
                          cfg->max_seq_len, cfg->use_fused_attention != 0,
                          cfg->is_remove_padding != 0, cfg->gamma_beta_fp32 != 0);
  BertTransformerParam<Op> p;
  p.intermediate_size = cfg->intermediate_size;
  enc.initialize(p);
  const bytetransformer::LayerPlan lp = enc.plan(batch_size, seq_len, false, rows_hint);
  for (int i = 0; i < 4; ++i) plan[i] = lp.copy[i] ? 1 : (lp.ln_copy[i] ? 2 : 0);
  plan[4] = lp.starts_with_qkv;
  plan[5] = lp.mask_direct;
}
}  // namespace

extern "C" int bt_encoder_layer_plan(const bt_encoder_config *cfg, int batch_size, int seq_len,
                                     int rows_hint, int *plan) {
  int rc = validate(cfg);
  if (rc != BT_OK) return rc;
  if (!plan || batch_size <= 0 || seq_len <= 0) {
    g_error = "[BT][ERROR] bt_encoder_layer_plan: null plan or non-positive size";
    return BT_ERR_INVALID_ARGUMENT;
  }
  if (cfg->dtype == BT_F32)
    layer_plan<OperationType::FP32>(cfg, batch_size, seq_len, rows_hint, plan);
  else
    layer_plan<OperationType::HALF>(cfg, batch_size, seq_len, rows_hint, plan);
  return BT_OK;
}

extern "C" unsigned long long bt_encoder_bufsize(const bt_encoder_config *cfg) {
  if (validate(cfg) != BT_OK) return 0;
  return cfg->dtype == BT_F32 ? layer_bufsize<OperationType::FP32>(cfg)
                              : layer_bufsize<OperationType::HALF>(cfg);
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
    if (cfg->dtype == BT_F32)
      layer_forward<OperationType::FP32>(cfg, weights, input, atten_mask, attention_bias, output,
                                         buf, batch_size, seq_len, stream);
    else
      layer_forward<OperationType::HALF>(cfg, weights, input, atten_mask, attention_bias, output,
                                         buf, batch_size, seq_len, stream);
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

template <OperationType Op>
int make_encoder(const bt_encoder_config *cfg, int num_layers, const bt_layer_weights *weights,
                 std::unique_ptr<BertEncoder<Op>> *out) {
  int rc = validate(cfg);
  if (rc != BT_OK) return rc;
  if (num_layers <= 0) {
    g_error = "[BT][ERROR] num_layers must be positive";
    return BT_ERR_INVALID_ARGUMENT;
  }
  out->reset(new BertEncoder<Op>(cfg->max_batch_size, cfg->head_num, cfg->size_per_head,
                                 cfg->max_seq_len, cfg->use_fused_attention != 0,
                                 cfg->is_remove_padding != 0, cfg->gamma_beta_fp32 != 0));
  if (cfg->layernorm_eps > 0.f) (*out)->layernorm_eps = cfg->layernorm_eps;
  std::vector<BertTransformerParam<Op>> layers((size_t)num_layers);
  for (int l = 0; l < num_layers; ++l) {
    if (weights) {
      const void *const *wp = (const void *const *)(weights + l);
      for (int i = 0; i < 12; ++i)
        if (!wp[i]) {
          g_error = "[BT][ERROR] null weight pointer #" + std::to_string(i) + " of layer " +
                    std::to_string(l);
          return BT_ERR_INVALID_ARGUMENT;
        }
      layers[(size_t)l] = make_param<Op>(cfg, weights + l);
    } else {
      layers[(size_t)l].intermediate_size = cfg->intermediate_size;
    }
  }
  (*out)->initialize(layers);
  return BT_OK;
}

template <OperationType Op>
unsigned long long encoder_sizes(const bt_encoder_config *cfg, int num_layers, bool prepack) {
  std::unique_ptr<BertEncoder<Op>> enc;
  if (make_encoder<Op>(cfg, num_layers, nullptr, &enc) != BT_OK) return 0;
  return prepack ? enc->prepack_bytes() : enc->cal_bufsize();
}

template <OperationType Op>
int encoder_prepack(const bt_encoder_config *cfg, int num_layers, const bt_layer_weights *weights,
                    void *prepacked, void *stream) {
  std::unique_ptr<BertEncoder<Op>> enc;
  int rc = make_encoder<Op>(cfg, num_layers, weights, &enc);
  if (rc != BT_OK) return rc;
  enc->prepack(prepacked, (hipStream_t)stream);
  return BT_OK;
}

template <OperationType Op>
int encoder_forward(const bt_encoder_config *cfg, int num_layers, const bt_layer_weights *weights,
                    const void *prepacked, const void *input, const void *atten_mask,
                    const void *attention_bias, void *output, void *buf, int batch_size,
                    int seq_len, int valid_rows_hint, void *stream) {
  using T = typename bytetransformer::Traits<Op>::DataType;
  std::unique_ptr<BertEncoder<Op>> enc;
  int rc = make_encoder<Op>(cfg, num_layers, weights, &enc);
  if (rc != BT_OK) return rc;
  BertEncoderInferParam<T> ip{(const T *)input, (const T *)atten_mask, (T *)output, buf,
                              batch_size,       seq_len,               (hipStream_t)stream};
  ip.attention_bias = (const T *)attention_bias;
  ip.prepacked = prepacked;
  ip.valid_rows_hint = valid_rows_hint;
  enc->infer(ip);
  return BT_OK;
}

bool is_f32(const bt_encoder_config *cfg) { return cfg && cfg->dtype == BT_F32; }
}  // namespace

extern "C" unsigned long long bt_encoder_forward_bufsize(const bt_encoder_config *cfg) {
  return is_f32(cfg) ? encoder_sizes<OperationType::FP32>(cfg, 1, false)
                     : encoder_sizes<OperationType::HALF>(cfg, 1, false);
}

extern "C" unsigned long long bt_encoder_prepack_bytes(const bt_encoder_config *cfg,
                                                       int num_layers) {
  return is_f32(cfg) ? encoder_sizes<OperationType::FP32>(cfg, num_layers, true)
                     : encoder_sizes<OperationType::HALF>(cfg, num_layers, true);
}

extern "C" int bt_encoder_prepack(const bt_encoder_config *cfg, int num_layers,
                                  const bt_layer_weights *weights, void *prepacked,
                                  void *stream) {
  if (!weights) {
    g_error = "[BT][ERROR] null weights";
    return BT_ERR_INVALID_ARGUMENT;
  }
  try {
    return is_f32(cfg)
               ? encoder_prepack<OperationType::FP32>(cfg, num_layers, weights, prepacked, stream)
               : encoder_prepack<OperationType::HALF>(cfg, num_layers, weights, prepacked, stream);
  } catch (const std::exception &e) {
    g_error = e.what();
    return BT_ERR_INVALID_ARGUMENT;
  }
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
  try {
    return is_f32(cfg)
               ? encoder_forward<OperationType::FP32>(cfg, num_layers, weights, prepacked, input,
                                                      atten_mask, attention_bias, output, buf,
                                                      batch_size, seq_len, valid_rows_hint, stream)
               : encoder_forward<OperationType::HALF>(cfg, num_layers, weights, prepacked, input,
                                                      atten_mask, attention_bias, output, buf,
                                                      batch_size, seq_len, valid_rows_hint, stream);
  } catch (const std::exception &e) {
    g_error = e.what();
    return BT_ERR_INVALID_ARGUMENT;
  }
}

namespace bt_host {
void set_error(const std::string &message) { g_error = message; }
}  // namespace bt_host

extern "C" const char *bt_encoder_last_error(void) { return g_error.c_str(); }
