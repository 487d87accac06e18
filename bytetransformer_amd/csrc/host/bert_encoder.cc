// BertEncoder<OpType>::infer - a stack of encoder layers over the C ABI with the
// hidden state kept packed between layers.  Per layer the operation order and
// residual choices are those of one reference layer (bert_transformer.cu:28-130);
// the compress / restore pair of every inner layer is dropped.
#include "bytetransformer/bert_encoder.h"

namespace bytetransformer {

template <OperationType OpType>
void BertEncoder<OpType>::prepack(void *prepacked, hipStream_t stream) const {
  if (OpType == OperationType::FP32) return;   // float weights are consumed as stored
  if (!prepacked) throw std::runtime_error("[BT][ERROR] BertEncoder::prepack: null destination");
  const int hidden = head_num_ * size_per_head_, inter = hidden * intermediate_size_;
  DataType_ *dst = (DataType_ *)prepacked;
  for (const auto &l : layers_) {
    DataType_ *wt_qkv = dst, *wt_proj = wt_qkv + (size_t)3 * hidden * hidden;
    DataType_ *wt_inter = wt_proj + (size_t)hidden * hidden, *wt_out = wt_inter + (size_t)hidden * inter;
    const void *src[4] = {l.attr_kernel_QKV, l.attr_output_kernel, l.inter_kernel, l.output_kernel};
    void *out[4] = {wt_qkv, wt_proj, wt_inter, wt_out};
    const int ks[4] = {hidden, hidden, hidden, inter};
    const int ns[4] = {3 * hidden, hidden, inter, hidden};
    check_bt_error(bt_transpose_weights(4, src, out, ks, ns, stream));
    dst += layer_weight_elems();
  }
}

template <OperationType OpType>
void BertEncoder<OpType>::infer(BertEncoderInferParam<DataType_> ip) {
  if (layers_.empty()) throw std::runtime_error("[BT][ERROR] BertEncoder: initialize() first");
  if (!ip.input_tensor || !ip.atten_mask || !ip.transformer_output || !ip.buf)
    throw std::runtime_error("[BT][ERROR] BertEncoder: null input/mask/output/buf pointer");
  const int batch_size = ip.batch_size, seq_len = ip.seq_len;
  if (batch_size <= 0 || seq_len <= 0 || batch_size > max_batch_size_ || seq_len > max_seq_len_)
    throw std::runtime_error(
        "[BT][ERROR] BertEncoder: batch_size/seq_len outside the constructed maximum");
  hipStream_t stream = ip.stream;

  const int hidden = head_num_ * size_per_head_, inter = hidden * intermediate_size_;
  const int rows = batch_size * seq_len;
  if (OpType == OperationType::HALF && hidden % 64 != 0)
    throw std::runtime_error("[BT][ERROR] BertEncoder: fp16 layers need head_num * size_per_head "
                             "to be a multiple of 64, got " + std::to_string(hidden));
  const size_t tensor = (size_t)rows * hidden;
  const unsigned long long max_rows = (unsigned long long)max_batch_size_ * max_seq_len_;
  const unsigned long long max_tensor = max_rows * hidden;

  uint8_t *base = (uint8_t *)ip.buf;
  DataType_ *qkv_buf = (DataType_ *)base;
  DataType_ *attr_out_buf = qkv_buf + 3 * tensor;
  DataType_ *attr_matmul_buf = qkv_buf + 4 * tensor;   // projection, then LN1 in place
  DataType_ *hidden_buf = qkv_buf + 5 * tensor;        // FFN2 out, then LN2 in place = next input
  DataType_ *inter_matmul_buf = qkv_buf + 6 * tensor;
  unsigned long long off = align_up((6 + intermediate_size_) * max_tensor * sizeof(DataType_), 256);
  ET_Param et_param;
  et_param.word_idx = (int *)(base + off);
  et_param.batch_idx = et_param.word_idx + max_rows;
  et_param.valid_word_num = rows;
  int *seq_order = et_param.batch_idx + max_batch_size_ + 1;
  int *mask_slots = seq_order + max_batch_size_;       // int[256], padded path only
  off += align_up((max_rows * 2 + 2 * (unsigned long long)max_batch_size_ + 2 + 256) * sizeof(int),
                  256);
  float *splitk_buf = (float *)(base + off);
  off += align_up(splitk_scratch_bytes(max_rows, (unsigned long long)hidden), 256);
  // the streaming attention's balanced work list: built once per forward beside the offsets
  void *work_list = nullptr;
  if (OpType == OperationType::HALF && size_per_head_ == 64 &&
      !attention_layer_->uses_short_kernel(seq_len) &&
      bt_attention_worklist_bytes(batch_size, seq_len, head_num_) > 0)
    work_list = base + off;

  // padded rows: the fp16 streaming attention applies the mask tensor unless one pass
  // over it (once for all layers) finds the plain prefix mask of the lengths
  const bool check_mask = !is_remove_padding_ && OpType == OperationType::HALF &&
                          size_per_head_ == 64;
  // offsets and that verdict in one launch, once per forward
  check_bt_error(bt_layer_prologue(ip.atten_mask, Traits_::dtype, batch_size, seq_len,
                                   et_param.batch_idx, et_param.word_idx, seq_order,
                                   check_mask ? mask_slots : nullptr, work_list, head_num_,
                                   is_remove_padding_ ? 0 : 1, 0, nullptr, nullptr, nullptr,
                                   nullptr, 0, nullptr, nullptr, stream));
  const int *valid_rows = is_remove_padding_ ? et_param.batch_idx + batch_size : nullptr;
  const int rows_hint = ip.valid_rows_hint;
  const int L = (int)layers_.size();

  for (int l = 0; l < L; ++l) {
    const auto &w = layers_[l];
    // layer 0 reads the caller's padded input (valid token t at row word_idx[t] when
    // packing), every later layer the packed hidden state
    const DataType_ *x = l == 0 ? ip.input_tensor : hidden_buf;
    const int *gather = (l == 0 && is_remove_padding_) ? et_param.word_idx : nullptr;

    const bool last = l == L - 1;
    // the last layer of the padded path writes straight into the caller's output
    DataType_ *ffn2_out = (last && !is_remove_padding_) ? ip.transformer_output : hidden_buf;
    attention_layer_->initialize(w.attention_param);

    if constexpr (OpType == OperationType::FP32) {
      check_bt_error(bt_gemm_f32(x, gather, w.attr_kernel_QKV, w.attention_param.attr_bias_QKV,
                                 qkv_buf, 0, valid_rows, rows, rows_hint, 3 * hidden, hidden, stream));
      struct AttentionInferParam<DataType_> att {
        qkv_buf, ip.atten_mask, attr_out_buf, nullptr, batch_size, seq_len, nullptr, stream,
            et_param
      };
      att.attention_bias = ip.attention_bias;
      att.seq_order = seq_order;
      attention_layer_->infer(att);
      check_bt_error(bt_gemm_f32(attr_out_buf, nullptr, w.attr_output_kernel, nullptr,
                                 attr_matmul_buf, 0, valid_rows, rows, rows_hint, hidden, hidden, stream));
      check_bt_error(bt_add_bias_residual_layernorm_f32(
          attr_matmul_buf, x, gather, w.attr_output_bias, w.attr_output_layernorm_gamma,
          w.attr_output_layernorm_beta, valid_rows, rows, hidden, layernorm_eps, stream));
      check_bt_error(bt_gemm_f32(attr_matmul_buf, nullptr, w.inter_kernel, w.inter_bias,
                                 inter_matmul_buf, 1, valid_rows, rows, rows_hint, inter, hidden, stream));
      check_bt_error(bt_gemm_f32(inter_matmul_buf, nullptr, w.output_kernel, nullptr, ffn2_out, 0,
                                 valid_rows, rows, rows_hint, hidden, inter, stream));
      if (last && is_remove_padding_)
        check_bt_error(bt_add_bias_residual_layernorm_restore_f32(
            ffn2_out, attr_matmul_buf, w.output_bias, w.output_layernorm_gamma,
            w.output_layernorm_beta, ip.transformer_output, et_param.batch_idx, batch_size,
            seq_len, hidden, layernorm_eps, stream));
      else
        check_bt_error(bt_add_bias_residual_layernorm_f32(
            ffn2_out, attr_matmul_buf, nullptr, w.output_bias, w.output_layernorm_gamma,
            w.output_layernorm_beta, valid_rows, rows, hidden, layernorm_eps, stream));
      continue;
    }

    // pre-packed copies made when the encoder was created (its weights are private and
    // immutable), else the [k, n] weights as they are stored
    const int weight_kn = ip.prepacked ? 0 : 1;
    const DataType_ *wt_qkv = w.attr_kernel_QKV, *wt_proj = w.attr_output_kernel,
                    *wt_inter = w.inter_kernel, *wt_out = w.output_kernel;
    if (ip.prepacked) {
      wt_qkv = (const DataType_ *)ip.prepacked + (size_t)l * layer_weight_elems();
      wt_proj = wt_qkv + (size_t)3 * hidden * hidden;
      wt_inter = wt_proj + (size_t)hidden * hidden;
      wt_out = wt_inter + (size_t)hidden * inter;
    }

    check_bt_error(bt_gemm_qkv_bias_split(x, gather, wt_qkv, w.attention_param.attr_bias_QKV,
                                          qkv_buf, valid_rows, rows, rows_hint, head_num_,
                                          size_per_head_, weight_kn, stream));

    struct AttentionInferParam<DataType_> att {
      qkv_buf, ip.atten_mask, attr_out_buf, nullptr, batch_size, seq_len, nullptr, stream, et_param
    };
    att.attention_bias = ip.attention_bias;
    att.seq_order = seq_order;
    if (check_mask) att.mask_prefix_slots = mask_slots;
    att.work_list = work_list;
    // warm the memory-side cache with what follows in memory order: the rest of this
    // layer's weights and, when all layers are pre-packed back to back, the next
    // layer's QKV matrix
    if (ip.prepacked) {
      att.prefetch[0] = wt_proj;
      att.prefetch_bytes[0] = ((size_t)hidden * hidden + 2 * (size_t)hidden * inter) * sizeof(DataType_);
      if (l + 1 < L) att.prefetch_bytes[0] += (size_t)3 * hidden * hidden * sizeof(DataType_);
      att.prefetch_count = 1;
    } else {
      const void *next[3] = {wt_proj, wt_inter, wt_out};
      const size_t elems[3] = {(size_t)hidden * hidden, (size_t)hidden * inter, (size_t)hidden * inter};
      for (int i = 0; i < 3; ++i) {
        att.prefetch[i] = next[i];
        att.prefetch_bytes[i] = elems[i] * sizeof(DataType_);
      }
      att.prefetch_count = 3;
      if (l + 1 < L) {
        att.prefetch[3] = layers_[l + 1].attr_kernel_QKV;
        att.prefetch_bytes[3] = (size_t)3 * hidden * hidden * sizeof(DataType_);
        att.prefetch_count = 4;
      }
    }
    attention_layer_->infer(att);

    check_bt_error(bt_gemm(attr_out_buf, wt_proj, attr_matmul_buf, valid_rows, rows, rows_hint,
                           hidden, hidden, weight_kn, stream));
    check_bt_error(bt_add_bias_residual_layernorm(
        attr_matmul_buf, x, gather, w.attr_output_bias, w.attr_output_layernorm_gamma,
        w.attr_output_layernorm_beta, use_fp32_ ? 1 : 0, valid_rows, rows, hidden, layernorm_eps,
        stream));
    check_bt_error(bt_gemm_bias_gelu(attr_matmul_buf, wt_inter, w.inter_bias, inter_matmul_buf,
                                     valid_rows, rows, rows_hint, inter, hidden, weight_kn,
                                     stream));

    // few rows, long k: FFN2 as split-k partial sums that the last LayerNorm folds in
    const long long rows_expected =
        !valid_rows ? rows : (rows_hint > 0 ? rows_hint : (rows * 3LL + 4) / 5);
    const int splits = splitk_splits(rows, rows_expected, inter);
    if (splits > 1) {
      const bool restore = last && is_remove_padding_;
      check_bt_error(bt_gemm_splitk(inter_matmul_buf, wt_out, splitk_buf, splits, valid_rows, rows,
                                    hidden, inter, weight_kn, stream));
      check_bt_error(bt_splitk_layernorm(
          splitk_buf, splits, attr_matmul_buf, nullptr, w.output_bias, w.output_layernorm_gamma,
          w.output_layernorm_beta, use_fp32_ ? 1 : 0,
          restore ? (void *)ip.transformer_output : (void *)ffn2_out,
          restore ? et_param.batch_idx : nullptr, restore ? nullptr : valid_rows, batch_size,
          seq_len, rows, hidden, layernorm_eps, stream));
      continue;
    }
    check_bt_error(bt_gemm(inter_matmul_buf, wt_out, ffn2_out, valid_rows, rows, rows_hint, hidden,
                           inter, weight_kn, stream));
    if (last && is_remove_padding_)
      check_bt_error(bt_add_bias_residual_layernorm_restore(
          ffn2_out, attr_matmul_buf, w.output_bias, w.output_layernorm_gamma,
          w.output_layernorm_beta, use_fp32_ ? 1 : 0, ip.transformer_output, et_param.batch_idx,
          et_param.word_idx, batch_size, seq_len, hidden, layernorm_eps, stream));
    else
      check_bt_error(bt_add_bias_residual_layernorm(
          ffn2_out, attr_matmul_buf, nullptr, w.output_bias, w.output_layernorm_gamma,
          w.output_layernorm_beta, use_fp32_ ? 1 : 0, valid_rows, rows, hidden, layernorm_eps,
          stream));
  }
}

template class BertEncoder<OperationType::FP32>;
template class BertEncoder<OperationType::HALF>;

}  // namespace bytetransformer
