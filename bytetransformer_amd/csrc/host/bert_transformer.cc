// BertTransformer<OpType>::bert_infer - host orchestration of one encoder
// layer over the C ABI.  Same operation order, residual choices and buffer
// reuse as the reference's bytetransformer/src/bert_transformer.cu:28-130; what
// differs is that nothing here waits for the device: the valid-token count
// stays in batch_idx[batch_size] and every kernel bounds itself with it.
#include "bytetransformer/bert_transformer.h"


namespace bytetransformer {

template <OperationType OpType>
LayerPlan BertTransformer<OpType>::plan(int batch_size, int seq_len, bool have_offsets,
                                        int valid_rows_hint) const {
  LayerPlan lp;
  const int hidden = head_num_ * size_per_head_;
  const int inter = hidden * param_.intermediate_size;
  const long long rows = (long long)batch_size * seq_len;
  const bool streaming_fp16 = OpType == OperationType::HALF && size_per_head_ == 64 &&
                              !attention_layer_->uses_short_kernel(seq_len);
  // Short sequences on padded rows: nothing but the attention would use the offsets there,
  // and the attention can apply the mask tensor itself (all seq_len keys, masked ones
  // shifted by -10000: the same probabilities) - so the layer goes without the prologue
  // launch, which at a few dozen tokens is an eighth of its run time.
  int direct_limit = 0;
  bt_get_option("padded_mask_direct", &direct_limit);
  // (only launches that take the plain workgroup order: the balanced one ranks the
  // sequences by their lengths)
  lp.mask_direct = streaming_fp16 && !is_remove_padding_ && !have_offsets &&
                   seq_len <= direct_limit &&
                   bt_attention_worklist_bytes(batch_size, seq_len, head_num_) == 0;
  // Padding-free fp16 layers that have to build their offsets: the QKV product can count the
  // mask rows itself and leave the offsets for the kernels after it, so that the layer goes
  // without the launch ahead of it - where that launch would have no per-call weight copy
  // to make (option qkv_mask_rows: -1 that rule, 0 never, 1 always and no copies).  Copies for
  // FFN1 and FFN2 need no such launch: the first LayerNorm's can carry them (ln_weight_copy) -
  // up to 32 sequences; beyond, counting the mask rows in every workgroup of several rounds
  // costs more than the launch it saves (batch 64 x 256: +1.4 % per forward).
  int qkv_mask_rows_opt = -1;
  bt_get_option("qkv_mask_rows", &qkv_mask_rows_opt);
  const bool fits = OpType == OperationType::HALF && is_remove_padding_ && !have_offsets &&
                    qkv_mask_rows_opt != 0 &&
                    bt_gemm_qkv_mask_rows_supported(batch_size, seq_len, Traits_::dtype);
  const bool have_prepack = OpType == OperationType::HALF && param_.prepacked_kernels[0] &&
                            param_.prepacked_kernels[1] && param_.prepacked_kernels[2] &&
                            param_.prepacked_kernels[3];
  if (!have_prepack && OpType == OperationType::HALF && !lp.mask_direct) {
    const long long live = valid_rows_hint > 0  ? valid_rows_hint
                           : is_remove_padding_ ? (rows * 3LL + 4) / 5
                                                : rows;
    int ln_weight_copy = 1;
    bt_get_option("ln_weight_copy", &ln_weight_copy);
    lp.copies = plan_weight_copies(live, rows, hidden, inter, size_per_head_ == 64,
                                   !fits ? 0 : (qkv_mask_rows_opt == 1 ? 2 : 1),
                                   fits && ln_weight_copy != 0 && batch_size <= 32, lp.copy,
                                   lp.ln_copy);
  }
  lp.starts_with_qkv = fits && lp.copies == 0;
  return lp;
}

template <OperationType OpType>
void BertTransformer<OpType>::bert_infer(BertTransformerInferParam infer_param) {
  if (inner_buf_size_ == 0) cal_bufsize();

  const DataType_ *from_tensor = infer_param.input_tensor;
  const DataType_ *atten_mask = infer_param.atten_mask;
  DataType_ *transformer_out = infer_param.transformer_output;
  const int batch_size = infer_param.batch_size;
  const int seq_len = infer_param.seq_len;
  hipStream_t stream = infer_param.stream;

  if (!from_tensor || !atten_mask || !transformer_out || !infer_param.buf)
    throw std::runtime_error("[BT][ERROR] BertTransformer: null input/mask/output/buf pointer");
  if (batch_size <= 0 || seq_len <= 0 || batch_size > max_batch_size_ || seq_len > max_seq_len_)
    throw std::runtime_error(
        "[BT][ERROR] BertTransformer: batch_size/seq_len outside the constructed maximum");

  const int hidden = head_num_ * size_per_head_;
  const int inter = hidden * param_.intermediate_size;
  const int rows = batch_size * seq_len;
  // the fp16 products step through k in tiles of 64 (the float layer has no such rule)
  if (OpType == OperationType::HALF && hidden % 64 != 0)
    throw std::runtime_error("[BT][ERROR] BertTransformer: fp16 layers need head_num * "
                             "size_per_head to be a multiple of 64, got " +
                             std::to_string(hidden));
  const size_t tensor = (size_t)rows * hidden;

  // carve the scratch with the maxima, exactly as cal_bufsize() laid it out
  const unsigned long long max_rows = (unsigned long long)max_batch_size_ * max_seq_len_;
  const unsigned long long max_tensor = max_rows * hidden;
  uint8_t *base = (uint8_t *)infer_param.buf;
  DataType_ *inner_buf = (DataType_ *)base;
  DataType_ *qkv_buf = inner_buf;
  DataType_ *attr_out_buf = inner_buf + 3 * tensor;
  DataType_ *attr_matmul_buf = inner_buf + 4 * tensor;
  DataType_ *inter_matmul_buf = inner_buf + 5 * tensor;
  unsigned long long off =
      align_up((5 + param_.intermediate_size) * max_tensor * sizeof(DataType_), 256);
  ET_Param et_param;
  et_param.word_idx = (int *)(base + off);
  et_param.batch_idx = et_param.word_idx + max_rows;
  et_param.valid_word_num = rows;
  int *seq_order = et_param.batch_idx + max_batch_size_ + 1;   // int[max_batch_size]
  off += align_up((max_rows * 2 + 2 * (unsigned long long)max_batch_size_ + 2) * sizeof(int), 256);
  const bool have_offsets =
      infer_param.offsets && infer_param.offsets->batch_idx && infer_param.offsets->word_idx;
  const bool streaming_fp16 = OpType == OperationType::HALF && size_per_head_ == 64 &&
                              !attention_layer_->uses_short_kernel(seq_len);
  const LayerPlan lp = plan(batch_size, seq_len, have_offsets, infer_param.valid_rows_hint);
  const bool mask_direct = lp.mask_direct;
  const bool qkv_mask_rows = lp.starts_with_qkv;
  // The four products read the [k, n] weights as the caller stores them, exactly as the
  // reference hands them to cuBLAS (gemm.cu:27-39): nothing is kept between calls and
  // nothing can go stale.  Where the measured tile table says that a product of this size
  // runs faster on a k-contiguous copy even after paying for the copy, the layer's first
  // launch makes that copy in the scratch, afresh in every call.  A caller that owns
  // k-contiguous copies of immutable weights (prepacked_kernels) passes those instead.
  const bool have_prepack = OpType == OperationType::HALF && param_.prepacked_kernels[0] &&
                            param_.prepacked_kernels[1] && param_.prepacked_kernels[2] &&
                            param_.prepacked_kernels[3];
  const DataType_ *w_use[4] = {param_.attr_kernel_QKV, param_.attr_output_kernel,
                               param_.inter_kernel, param_.output_kernel};
  int w_kn[4] = {1, 1, 1, 1};
  const int w_k[4] = {hidden, hidden, hidden, inter};
  const int w_n[4] = {3 * hidden, hidden, inter, hidden};
  const void *pack_src[4], *ln_src[4];
  void *pack_dst[4], *ln_dst[4];
  int pack_k[4], pack_n[4], pack_count = 0, ln_k[4], ln_n[4], ln_count = 0;
  if (have_prepack) {
    for (int i = 0; i < 4; ++i) {
      w_use[i] = param_.prepacked_kernels[i];
      w_kn[i] = 0;
    }
  } else {
    // (copies made by the launch ahead of the layer, or by the first LayerNorm's launch)
    DataType_ *slot = (DataType_ *)(base + off);
    for (int i = 0; i < 4; ++i) {
      if (lp.copy[i]) {
        pack_src[pack_count] = w_use[i];
        pack_dst[pack_count] = slot;
        pack_k[pack_count] = w_k[i];
        pack_n[pack_count] = w_n[i];
        ++pack_count;
        w_use[i] = slot;
        w_kn[i] = 0;
      } else if (lp.ln_copy[i]) {
        ln_src[ln_count] = w_use[i];
        ln_dst[ln_count] = slot;
        ln_k[ln_count] = w_k[i];
        ln_n[ln_count] = w_n[i];
        ++ln_count;
        w_use[i] = slot;
        w_kn[i] = 0;
      }
      slot += (size_t)w_k[i] * w_n[i];
    }
  }
  off += align_up((4 + 2 * (unsigned long long)param_.intermediate_size) * hidden * hidden *
                      sizeof(DataType_),
                  256);
  float *splitk_buf = (float *)(base + off);

  // Padded rows, fp16 streaming attention: the mask tensor is applied unless one pass over
  // it finds the plain prefix mask of its lengths; the prologue leaves that verdict in the
  // attention's scratch and the kernel decides on the device.
  int *mask_slots = nullptr;
  if (streaming_fp16 && !is_remove_padding_ && !mask_direct &&
      !(have_offsets && infer_param.mask_prefix >= 0))
    mask_slots = (int *)(base + inner_buf_size_);

  // One launch ahead of the layer: lengths and offsets from the mask (needed on both
  // paths: keys past len_b are excluded), the prefix-mask verdict, the weight copies.
  // Rebuilt on every call, as the reference does (bert_transformer.cu:62-66), unless the
  // caller vouches for offsets of its own.
  int rows_hint = infer_param.valid_rows_hint > 0 ? infer_param.valid_rows_hint : 0;
  // ... and, for the weights that are read as stored, a first touch: the launch has
  // workgroups to spare, and a product that finds its weight in the memory-side cache
  // instead of in HBM starts sooner (what a few hundred rows spend most of their time on).
  const void *warm[4];
  unsigned long long warm_bytes[4];
  int warm_count = 0;
  // (a layer that starts with the QKV product has no launch to do this in)
  if (OpType == OperationType::HALF && !have_prepack && !qkv_mask_rows)
    for (int i = 0; i < 4; ++i)
      if (w_kn[i]) {
        warm[warm_count] = w_use[i];
        warm_bytes[warm_count++] = (unsigned long long)w_k[i] * w_n[i] * sizeof(DataType_);
      }
  if (!mask_direct && !qkv_mask_rows && (!have_offsets || mask_slots || pack_count > 0))
    check_bt_error(bt_layer_prologue(atten_mask, Traits_::dtype, batch_size, seq_len,
                                     et_param.batch_idx, et_param.word_idx, seq_order,
                                     mask_slots, nullptr, head_num_, is_remove_padding_ ? 0 : 1,
                                     pack_count, pack_src, pack_dst, pack_k, pack_n, warm_count,
                                     warm, warm_bytes, stream));
  if (have_offsets) {
    et_param = *infer_param.offsets;
    rows_hint = et_param.valid_word_num;
    seq_order = const_cast<int *>(infer_param.seq_order);
  }
  const int *valid_rows = nullptr;
  const int *gather = nullptr;
  DataType_ *restore_target = nullptr;
  // Row capacity of the launches over packed rows that follow the attention.  A caller
  // that passes offsets of its own vouches for their exact live count, so these launches
  // are then sized for it instead of batch * seq_len: no workgroups
  // that only find out on the device that their rows do not exist (1.7-2.2 us per layer
  // at batch 16 x 512), and a short sequence in a long padded row still takes the split-k
  // FFN2.  The QKV product and the attention keep batch * seq_len: it is the row stride
  // of the per-head Q/K/V layout and the extent of the gathered input.
  int packed_cap = rows;
  if (is_remove_padding_) {
    // The packed copy of the input is never materialised: the QKV GEMM and the
    // first LayerNorm read valid token t from the padded input at row word_idx[t]
    // (the compress step of bert_transformer.cu:68-78 folded into its consumers).
    gather = et_param.word_idx;
    restore_target = transformer_out;
    transformer_out = inner_buf;  // FFN2 output reuses the dead qkv region
    valid_rows = et_param.batch_idx + batch_size;
    if (have_offsets && rows_hint > 0 && rows_hint < rows) packed_cap = rows_hint;
  }

  if constexpr (OpType == OperationType::FP32) {
    // float: weights are consumed as stored, Q/K/V stay token-major [rows, 3H], gamma
    // and beta are float by definition
    check_bt_error(bt_gemm_f32(from_tensor, gather, param_.attr_kernel_QKV,
                               param_.attention_param.attr_bias_QKV, qkv_buf, 0, valid_rows, rows, rows_hint,
                               3 * hidden, hidden, stream));
    if (infer_param.valid_word_num_out && is_remove_padding_ && !have_offsets)
      check_bt_error(bt_publish_int(et_param.batch_idx + batch_size,
                                    infer_param.valid_word_num_out, stream));
    struct AttentionInferParam<DataType_> attention_infer_param {
      qkv_buf, atten_mask, attr_out_buf, base + inner_buf_size_, batch_size, seq_len,
          infer_param.cublas_handle, stream, et_param
    };
    attention_infer_param.attention_bias = infer_param.attention_bias;
    attention_infer_param.seq_order = seq_order;
    attention_infer_param.mask_prefix = have_offsets ? infer_param.mask_prefix : -1;
    attention_layer_->infer(attention_infer_param);
    check_bt_error(bt_gemm_f32(attr_out_buf, nullptr, param_.attr_output_kernel, nullptr,
                               attr_matmul_buf, 0, valid_rows, packed_cap, rows_hint, hidden, hidden,
                               stream));
    check_bt_error(bt_add_bias_residual_layernorm_f32(
        attr_matmul_buf, from_tensor, gather, param_.attr_output_bias,
        param_.attr_output_layernorm_gamma, param_.attr_output_layernorm_beta, valid_rows,
        packed_cap, hidden, layernorm_eps, stream));
    check_bt_error(bt_gemm_f32(attr_matmul_buf, nullptr, param_.inter_kernel, param_.inter_bias,
                               inter_matmul_buf, 1, valid_rows, packed_cap, rows_hint, inter, hidden,
                               stream));
    check_bt_error(bt_gemm_f32(inter_matmul_buf, nullptr, param_.output_kernel, nullptr,
                               transformer_out, 0, valid_rows, packed_cap, rows_hint, hidden, inter,
                               stream));
    if (is_remove_padding_)
      check_bt_error(bt_add_bias_residual_layernorm_restore_f32(
          transformer_out, attr_matmul_buf, param_.output_bias, param_.output_layernorm_gamma,
          param_.output_layernorm_beta, restore_target, et_param.batch_idx, batch_size, seq_len,
          hidden, layernorm_eps, stream));
    else
      check_bt_error(bt_add_bias_residual_layernorm_f32(
          transformer_out, attr_matmul_buf, nullptr, param_.output_bias,
          param_.output_layernorm_gamma, param_.output_layernorm_beta, nullptr, rows, hidden,
          layernorm_eps, stream));
    return;
  }

  const DataType_ *wt_qkv = w_use[0], *wt_proj = w_use[1], *wt_inter = w_use[2], *wt_out = w_use[3];

  if (qkv_mask_rows)
    check_bt_error(bt_gemm_qkv_bias_split_mask_rows(
        from_tensor, atten_mask, Traits_::dtype, batch_size, seq_len, wt_qkv,
        param_.attention_param.attr_bias_QKV, qkv_buf, et_param.batch_idx, et_param.word_idx,
        seq_order, rows_hint, head_num_, size_per_head_, w_kn[0], stream));
  else
    check_bt_error(bt_gemm_qkv_bias_split(from_tensor, gather, wt_qkv,
                                          param_.attention_param.attr_bias_QKV, qkv_buf,
                                          valid_rows, rows, rows_hint, head_num_, size_per_head_,
                                          w_kn[0], stream));

  // the count that this call's first launch has left in batch_idx[batch_size], for a host that
  // wants it without waiting (one more launch of one wave, only when asked for)
  if (infer_param.valid_word_num_out && is_remove_padding_ && !have_offsets)
    check_bt_error(bt_publish_int(et_param.batch_idx + batch_size, infer_param.valid_word_num_out,
                                  stream));

  struct AttentionInferParam<DataType_> attention_infer_param {
    qkv_buf, atten_mask, attr_out_buf, base + inner_buf_size_, batch_size, seq_len,
        infer_param.cublas_handle, stream, et_param
  };
  attention_infer_param.attention_bias = infer_param.attention_bias;
  attention_infer_param.seq_order = mask_direct ? nullptr : seq_order;   // (no offsets: none was written)
  // (0 = "not known to be the prefix mask": the tensor is applied)
  attention_infer_param.mask_prefix = have_offsets ? infer_param.mask_prefix : (mask_direct ? 0 : -1);
  attention_infer_param.mask_prefix_slots = mask_slots;
  // (no work list: building one per layer costs its launch more than the attention saves; the
  // kernel finds its balanced order by a look-up of its own)
  attention_infer_param.work_list = nullptr;
  attention_infer_param.no_offsets = mask_direct;   // (nothing has written them)
  // the weight matrices the rest of the layer reads (as stored, or the copies that the first
  // launch has made): the attention kernel pulls them into the memory-side cache while it
  // runs.  A matrix that the first LayerNorm's launch copies is left alone: the copy reads
  // its source once either way, and the product reads the copy (same box, with / without
  // touching it: batch 16 x 512 1.519 / 1.514 ms, 16 x 1024 2.586 / 2.574, BERT-large 6.610 / 6.589).
  {
    const size_t elems[3] = {(size_t)hidden * hidden, (size_t)hidden * inter, (size_t)hidden * inter};
    int pc = 0;
    for (int i = 0; i < 3; ++i) {
      if (lp.ln_copy[i + 1]) continue;
      attention_infer_param.prefetch[pc] = w_use[i + 1];
      attention_infer_param.prefetch_bytes[pc] = elems[i] * sizeof(DataType_);
      ++pc;
    }
    attention_infer_param.prefetch_count = pc;
  }
  attention_layer_->infer(attention_infer_param);

  check_bt_error(
      bt_gemm(attr_out_buf, wt_proj, attr_matmul_buf, valid_rows, packed_cap, rows_hint, hidden,
              hidden, w_kn[1], stream));

  if (ln_count > 0)
    check_bt_error(bt_add_bias_residual_layernorm_copy(
        attr_matmul_buf, from_tensor, gather, param_.attr_output_bias,
        param_.attr_output_layernorm_gamma, param_.attr_output_layernorm_beta, use_fp32_ ? 1 : 0,
        valid_rows, packed_cap, hidden, layernorm_eps, ln_count, ln_src, ln_dst, ln_k, ln_n, stream));
  else
    check_bt_error(bt_add_bias_residual_layernorm(
        attr_matmul_buf, from_tensor, gather, param_.attr_output_bias,
        param_.attr_output_layernorm_gamma, param_.attr_output_layernorm_beta, use_fp32_ ? 1 : 0,
        valid_rows, packed_cap, hidden, layernorm_eps, stream));

  check_bt_error(bt_gemm_bias_gelu(attr_matmul_buf, wt_inter, param_.inter_bias, inter_matmul_buf,
                                   valid_rows, packed_cap, rows_hint, inter, hidden, w_kn[2],
                                   stream));

  // few rows, long k: FFN2 as split-k partial sums that the last LayerNorm folds in
  const long long rows_expected =
      !valid_rows ? rows : (rows_hint > 0 ? rows_hint : (rows * 3LL + 4) / 5);
  const int splits = splitk_splits(packed_cap, rows_expected, inter);
  if (splits > 1) {
    check_bt_error(bt_gemm_splitk(inter_matmul_buf, wt_out, splitk_buf, splits, valid_rows,
                                  packed_cap, hidden, inter, w_kn[3], stream));
    check_bt_error(bt_splitk_layernorm(
        splitk_buf, splits, attr_matmul_buf, nullptr, param_.output_bias,
        param_.output_layernorm_gamma, param_.output_layernorm_beta, use_fp32_ ? 1 : 0,
        is_remove_padding_ ? restore_target : transformer_out,
        is_remove_padding_ ? et_param.batch_idx : nullptr, nullptr, batch_size, seq_len,
        packed_cap, hidden, layernorm_eps, stream));
    return;
  }

  check_bt_error(
      bt_gemm(inter_matmul_buf, wt_out, transformer_out, valid_rows, packed_cap, rows_hint, hidden,
              inter, w_kn[3], stream));

  if (is_remove_padding_)
    check_bt_error(bt_add_bias_residual_layernorm_restore(
        transformer_out, attr_matmul_buf, param_.output_bias, param_.output_layernorm_gamma,
        param_.output_layernorm_beta, use_fp32_ ? 1 : 0, restore_target, et_param.batch_idx,
        // the row map is this call's own word_idx (complete by construction); a caller's
        // offsets keep the look-up through batch_idx
        have_offsets ? nullptr : et_param.word_idx, batch_size, seq_len, hidden, layernorm_eps,
        stream));
  else
    check_bt_error(bt_add_bias_residual_layernorm(
        transformer_out, attr_matmul_buf, nullptr, param_.output_bias, param_.output_layernorm_gamma,
        param_.output_layernorm_beta, use_fp32_ ? 1 : 0, nullptr, rows, hidden, layernorm_eps,
        stream));
}

template class BertTransformer<OperationType::FP32>;
template class BertTransformer<OperationType::HALF>;

}  // namespace bytetransformer
