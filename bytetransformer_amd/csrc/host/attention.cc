// Attention<OpType>::infer - picks one of the two fused MHA kernels.
// Dispatch role of the reference's attention.h:124-139 and of the path
// selection in bert_transformer.h:132-185, reduced to what exists on gfx950:
// an LDS-resident short-sequence kernel and a streaming grouped kernel.
#include "bytetransformer/attention.h"

#include <cmath>

namespace bytetransformer {

template <OperationType OpType>
void Attention<OpType>::infer(AttentionInferParam infer_param) {
  if (infer_param.et_param.batch_idx == nullptr && !infer_param.no_offsets)
    throw std::runtime_error("[BT][ERROR] Attention: et_param.batch_idx must be set");
  if (infer_param.no_offsets &&
      (OpType != OperationType::HALF || is_remove_padding_ || size_per_head_ != 64 ||
       infer_param.mask_prefix != 0 || uses_short_kernel(infer_param.seq_len)))
    throw std::runtime_error("[BT][ERROR] Attention: no_offsets is for the streaming fp16 kernel "
                             "on padded rows with the mask tensor applied (mask_prefix == 0)");
  if (infer_param.batch_size > max_batch_size_ || infer_param.seq_len > max_seq_len_)
    throw std::runtime_error("[BT][ERROR] Attention: batch_size/seq_len exceed the constructed maximum");

  const int rows_cap = infer_param.batch_size * infer_param.seq_len;
  const float scale = 1.0f / std::sqrt((float)size_per_head_) / param_.tao;
  const int padded_rows = is_remove_padding_ ? 0 : 1;
  if constexpr (OpType == OperationType::FP32) {
    // float: one streaming kernel over token-major [rows, 3H] projections; the mask tensor
    // is applied on both row layouts, as the reference's float path does
    // (attention_nofused.cu:85-94) - unless the caller has found it to be the plain
    // prefix mask, whose terms are 0 for the keys of the sequence and vanish for the rest
    check_bt_error(bt_attention_f32(infer_param.qkv, infer_param.attention_output,
                                    infer_param.et_param.batch_idx, infer_param.seq_order,
                                    infer_param.mask_prefix == 1 ? nullptr : infer_param.atten_mask,
                                    infer_param.attention_bias,
                                    infer_param.batch_size,
                                    infer_param.seq_len, rows_cap, head_num_, size_per_head_,
                                    scale, padded_rows, infer_param.stream));
    return;
  }
  // on padded rows the mask tensor itself is applied (any 0/1 pattern), as in the
  // reference's non-remove-padding kernels; packed rows use the prefix lengths
  // (unless the caller has checked that it is the plain prefix mask: stopping at the
  // lengths then gives the same result without reading batch x seq_len^2 mask elements
  // per head)
  const void *mask = is_remove_padding_ || infer_param.mask_prefix == 1
                         ? nullptr
                         : (const void *)infer_param.atten_mask;
  if (size_per_head_ != 64) {
    // the fp16 kernels are built for 64-wide heads; other head sizes (multiples of 8 up to 128) take the
    // generic kernel over token-major projections (the reference's unfused path for them)
    check_bt_error(bt_attention_generic_f16(
        infer_param.qkv, infer_param.attention_output, infer_param.et_param.batch_idx,
        infer_param.seq_order, mask, infer_param.attention_bias, infer_param.batch_size,
        infer_param.seq_len, rows_cap, head_num_, size_per_head_, scale, padded_rows,
        infer_param.stream));
    return;
  }
  if (uses_short_kernel(infer_param.seq_len))
    check_bt_error(bt_attention_short(infer_param.qkv, infer_param.attention_output,
                                      infer_param.et_param.batch_idx, infer_param.seq_order, mask,
                                      infer_param.attention_bias, infer_param.batch_size, infer_param.seq_len, rows_cap, head_num_, size_per_head_,
                                      scale, padded_rows, infer_param.prefetch,
                                      infer_param.prefetch_bytes, infer_param.prefetch_count,
                                      infer_param.stream));
  else {
    // A mask tensor in use and no verdict from the caller: one pass over it on the device
    // (every launch of the layer, a few microseconds) lets the kernel drop it when it is the
    // plain prefix mask - the usual case, worth 3-15 us of attention per layer.
    const int *slots = mask ? infer_param.mask_prefix_slots : nullptr;
    if (mask && !slots && infer_param.mask_prefix < 0 && infer_param.buf) {
      int *verdict = (int *)infer_param.buf;
      check_bt_error(bt_mask_prefix_slots(mask, Traits_::dtype, infer_param.batch_size,
                                          infer_param.seq_len, infer_param.et_param.batch_idx,
                                          verdict, infer_param.stream));
      slots = verdict;
    }
    check_bt_error(bt_attention_grouped(
        infer_param.qkv, infer_param.attention_output,
        infer_param.no_offsets ? nullptr : infer_param.et_param.batch_idx,
        infer_param.seq_order, mask, infer_param.attention_bias, infer_param.batch_size,
        infer_param.seq_len, rows_cap, head_num_, size_per_head_, scale, padded_rows,
        infer_param.prefetch, infer_param.prefetch_bytes, infer_param.prefetch_count, slots,
        infer_param.work_list,
        infer_param.stream));
  }
}

template class Attention<OperationType::FP32>;
template class Attention<OperationType::HALF>;

}  // namespace bytetransformer
