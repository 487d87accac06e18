// BertTransformer<OpType>: one post-LN BERT encoder layer, padded [B,S,H] in,
// padded [B,S,H] out, optionally running on the packed (padding-free) rows in
// between.  Public surface follows the reference's
// bytetransformer/include/bert_transformer.h:30-224: BertTransformerParam,
// BertTransformerInferParam (same field order, so positional aggregate
// initialisation keeps working), and BertTransformer with
// ctor / initialize / cal_bufsize / infer.
#pragma once
#include "attention.h"
#include "common.h"

namespace bytetransformer {

template <OperationType OpType>
class BertTransformerParam {
 private:
  typedef Traits<OpType> Traits_;
  typedef typename Traits_::DataType DataType_;

 public:
  AttentionParam<OpType> attention_param;

  const DataType_ *attr_kernel_QKV = nullptr;  // [H, 3H]

  const DataType_ *attr_output_kernel = nullptr;  // [H, H]
  const DataType_ *attr_output_bias = nullptr;
  const void *attr_output_layernorm_gamma = nullptr;  // DataType_ or float (use_fp32)
  const void *attr_output_layernorm_beta = nullptr;

  const DataType_ *inter_kernel = nullptr;  // [H, intermediate_size * H]
  const DataType_ *inter_bias = nullptr;

  const DataType_ *output_kernel = nullptr;  // [intermediate_size * H, H]
  const DataType_ *output_bias = nullptr;
  const void *output_layernorm_gamma = nullptr;
  const void *output_layernorm_beta = nullptr;

  int intermediate_size = 4;

  int cublas_Algo[3] = {Traits_::algo, Traits_::algo, Traits_::algo};  // unused, kept for callers

  // Extension (no counterpart in the reference): k-contiguous copies of the four weight
  // matrices as bt_transpose_weights makes them, in the order QKV [3H,H], attention
  // output [H,H], FFN1 [F,H], FFN2 [H,F], for a caller that owns copies of immutable
  // weights and vouches that they match the *_kernel tensors above.  Left null, infer()
  // reads the *_kernel tensors as they are stored, in every call.
  const DataType_ *prepacked_kernels[4] = {nullptr, nullptr, nullptr, nullptr};
};

template <typename T>
struct BertTransformerInferParam {
  const T *input_tensor;  // [batch_size, seq_len, hidden_dim]
  const T *atten_mask;    // [batch_size, seq_len, seq_len], 1 = attend, 0 = padding
  T *transformer_output;  // [batch_size, seq_len, hidden_dim]; may alias input_tensor
  void *buf;              // >= cal_bufsize() bytes of device memory, 256-byte aligned
  int batch_size;
  int seq_len;
  BlasHandle cublas_handle;  // ignored
  hipStream_t stream;
  const T *attention_bias = NULL;         // [head_num, seq_len, seq_len], added to the scaled logits
  const uint32_t *position_ids = NULL;    // never read
  const uint32_t *token_type_ids = NULL;  // never read
  // Extension (no counterpart in the reference): offsets already built from this
  // very atten_mask by bt_build_offsets (batch_idx int[batch_size+1], word_idx
  // int[batch_size*seq_len], valid_word_num = their total).  When set, infer()
  // skips its own mask prefix sum.  valid_word_num must be the exact total (as the
  // reference's ET_Param carries it) or 0 when the host does not know it: a positive
  // value sizes the launches over packed rows and picks their tile shapes.
  const ET_Param *offsets = NULL;
  // ... and the matching sequence order (int[batch_size], longest first), or NULL.
  const int *seq_order = NULL;
  // ... and the caller's finding (bt_mask_is_prefix) about atten_mask: 1 = it is exactly the
  // prefix mask of those offsets - on the padded rows the attention then stops at each
  // length instead of reading the tensor, the same result, the masked terms being exactly
  // zero; 0 = it is not; -1 = not checked (the layer then checks on the device).
  int mask_prefix = -1;
  // Extension: the number of valid tokens the caller expects (0 = unknown) when it passes
  // no offsets.  A hint: it picks tile shapes and the split-k FFN2, never a launch size, so
  // a wrong value costs time and nothing else.
  int valid_rows_hint = 0;
  // Extension: where the layer leaves the number of valid tokens it counted (padding-free
  // layers that build their own offsets), or NULL.  Memory the device can write and the host
  // can read (hipHostMalloc): written by a one-wave launch behind the layer's first launch,
  // so a host that polls it learns the count without waiting for the stream - and can pass
  // it as valid_rows_hint from then on.
  int *valid_word_num_out = NULL;
};

// What one call of a layer will launch ahead of and around its QKV product (decided on the
// host from sizes, options and the measured tile table; never changes a result).
struct LayerPlan {
  bool mask_direct = false;      // padded rows, short sequences: no offsets at all
  bool starts_with_qkv = false;  // the QKV product counts the mask rows itself: no launch ahead of it
  bool copy[4] = {false, false, false, false};   // QKV, projection, FFN1, FFN2 run on a per-call copy
  int copies = 0;                                // ... made by the launch ahead of the layer
  bool ln_copy[4] = {false, false, false, false};   // FFN1, FFN2: ... made by the first LayerNorm's launch
};

template <OperationType OpType>
class BertTransformer {
 private:
  typedef Traits<OpType> Traits_;
  typedef typename Traits_::DataType DataType_;

  BertTransformerParam<OpType> param_;
  using BertTransformerInferParam = struct BertTransformerInferParam<DataType_>;

  Attention<OpType> *attention_layer_ = nullptr;

  const int max_batch_size_, max_seq_len_, head_num_, size_per_head_;

  unsigned long long inner_buf_size_ = 0;

  bool use_fused_attention_;
  bool is_remove_padding_;
  const bool use_fp32_;  // gamma & beta datatype
  const ModelType model_type_;

  static unsigned long long align_up(unsigned long long v, unsigned long long a) {
    return (v + a - 1) / a * a;
  }

 public:
  // LayerNorm epsilon of the reference kernels (layernorm.h:35,58,103,133).
  float layernorm_eps = 1e-6f;

  BertTransformer(const int max_batch_size, const int head_num, const int size_per_head,
                  const int max_seq_len, const bool use_fused_attention = true,
                  const bool is_remove_padding = true, const bool use_fp32 = false,
                  const ModelType model_type = ModelType::Bert)
      : max_batch_size_(max_batch_size),
        max_seq_len_(max_seq_len),
        head_num_(head_num),
        size_per_head_(size_per_head),
        use_fused_attention_(use_fused_attention),
        is_remove_padding_(is_remove_padding),
        use_fp32_(use_fp32),
        model_type_(model_type) {
    // Same side rule as the reference (bert_transformer.h:135-136): tiny batches
    // run on the padded rows.
    if (max_batch_size_ <= 2) is_remove_padding_ = false;
    attention_layer_ =
        new Attention<OpType>(max_batch_size, head_num, size_per_head, max_seq_len,
                              use_fused_attention_, is_remove_padding_, model_type_);
  }

  BertTransformer(const BertTransformer &) = delete;
  BertTransformer &operator=(const BertTransformer &) = delete;

  void initialize(BertTransformerParam<OpType> param) {
    param_ = param;
    attention_layer_->initialize(param_.attention_param);
  }

  bool is_remove_padding() const { return is_remove_padding_; }

  // Scratch layout (elements of DataType_, T = max_batch*max_seq*hidden):
  //   [0,3T) qkv heads | [3T,4T) attention out | [4T,5T) projection / LN1 |
  //   [5T,(5+mult)T) FFN1 | word_idx int[B*S] | batch_idx int[B+1] | seq order int[B] |
  //   pre-packed weights (3+1+2*mult)*H*H | split-k partial sums | attention scratch (256 ints)
  unsigned long long cal_bufsize() {
    const unsigned long long rows = (unsigned long long)max_batch_size_ * max_seq_len_;
    const unsigned long long hidden = (unsigned long long)head_num_ * size_per_head_;
    const unsigned long long tensor = rows * hidden;
    inner_buf_size_ = (5 + param_.intermediate_size) * tensor * sizeof(DataType_);
    inner_buf_size_ = align_up(inner_buf_size_, 256);
    inner_buf_size_ += align_up((rows * 2 + 2 * max_batch_size_ + 2) * sizeof(int), 256);
    inner_buf_size_ += align_up(
        (4 + 2 * (unsigned long long)param_.intermediate_size) * hidden * hidden *
            sizeof(DataType_),
        256);
    inner_buf_size_ += align_up(splitk_scratch_bytes(rows, hidden), 256);
    return inner_buf_size_ + attention_layer_->cal_bufsize();
  }

  void infer(BertTransformerInferParam infer_param) { bert_infer(infer_param); }

  // The plan of a call with these sizes (have_offsets: the caller passes offsets of its own).
  LayerPlan plan(int batch_size, int seq_len, bool have_offsets, int valid_rows_hint) const;

  void bert_infer(BertTransformerInferParam infer_param);

  ~BertTransformer() { delete attention_layer_; }
};

}  // namespace bytetransformer
