// Attention<OpType>: parameter structs and the dispatcher between the two
// fused multi-head-attention kernels.  Public surface follows the reference's
// bytetransformer/include/attention.h:25-149 (AttentionParam,
// AttentionInferParam, Attention with ctor / initialize / cal_bufsize / infer).
#pragma once
#include "common.h"

namespace bytetransformer {

template <OperationType OpType>
class AttentionParam {
 private:
  using Traits_ = Traits<OpType>;
  using DataType_ = typename Traits_::DataType;

 public:
  const DataType_ *attr_bias_QKV = nullptr;  // [3 * hidden_dim]
  float tao = 1.0f;                          // softmax temperature: scale = 1/sqrt(d)/tao
  int cublas_Algo[2] = {Traits_::algo, Traits_::algo};  // kept for source compatibility, unused
};

template <typename T>
struct AttentionInferParam {
  // Projections with the QKV bias already added, as the QKV GEMM writes them:
  // fp16 head-major [3][head_num][batch_size * seq_len][size_per_head],
  // float token-major [batch_size * seq_len][3 * hidden_dim].
  const T *qkv;
  const T *atten_mask;  // [batch_size, seq_len, seq_len]; lengths come from et_param.batch_idx
  T *attention_output;  // token-major [rows, hidden_dim]
  void *buf;
  int batch_size = 0;
  int seq_len = 0;
  BlasHandle cublas_handle = nullptr;
  hipStream_t stream = nullptr;
  ET_Param et_param = {nullptr, nullptr, 0};
  const T *attention_bias = nullptr;         // [head_num, seq_len, seq_len], added to the scaled logits
  const uint32_t *position_ids = nullptr;    // never read
  const uint32_t *token_type_ids = nullptr;  // never read
  // Extension: sequence indices by descending length from bt_build_offsets; the
  // kernels then start the longest sequences first.  May be null.
  const int *seq_order = nullptr;
  // Extension: a device range later kernels of the stream will read (the layer's
  // remaining weights); the attention kernel warms the memory-side cache with it.
  const void *prefetch[4] = {nullptr, nullptr, nullptr, nullptr};
  unsigned long long prefetch_bytes[4] = {0, 0, 0, 0};
  int prefetch_count = 0;
  // Extension: what the caller knows about atten_mask: 1 = the plain prefix mask of
  // et_param's lengths (the padded rows then need no mask tensor: keys stop at each length,
  // the same result), 0 = something else, -1 = not checked.
  int mask_prefix = -1;
  // Extension: or the verdict slots of the device-side check (bt_mask_prefix_slots) of
  // this mask, already enqueued on the stream; else, with mask_prefix == -1, the layer runs
  // the check itself into `buf` whenever the mask tensor is in use.
  const int *mask_prefix_slots = nullptr;
  // Extension: the balanced workgroup order of the streaming kernel as a list
  // (bt_attention_worklist for this shape and these offsets), or null: the kernel then
  // looks its work up itself.
  const void *work_list = nullptr;
  // Extension: et_param's offsets have not been built (a short layer on padded rows that
  // goes without the launch that builds them): the streaming fp16 kernel then applies the
  // mask tensor to all seq_len keys and reads no offsets.  Needs padded rows and
  // mask_prefix == 0.
  bool no_offsets = false;
};

template <OperationType OpType>
class Attention {
 protected:
  typedef Traits<OpType> Traits_;
  typedef typename Traits_::DataType DataType_;
  const int max_batch_size_, max_seq_len_, head_num_, size_per_head_;
  AttentionParam<OpType> param_;

  using AttentionInferParam = struct AttentionInferParam<DataType_>;

  bool use_fused_attention_;
  const bool is_remove_padding_;
  const ModelType model_type_;

 public:
  // Sequences up to this length take the LDS-resident short kernel (whole K / V in LDS,
  // exact two-pass softmax) when use_fused_attention is set; longer ones, or
  // use_fused_attention = false, take the streaming grouped kernel.  The limit is the
  // process-wide option "attention_short_limit" of the kernel library and defaults to 0:
  // on MI355X the streaming kernel measures faster at every length and batch size (its
  // first key tile is in flight while the short kernel still waits for all of K and V).
  static int short_seq_limit() {
    int v = 0;
    return bt_get_option("attention_short_limit", &v) == BT_OK ? v : 0;
  }

  Attention(const int max_batch_size, const int head_num, const int size_per_head,
            const int max_seq_len, const bool use_fused_attention = true,
            const bool is_remove_padding = false, const ModelType model_type = ModelType::Bert)
      : max_batch_size_(max_batch_size),
        max_seq_len_(max_seq_len),
        head_num_(head_num),
        size_per_head_(size_per_head),
        use_fused_attention_(use_fused_attention),
        is_remove_padding_(is_remove_padding),
        model_type_(model_type) {}

  void initialize(AttentionParam<OpType> param) { param_ = param; }

  // Both kernels keep logits and probabilities on chip.  Scratch: 256 ints, the verdict slots
  // of the device-side prefix-mask check (padded rows), then the streaming kernel's work
  // list (16 bytes per workgroup of its largest launch).
  static unsigned long long work_list_offset() { return 256 * sizeof(int); }
  unsigned long long work_list_capacity() const {
    const unsigned long long pairs8 = ((unsigned long long)max_batch_size_ * head_num_ + 7) / 8;
    const unsigned long long slots = (pairs8 * ((max_seq_len_ + 63) / 64) + 31) / 32 * 32 * 8;
    return slots * 16;
  }
  virtual unsigned long long cal_bufsize() const {
    return work_list_offset() + work_list_capacity();
  }

  bool uses_short_kernel(int seq_len) const {
    return use_fused_attention_ && seq_len <= short_seq_limit();
  }

  virtual void infer(AttentionInferParam infer_param);

  virtual ~Attention() {}
};

}  // namespace bytetransformer
