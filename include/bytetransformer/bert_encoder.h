// BertEncoder<OpType>: a stack of post-LN BERT encoder layers run as ONE call,
// with the activations kept on the packed (padding-free) rows between layers.
//
// This class has no counterpart in the reference, whose API is one layer per call
// (bert_transformer.h:30-224): there every layer compresses its padded input and
// restores its padded output (bert_transformer.cu:68-78,119-127).  Here the mask
// prefix sum runs once, layer 0 gathers its rows from the padded input, layers in
// between read and write packed rows only, and the last layer scatters back to the
// padded [B,S,H] output (zero rows past each length).  The call never waits for the
// device and never allocates, so it can be captured into a HIP graph and replayed
// with other lengths in the same mask buffer.
#pragma once
#include <vector>

#include "bert_transformer.h"

namespace bytetransformer {

template <typename T>
struct BertEncoderInferParam {
  const T *input_tensor;   // [batch_size, seq_len, hidden_dim]
  const T *atten_mask;     // [batch_size, seq_len, seq_len]
  T *transformer_output;   // [batch_size, seq_len, hidden_dim]; may alias input_tensor
  void *buf;               // >= cal_bufsize() bytes, 256-byte aligned
  int batch_size;
  int seq_len;
  hipStream_t stream;
  const T *attention_bias = nullptr;   // [head_num, seq_len, seq_len] or null, same for every layer
  // all layers' pre-packed weights as written by BertEncoder::prepack, or null: the
  // products then read the weights as they are stored
  const void *prepacked = nullptr;
  int valid_rows_hint = 0;             // expected number of valid tokens (0 = unknown); tile choice only
};

template <OperationType OpType>
class BertEncoder {
  typedef Traits<OpType> Traits_;
  typedef typename Traits_::DataType DataType_;

  std::vector<BertTransformerParam<OpType>> layers_;
  Attention<OpType> *attention_layer_ = nullptr;
  const int max_batch_size_, max_seq_len_, head_num_, size_per_head_;
  bool use_fused_attention_, is_remove_padding_;
  const bool use_fp32_;
  int intermediate_size_ = 4;

  static unsigned long long align_up(unsigned long long v, unsigned long long a) {
    return (v + a - 1) / a * a;
  }
  unsigned long long layer_weight_elems() const {
    const unsigned long long hidden = (unsigned long long)head_num_ * size_per_head_;
    return (4 + 2 * (unsigned long long)intermediate_size_) * hidden * hidden;
  }

 public:
  float layernorm_eps = 1e-6f;

  BertEncoder(int max_batch_size, int head_num, int size_per_head, int max_seq_len,
              bool use_fused_attention = true, bool is_remove_padding = true,
              bool use_fp32 = false)
      : max_batch_size_(max_batch_size),
        max_seq_len_(max_seq_len),
        head_num_(head_num),
        size_per_head_(size_per_head),
        use_fused_attention_(use_fused_attention),
        is_remove_padding_(is_remove_padding),
        use_fp32_(use_fp32) {
    if (max_batch_size_ <= 2) is_remove_padding_ = false;   // bert_transformer.h:135-136
    attention_layer_ = new Attention<OpType>(max_batch_size, head_num, size_per_head, max_seq_len,
                                             use_fused_attention_, is_remove_padding_);
  }
  BertEncoder(const BertEncoder &) = delete;
  BertEncoder &operator=(const BertEncoder &) = delete;
  ~BertEncoder() { delete attention_layer_; }

  // every layer must use the same intermediate_size and attention parameters' tao
  void initialize(const std::vector<BertTransformerParam<OpType>> &layers) {
    if (layers.empty()) throw std::runtime_error("[BT][ERROR] BertEncoder: no layers");
    for (const auto &l : layers)
      if (l.intermediate_size != layers[0].intermediate_size)
        throw std::runtime_error("[BT][ERROR] BertEncoder: layers differ in intermediate_size");
    layers_ = layers;
    intermediate_size_ = layers[0].intermediate_size;
  }

  int num_layers() const { return (int)layers_.size(); }
  bool is_remove_padding() const { return is_remove_padding_; }

  // Scratch (elements of DataType_, T = max_batch*max_seq*hidden): [0,3T) qkv heads |
  // [3T,4T) attention out | [4T,5T) projection / LN1 | [5T,6T) packed hidden state |
  // [6T,(6+mult)T) FFN1 | word_idx int[B*S] | batch_idx int[B+1] | seq order int[B] |
  // split-k partial sums | the streaming attention's work list
  unsigned long long cal_bufsize() const {
    const unsigned long long rows = (unsigned long long)max_batch_size_ * max_seq_len_;
    const unsigned long long tensor = rows * head_num_ * size_per_head_;
    unsigned long long n = align_up((6 + intermediate_size_) * tensor * sizeof(DataType_), 256);
    // (+ 256 ints: the verdict slots of the prefix-mask check of the padded path)
    n += align_up((rows * 2 + 2 * (unsigned long long)max_batch_size_ + 2 + 256) * sizeof(int), 256);
    n += align_up(splitk_scratch_bytes(rows, (unsigned long long)head_num_ * size_per_head_), 256);
    n += align_up(attention_layer_->work_list_capacity(), 256);   // the attention's work list
    return n;
  }

  // bytes of the `prepacked` area for all layers, and the launch that fills it
  unsigned long long prepack_bytes() const {
    return (unsigned long long)layers_.size() * layer_weight_elems() * sizeof(DataType_);
  }
  void prepack(void *prepacked, hipStream_t stream) const;

  void infer(BertEncoderInferParam<DataType_> infer_param);
};

}  // namespace bytetransformer
