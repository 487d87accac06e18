/*
 * bt_encoder.h - C entry points of the host library (libbytetransformer.so)
 * for callers that cannot instantiate the C++ BertTransformer<OpType> class
 * template (ctypes, cgo, JNI ...).  One call = one encoder layer, exactly what
 * BertTransformer::infer does (reference: bytetransformer/include/
 * bert_transformer.h:98-224, bytetransformer/src/bert_transformer.cu:28-130).
 *
 * Pointers are device pointers unless stated; `stream` is a hipStream_t passed
 * as void*.  Returns 0 or a bt_status code; the message of a failure is
 * available from bt_encoder_last_error().  Never allocates device memory.
 */
#ifndef BT_ENCODER_H_
#define BT_ENCODER_H_

#ifdef __cplusplus
extern "C" {
#endif

/* The twelve per-layer tensors, in the order of the PyTorch operator's
 * arguments (reference: bytetransformer/th_op/ths_op_f.cc:28-34). */
typedef struct bt_layer_weights {
  const void *qkv_kernel;                  /* [H, 3H]  */
  const void *qkv_bias;                    /* [3H]     */
  const void *attr_output_kernel;          /* [H, H]   */
  const void *attr_output_bias;            /* [H]      */
  const void *attr_output_layernorm_gamma; /* [H] dtype or fp32 (gamma_beta_fp32) */
  const void *attr_output_layernorm_beta;
  const void *inter_kernel;                /* [H, mult*H] */
  const void *inter_bias;                  /* [mult*H]    */
  const void *output_kernel;               /* [mult*H, H] */
  const void *output_bias;                 /* [H]         */
  const void *output_layernorm_gamma;
  const void *output_layernorm_beta;
} bt_layer_weights;

typedef struct bt_encoder_config {
  int dtype;               /* BT_F16 or BT_F32: element type of every tensor (OperationType) */
  int max_batch_size;
  int max_seq_len;
  int head_num;
  int size_per_head;
  int intermediate_size;   /* FFN width as a multiple of hidden_dim; reference default 4 */
  int use_fused_attention; /* reference default 1 */
  int is_remove_padding;   /* reference default 1; forced off when max_batch_size <= 2 */
  int gamma_beta_fp32;     /* LayerNorm gamma/beta are float even when dtype is fp16 */
  float tao;               /* softmax temperature, reference default 1 */
  float layernorm_eps;     /* reference kernels: 1e-6 */
} bt_encoder_config;

/* Bytes of scratch `buf` that bt_encoder_layer_forward needs (cal_bufsize()). */
unsigned long long bt_encoder_bufsize(const bt_encoder_config *cfg);

/* One encoder layer: padded input [B,S,H] + mask [B,S,S] -> padded output
 * [B,S,H] (rows past each sequence's length are zero on the remove-padding
 * path).  `output` may alias `input` (the input is fully consumed before the
 * final LayerNorm writes). */
int bt_encoder_layer_forward(const bt_encoder_config *cfg, const bt_layer_weights *weights,
                             const void *input, const void *atten_mask, void *output, void *buf,
                             int batch_size, int seq_len, void *stream);

/*
 * What a call of bt_encoder_layer_forward with these sizes will launch around its QKV
 * product, for benchmarks that time the kernels one by one (host decisions only - sizes,
 * options, the measured tile table -, never a matter of results; no counterpart in the
 * reference).  rows_hint: the expected number of valid tokens, 0 = unknown.  plan[0..3]:
 * where the QKV / projection / FFN1 / FFN2 product runs on a k-contiguous copy of its
 * weight made during the call, 1 = by the call's first launch (bt_layer_prologue), 2 = by the
 * launch of the first LayerNorm (FFN1, FFN2), 0 = read as stored; plan[4]: 1 when the layer starts with the QKV
 * product that counts the mask rows itself (bt_gemm_qkv_bias_split_mask_rows) instead of
 * bt_layer_prologue; plan[5]: 1 when a layer on padded rows goes without offsets altogether.
 */
int bt_encoder_layer_plan(const bt_encoder_config *cfg, int batch_size, int seq_len,
                          int rows_hint, int *plan);

/* The same with the optional attention bias of the reference's infer parameters
 * (bert_transformer.h:93, attention.h:56): [head_num, seq_len, seq_len] of cfg->dtype,
 * added to the scaled logits before the mask term (softmax.h:41-46).  NULL = none. */
int bt_encoder_layer_forward_bias(const bt_encoder_config *cfg, const bt_layer_weights *weights,
                                  const void *input, const void *atten_mask,
                                  const void *attention_bias, void *output, void *buf,
                                  int batch_size, int seq_len, void *stream);

/*
 * One encoder layer with NO caller-owned scratch: bt_encoder_layer_forward_bias with
 * `buf` replaced by a device array that the library itself holds (BT_STATIC_SCRATCH_BYTES
 * per GPU the library runs on, from the first call on that GPU until the process ends).
 * No counterpart in the reference; it is for callers that cannot allocate device memory
 * for the workspace: code under HIP-graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  The call allocates nothing (no hipMalloc / hipFree, no allocating
 * library routine) and never waits for the device.
 *   - cfg's scratch need (bt_encoder_bufsize) must not exceed BT_STATIC_SCRATCH_BYTES,
 *     else BT_ERR_UNSUPPORTED with a message stating both sizes (BERT-base fp16 fits up
 *     to about 1300 padded rows, e.g. batch 1-2 x 512 or batch 4 x 256);
 *   - every call on one GPU shares that GPU's array: calls that overlap on one GPU (two
 *     streams, two threads) race; calls on one stream are ordered and safe;
 *   - the first call on a GPU looks the array's address up (hipGetSymbolAddress): make
 *     it outside stream capture.
 * attention_bias is nullable as in bt_encoder_layer_forward_bias; results are identical
 * to that entry point's.
 */
#define BT_STATIC_SCRATCH_BYTES (32ull << 20)
int bt_encoder_layer_forward_static(const bt_encoder_config *cfg, const bt_layer_weights *weights,
                                    const void *input, const void *atten_mask,
                                    const void *attention_bias, void *output, int batch_size,
                                    int seq_len, void *stream);

/*
 * Whole encoder in one call: num_layers layers (weights[l] = layer l) over one padded
 * batch, hidden state kept on the packed rows between layers.  No counterpart in the
 * reference, whose interface is one layer per call: the mask prefix sum runs once,
 * layer 0 gathers from the padded input, the last layer scatters to the padded output
 * (rows past each length zero), inner layers neither compress nor restore.  Never
 * waits for the device and never allocates, so a caller may capture it into a HIP
 * graph and replay it with other lengths written into the same mask buffer.
 *
 *   bt_encoder_forward_bufsize  bytes of scratch `buf` (independent of num_layers)
 *   bt_encoder_prepack_bytes    bytes of the pre-packed weight area of all layers
 *   bt_encoder_prepack          fills that area (one launch per layer); do it once per
 *                               weight set and pass it to every forward
 *   bt_encoder_forward          prepacked == NULL: the products read each layer's weights
 *                               as they are stored; attention_bias nullable, shared by
 *                               all layers; valid_rows_hint = expected number of valid
 *                               tokens or 0 (steers tile shapes only)
 * cfg->max_batch_size <= 2 or is_remove_padding == 0 runs every layer on the padded rows.
 */
unsigned long long bt_encoder_forward_bufsize(const bt_encoder_config *cfg);
unsigned long long bt_encoder_prepack_bytes(const bt_encoder_config *cfg, int num_layers);
int bt_encoder_prepack(const bt_encoder_config *cfg, int num_layers,
                       const bt_layer_weights *weights, void *prepacked, void *stream);
int bt_encoder_forward(const bt_encoder_config *cfg, int num_layers,
                       const bt_layer_weights *weights, const void *prepacked, const void *input,
                       const void *atten_mask, const void *attention_bias, void *output,
                       void *buf, int batch_size, int seq_len, int valid_rows_hint, void *stream);

const char *bt_encoder_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* BT_ENCODER_H_ */
