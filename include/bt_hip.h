/*
 * bt_hip.h - C ABI of the gfx950 kernel library (libbt_hip.so) behind the
 * padding-free BERT encoder-layer forward.
 *
 * Conventions for every entry point:
 *   - plain C types only; `stream` is a hipStream_t passed as void* (NULL = the
 *     null stream); all work is enqueued asynchronously on it;
 *   - returns BT_OK (0) or a BT_ERR_* code, never throws, never allocates
 *     device memory; the caller owns every buffer, scratch included;
 *   - after a non-zero return bt_last_error_string() describes the failure
 *     (thread-local);
 *   - tensor pointers must be 16-byte aligned (every kernel moves data in 16-byte pieces);
 *   - activations and weights are fp16 (IEEE binary16) unless a dtype argument
 *     says otherwise; "packed" means the M valid token rows of the batch laid
 *     out back to back in (batch, position) order;
 *   - `valid_rows` arguments point at ONE int in device memory holding the
 *     number of live rows M (normally batch_idx + batch_size); kernels size
 *     their grids for `rows_cap` rows and retire rows >= M on the device, so
 *     the host never waits for M.  NULL means all rows_cap rows are live.
 *   - `rows_hint` arguments are the host's estimate of M (0 = none); they only
 *     steer the choice of tile shape and never affect results.
 *
 * Each declaration cites the reference interface it replaces (paths relative
 * to the ByteTransformer tree).
 */
#ifndef BT_HIP_H_
#define BT_HIP_H_

#ifdef __cplusplus
extern "C" {
#endif

enum bt_status {
  BT_OK = 0,
  BT_ERR_INVALID_ARGUMENT = 1,
  BT_ERR_UNSUPPORTED = 2,
  BT_ERR_HIP = 3
};

enum bt_dtype { BT_F32 = 0, BT_F16 = 1 };

/* ABI revision of the loaded library. */
int bt_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char *bt_last_error_string(void);

/*
 * Tuning knob for experiments and tests; no counterpart in the reference.
 *   "gemm_tile"     -1 heuristic | 0: 256x256 tile, 8 waves | 1: 128x128, 4 computing + 4 loader
 *                   waves | 2: 256x128, 8 + 4 waves | 3: 256x192, 8 + 4 waves | 4: 32x64, 2 + 2 waves
 *                   | 5: 128x128 with a two-deep ring (two workgroups per CU)
 *                   | 6, 7, 8: tiles 2, 1, 0 as persistent workgroups (about one per CU, each
 *                   running one load pipeline over several tiles of its XCD's range)
 *   "gemm_table_margin"  4 (default), 0..100: per cent by which a tile's measured time must beat
 *                   that of the cost model's choice before the measured table overrides the
 *                   model (100 = the model alone decides)
 *   "attention_qb"  -1 heuristic | 1 | 2: 16-query blocks per wave in the grouped kernel
 *   "attention_key_split"  -1 heuristic | 0 | 1: the 64-query streaming attention with four waves,
 *                   or with eight: two groups of four take alternate 64-key halves of every ring
 *                   slot and are merged at the end
 *   "layer_prepack" -1 (default) | 0 | 1: answer of bt_gemm_prepack_pays: by the measured
 *                   table | never | always
 *   "padded_mask_direct"  320 (default): on padded rows (batches of one and two) a layer of
 *                   up to this many tokens per sequence goes without bt_layer_prologue: its
 *                   attention applies the mask tensor itself, which needs no offsets, and a
 *                   launch less is worth more there than the keys the lengths would skip;
 *                   0 = every layer starts with the prologue.  Same results either way.
 *   "qkv_mask_rows" -1 (default) | 0 | 1: a padding-free fp16 layer that has to build its
 *                   offsets starts with bt_gemm_qkv_bias_split_mask_rows (one launch less,
 *                   every weight read as stored) where that entry takes the shape and no
 *                   per-call weight copy pays | always with bt_layer_prologue | with the
 *                   fused entry wherever it takes the shape, without copies.  Same results
 *                   either way.
 *   "ln_weight_copy"  1 (default) | 0: a padding-free fp16 layer that goes without
 *                   bt_layer_prologue lets the launch of its first LayerNorm make the k-contiguous
 *                   copies that pay for FFN1 and FFN2 (bt_add_bias_residual_layernorm_copy) | such
 *                   a layer makes no copies (or keeps the prologue for them).  Same results.
 *   "prefetch"      1 (default) | 0: honour / ignore the prefetch hint of the attention entries
 *   "prefetch_min_grid"  512 (default): attention launches of fewer workgroups ignore the hint
 *                   (there the warm-up costs more than it returns); 1 = every launch honours it
 *   "f32_gemm_tile" -1 heuristic | 0: 128x128 tile, 8 waves | 1: 128x64, 4 waves | 2: 64x64, 4 waves
 *                   (bt_gemm_f32 only)
 *   "attention_short_limit"  0 (default) .. 512: the host library sends sequences up to this
 *                   length to bt_attention_short when use_fused_attention is set; 0 = always
 *                   the streaming kernel, which measures faster at every length
 *   "attention_xcd_map"  workgroup order of the attention kernels: 0 plain (fp16 kernels
 *                   only) | 1 XCD-aware | 2 (default) XCD-aware, and in the streaming
 *                   kernels (fp16, float, generic head sizes) the live query
 *                   tiles are dealt evenly to the CUs once the launch has more than two
 *                   rounds of workgroups per CU (batches up to 128 sequences) | 3: that
 *                   balanced order at any size
 * Process-wide; results do not depend on it beyond fp32 summation order.
 */
int bt_set_option(const char *name, int value);
int bt_get_option(const char *name, int *value);

/*
 * Mask prefix sum.  Replaces build_sequence_length_padding_offset_kernelLauncher
 * and parallel_prefix (bytetransformer/include/remove_padding.h:36-101).
 *   atten_mask  [batch_size, seq_len, seq_len], dtype mask_dtype (BT_F16/BT_F32);
 *               only row 0 of each batch is read; an element counts when >= 0.5
 *   batch_idx   int[batch_size + 1]  exclusive prefix sum of the lengths, total last
 *   word_idx    int[batch_size * seq_len]; first M entries = b*seq_len + i, i < len_b (the valid
 *               positions in order), then the batch_size * seq_len - M padded positions
 *   seq_order   NULL, or int[batch_size]: the sequence indices by descending
 *               length (ties by index); the attention kernels use it to start the
 *               longest sequences first (no counterpart in the reference)
 *   valid_word_num_host  NULL, or a host int that receives M; passing it makes
 *               the call wait for the stream (the reference always does)
 */
int bt_build_offsets(const void *atten_mask, int mask_dtype, int batch_size, int seq_len,
                     int *batch_idx, int *word_idx, int *seq_order, int *valid_word_num_host,
                     void *stream);

/*
 * *dst = *src by one lane of a one-wave launch on `stream`.  `dst` may be host memory that
 * the device can write (hipHostMalloc): a host that polls it learns the valid-token count
 * (src = batch_idx + batch_size) some time after the launch without ever waiting for the
 * stream - the asynchronous form of the reference's blocking copy of valid_word_num
 * (remove_padding.h:99-100).
 */
int bt_publish_int(const int *src, int *dst, void *stream);

/*
 * Is atten_mask exactly the prefix mask of the lengths in batch_idx, i.e. for every
 * batch b and EVERY row i: mask[b, i, j] == 1 for j < len_b and == 0 from there on, with
 * no empty sequence?  Then the padded-row attention may ignore the tensor and stop at
 * len_b keys, which gives the same result as applying it (the logits of the ones are not
 * shifted, the exp of the others is exactly 0).
 * The reference always applies the tensor on that path (attention_fused.cu:234-237); no
 * counterpart there.
 *   bt_mask_prefix_slots  asynchronous: 256 workgroups each write 1 ("nothing wrong in
 *                         my share of the rows") or 0 to slots[0..255] (device); the
 *                         mask is the prefix mask when every slot is 1.  The attention
 *                         entry below takes such an array and decides on the device.
 *   bt_mask_is_prefix     the same pass into scratch (device int[256]), then waits for
 *                         the stream and writes the verdict 0 / 1 to *is_prefix_host.
 */
int bt_mask_prefix_slots(const void *atten_mask, int mask_dtype, int batch_size, int seq_len,
                         const int *batch_idx, int *slots, void *stream);
int bt_mask_is_prefix(const void *atten_mask, int mask_dtype, int batch_size, int seq_len,
                      const int *batch_idx, int *scratch, int *is_prefix_host, void *stream);

/*
 * Layer prologue: what one layer has to know before its first product, in ONE launch.
 * No counterpart in the reference, which rebuilds the offsets on every call
 * (bert_transformer.cu:62-66) and reads the weights as stored.
 *   - the offsets of bt_build_offsets (batch_idx, word_idx, seq_order; same rules);
 *   - mask_prefix_slots (nullable): the int[256] verdict of bt_mask_prefix_slots for the
 *     lengths of this very mask;
 *   - attention_work_list (nullable; needs head_num and padded_rows): the list of
 *     bt_attention_worklist for these offsets, when launches of this shape use one
 *     (bt_attention_worklist_bytes > 0; else nothing is written);
 *   - weight_count in [0, 4] matrices w[i] ([k[i], n[i]] as the caller stores them) to
 *     pre-pack into wt[i] ([n[i], k[i]], as bt_transpose_weights does) for the products of
 *     this call (see bt_gemm_prepack_pays): made afresh in every call from the weights as
 *     they are at that moment - nothing is remembered between calls, so nothing can go
 *     stale;
 *   - warm_count in [0, 4] readable device ranges (host arrays of pointers and sizes) that
 *     the layer's launches will read later - the weights that are used as stored: touched
 *     line by line so that they sit in the memory-side cache by then.  Purely a hint
 *     (bt_set_option("prefetch", 0) ignores it); the results do not depend on it.
 */
int bt_layer_prologue(const void *atten_mask, int mask_dtype, int batch_size, int seq_len,
                      int *batch_idx, int *word_idx, int *seq_order, int *mask_prefix_slots,
                      void *attention_work_list, int head_num, int padded_rows, int weight_count,
                      const void *const *w, void *const *wt, const int *k, const int *n,
                      int warm_count, const void *const *warm,
                      const unsigned long long *warm_bytes, void *stream);

/*
 * Gather valid rows: to_tensor[t, :] = from_tensor[word_idx[t], :], t < M.
 * Replaces compressBertInput_kernelLauncher (remove_padding.h:104-121).
 * hidden_dim % 8 == 0.  M is read on the device from batch_idx[batch_size].
 */
int bt_compress(const void *from_tensor, void *to_tensor, const int *batch_idx,
                const int *word_idx, int batch_size, int seq_len, int hidden_dim, void *stream);

/*
 * Weight pre-pack: wt[n, k] = w[k, n].  The reference hands cuBLAS the
 * [in, out] row-major weight directly (gemm.cu:27-39), and so do the per-layer entries
 * here (weight_kn = 1 of the products below).  A caller that owns an immutable copy of
 * its weights can pre-pack them once with this and pass weight_kn = 0: both operands
 * are then contiguous along k.  k % 8 == 0, n % 8 == 0.
 */
int bt_transpose_weight(const void *w, void *wt, int k, int n, void *stream);

/* The same pre-pack for up to four matrices in ONE launch (a layer has four:
 * QKV, attention output, FFN1, FFN2): wt[i][n, k] = w[i][k, n]. */
int bt_transpose_weights(int count, const void *const *w, void *const *wt, const int *k,
                         const int *n, void *stream);

/*
 * c[rows, n] = a[rows, k] . w[k, n], fp16 in/out, fp32 accumulate on MFMA.
 * Replaces dense_layer_kernel_launcher (bytetransformer/src/gemm.cu:32-39) at
 * its attention-output-projection and FFN2 call sites
 * (bert_transformer.cu:102-104,115-117).  k % 64 == 0, n % 8 == 0.
 * weight_kn (all fp16 products): 1 = `wt` is the row-major [k, n] weight itself, as the
 * reference hands it to cuBLAS - nothing to prepare, nothing that could go stale;
 * 0 = `wt` is the [n, k] copy made by bt_transpose_weights, for callers that own an
 * immutable copy of the weights (the whole-encoder object): the 256 x 256 tile runs
 * about 10 % faster on it.  Results are bit-identical either way.
 */
int bt_gemm(const void *a, const void *wt, void *c, const int *valid_rows, int rows_cap,
            int rows_hint, int n, int k, int weight_kn, void *stream);

/* Epilogue codes of the question below. */
#define BT_EPILOGUE_PLAIN 0
#define BT_EPILOGUE_BIAS_GELU 1
#define BT_EPILOGUE_QKV_SPLIT 2
/*
 * 1 when, by the measured tile table, the product of about `rows` live rows with an
 * [k, n] weight and this epilogue runs faster on a pre-packed copy even after paying for
 * the copy (made per call inside bt_layer_prologue), else 0 - shapes outside the table
 * included.  bt_set_option("layer_prepack", 0 | 1) overrides the table.  Only ever a
 * matter of time: the products' results do not depend on the layout.  No counterpart in
 * the reference.
 */
int bt_gemm_prepack_pays(long long rows, int n, int k, int epilogue);
/*
 * The same answer as a quantity: the microseconds per launch that the product saves on a
 * pre-packed copy after paying for the copy (bt_gemm_prepack_pays = more than one); 0 for
 * shapes outside the table, +-1e9 under bt_set_option("layer_prepack", 1 | 0).  A layer
 * that could go without its prologue launch altogether if it made no copy asks for more
 * than that launch costs.
 */
float bt_gemm_prepack_gain_us(long long rows, int n, int k, int epilogue);

/*
 * c = gelu_tanh(a . w + bias).  Replaces gemm_bias_gelu
 * (bytetransformer/src/gemm_bias_act.cu:76-148; tanh constants
 * gemm_bias_act.h:80-87).
 */
int bt_gemm_bias_gelu(const void *a, const void *wt, const void *bias, void *c,
                      const int *valid_rows, int rows_cap, int rows_hint, int n, int k,
                      int weight_kn, void *stream);

/*
 * QKV projection with the bias add and the head split fused into the store:
 *   qkv_heads[which][g][t][0:d] = (a . w_qkv + bias)[t, which*H + g*d : +d]
 * with which in {Q, K, V}, H = head_num*size_per_head, layout
 * [3][head_num][rows_cap][size_per_head].  Replaces the bias-free QKV
 * dense_layer_kernel_launcher call (bert_transformer.cu:85-87) plus
 * add_QKV_bias_padding (attention_nofused_utils.cu:143-184) / the in-kernel
 * bias add of attention_fused.cu:318-325.  The head split needs size_per_head == 64.
 * a_row_index (nullable, needs valid_rows): live row t of A is a[a_row_index[t], :] -
 * passing word_idx reads the valid tokens straight out of the padded input, which
 * folds compressBertInput (remove_padding.h:104-121) into this GEMM's operand fetch.
 * size_per_head != 64: the projections stay token-major, qkv_heads = [rows_cap, 3 * hidden]
 * (Q | K | V per row), the layout bt_attention_generic_f16 reads.
 */
int bt_gemm_qkv_bias_split(const void *a, const int *a_row_index, const void *wt_qkv,
                           const void *bias_qkv, void *qkv_heads, const int *valid_rows,
                           int rows_cap, int rows_hint, int head_num, int size_per_head,
                           int weight_kn, void *stream);

/*
 * The same product for a padding-free layer that has not built its offsets yet: the live
 * rows of the padded from_tensor [batch_size * seq_len, hidden] and their order are taken
 * from the mask inside the launch (every workgroup counts row 0 of each sequence's mask
 * itself, remove_padding.h:36-86's length rule), so no launch ahead of the product has
 * to produce word_idx first.  Workgroup 0 also writes batch_idx [batch_size + 1], word_idx
 * [batch_size * seq_len] and seq_order [batch_size] exactly as bt_build_offsets /
 * bt_layer_prologue would (word_idx and seq_order may be null), for the kernels that follow
 * on the stream.  rows_cap of qkv_heads is batch_size * seq_len.  Covers
 * build_sequence_length_padding_offset_kernelLauncher + compressBertInput + the QKV GEMM +
 * the bias add of one layer call (bert_transformer.cu:62-87) in one launch.
 * bt_gemm_qkv_mask_rows_supported: 1 when the launch takes this shape (at most 64
 * sequences whose mask rows fit 64 KB), else 0 - then build the offsets first.
 */
int bt_gemm_qkv_mask_rows_supported(int batch_size, int seq_len, int mask_dtype);
int bt_gemm_qkv_bias_split_mask_rows(const void *from_tensor, const void *atten_mask,
                                     int mask_dtype, int batch_size, int seq_len,
                                     const void *wt_qkv, const void *bias_qkv, void *qkv_heads,
                                     int *batch_idx, int *word_idx, int *seq_order,
                                     int rows_hint, int head_num, int size_per_head,
                                     int weight_kn, void *stream);

/*
 * Fused multi-head attention over the head-major Q/K/V written by
 * bt_gemm_qkv_bias_split; output is token-major [rows, H] with head g at
 * columns [g*d, g*d+d).  Per sequence b and head g:
 *   P = exp(scale*Q.K^T - rowmax) / (rowsum + 1e-6),  O = fp16(P) . V
 * keys >= len_b are excluded by index, len_b = batch_idx[b+1] - batch_idx[b].
 *   padded_rows == 0: sequence b owns packed rows [batch_idx[b], batch_idx[b+1])
 *   padded_rows != 0: sequence b owns rows [b*seq_len, (b+1)*seq_len), all
 *                     seq_len query rows are computed against the len_b keys
 *   atten_mask (nullable, padded rows only): the fp16 [batch_size, seq_len, seq_len]
 *                     0/1 mask.  When given, ALL seq_len keys of the sequence take
 *                     part and every logit is shifted by (mask[b,q,k] - 1) * 10000
 *                     before the softmax - the arbitrary-mask semantics of the
 *                     reference's non-remove-padding kernels (attention_fused.cu:234-237,
 *                     attention_fused_long.cu) - instead of the prefix-length rule.
 *   attention_bias (nullable): fp16 [head_num, seq_len, seq_len], added to the scaled
 *                     logit of (head, query position, key position) before the mask
 *                     term, as the reference's unfused softmax does (softmax.h:41-46,
 *                     attention_nofused.cu:78-95); positions are relative to the
 *                     start of the sequence in both row layouts.
 *   prefetch, prefetch_bytes, prefetch_count (nullable / 0): up to 4 readable device
 *                     ranges (host arrays of pointers and sizes) that LATER kernels of the
 *                     stream will read, typically the layer's remaining weight matrices.
 *                     Workgroups that retire early touch them line by line so that they
 *                     sit in the memory-side cache by then; purely a hint, the results do
 *                     not depend on it.  No counterpart in the reference.
 *   seq_order (nullable): a permutation of the sequence indices from
 *                     bt_build_offsets; workgroups are issued in that order so the
 *                     longest sequences start first.  Results do not depend on it.
 *   work_list (bt_attention_grouped; nullable): see bt_attention_worklist below.
 *   mask_prefix_slots (bt_attention_grouped; nullable): the int[256] that
 *                     bt_mask_prefix_slots filled for this atten_mask earlier on the
 *                     stream.  When all are 1 the kernel ignores the tensor and stops at
 *                     the lengths, which gives the same result; decided on the device,
 *                     so the call stays asynchronous.
 *   batch_idx == NULL (bt_attention_grouped only): allowed on padded rows with an
 *                     atten_mask and no mask_prefix_slots - every one of the seq_len keys
 *                     takes part under the mask tensor, so no length is read (seq_order and
 *                     work_list are then ignored).
 *
 * bt_attention_short keeps the whole logits row of a query tile in registers
 * (exact two-pass softmax, seq_len <= 512).  Replaces wmma_attention[_rm]_kernel
 * and wmma_attention_long[_rm]_kernel with their dispatch tables
 * (attention_fused.cu:168-491, attention_fused_long.cu:30-488).
 *
 * bt_attention_grouped streams K/V tiles with an online softmax over a
 * variable-length work list, any seq_len.  Replaces
 * CutlassAttention::infer_impl (cutlass_attention.cu:150-210): the grouped
 * GEMM0 + partial softmax, softmax_reduction_kernel and grouped GEMM1, without
 * the logits round trip through HBM.
 */
int bt_attention_short(const void *qkv_heads, void *attention_output, const int *batch_idx,
                       const int *seq_order, const void *atten_mask, const void *attention_bias,
                       int batch_size, int seq_len, int rows_cap, int head_num, int size_per_head,
                       float scale, int padded_rows, const void *const *prefetch,
                       const unsigned long long *prefetch_bytes, int prefetch_count,
                       void *stream);

int bt_attention_grouped(const void *qkv_heads, void *attention_output, const int *batch_idx,
                         const int *seq_order, const void *atten_mask, const void *attention_bias,
                         int batch_size, int seq_len, int rows_cap, int head_num,
                         int size_per_head, float scale, int padded_rows,
                         const void *const *prefetch, const unsigned long long *prefetch_bytes,
                         int prefetch_count, const int *mask_prefix_slots,
                         const void *work_list, void *stream);

/*
 * The balanced workgroup order of bt_attention_grouped (option "attention_xcd_map" 2) as a
 * list, so that a forward of many layers looks it up once instead of in every workgroup of
 * every layer: entry w = what workgroup w works on.  No counterpart in the reference.
 *   bt_attention_worklist_bytes  bytes of the list for a launch of this shape, 0 when such a
 *                                launch does not use the balanced order (few workgroups, more
 *                                than 128 sequences, another option value)
 *   bt_attention_worklist        fills it from batch_idx / seq_order (asynchronous); pass the
 *                                same shape, padded_rows and offsets to bt_attention_grouped
 *                                with the list (work_list there is nullable and only a time
 *                                saver: results do not depend on it)
 */
unsigned long long bt_attention_worklist_bytes(int batch_size, int seq_len, int head_num);
int bt_attention_worklist(const int *batch_idx, const int *seq_order, int batch_size, int seq_len,
                          int head_num, int padded_rows, void *work_list, void *stream);

/*
 * out = LayerNorm((out + residual) + bias) * gamma + beta, in place on `out`,
 * both adds rounded to fp16, statistics in fp32 (two-pass), eps inside the
 * rsqrt.  Replaces add_bias_input_layernorm_kernel_launcher
 * (bytetransformer/include/layernorm.h:410-428, kernels :114-159,273-296).
 * gamma/beta are fp32 when gamma_beta_fp32 != 0, else fp16.  hidden_dim % 8 == 0.
 * residual_row_index (nullable, needs valid_rows): row t adds residual[residual_row_index[t], :]
 * instead of residual[t, :] (word_idx: the residual is read from the padded input).
 */
int bt_add_bias_residual_layernorm(void *out, const void *residual,
                                   const int *residual_row_index, const void *bias,
                                   const void *gamma, const void *beta, int gamma_beta_fp32,
                                   const int *valid_rows, int rows_cap, int hidden_dim,
                                   float eps, void *stream);

/*
 * The same launch with k-contiguous weight copies riding along: weight_count (0..4) matrices
 * w[i] [k[i], n[i]] are copied into wt[i] [n[i], k[i]] (bt_transpose_weights) by workgroups of
 * their own at the head of the grid, complete when the launch is.  A LayerNorm over a few
 * thousand rows leaves most of the memory system idle, so the copies cost this launch less than
 * a launch of their own would - the layer uses it for the weight of the product that follows
 * (FFN1; the role of the reference's one-off weight layout choice, gemm.cu:27-39, made per
 * call so that nothing is kept between calls).  With weight_count == 0 it is
 * bt_add_bias_residual_layernorm.
 */
int bt_add_bias_residual_layernorm_copy(void *out, const void *residual,
                                        const int *residual_row_index, const void *bias,
                                        const void *gamma, const void *beta, int gamma_beta_fp32,
                                        const int *valid_rows, int rows_cap, int hidden_dim,
                                        float eps, int weight_count, const void *const *w,
                                        void *const *wt, const int *k, const int *n,
                                        void *stream);

/*
 * Same LayerNorm, but reading packed rows and writing the padded layout:
 * out_padded[b, s, :] = LN(out[p] + residual[p] + bias) with p = batch_idx[b]+s
 * when s < len_b, else zeros.  Replaces
 * add_bias_input_layernorm_restore_output_kernel_launcher (layernorm.h:430-446,
 * kernels :334-373).
 * word_idx (nullable): the word_idx that bt_build_offsets / bt_layer_prologue wrote beside
 * this batch_idx, all batch_size * seq_len entries of it (valid positions first, the empty
 * ones after them).  With it a wave knows its output row from one load that travels together
 * with its input rows instead of ahead of them; `out` and `residual` must then hold
 * batch_size * seq_len rows.  Same result.
 */
int bt_add_bias_residual_layernorm_restore(const void *out, const void *residual,
                                           const void *bias, const void *gamma,
                                           const void *beta, int gamma_beta_fp32,
                                           void *out_padded, const int *batch_idx,
                                           const int *word_idx, int batch_size, int seq_len,
                                           int hidden_dim, float eps, void *stream);

/*
 * Split-k pair for launches with few rows and a long k (FFN2 at a few hundred tokens),
 * where one tile's k loop is the whole run time.  No counterpart in the reference.
 *
 * bt_gemm_splitk: partials[s][m][:] = a[m, ks:ke] . wt[:, ks:ke]^T as fp32, split s covering
 * k range [s, s+1) * k / splits; partials is float [splits][rows_cap][n]; splits in [1, 16]
 * dividing k / 64.
 *
 * bt_splitk_layernorm: the add-bias + residual + LayerNorm entry points with the fp32
 * partials (summed, rounded to fp16 once) in the place of `out`; splits 2 or 4.
 * batch_idx == NULL: packed rows, dst [rows_cap, hidden] (valid_rows / residual_row_index as
 * in bt_add_bias_residual_layernorm); batch_idx != NULL: dst is the padded
 * [batch_size, seq_len, hidden] output with zero fill, and rows_cap (<= batch_size *
 * seq_len, >= the live rows) is the row count of one slice of the partials, i.e. the
 * rows_cap that bt_gemm_splitk was given.
 */
int bt_gemm_splitk(const void *a, const void *wt, void *partials, int splits,
                   const int *valid_rows, int rows_cap, int n, int k, int weight_kn, void *stream);

int bt_splitk_layernorm(const void *partials, int splits, const void *residual,
                        const int *residual_row_index, const void *bias, const void *gamma,
                        const void *beta, int gamma_beta_fp32, void *dst, const int *batch_idx,
                        const int *valid_rows, int batch_size, int seq_len, int rows_cap,
                        int hidden_dim, float eps, void *stream);

/*
 * ---- OperationType::FP32 ------------------------------------------------------
 * The float flavour of the layer: every tensor (activations, weights, biases, gamma,
 * beta, mask, attention bias) is float, products run on the fp32 MFMA with fp32
 * operands and accumulators.  Weights are read as the caller stores them ([K, N]
 * row-major): there is no pre-pack.
 *
 * bt_gemm_f32: c[M, n] = a[M, k] . w[k, n] (+ bias[n]) (then tanh-GELU when gelu != 0,
 * which needs a bias).  a_row_index (nullable, needs valid_rows): row r of A is
 * a[a_row_index[r], :].  rows_hint: expected live rows or 0, steers the tile shape only.
 * n % 4 == 0, k % 4 == 0.  Replaces the cuBLAS calls of
 * dense_layer_kernel_launcher<float> (bytetransformer/src/gemm.cu:32-39), the QKV bias
 * add of add_QKV_bias (attention_nofused_utils.cu:143-184) and
 * gemm_bias_gelu<float> (gemm_bias_act.cu:24-75).
 */
int bt_gemm_f32(const void *a, const int *a_row_index, const void *w, const void *bias, void *c,
                int gelu, const int *valid_rows, int rows_cap, int rows_hint, int n, int k,
                void *stream);

/*
 * Fused multi-head attention on float, token-major projections qkv [rows, 3 * hidden]
 * (Q | K | V per row, QKV bias already added) -> attention_output [rows, hidden].
 * P = exp(x - max) / (sum + 1e-6) with x = scale q.k + attention_bias[head, q, key]
 * + (atten_mask[b, q, key] - 1) * 10000, the arithmetic of softmax_kernel_warp[_et]
 * (bytetransformer/include/softmax.h:25-60,103-140); replaces the whole unfused path
 * Attention<FP32>::nofused_infer (attention_nofused.cu:27-114) without its logits
 * buffer.  atten_mask (nullable, float [B,S,S]) is applied on both row layouts; keys at
 * or past the sequence length are excluded by index on packed rows (they do not exist
 * there) and, without a mask, on padded rows.  seq_order (nullable) as in the fp16
 * entries: issue order only.  size_per_head a multiple of 8 up to 128.
 */
/* The same kernel on fp16 tensors (operands widened to float on chip), for fp16 layers whose
 * head size the fp16 attention entries do not cover: size_per_head a multiple of 8 up to 128.
 * Role of the reference's unfused path for size_per_head != 64 (bert_transformer.h:132-133,
 * attention_nofused.cu:27-114). */
int bt_attention_generic_f16(const void *qkv, void *attention_output, const int *batch_idx,
                             const int *seq_order, const void *atten_mask,
                             const void *attention_bias, int batch_size, int seq_len,
                             int rows_cap, int head_num, int size_per_head, float scale,
                             int padded_rows, void *stream);

int bt_attention_f32(const void *qkv, void *attention_output, const int *batch_idx,
                     const int *seq_order, const void *atten_mask, const void *attention_bias, int batch_size,
                     int seq_len, int rows_cap, int head_num, int size_per_head, float scale,
                     int padded_rows, void *stream);

/*
 * The two LayerNorm entry points on float: x = out + residual + bias in fp32, two-pass
 * statistics, hidden_dim % 4 == 0 (layernorm.h:20-40, layernorm.cu:89-148 for float).
 */
int bt_add_bias_residual_layernorm_f32(void *out, const void *residual,
                                       const int *residual_row_index, const void *bias,
                                       const void *gamma, const void *beta,
                                       const int *valid_rows, int rows_cap, int hidden_dim,
                                       float eps, void *stream);

int bt_add_bias_residual_layernorm_restore_f32(const void *out, const void *residual,
                                               const void *bias, const void *gamma,
                                               const void *beta, void *out_padded,
                                               const int *batch_idx, int batch_size,
                                               int seq_len, int hidden_dim, float eps,
                                               void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BT_HIP_H_ */
