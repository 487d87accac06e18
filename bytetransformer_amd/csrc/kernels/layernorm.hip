// add-bias + residual + LayerNorm, packed in place and packed -> padded with
// zero fill.  Memory-bound: one wave64 per row, 16-byte lanes, the row lives in
// registers between the two statistics passes, reductions are wave shuffles
// (no LDS, no block barrier).
//
// Numerics follow bytetransformer/include/layernorm.h:114-159,273-296,334-373:
// x = (out + residual) + bias with both adds rounded to fp16, mean and biased
// variance in fp32 (two-pass), y = (x - mean) * rsqrt(var + eps) * gamma + beta.
#include "common.h"

namespace bt {

constexpr int kLnRowsPerBlock = 4;   // 2, 8 and 16 rows per workgroup measured 0-20 % slower

// Statistics and store of one row held in registers (x = (a + r) + bias, two fp16-rounded adds).
template <int NC, bool GB32, bool kAffineEarly, int NG>
__device__ __forceinline__ void ln_finish(const half8_t (&av)[NC], const half8_t (&rv)[NC],
                                          const half8_t (&bias_v)[NC], const half8_t (&gh)[NC],
                                          const half8_t (&bh)[NC], const float4_t (&g32)[NG][2],
                                          const float4_t (&b32)[NG][2], const void *gamma,
                                          const void *beta, const int (&cc)[NC],
                                          const bool (&live)[NC], half8_t *o, float inv_n,
                                          float eps) {
  float v[NC][8];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const half8_t x = (av[i] + rv[i]) + bias_v[i];  // two fp16-rounded adds
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      v[i][j] = live[i] ? (float)x[j] : 0.f;
      sum += v[i][j];
    }
  }
  const float mean = wave_sum(sum) * inv_n;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      v[i][j] = live[i] ? v[i][j] - mean : 0.f;
      sq += v[i][j] * v[i][j];
    }
  }
  const float rstd = rsqrtf(wave_sum(sq) * inv_n + eps);

#pragma unroll
  for (int i = 0; i < NC; ++i) {
    float g[8], bt_[8];
    if (GB32) {
      float4_t g0, g1, b0, b1;
      if (kAffineEarly) {
        g0 = g32[i][0], g1 = g32[i][1], b0 = b32[i][0], b1 = b32[i][1];
      } else {
        const float4_t *gp = (const float4_t *)gamma + 2 * cc[i];
        const float4_t *bp = (const float4_t *)beta + 2 * cc[i];
        g0 = gp[0], g1 = gp[1], b0 = bp[0], b1 = bp[1];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        g[j] = g0[j];
        g[4 + j] = g1[j];
        bt_[j] = b0[j];
        bt_[4 + j] = b1[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        g[j] = (float)gh[i][j];
        bt_[j] = (float)bh[i][j];
      }
    }
    half8_t y;
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = (half_t)(v[i][j] * rstd * g[j] + bt_[j]);
    if (live[i]) o[cc[i]] = y;
  }
}

// SPLITS > 0: `src` holds SPLITS fp32 partial sums of the row ([SPLITS][split_rows][H], the
// output of a split-k GEMM); their sum, rounded to fp16 once, takes the place of `out`.
//
// A launch of a few thousand rows is one round of waves, each living for the length of its
// chain of dependent memory accesses, so the kernel is written to keep that chain short:
// everything whose address does not depend on loaded data (bias, gamma, beta, the row
// index or the sequence offsets, and on packed rows the row of `src` itself) is requested
// at the top in one batch, a lane past the end of the row loads the last chunk again
// instead of branching, and the only dependent step left is the row(s) behind an index.
template <int NC, bool RESTORE, bool GB32, int SPLITS>
__device__ __forceinline__ void layernorm_block(
    int block, const half8_t *src, const half8_t *__restrict__ residual,
    const half8_t *__restrict__ bias, const void *__restrict__ gamma,
    const void *__restrict__ beta, half8_t *dst, const int *__restrict__ idx,
    const int *__restrict__ residual_row_index, int B, int S, int rows_cap, int split_rows,
    int chunks, float inv_n, float eps) {
  const int r = block * kLnRowsPerBlock + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows_cap) return;
  // fp32 gamma / beta of wide rows would not fit the registers next to the row: those
  // instantiations fetch them after the statistics, as before
  constexpr bool kAffineEarly = !GB32 || NC <= 2;

  int cc[NC];        // this lane's chunks, clamped into the row
  bool live[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = lane + i * kWave;
    live[i] = c < chunks;
    cc[i] = live[i] ? c : chunks - 1;
  }

  // ---- first batch: nothing here depends on loaded data ----
  half8_t bias_v[NC];
  half8_t gh[NC], bh[NC];
  float4_t g32[kAffineEarly && GB32 ? NC : 1][2], b32[kAffineEarly && GB32 ? NC : 1][2];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    bias_v[i] = bias[cc[i]];
    if (kAffineEarly) {
      if (GB32) {
        g32[i][0] = ((const float4_t *)gamma)[2 * cc[i]];
        g32[i][1] = ((const float4_t *)gamma)[2 * cc[i] + 1];
        b32[i][0] = ((const float4_t *)beta)[2 * cc[i]];
        b32[i][1] = ((const float4_t *)beta)[2 * cc[i] + 1];
      } else {
        gh[i] = ((const half8_t *)gamma)[cc[i]];
        bh[i] = ((const half8_t *)beta)[cc[i]];
      }
    }
  }

  size_t src_row, dst_row = r;
  half8_t av[NC];
  if (RESTORE && residual_row_index && SPLITS == 0) {
    // restore through the row map (word_idx of the offsets: entry r < M is the padded
    // position of packed row r, the entries from M on are the padded positions that stay
    // empty): only the store address depends on a loaded value, so the rows are requested
    // together with it.  idx = batch_idx, M = idx[B].
    src_row = r;
#pragma unroll
    for (int i = 0; i < NC; ++i) av[i] = src[src_row * chunks + cc[i]];
    half8_t rv0[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) rv0[i] = residual[src_row * chunks + cc[i]];
    dst_row = (size_t)residual_row_index[r];
    const int M = idx[B];
    if (r >= M) {
      const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
      for (int c = lane; c < chunks; c += kWave) dst[dst_row * chunks + c] = z;
      return;
    }
    ln_finish<NC, GB32, kAffineEarly>(av, rv0, bias_v, gh, bh, g32, b32, gamma, beta, cc, live,
                                      dst + dst_row * chunks, inv_n, eps);
    return;
  }
  if (RESTORE) {
    // r walks the padded [B, S] grid; idx = batch_idx
    const int b = r / S, s = r - b * S;
    const int start = idx[b], len = idx[b + 1] - start;
    if (s >= len) {
      const half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
      for (int c = lane; c < chunks; c += kWave) dst[dst_row * chunks + c] = z;
      return;
    }
    src_row = (size_t)start + s;
  } else {
    // idx = pointer to the live-row count (or null: all rows live): one scalar load, the same
    // address for every wave of the launch, and the one thing a wave waits for before it asks
    // for its rows - the waves of the rows past the count (40 % of a launch sized for the
    // padded batch) would otherwise read 1.5 KB each for nothing.
    src_row = r;
    const int M = idx ? *idx : rows_cap;
    if (r >= M) return;
    if (SPLITS == 0) {
#pragma unroll
      for (int i = 0; i < NC; ++i) av[i] = src[src_row * chunks + cc[i]];
    }
    const size_t res_row = residual_row_index ? (size_t)residual_row_index[src_row] : src_row;
    residual += res_row * chunks;
  }
  if (RESTORE) {
    residual += src_row * chunks;
    if (SPLITS == 0) {
#pragma unroll
      for (int i = 0; i < NC; ++i) av[i] = src[src_row * chunks + cc[i]];
    }
  }
  half8_t rv[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) rv[i] = residual[cc[i]];
  if (SPLITS > 0) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const float4_t *pp = (const float4_t *)src + (src_row * chunks + cc[i]) * 2;
      float4_t lo = pp[0], hi = pp[1];
#pragma unroll
      for (int sp = 1; sp < SPLITS; ++sp) {
        lo += pp[(size_t)sp * split_rows * chunks * 2];
        hi += pp[(size_t)sp * split_rows * chunks * 2 + 1];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        av[i][j] = (half_t)lo[j];
        av[i][4 + j] = (half_t)hi[j];
      }
    }
  }

  ln_finish<NC, GB32, kAffineEarly>(av, rv, bias_v, gh, bh, g32, b32, gamma, beta, cc, live,
                                    dst + dst_row * chunks, inv_n, eps);
}

template <int NC, bool RESTORE, bool GB32, int SPLITS>
__global__ __launch_bounds__(kLnRowsPerBlock *kWave) void layernorm_kernel(
    const half8_t *src, const half8_t *__restrict__ residual,
    const half8_t *__restrict__ bias, const void *__restrict__ gamma,
    const void *__restrict__ beta, half8_t *dst, const int *__restrict__ idx,
    const int *__restrict__ residual_row_index, int B, int S, int rows_cap, int split_rows,
    int chunks, float inv_n, float eps) {
  layernorm_block<NC, RESTORE, GB32, SPLITS>(blockIdx.x, src, residual, bias, gamma, beta, dst, idx,
                                             residual_row_index, B, S, rows_cap, split_rows, chunks,
                                             inv_n, eps);
}

// The packed LayerNorm with k-contiguous weight copies riding along: the first `copy_blocks`
// workgroups of the grid move 64 x 64 tiles of the [K, N] matrices of `jobs` into their [N, K]
// copies (through LDS, as the layer's prologue launch does), the others are the LayerNorm's.
// A launch of a few thousand rows moves its 20 MB at half of what the memory system
// sustains, so the copy of a few MB costs this launch less than a launch of its own would,
// and the product behind it (FFN1) reads its weight k-contiguous.
template <int NC, bool GB32>
__global__ __launch_bounds__(kLnRowsPerBlock *kWave) void layernorm_copy_kernel(
    const half8_t *src, const half8_t *__restrict__ residual,
    const half8_t *__restrict__ bias, const void *__restrict__ gamma,
    const void *__restrict__ beta, half8_t *dst, const int *__restrict__ idx,
    const int *__restrict__ residual_row_index, int rows_cap, int chunks, float inv_n, float eps,
    WeightJobs jobs, int copy_blocks) {
  static_assert(kLnRowsPerBlock * kWave == 256, "a tile is moved by 256 threads");
  if ((int)blockIdx.x < copy_blocks) {
    __shared__ half_t tiles[64][kTransposePitch];
    const int t_end = jobs.tile_end[jobs.count - 1];
    for (int t0 = blockIdx.x; t0 < t_end; t0 += copy_blocks)
      transpose_tiles_64<1>(jobs, t0, tiles, threadIdx.x);
    return;
  }
  layernorm_block<NC, false, GB32, 0>((int)blockIdx.x - copy_blocks, src, residual, bias, gamma,
                                      beta, dst, idx, residual_row_index, 0, 1, rows_cap, rows_cap,
                                      chunks, inv_n, eps);
}

template <bool RESTORE, int SPLITS = 0>
static int launch_ln(const void *src, const void *residual, const void *bias, const void *gamma,
                     const void *beta, int gb32, void *dst, const int *idx,
                     const int *residual_row_index, int B, int S, int rows_cap, int H, float eps,
                     hipStream_t s, const char *who, int split_rows = 0) {
  BT_REQUIRE(H > 0 && H % 8 == 0, BT_ERR_UNSUPPORTED, "%s: hidden_dim %d must be a multiple of 8",
             who, H);
  BT_REQUIRE(aligned16({src, residual, bias, gamma, beta, dst}), BT_ERR_INVALID_ARGUMENT,
             "%s: tensor pointers must be 16-byte aligned", who);
  const int chunks = H / 8;
  const int nc = (chunks + kWave - 1) / kWave;
  BT_REQUIRE(nc <= 8, BT_ERR_UNSUPPORTED, "%s: hidden_dim %d exceeds 4096", who, H);
  if (rows_cap == 0) return BT_OK;
  const int grid = (rows_cap + kLnRowsPerBlock - 1) / kLnRowsPerBlock;
  const float inv_n = 1.0f / (float)H;
#define BT_LN_LAUNCH(NC_, GB_)                                                                  \
  layernorm_kernel<NC_, RESTORE, GB_, SPLITS><<<grid, kLnRowsPerBlock * kWave, 0, s>>>(         \
      (const half8_t *)src, (const half8_t *)residual, (const half8_t *)bias, gamma, beta,      \
      (half8_t *)dst, idx, residual_row_index, B, S, rows_cap, split_rows ? split_rows : rows_cap, \
      chunks, inv_n, eps)
#define BT_LN_NC(NC_)              \
  do {                             \
    if (gb32)                      \
      BT_LN_LAUNCH(NC_, true);     \
    else                           \
      BT_LN_LAUNCH(NC_, false);    \
  } while (0)
  if (nc <= 1)
    BT_LN_NC(1);
  else if (nc <= 2)
    BT_LN_NC(2);
  else if (nc <= 4)
    BT_LN_NC(4);
  else
    BT_LN_NC(8);
#undef BT_LN_NC
#undef BT_LN_LAUNCH
  BT_CHECK_LAUNCH(who);
  return BT_OK;
}

}  // namespace bt

using namespace bt;

extern "C" int bt_add_bias_residual_layernorm(void *out, const void *residual,
                                              const int *residual_row_index, const void *bias,
                                              const void *gamma, const void *beta,
                                              int gamma_beta_fp32, const int *valid_rows,
                                              int rows_cap, int hidden_dim, float eps,
                                              void *stream) {
  BT_REQUIRE(out && residual && bias && gamma && beta, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm: null pointer argument");
  BT_REQUIRE(rows_cap >= 0, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm: negative rows_cap");
  BT_REQUIRE(!residual_row_index || valid_rows, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm: residual_row_index needs valid_rows");
  return launch_ln<false>(out, residual, bias, gamma, beta, gamma_beta_fp32, out, valid_rows,
                          residual_row_index, 0, 1, rows_cap, hidden_dim, eps, as_stream(stream),
                          "bt_add_bias_residual_layernorm");
}

extern "C" int bt_add_bias_residual_layernorm_copy(
    void *out, const void *residual, const int *residual_row_index, const void *bias,
    const void *gamma, const void *beta, int gamma_beta_fp32, const int *valid_rows, int rows_cap,
    int hidden_dim, float eps, int weight_count, const void *const *w, void *const *wt,
    const int *k, const int *n, void *stream) {
  const char *who = "bt_add_bias_residual_layernorm_copy";
  BT_REQUIRE(out && residual && bias && gamma && beta, BT_ERR_INVALID_ARGUMENT,
             "%s: null pointer argument", who);
  BT_REQUIRE(rows_cap >= 0, BT_ERR_INVALID_ARGUMENT, "%s: negative rows_cap", who);
  BT_REQUIRE(!residual_row_index || valid_rows, BT_ERR_INVALID_ARGUMENT,
             "%s: residual_row_index needs valid_rows", who);
  WeightJobs jobs;
  const int rc = make_weight_jobs(who, &jobs, weight_count, w, wt, k, n, 0, nullptr, nullptr);
  if (rc != BT_OK) return rc;
  if (jobs.count == 0)
    return launch_ln<false>(out, residual, bias, gamma, beta, gamma_beta_fp32, out, valid_rows,
                            residual_row_index, 0, 1, rows_cap, hidden_dim, eps, as_stream(stream),
                            who);
  const int H = hidden_dim;
  BT_REQUIRE(H > 0 && H % 8 == 0, BT_ERR_UNSUPPORTED, "%s: hidden_dim %d must be a multiple of 8",
             who, H);
  BT_REQUIRE(aligned16({out, residual, bias, gamma, beta}), BT_ERR_INVALID_ARGUMENT,
             "%s: tensor pointers must be 16-byte aligned", who);
  const int chunks = H / 8;
  const int nc = (chunks + kWave - 1) / kWave;
  BT_REQUIRE(nc <= 8, BT_ERR_UNSUPPORTED, "%s: hidden_dim %d exceeds 4096", who, H);
  // one tile per copying workgroup up to 1024 of them (a BERT-large FFN weight has 1024 tiles)
  const int tiles = jobs.tile_end[jobs.count - 1];
  const int copy_blocks = tiles < 1024 ? tiles : 1024;
  const int grid = copy_blocks + (rows_cap + kLnRowsPerBlock - 1) / kLnRowsPerBlock;
  const float inv_n = 1.0f / (float)H;
  hipStream_t s = as_stream(stream);
#define BT_LN_LAUNCH(NC_, GB_)                                                                  \
  layernorm_copy_kernel<NC_, GB_><<<grid, kLnRowsPerBlock * kWave, 0, s>>>(                     \
      (const half8_t *)out, (const half8_t *)residual, (const half8_t *)bias, gamma, beta,      \
      (half8_t *)out, valid_rows, residual_row_index, rows_cap, chunks, inv_n, eps, jobs,       \
      copy_blocks)
#define BT_LN_NC(NC_)              \
  do {                             \
    if (gamma_beta_fp32)           \
      BT_LN_LAUNCH(NC_, true);     \
    else                           \
      BT_LN_LAUNCH(NC_, false);    \
  } while (0)
  if (nc <= 1)
    BT_LN_NC(1);
  else if (nc <= 2)
    BT_LN_NC(2);
  else if (nc <= 4)
    BT_LN_NC(4);
  else
    BT_LN_NC(8);
#undef BT_LN_NC
#undef BT_LN_LAUNCH
  BT_CHECK_LAUNCH(who);
  return BT_OK;
}

extern "C" int bt_add_bias_residual_layernorm_restore(
    const void *out, const void *residual, const void *bias, const void *gamma, const void *beta,
    int gamma_beta_fp32, void *out_padded, const int *batch_idx, const int *word_idx,
    int batch_size, int seq_len, int hidden_dim, float eps, void *stream) {
  BT_REQUIRE(out && residual && bias && gamma && beta && out_padded && batch_idx,
             BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm_restore: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm_restore: sizes must be positive");
  BT_REQUIRE((long long)batch_size * seq_len < (1ll << 31), BT_ERR_UNSUPPORTED,
             "bt_add_bias_residual_layernorm_restore: too many rows");
  return launch_ln<true>(out, residual, bias, gamma, beta, gamma_beta_fp32, out_padded, batch_idx,
                         word_idx, batch_size, seq_len, batch_size * seq_len, hidden_dim, eps,
                         as_stream(stream), "bt_add_bias_residual_layernorm_restore");
}

extern "C" int bt_splitk_layernorm(const void *partials, int splits, const void *residual,
                                   const int *residual_row_index, const void *bias,
                                   const void *gamma, const void *beta, int gamma_beta_fp32,
                                   void *dst, const int *batch_idx, const int *valid_rows,
                                   int batch_size, int seq_len, int rows_cap, int hidden_dim,
                                   float eps, void *stream) {
  BT_REQUIRE(partials && residual && bias && gamma && beta && dst, BT_ERR_INVALID_ARGUMENT,
             "bt_splitk_layernorm: null pointer argument");
  BT_REQUIRE(splits == 2 || splits == 4, BT_ERR_UNSUPPORTED,
             "bt_splitk_layernorm: splits=%d (supported: 2, 4)", splits);
  BT_REQUIRE(rows_cap >= 0, BT_ERR_INVALID_ARGUMENT, "bt_splitk_layernorm: negative rows_cap");
  hipStream_t s = as_stream(stream);
  if (batch_idx) {
    // restore mode: dst is the padded [batch_size, seq_len, hidden] output
    // rows_cap is the row count of one partial-sum slice (what bt_gemm_splitk was given)
    BT_REQUIRE(batch_size > 0 && seq_len > 0 && (long long)batch_size * seq_len < (1ll << 31) &&
                   rows_cap > 0 && rows_cap <= batch_size * seq_len,
               BT_ERR_INVALID_ARGUMENT,
               "bt_splitk_layernorm: restore needs 0 < rows_cap <= batch_size * seq_len");
    BT_REQUIRE(!residual_row_index, BT_ERR_INVALID_ARGUMENT,
               "bt_splitk_layernorm: no residual gather in restore mode");
    const int padded = batch_size * seq_len;
    return splits == 2
               ? launch_ln<true, 2>(partials, residual, bias, gamma, beta, gamma_beta_fp32, dst,
                                    batch_idx, nullptr, batch_size, seq_len, padded, hidden_dim,
                                    eps, s, "bt_splitk_layernorm", rows_cap)
               : launch_ln<true, 4>(partials, residual, bias, gamma, beta, gamma_beta_fp32, dst,
                                    batch_idx, nullptr, batch_size, seq_len, padded, hidden_dim,
                                    eps, s, "bt_splitk_layernorm", rows_cap);
  }
  BT_REQUIRE(!residual_row_index || valid_rows, BT_ERR_INVALID_ARGUMENT,
             "bt_splitk_layernorm: residual_row_index needs valid_rows");
  return splits == 2
             ? launch_ln<false, 2>(partials, residual, bias, gamma, beta, gamma_beta_fp32, dst,
                                   valid_rows, residual_row_index, 0, 1, rows_cap, hidden_dim, eps,
                                   s, "bt_splitk_layernorm")
             : launch_ln<false, 4>(partials, residual, bias, gamma, beta, gamma_beta_fp32, dst,
                                   valid_rows, residual_row_index, 0, 1, rows_cap, hidden_dim, eps,
                                   s, "bt_splitk_layernorm");
}
