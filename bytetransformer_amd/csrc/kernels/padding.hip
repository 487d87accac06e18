// Padding removal: mask prefix sum -> packed-token offsets, and the gather of
// valid rows into the packed layout.  Integer outputs are bit-exact with the
// reference's parallel_prefix (bytetransformer/include/remove_padding.h:36-86).
#include "common.h"

#include <atomic>
#include <cstring>
#include <string>

namespace bt {

// ---- error plumbing shared by every translation unit ------------------------
static thread_local std::string g_last_error;

void set_error(const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
}

int hip_fail(hipError_t e, const char *what) {
  set_error("[BT][ERROR] HIP runtime error: %s (%s)", hipGetErrorString(e), what);
  return BT_ERR_HIP;
}

// ---- tuning options ---------------------------------------------------------
static std::atomic<int> g_gemm_tile{-1};
static std::atomic<int> g_attention_qb{-1};
static std::atomic<int> g_prefetch{1};
static std::atomic<int> g_prefetch_min_grid{512};
static std::atomic<int> g_attention_key_split{-1};
static std::atomic<int> g_layer_prepack{-1};
static std::atomic<int> g_padded_mask_direct{320};
static std::atomic<int> g_qkv_mask_rows{-1};
static std::atomic<int> g_f32_gemm_tile{-1};
static std::atomic<int> g_attention_short_limit{0};
static std::atomic<int> g_attention_xcd_map{2};
static std::atomic<int> g_gemm_table_margin{4};
static std::atomic<int> g_ln_weight_copy{1};
int option_gemm_table_margin() { return g_gemm_table_margin.load(std::memory_order_relaxed); }
int option_attention_xcd_map() { return g_attention_xcd_map.load(std::memory_order_relaxed); }
int option_f32_gemm_tile() { return g_f32_gemm_tile.load(std::memory_order_relaxed); }
int option_gemm_tile() { return g_gemm_tile.load(std::memory_order_relaxed); }
int option_attention_qb() { return g_attention_qb.load(std::memory_order_relaxed); }
int option_prefetch() { return g_prefetch.load(std::memory_order_relaxed); }
int option_prefetch_min_grid() { return g_prefetch_min_grid.load(std::memory_order_relaxed); }
int option_attention_key_split() { return g_attention_key_split.load(std::memory_order_relaxed); }
int option_layer_prepack() { return g_layer_prepack.load(std::memory_order_relaxed); }

// ---- offsets ----------------------------------------------------------------
constexpr int kOffsetThreads = 1024;
constexpr int kOffsetWaves = kOffsetThreads / kWave;

// Every block recomputes all B lengths (B*S mask elements, a few KB) and the
// exclusive scan, then writes word_idx for the sequences it owns; block 0 also
// writes batch_idx.  No inter-block communication, so the grid can be as wide
// as the batch.
template <typename T>
__global__ __launch_bounds__(kOffsetThreads) void build_offsets_kernel(
    const T *__restrict__ mask, int *__restrict__ batch_idx, int *__restrict__ word_idx,
    int *__restrict__ seq_order, int B, int S) {
  extern __shared__ int smem[];
  int *s_len = smem;          // [B]
  int *s_off = smem + B;      // [B + 1]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  // one wave per sequence: count row-0 mask elements >= 0.5 with a 64-wide ballot
  for (int b = wave; b < B; b += kOffsetWaves) {
    const int count = wave_row_length(mask + (size_t)b * S * S, S, lane);
    if (lane == 0) s_len[b] = count;
  }
  __syncthreads();

  // wave 0: exclusive scan of the lengths in chunks of 64
  if (wave == 0) {
    int carry = 0;
    for (int i0 = 0; i0 < B; i0 += kWave) {
      int i = i0 + lane;
      int len = i < B ? s_len[i] : 0;
      int incl = wave_inclusive_scan(len, lane);
      if (i < B) s_off[i] = carry + incl - len;
      carry += __shfl(incl, 63, 64);
    }
    if (lane == 0) s_off[B] = carry;
  }
  __syncthreads();

  if (blockIdx.x == 0) {
    for (int i = tid; i <= B; i += kOffsetThreads) batch_idx[i] = s_off[i];
    // sequences by descending length (ties by index): rank by counting
    if (seq_order)
      for (int b = tid; b < B; b += kOffsetThreads) {
        const int len = s_len[b];
        int rank = 0;
        for (int o = 0; o < B; ++o) {
          const int lo = s_len[o];
          rank += (lo > len) || (lo == len && o < b);
        }
        seq_order[rank] = b;
      }
  }

  for (int b = blockIdx.x; b < B; b += gridDim.x) {
    const int off = s_off[b], len = s_len[b];
    // valid tokens first, in order; the padded positions fill the tail from M on (pad_at =
    // number of padded positions of the sequences before b)
    const int pad_at = s_off[B] + b * S - off;
    for (int i = tid; i < S; i += kOffsetThreads)
      word_idx[i < len ? off + i : pad_at + i - len] = b * S + i;
  }
}

// ---- is the mask the plain prefix mask of its lengths? ------------------------
// One wave per mask row (b, i): any element that is not exactly 1 before len_b or not
// exactly 0 from there on, or an empty sequence, clears the workgroup's slot of `ok`
// (the padded-row attention shifts a logit by (mask - 1) * 10000: only 1 leaves it alone
// and only a shift of the full -10000 is certain to vanish in the softmax).  Every
// workgroup writes its own slot each time, so nothing needs clearing beforehand.
constexpr int kPrefixBlocks = 256;
constexpr int kPrefixWaves = 4;

template <typename T>
__global__ __launch_bounds__(kPrefixWaves *kWave) void mask_prefix_kernel(
    const T *__restrict__ mask, const int *__restrict__ batch_idx, int *__restrict__ ok, int B,
    int S) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long rows = (long long)B * S;
  int bad = 0;
  for (long long r = (long long)blockIdx.x * kPrefixWaves + wave; r < rows;
       r += (long long)gridDim.x * kPrefixWaves) {
    const int b = (int)(r / S);
    const int len = batch_idx[b + 1] - batch_idx[b];
    bad |= len == 0;
    const T *row = mask + (size_t)r * S;
    for (int j = lane; j < S; j += kWave) bad |= (float)row[j] != (j < len ? 1.0f : 0.0f);
  }
  const int any_bad = __syncthreads_or(bad);
  if (threadIdx.x == 0) ok[blockIdx.x] = !any_bad;
}

// ---- layer prologue ------------------------------------------------------------
// Everything a layer needs before its first product, in ONE launch: the offsets
// (blocks below `offset_blocks`, the code of build_offsets_kernel), the prefix-mask
// verdict slots (every block, one wave per mask row; a wave counts the length of its row's
// sequence itself, so no block waits for another) and the k-contiguous copies of those
// weight matrices whose product runs faster on one (made afresh in every call, from the
// weights as they are at that moment: nothing is kept between calls).
constexpr int kPrologueThreads = 1024;
constexpr int kPrologueWaves = kPrologueThreads / kWave;
constexpr int kPackGroups = kPrologueThreads / 256;   // 64 x 64 tiles one block transposes at a time

// The pre-pack job belongs to a fixed set of blocks (kPackFirst .. kPackFirst + kPackBlocks
// - 1, whatever the batch size), each with an equal share of the 64 x 64 tiles.
constexpr int kPackFirst = 64;     // blocks below build offsets (at most 64 of them)
constexpr int kPackBlocks = 192;

// The attention's balanced work list, built by blocks of their own beyond the others
// (kListBlocks of them, each with its own copy of the lengths in LDS): one wave per entry.
constexpr int kListBlocks = 48;
struct PrologueList {
  int4 *list;           // null: none
  unsigned entries;
  int bq, nqb, heads, padded_rows;
};

template <typename T>
__global__ __launch_bounds__(kPrologueThreads) void layer_prologue_kernel(
    const T *__restrict__ mask, int *__restrict__ batch_idx, int *__restrict__ word_idx,
    int *__restrict__ seq_order, int *__restrict__ slots, int B, int S, int offset_blocks,
    WeightJobs pw, PrologueList pl) {
  extern __shared__ __attribute__((aligned(16))) int smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  // ---- offsets (and, in the list blocks, the attention's work list) ----
  const bool list_block = pl.list && blockIdx.x >= gridDim.x - kListBlocks;
  if ((int)blockIdx.x < offset_blocks || list_block) {
    int *s_len = smem;          // [B]
    int *s_off = smem + B;      // [B + 1]
    int *s_order = smem + 2 * B + 1;   // [B] rank -> sequence, longest first
    for (int b = wave; b < B; b += kPrologueWaves) {
      const int count = wave_row_length(mask + (size_t)b * S * S, S, lane);
      if (lane == 0) s_len[b] = count;
    }
    __syncthreads();
    if (wave == 0) {
      int carry = 0;
      for (int i0 = 0; i0 < B; i0 += kWave) {
        const int i = i0 + lane;
        const int len = i < B ? s_len[i] : 0;
        const int incl = wave_inclusive_scan(len, lane);
        if (i < B) s_off[i] = carry + incl - len;
        carry += __shfl(incl, 63, 64);
      }
      if (lane == 0) s_off[B] = carry;
    }
    // sequences by descending length (ties by index): rank by counting
    if (blockIdx.x == 0 || list_block)
      for (int b = tid; b < B; b += kPrologueThreads) {
        const int len = s_len[b];
        int rank = 0;
        for (int o = 0; o < B; ++o) {
          const int lo = s_len[o];
          rank += (lo > len) || (lo == len && o < b);
        }
        s_order[rank] = b;
      }
    __syncthreads();
    if (list_block) {
      AttListArgs la{B, S, pl.heads, pl.nqb, pl.padded_rows, s_off, s_order};
      const unsigned first = (blockIdx.x - (gridDim.x - kListBlocks)) * kPrologueWaves + wave;
      for (unsigned e = first; e < pl.entries; e += kListBlocks * kPrologueWaves) {
        const AttWork w = pl.bq == 128 ? att_work_balanced<128>(la, e) : att_work_balanced<64>(la, e);
        if (lane == 0)
          pl.list[e] = w.exists ? int4{w.b, w.head | (w.qb << 16), w.seq_start, w.len}
                                : int4{-1, 0, 0, 0};
      }
      return;     // a list block has no other job
    }
    if (blockIdx.x == 0) {
      for (int i = tid; i <= B; i += kPrologueThreads) batch_idx[i] = s_off[i];
      if (seq_order)
        for (int b = tid; b < B; b += kPrologueThreads) seq_order[b] = s_order[b];
    }
    for (int b = blockIdx.x; b < B; b += offset_blocks) {
      const int off = s_off[b], len = s_len[b];
      const int pad_at = s_off[B] + b * S - off;   // the padded positions fill the tail from M on
      for (int i = tid; i < S; i += kPrologueThreads)
        word_idx[i < len ? off + i : pad_at + i - len] = b * S + i;
    }
  }

  // ---- is the mask the plain prefix mask of its lengths? (mask_prefix_kernel's rule) ----
  if (slots) {
    const long long rows = (long long)B * S;
    constexpr int kVec = 16 / (int)sizeof(T);       // elements per 16-byte load
    const bool vec = S % kVec == 0 && (reinterpret_cast<uintptr_t>(mask) & 15) == 0;
    int bad = 0, len_of = -1, len = 0;
    for (long long r = (long long)blockIdx.x * kPrologueWaves + wave; r < rows;
         r += (long long)kPrefixBlocks * kPrologueWaves) {
      const int b = (int)(r / S);
      if (b != len_of) {
        len = wave_row_length(mask + (size_t)b * S * S, S, lane);
        len_of = b;
      }
      bad |= len == 0;
      const T *row = mask + (size_t)r * S;
      if (vec) {
        for (int j0 = lane * kVec; j0 < S; j0 += kWave * kVec) {
          const uint4_t raw = *(const uint4_t *)(row + j0);
          const T *e = (const T *)&raw;
#pragma unroll
          for (int i = 0; i < kVec; ++i) bad |= (float)e[i] != (j0 + i < len ? 1.0f : 0.0f);
        }
      } else {
        for (int j = lane; j < S; j += kWave) bad |= (float)row[j] != (j < len ? 1.0f : 0.0f);
      }
    }
    const int any_bad = __syncthreads_or(bad);
    if (tid == 0) slots[blockIdx.x] = !any_bad;
  }

  // ---- k-contiguous copies of the weights that were asked for ----
  if (pw.count > 0 && (int)blockIdx.x >= kPackFirst) {
    const int pb = blockIdx.x - kPackFirst;
    const int tiles_all = pw.tile_end[pw.count - 1];
    const int tile_lo = (int)((long long)tiles_all * pb / kPackBlocks);
    const int tile_hi = (int)((long long)tiles_all * (pb + 1) / kPackBlocks);
    // a group of 256 lanes takes one tile at a time; which matrix and where in it is the
    // same for the whole group (scalar arithmetic)
    half_t(*tile)[kTransposePitch] =
        (half_t(*)[kTransposePitch])((half_t *)smem + (size_t)(tid >> 8) * 64 * kTransposePitch);
#pragma unroll 1
    for (int t0 = tile_lo; t0 < tile_hi; t0 += kPackGroups) {
      const int t = t0 + (tid >> 8);
      int j = 0, first = 0;
#pragma unroll
      for (int q = 1; q < 4; ++q)
        if (q < pw.count && t >= pw.tile_end[q - 1]) {
          j = q;
          first = pw.tile_end[q - 1];
        }
      const int tl = t - first;
      transpose_tile_64(pw.w[j], pw.wt[j], pw.K[j], pw.N[j], (tl / pw.tiles_n[j]) * 64,
                        (tl % pw.tiles_n[j]) * 64, tile, tid & 255, t < tile_hi);
      __syncthreads();
    }
  }

  // ---- warm-up of the weights that are read as stored ----
  const unsigned n_lines = pw.warm_end[3];
  if (n_lines && (int)blockIdx.x >= kPackFirst && (int)blockIdx.x < kPackFirst + kPackBlocks) {
    const unsigned pb = blockIdx.x - kPackFirst;
    const unsigned per = (n_lines + kPackBlocks - 1) / kPackBlocks;
    const unsigned first = pb * per;
    const unsigned last = first + per < n_lines ? first + per : n_lines;
    warm_lines(pw, first + tid, last, kPrologueThreads);
  }
}

// ---- one int from device memory to wherever the caller reads it -----------------
// (pinned host memory that the device can write: the host then learns a count without ever
// waiting for the stream)
__global__ void publish_int_kernel(const int *__restrict__ src, int *__restrict__ dst) {
  if (threadIdx.x == 0) *dst = *src;
}

// ---- compress ---------------------------------------------------------------
// One wave per packed row, 16-byte lanes.  M is read from batch_idx[B]; rows
// past it retire immediately, so the grid is sized for B*S without a host sync.
constexpr int kRowsPerBlock = 4;

__global__ __launch_bounds__(kRowsPerBlock *kWave) void compress_kernel(
    const uint4_t *__restrict__ from, uint4_t *__restrict__ to, const int *__restrict__ batch_idx,
    const int *__restrict__ word_idx, int B, int chunks /* H/8 */) {
  const int t = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  const int M = batch_idx[B];
  if (t >= M) return;
  const int lane = threadIdx.x & 63;
  const size_t src = (size_t)word_idx[t] * chunks;
  const size_t dst = (size_t)t * chunks;
  for (int c = lane; c < chunks; c += kWave) to[dst + c] = from[src + c];
}

int make_weight_jobs(const char *who, WeightJobs *out, int weight_count, const void *const *w,
                     void *const *wt, const int *k, const int *n, int warm_count,
                     const void *const *warm, const unsigned long long *warm_bytes) {
  WeightJobs &pw = *out;
  memset(&pw, 0, sizeof(pw));
  BT_REQUIRE(weight_count >= 0 && weight_count <= 4, BT_ERR_INVALID_ARGUMENT,
             "%s: weight_count=%d outside [0, 4]", who, weight_count);
  pw.count = weight_count;
  if (weight_count > 0) {
    BT_REQUIRE(w && wt && k && n, BT_ERR_INVALID_ARGUMENT,
               "%s: weights to pre-pack need w, wt, k and n", who);
    long long tiles = 0;
    for (int i = 0; i < weight_count; ++i) {
      BT_REQUIRE(w[i] && wt[i], BT_ERR_INVALID_ARGUMENT, "%s: null matrix pointer #%d", who, i);
      BT_REQUIRE(aligned16({w[i], wt[i]}), BT_ERR_INVALID_ARGUMENT,
                 "%s: matrix pointers must be 16-byte aligned", who);
      BT_REQUIRE(k[i] > 0 && n[i] > 0 && k[i] % 8 == 0 && n[i] % 8 == 0, BT_ERR_UNSUPPORTED,
                 "%s: k=%d n=%d must be positive multiples of 8", who, k[i], n[i]);
      tiles += (long long)((k[i] + 63) / 64) * ((n[i] + 63) / 64);
      BT_REQUIRE(tiles < (1ll << 21), BT_ERR_UNSUPPORTED,
                 "%s: weight matrices beyond 2^21 tiles of 64 x 64", who);
      pw.w[i] = (const half_t *)w[i];
      pw.wt[i] = (half_t *)wt[i];
      pw.K[i] = k[i];
      pw.N[i] = n[i];
      pw.tiles_n[i] = (n[i] + 63) / 64;
      pw.tile_end[i] = (int)tiles;
    }
    for (int i = weight_count; i < 4; ++i) {
      pw.tiles_n[i] = 1;
      pw.tile_end[i] = (int)tiles;
    }
  }
  BT_REQUIRE(warm_count >= 0 && warm_count <= 4 && (warm_count == 0 || (warm && warm_bytes)),
             BT_ERR_INVALID_ARGUMENT, "%s: warm_count=%d outside [0, 4], or no ranges", who,
             warm_count);
  if (option_prefetch()) {
    unsigned end = 0;
    for (int r = 0; r < 4; ++r) {
      if (r < warm_count && warm[r]) {
        // one dword at the start of each 128-byte line; a last line of fewer than four bytes
        // is left alone, so no byte outside the range is read
        const unsigned long long lines = (warm_bytes[r] + 124) / 128;
        BT_REQUIRE(lines < (1ull << 24), BT_ERR_UNSUPPORTED, "%s: a range to warm beyond 2 GiB",
                   who);
        pw.warm[r] = (const char *)warm[r];
        end += (unsigned)lines;
      }
      pw.warm_end[r] = end;
    }
  }
  return BT_OK;
}

}  // namespace bt

using namespace bt;

extern "C" int bt_version(void) { return 1; }

extern "C" const char *bt_last_error_string(void) { return g_last_error.c_str(); }

extern "C" int bt_set_option(const char *name, int value) {
  BT_REQUIRE(name, BT_ERR_INVALID_ARGUMENT, "bt_set_option: null name");
  if (!strcmp(name, "gemm_tile")) {
    BT_REQUIRE(value >= -1 && value <= 8, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: gemm_tile=%d outside [-1, 8]", value);
    g_gemm_tile.store(value);
  } else if (!strcmp(name, "ln_weight_copy")) {
    BT_REQUIRE(value == 0 || value == 1, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: ln_weight_copy=%d must be 0 or 1", value);
    g_ln_weight_copy.store(value);
  } else if (!strcmp(name, "gemm_table_margin")) {
    BT_REQUIRE(value >= 0 && value <= 100, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: gemm_table_margin=%d outside [0, 100]", value);
    g_gemm_table_margin.store(value);
  } else if (!strcmp(name, "attention_qb")) {
    BT_REQUIRE(value == -1 || value == 1 || value == 2, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: attention_qb=%d must be -1, 1 or 2", value);
    g_attention_qb.store(value);
  } else if (!strcmp(name, "f32_gemm_tile")) {
    BT_REQUIRE(value >= -1 && value <= 2, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: f32_gemm_tile=%d outside [-1, 2]", value);
    g_f32_gemm_tile.store(value);
  } else if (!strcmp(name, "attention_short_limit")) {
    BT_REQUIRE(value >= 0 && value <= 512, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: attention_short_limit=%d outside [0, 512]", value);
    g_attention_short_limit.store(value);
  } else if (!strcmp(name, "attention_xcd_map")) {
    BT_REQUIRE(value >= 0 && value <= 3, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: attention_xcd_map=%d outside [0, 3]", value);
    g_attention_xcd_map.store(value);
  } else if (!strcmp(name, "prefetch")) {
    BT_REQUIRE(value == 0 || value == 1, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: prefetch=%d must be 0 or 1", value);
    g_prefetch.store(value);
  } else if (!strcmp(name, "attention_key_split")) {
    BT_REQUIRE(value >= -1 && value <= 1, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: attention_key_split=%d must be -1, 0 or 1", value);
    g_attention_key_split.store(value);
  } else if (!strcmp(name, "layer_prepack")) {
    BT_REQUIRE(value >= -1 && value <= 1, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: layer_prepack=%d must be -1, 0 or 1", value);
    g_layer_prepack.store(value);
  } else if (!strcmp(name, "padded_mask_direct")) {
    BT_REQUIRE(value >= 0 && value <= (1 << 20), BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: padded_mask_direct=%d outside [0, 2^20]", value);
    g_padded_mask_direct.store(value);
  } else if (!strcmp(name, "qkv_mask_rows")) {
    BT_REQUIRE(value >= -1 && value <= 1, BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: qkv_mask_rows=%d must be -1, 0 or 1", value);
    g_qkv_mask_rows.store(value);
  } else if (!strcmp(name, "prefetch_min_grid")) {
    BT_REQUIRE(value >= 1 && value <= (1 << 20), BT_ERR_INVALID_ARGUMENT,
               "bt_set_option: prefetch_min_grid=%d outside [1, 2^20]", value);
    g_prefetch_min_grid.store(value);
  } else {
    set_error("bt_set_option: unknown option '%s'", name);
    return BT_ERR_INVALID_ARGUMENT;
  }
  return BT_OK;
}

extern "C" int bt_get_option(const char *name, int *value) {
  BT_REQUIRE(name && value, BT_ERR_INVALID_ARGUMENT, "bt_get_option: null argument");
  if (!strcmp(name, "gemm_tile")) {
    *value = g_gemm_tile.load();
  } else if (!strcmp(name, "ln_weight_copy")) {
    *value = g_ln_weight_copy.load();
  } else if (!strcmp(name, "gemm_table_margin")) {
    *value = g_gemm_table_margin.load();
  } else if (!strcmp(name, "attention_qb")) {
    *value = g_attention_qb.load();
  } else if (!strcmp(name, "prefetch")) {
    *value = g_prefetch.load();
  } else if (!strcmp(name, "prefetch_min_grid")) {
    *value = g_prefetch_min_grid.load();
  } else if (!strcmp(name, "attention_key_split")) {
    *value = g_attention_key_split.load();
  } else if (!strcmp(name, "layer_prepack")) {
    *value = g_layer_prepack.load();
  } else if (!strcmp(name, "padded_mask_direct")) {
    *value = g_padded_mask_direct.load();
  } else if (!strcmp(name, "qkv_mask_rows")) {
    *value = g_qkv_mask_rows.load();
  } else if (!strcmp(name, "f32_gemm_tile")) {
    *value = g_f32_gemm_tile.load();
  } else if (!strcmp(name, "attention_short_limit")) {
    *value = g_attention_short_limit.load();
  } else if (!strcmp(name, "attention_xcd_map")) {
    *value = g_attention_xcd_map.load();
  } else {
    set_error("bt_get_option: unknown option '%s'", name);
    return BT_ERR_INVALID_ARGUMENT;
  }
  return BT_OK;
}

extern "C" int bt_build_offsets(const void *atten_mask, int mask_dtype, int batch_size,
                                int seq_len, int *batch_idx, int *word_idx, int *seq_order,
                                int *valid_word_num_host, void *stream) {
  BT_REQUIRE(atten_mask && batch_idx && word_idx, BT_ERR_INVALID_ARGUMENT,
             "bt_build_offsets: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_build_offsets: batch_size=%d seq_len=%d must be positive", batch_size, seq_len);
  BT_REQUIRE(mask_dtype == BT_F16 || mask_dtype == BT_F32, BT_ERR_INVALID_ARGUMENT,
             "bt_build_offsets: unknown mask dtype %d", mask_dtype);
  BT_REQUIRE((long long)batch_size * seq_len < (1ll << 31), BT_ERR_UNSUPPORTED,
             "bt_build_offsets: batch_size*seq_len overflows int32");
  const size_t smem = (2 * (size_t)batch_size + 1) * sizeof(int);
  BT_REQUIRE(smem <= 64 * 1024, BT_ERR_UNSUPPORTED,
             "bt_build_offsets: batch_size %d too large (limit 8191)", batch_size);
  hipStream_t s = as_stream(stream);
  const int grid = batch_size < 64 ? batch_size : 64;
  if (mask_dtype == BT_F16)
    build_offsets_kernel<half_t><<<grid, kOffsetThreads, smem, s>>>(
        (const half_t *)atten_mask, batch_idx, word_idx, seq_order, batch_size, seq_len);
  else
    build_offsets_kernel<float><<<grid, kOffsetThreads, smem, s>>>(
        (const float *)atten_mask, batch_idx, word_idx, seq_order, batch_size, seq_len);
  BT_CHECK_LAUNCH("build_offsets_kernel");
  if (valid_word_num_host) {
    hipError_t e = hipMemcpyAsync(valid_word_num_host, batch_idx + batch_size, sizeof(int),
                                  hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return hip_fail(e, "copy of valid_word_num");
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(e, "stream synchronize for valid_word_num");
  }
  return BT_OK;
}

extern "C" int bt_publish_int(const int *src, int *dst, void *stream) {
  BT_REQUIRE(src && dst, BT_ERR_INVALID_ARGUMENT, "bt_publish_int: null pointer argument");
  publish_int_kernel<<<1, kWave, 0, as_stream(stream)>>>(src, dst);
  BT_CHECK_LAUNCH("publish_int_kernel");
  return BT_OK;
}

extern "C" int bt_layer_prologue(const void *atten_mask, int mask_dtype, int batch_size,
                                 int seq_len, int *batch_idx, int *word_idx, int *seq_order,
                                 int *mask_prefix_slots, void *attention_work_list, int head_num,
                                 int padded_rows, int weight_count, const void *const *w,
                                 void *const *wt, const int *k, const int *n, int warm_count,
                                 const void *const *warm, const unsigned long long *warm_bytes,
                                 void *stream) {
  BT_REQUIRE(atten_mask && batch_idx && word_idx, BT_ERR_INVALID_ARGUMENT,
             "bt_layer_prologue: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_layer_prologue: batch_size=%d seq_len=%d must be positive", batch_size, seq_len);
  BT_REQUIRE(mask_dtype == BT_F16 || mask_dtype == BT_F32, BT_ERR_INVALID_ARGUMENT,
             "bt_layer_prologue: unknown mask dtype %d", mask_dtype);
  BT_REQUIRE((long long)batch_size * seq_len < (1ll << 31), BT_ERR_UNSUPPORTED,
             "bt_layer_prologue: batch_size*seq_len overflows int32");
  WeightJobs pw;
  const int rc_jobs = make_weight_jobs("bt_layer_prologue", &pw, weight_count, w, wt, k, n,
                                       warm_count, warm, warm_bytes);
  if (rc_jobs != BT_OK) return rc_jobs;
  const bool warming = pw.warm_end[3] > 0;
  // the attention's balanced work list, when a launch of this shape uses one
  PrologueList pl;
  memset(&pl, 0, sizeof(pl));
  if (attention_work_list) {
    BT_REQUIRE(head_num > 0, BT_ERR_INVALID_ARGUMENT,
               "bt_layer_prologue: attention_work_list needs head_num");
    BT_REQUIRE(aligned16({attention_work_list}), BT_ERR_INVALID_ARGUMENT,
               "bt_layer_prologue: attention_work_list must be 16-byte aligned");
    const AttListPlan plan = att_worklist_plan(batch_size, seq_len, head_num);
    if (plan.entries > 0) {
      pl.list = (int4 *)attention_work_list;
      pl.entries = plan.entries;
      pl.bq = plan.bq;
      pl.nqb = plan.nqb;
      pl.heads = head_num;
      pl.padded_rows = padded_rows;
    }
  }
  size_t smem = (3 * (size_t)batch_size + 1) * sizeof(int);
  const size_t pack = (size_t)kPackGroups * 64 * kTransposePitch * sizeof(half_t);
  if (weight_count > 0 && smem < pack) smem = pack;
  BT_REQUIRE(smem <= 60 * 1024, BT_ERR_UNSUPPORTED,
             "bt_layer_prologue: batch_size %d too large (limit 5119)", batch_size);
  hipStream_t s = as_stream(stream);
  const int offset_blocks = batch_size < 64 ? batch_size : 64;
  // the verdict slots are an array of kPrefixBlocks entries, one per block; the
  // pre-pack blocks are the last kPackBlocks of the same grid
  static_assert(kPackFirst + kPackBlocks == kPrefixBlocks, "one grid for both jobs");
  const int grid = ((mask_prefix_slots || weight_count > 0 || warming) ? kPrefixBlocks : offset_blocks) +
                   (pl.list ? kListBlocks : 0);
  if (mask_dtype == BT_F16)
    layer_prologue_kernel<half_t><<<grid, kPrologueThreads, smem, s>>>(
        (const half_t *)atten_mask, batch_idx, word_idx, seq_order, mask_prefix_slots, batch_size,
        seq_len, offset_blocks, pw, pl);
  else
    layer_prologue_kernel<float><<<grid, kPrologueThreads, smem, s>>>(
        (const float *)atten_mask, batch_idx, word_idx, seq_order, mask_prefix_slots, batch_size,
        seq_len, offset_blocks, pw, pl);
  BT_CHECK_LAUNCH("layer_prologue_kernel");
  return BT_OK;
}

extern "C" int bt_mask_prefix_slots(const void *atten_mask, int mask_dtype, int batch_size,
                                    int seq_len, const int *batch_idx, int *slots, void *stream) {
  BT_REQUIRE(atten_mask && batch_idx && slots, BT_ERR_INVALID_ARGUMENT,
             "bt_mask_prefix_slots: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_mask_prefix_slots: batch_size=%d seq_len=%d must be positive", batch_size,
             seq_len);
  BT_REQUIRE(mask_dtype == BT_F16 || mask_dtype == BT_F32, BT_ERR_INVALID_ARGUMENT,
             "bt_mask_prefix_slots: unknown mask dtype %d", mask_dtype);
  BT_REQUIRE((long long)batch_size * seq_len < (1ll << 31), BT_ERR_UNSUPPORTED,
             "bt_mask_prefix_slots: too many rows");
  hipStream_t s = as_stream(stream);
  // always all 256 workgroups: one without rows reports "nothing wrong"
  if (mask_dtype == BT_F16)
    mask_prefix_kernel<half_t><<<kPrefixBlocks, kPrefixWaves * kWave, 0, s>>>(
        (const half_t *)atten_mask, batch_idx, slots, batch_size, seq_len);
  else
    mask_prefix_kernel<float><<<kPrefixBlocks, kPrefixWaves * kWave, 0, s>>>(
        (const float *)atten_mask, batch_idx, slots, batch_size, seq_len);
  BT_CHECK_LAUNCH("mask_prefix_kernel");
  return BT_OK;
}

extern "C" int bt_mask_is_prefix(const void *atten_mask, int mask_dtype, int batch_size,
                                 int seq_len, const int *batch_idx, int *scratch,
                                 int *is_prefix_host, void *stream) {
  BT_REQUIRE(is_prefix_host, BT_ERR_INVALID_ARGUMENT, "bt_mask_is_prefix: null pointer argument");
  const int rc = bt_mask_prefix_slots(atten_mask, mask_dtype, batch_size, seq_len, batch_idx,
                                      scratch, stream);
  if (rc != BT_OK) return rc;
  hipStream_t s = as_stream(stream);
  int slots[kPrefixBlocks];
  hipError_t e = hipMemcpyAsync(slots, scratch, sizeof(slots), hipMemcpyDeviceToHost, s);
  if (e != hipSuccess) return hip_fail(e, "copy of the prefix-mask verdict");
  e = hipStreamSynchronize(s);
  if (e != hipSuccess) return hip_fail(e, "stream synchronize for the prefix-mask verdict");
  int all = 1;
  for (int i = 0; i < kPrefixBlocks; ++i) all &= slots[i] != 0;
  *is_prefix_host = all;
  return BT_OK;
}

extern "C" int bt_compress(const void *from_tensor, void *to_tensor, const int *batch_idx,
                           const int *word_idx, int batch_size, int seq_len, int hidden_dim,
                           void *stream) {
  BT_REQUIRE(from_tensor && to_tensor && batch_idx && word_idx, BT_ERR_INVALID_ARGUMENT,
             "bt_compress: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0 && hidden_dim > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_compress: sizes must be positive");
  BT_REQUIRE(hidden_dim % 8 == 0, BT_ERR_UNSUPPORTED,
             "bt_compress: hidden_dim %d must be a multiple of 8", hidden_dim);
  BT_REQUIRE(aligned16({from_tensor, to_tensor}), BT_ERR_INVALID_ARGUMENT,
             "bt_compress: tensor pointers must be 16-byte aligned");
  const long long rows = (long long)batch_size * seq_len;
  BT_REQUIRE(rows < (1ll << 31), BT_ERR_UNSUPPORTED, "bt_compress: too many rows");
  const int grid = (int)((rows + kRowsPerBlock - 1) / kRowsPerBlock);
  compress_kernel<<<grid, kRowsPerBlock * kWave, 0, as_stream(stream)>>>(
      (const uint4_t *)from_tensor, (uint4_t *)to_tensor, batch_idx, word_idx, batch_size,
      hidden_dim / 8);
  BT_CHECK_LAUNCH("compress_kernel");
  return BT_OK;
}
