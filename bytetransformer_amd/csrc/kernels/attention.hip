// Fused multi-head attention for gfx950 over head-major Q/K/V
// ([3][heads][rows_cap][64], fp16), one workgroup per (query tile, head,
// sequence), wave64 + v_mfma_f32_16x16x32_f16.
//
// Both kernels compute the logits TRANSPOSED, S^T = K.Q^T, so that the MFMA
// accumulator of a 16-key block (lane = query, 4 consecutive keys per lane) is
// already laid out as the "B" operand of the second product O^T = V^T.P^T: the
// probabilities never leave registers.  K and V rows travel global -> LDS with
// direct-to-LDS 16-byte loads (no staging registers) into XOR-swizzled
// row-major tiles; the "A" operand of the second product, V^T, is fetched with
// the LDS transpose read (ds_read_b64_tr_b16), so V is never transposed in
// memory.
//
//   attention_short_kernel    whole K / V of the sequence resident in LDS,
//                             all logits of a query tile in registers, exact
//                             two-pass softmax: P = exp(s-max)/(sum+1e-6) is
//                             rounded to fp16 before P.V exactly as
//                             attention_fused.cu:348-381 does.
//   attention_grouped_kernel  K / V streamed in 64-key tiles through a 2- or 3-stage
//                             LDS ring with an online softmax; handles any
//                             length; the [S, S] logits never exist.
//
// Keys at or past the sequence length are excluded by index (the mask tensor is
// not read), the convention of the reference's remove-padding kernels
// (attention_fused.cu:359, attention_fused_long.cu:254).  Tile rows past the
// length are fetched from the last valid row (finite data, never out of
// bounds) and their probabilities are forced to zero.
#include "common.h"

#include <type_traits>

namespace bt {

constexpr int kAttThreads = 256;
constexpr int kHeadDim = 64;
constexpr float kNegBig = -1.0e30f;
constexpr float kLog2e = 1.4426950408889634f;

typedef float float2_t __attribute__((ext_vector_type(2)));

constexpr int kPrefetchRanges = 4;

struct AttArgs {
  const half_t *qkv;   // [3][heads][rows_cap][64]
  half_t *out;         // [rows, heads*64]
  const int *batch_idx;
  const int *seq_order;   // optional: grid z -> sequence, longest first (null = identity)
  const half_t *mask;     // optional [B,S,S] 0/1 mask, padded rows only: every key of the
                          // sequence's S rows takes part, shifted by (mask-1)*10000
  const half_t *bias;     // optional [heads,S,S] term added to the scaled logits
  // optional: up to kPrefetchRanges ranges that the NEXT kernels will read (weights),
  // touched line by line so they sit in the memory-side cache: range r holds the 128-byte
  // lines [pf_end[r - 1], pf_end[r]) of their concatenation (pf_end[last] = 0: none)
  const char *pf_base[kPrefetchRanges];
  unsigned pf_end[kPrefetchRanges];
  int B, S, rows_cap, heads;
  float scale_log2e;   // scale * log2(e)
  int padded_rows;
  int nqb;             // query tiles per sequence (set by the launcher)
  unsigned nqb_grid;   // host only: workgroups of the launch
  int xcd_map;         // 0: plain (tile, head, sequence) order, 1: XCD-aware, 2: XCD-aware and balanced over the CUs
  const int *mask_ok;  // optional int[256] from bt_mask_prefix_slots: all non-zero = the mask
                       // is the plain prefix mask of the lengths, and is then ignored
  const int4 *work_list;   // optional: entry w of bt_attention_worklist = what workgroup w of the
                           // balanced order works on {sequence or -1, head | tile << 16, first row, length}
};

// Which (sequence rank, head, query tile) a workgroup of the 1-D grid works on.  The
// hardware deals consecutive workgroup ids round-robin to the 8 XCDs.  In a plain
// (tile fastest) order the XCD of a workgroup is a function of its query-tile index, and
// with ragged lengths the high tiles are mostly dead: some XCDs get a fraction of the
// work of others.  The XCD-aware order gives XCD x the (sequence, head) pairs
// p = x (mod 8) - pairs counted sequence-major over the longest-first order, so every
// XCD sees the same mix of lengths - and runs the query tiles of one pair back to back
// on that XCD, whose L2 then serves the pair's K / V to all of them.
struct AttItem {
  int rank, head, qb;
  bool exists;
};
__device__ __forceinline__ AttItem att_item(const AttArgs &p) {
  AttItem it;
  const unsigned lin = blockIdx.x;
  if (p.xcd_map) {
    const unsigned slot = lin >> 3, pair = (slot / p.nqb) * 8 + (lin & 7);
    it.qb = slot % p.nqb;
    it.exists = pair < (unsigned)(p.B * p.heads);
    it.rank = pair / p.heads;
    it.head = pair % p.heads;
  } else {
    it.qb = lin % p.nqb;
    it.head = (lin / p.nqb) % p.heads;
    it.rank = lin / (p.nqb * p.heads);
    it.exists = true;
  }
  return it;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Reductions over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48) with the
// row-swap VALU instructions: after a swap of two copies of x, the pair holds x of
// rows {0,0,2,2} / {1,1,3,3} (16-lane swap) or {0,1,0,1} / {2,3,2,3} (32-lane swap),
// so one max / add per step folds the partner row in - no LDS round trip.  The empty
// asm keeps the optimiser from treating the two results of a swap of equal inputs as
// equal (it then drops the max / add).
__device__ __forceinline__ void swap_rows16(float x, float &lo, float &hi) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  unsigned r0 = r[0], r1 = r[1];
  asm volatile("" : "+v"(r0), "+v"(r1));
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ void swap_rows32(float x, float &lo, float &hi) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  unsigned r0 = r[0], r1 = r[1];
  asm volatile("" : "+v"(r0), "+v"(r1));
  lo = __builtin_bit_cast(float, r0);
  hi = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float rows_max(float x) {
  float a, b;
  swap_rows16(x, a, b);
  swap_rows32(fmaxf(a, b), a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float rows_sum(float x) {
  float a, b;
  swap_rows16(x, a, b);
  swap_rows32(a + b, a, b);
  return a + b;
}

// Cache warm-up on behalf of later kernels: the workgroups of the last quarter of the
// issue order (short sequences and dead tiles, which retire early) each touch one
// dword per 128-byte line of their slice of the ranges.  The loads are the wave's last
// instructions; nothing reads their results.
__device__ __forceinline__ void prefetch_slice(const AttArgs &p) {
  const unsigned lines = p.pf_end[kPrefetchRanges - 1];
  if (!lines) return;
  const unsigned z0 = (unsigned)((unsigned long long)gridDim.x * 3 / 4);
  if (blockIdx.x < z0) return;
  const unsigned duty = gridDim.x - z0;
  const unsigned me = blockIdx.x - z0;
  const unsigned per = (lines + duty - 1) / duty;
  const unsigned first = me * per;
  const unsigned last = first + per < lines ? first + per : lines;
  for (unsigned l = first + threadIdx.x; l < last; l += blockDim.x) {
    const char *base = p.pf_base[0];
    unsigned begin = 0;
#pragma unroll
    for (int r = 1; r < kPrefetchRanges; ++r)
      if (l >= p.pf_end[r - 1]) {
        base = p.pf_base[r];
        begin = p.pf_end[r - 1];
      }
    unsigned sink;
    const char *addr = base + (unsigned long long)(l - begin) * 128;
    asm volatile("global_load_dword %0, %1, off" : "=v"(sink) : "v"(addr) : "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// 16-byte chunk swizzles of a [rows][64] fp16 tile (8 chunks per 128-byte row).
// K is read with ds_read_b128 by 16 consecutive rows at one chunk: slot =
// chunk ^ (row>>1 & 7) spreads them over all 64 banks.  V is read with the
// transpose read, 4 consecutive rows x 32 bytes per 16 lanes: slot =
// chunk ^ 2*(row>>1 & 3) puts those four rows on distinct banks.
__device__ __forceinline__ int swz_k(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz_v(int row) { return ((row >> 1) & 3) << 1; }

template <int N>
__device__ __forceinline__ void att_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

__device__ __forceinline__ void lds_dma16(const half_t *src, half_t *dst) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                   (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
}

// V^T fragment for d-block db and key pair-block kk of a [keys][64] swizzled V
// tile: 8 keys {32kk+4g+r, 32kk+16+4g+r} for d = 16db + (lane&15), g = lane>>4.
__device__ __forceinline__ half8_t load_vt_frag(const half_t *sV, int kk, int db, int lq, int lg) {
  const int row0 = 32 * kk + 4 * lg + (lq >> 2);
  const int c = 2 * db + ((lq & 3) >> 1), sub = 4 * (lq & 1);
  const half_t *p0 = sV + row0 * kHeadDim + ((c ^ swz_v(row0)) << 3) + sub;
  const int row1 = row0 + 16;
  const half_t *p1 = sV + row1 * kHeadDim + ((c ^ swz_v(row1)) << 3) + sub;
  const fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t *)p0);
  const fp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t *)p1);
  const half4_t l4 = __builtin_bit_cast(half4_t, lo), h4 = __builtin_bit_cast(half4_t, hi);
  return half8_t{l4[0], l4[1], l4[2], l4[3], h4[0], h4[1], h4[2], h4[3]};
}

// The same fragment from the address of its first read (a tile's first key pair-block plus
// the lane's own offset): the second read lies 16 rows further on.
__device__ __forceinline__ half8_t load_vt_frag_at(const half_t *p0) {
  const fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t *)p0);
  const fp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t *)(p0 + 16 * kHeadDim));
  const half4_t l4 = __builtin_bit_cast(half4_t, lo), h4 = __builtin_bit_cast(half4_t, hi);
  return half8_t{l4[0], l4[1], l4[2], l4[3], h4[0], h4[1], h4[2], h4[3]};
}

__device__ __forceinline__ half8_t load_k_frag(const half_t *sK, int kb, int dh, int lq, int lg) {
  const int row = 16 * kb + lq;
  return *(const half8_t *)(sK + row * kHeadDim + (((4 * dh + lg) ^ swz_k(row)) << 3));
}

// Additive mask term of four consecutive keys of one query row, in the exp2
// domain: (mask - 1) * 10000 * log2(e)  (the reference's non-remove-padding
// kernels, attention_fused.cu:234-237).  Keys at or past S get no term here; the
// caller excludes them by index.
__device__ __forceinline__ float4_t row4(const half_t *row, int key, int S, bool vec, float fill) {
  float4_t m = {fill, fill, fill, fill};
  if (vec && key + 3 < S) {
    const half4_t h = *(const half4_t *)(row + key);
#pragma unroll
    for (int r = 0; r < 4; ++r) m[r] = (float)h[r];
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (key + r < S) m[r] = (float)row[key + r];
  }
  return m;
}
__device__ __forceinline__ float4_t mask_bias4(const half_t *mask_row, int key, int S, bool vec) {
  constexpr float kShift = 10000.0f * kLog2e;
  return (row4(mask_row, key, S, vec, 1.f) - 1.0f) * kShift;
}
// Additive term of four consecutive keys in the exp2 domain: the mask shift (when a
// mask row is given) plus the attention bias (softmax.h:41-46 adds it to the
// scaled logits before the mask term).
__device__ __forceinline__ float4_t add_terms4(const half_t *mask_row, const half_t *bias_row,
                                               int key, int S, bool vec) {
  float4_t t = {0.f, 0.f, 0.f, 0.f};
  if (mask_row) t = mask_bias4(mask_row, key, S, vec);
  if (bias_row) t += row4(bias_row, key, S, vec, 0.f) * kLog2e;
  return t;
}

// ---------------------------------------------------------------------------
// grouped / streaming kernel
// ---------------------------------------------------------------------------
constexpr int kKT = 64;                          // keys per streamed tile
#ifndef BT_LAZY_MAX
#define BT_LAZY_MAX 8.0f
#endif
constexpr float kLazyMax = BT_LAZY_MAX;          // see the running maximum in the tile loop
constexpr int kTileHalfs = kKT * kHeadDim;       // one K or V tile

// QB 16-query blocks per wave; workgroup covers 4*QB*16 queries.  ADD: a mask tensor and / or an
// attention bias contribute additive terms to the logits.
// KS = 2 (key split): eight waves; waves 4-7 work on the same queries as waves 0-3 but on
// the other 64-key half of every 128-key ring slot, with their own running maximum, sum
// and output, and the two halves are merged through LDS at the end.  The dependency chain
// of a query tile - what bounds a launch of a few workgroups per CU, where the longest
// sequence's workgroups finish last - is half as long, and twice the waves hide it.
template <int QB, bool ADD, int STAGES, int KS = 1>
__global__ __launch_bounds__(kAttThreads * KS, KS == 1 ? 2 : 4) void attention_grouped_kernel(AttArgs p) {
  constexpr int BQ = 4 * QB * 16;
  constexpr int AHEAD = STAGES - 1;     // tiles in flight beyond the one being consumed
  constexpr int kSlotKeys = kKT * KS;   // keys per ring slot
  constexpr int kSlotHalfs = KS * 2 * kTileHalfs;
  static_assert(STAGES == 2 || STAGES == 3, "ring depth");
  static_assert(KS == 1 || KS == 2, "key split");
  __shared__ __attribute__((aligned(1024))) half_t ring[STAGES * kSlotHalfs];

  int b, head, seq_start, seq_len, qb_index;
  if (p.xcd_map == 2 && p.work_list) {
    // the balanced order, looked up by an earlier launch: one scalar load
    const int4 w = p.work_list[blockIdx.x];
    if (w.x < 0) {
      prefetch_slice(p);
      return;
    }
    b = w.x, head = w.y & 0xffff, qb_index = w.y >> 16, seq_start = w.z, seq_len = w.w;
  } else if (p.xcd_map == 2) {
    const AttWork w = att_work_balanced<BQ>(p, blockIdx.x);
    if (!w.exists) {
      prefetch_slice(p);
      return;
    }
    b = w.b, head = w.head, seq_start = w.seq_start, seq_len = w.len, qb_index = w.qb;
  } else {
    const AttItem item = att_item(p);
    if (!item.exists) {
      prefetch_slice(p);
      return;
    }
    b = p.seq_order ? p.seq_order[item.rank] : item.rank, head = item.head;
    if (p.batch_idx) {
      seq_start = p.batch_idx[b];
      seq_len = p.batch_idx[b + 1] - seq_start;
    } else {   // no offsets: padded rows under a mask tensor, which says everything
      seq_start = b * p.S;
      seq_len = p.S;
    }
    qb_index = item.qb;
  }
  // A mask tensor that the device-side check found to be the plain prefix mask adds 0 to
  // the logits of the sequence's keys and removes the others: the lengths say the same.
  const half_t *mask = ADD ? p.mask : nullptr;
  if (ADD && mask && p.mask_ok) {
    const int l = threadIdx.x & 63;
    const int ok = p.mask_ok[l] & p.mask_ok[l + 64] & p.mask_ok[l + 128] & p.mask_ok[l + 192];
    if (__builtin_amdgcn_ballot_w64(ok == 0) == 0) mask = nullptr;
  }
  // with a mask tensor every one of the S key rows takes part
  const int klen = mask ? p.S : seq_len;
  const int row_start = p.padded_rows ? b * p.S : seq_start;
  const int nq = p.padded_rows ? p.S : klen;
  const int q0 = qb_index * BQ;
  if (q0 >= nq) {
    prefetch_slice(p);
    return;
  }

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave = wave_all & 3;        // which 16-query blocks
  const int grp = KS > 1 ? wave_all >> 2 : 0;   // which 64-key half of a ring slot (KS = 2)
  const int lq = lane & 15, lg = lane >> 4;

  const size_t head_stride = (size_t)p.rows_cap * kHeadDim;
  const half_t *Q = p.qkv + (size_t)head * head_stride + (size_t)row_start * kHeadDim;
  const half_t *K = Q + (size_t)p.heads * head_stride;
  const half_t *V = K + (size_t)p.heads * head_stride;

  // Q fragments: "B" operand, lane (query lq, k-group lg) holds d = 32*dh + 8*lg .. +8
  half8_t qf[QB][2];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int q = q0 + (wave * QB + qb) * 16 + lq;
#pragma unroll
    for (int dh = 0; dh < 2; ++dh) {
      uint4_t v = {0u, 0u, 0u, 0u};
      if (q < nq) v = *(const uint4_t *)(Q + (size_t)q * kHeadDim + 32 * dh + 8 * lg);
      qf[qb][dh] = __builtin_bit_cast(half8_t, v);
    }
  }

  // Where this lane's operand fragments sit inside a K or V tile, in halfs: the swizzle
  // term of a fragment's row does not depend on the key block (K: row = 16 kb + lq, V: row
  // = 32 kk + 4 lg + (lq >> 2); the block index drops out of swz_k / swz_v), so the whole
  // address is one of these six lane constants plus a compile-time offset - ring stage,
  // key block - that fits the instruction's immediate field: no address arithmetic is
  // left in the loop over the key tiles (it was a quarter of its vector instructions).
  int koff[2], voff[4];
#pragma unroll
  for (int dh = 0; dh < 2; ++dh) koff[dh] = lq * kHeadDim + (((4 * dh + lg) ^ swz_k(lq)) << 3);
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    const int row0 = 4 * lg + (lq >> 2);
    const int c = 2 * db + ((lq & 3) >> 1);
    voff[db] = row0 * kHeadDim + ((c ^ swz_v(row0)) << 3) + 4 * (lq & 1);
  }

  // Slot copy: 16 load instructions per 64-key tile (8 rows each; 0-7 = K, 8-15 = V),
  // four per wave.  Lane -> (row, slot) and fetches the chunk the swizzle puts
  // in that slot.
  const int ld_row = lane >> 3, ld_slot = lane & 7;
  auto issue_tile = [&](int t, int stage) {
    half_t *sbase = ring + stage * kSlotHalfs;
    const int k0 = t * kSlotKeys;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id_all = i * 4 * KS + wave_all;   // 0 .. 16 KS - 1
      const int sub = id_all >> 4, id = id_all & 15;
      const int row = (id & 7) * 8 + ld_row;
      const int key = min(k0 + sub * kKT + row, klen - 1);
      if (id < 8)
        lds_dma16(K + (size_t)key * kHeadDim + ((ld_slot ^ swz_k(row)) << 3),
                  sbase + sub * 2 * kTileHalfs + (id & 7) * 8 * kHeadDim);
      else
        lds_dma16(V + (size_t)key * kHeadDim + ((ld_slot ^ swz_v(row)) << 3),
                  sbase + sub * 2 * kTileHalfs + kTileHalfs + (id & 7) * 8 * kHeadDim);
    }
  };

  // o[4] is a fifth "d block" fed with an all-ones V^T fragment: the MFMA then
  // accumulates the row sums of the (fp16-rounded) probabilities, already
  // reduced over the wave, in the same rescaled form as O.
  float4_t o[5][QB];
  float m_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = kNegBig;
#pragma unroll
    for (int db = 0; db < 5; ++db) o[db][qb] = float4_t{0.f, 0.f, 0.f, 0.f};
  }
  const half8_t ones = {1, 1, 1, 1, 1, 1, 1, 1};

  const bool wave_live = q0 + wave * QB * 16 < nq;
  const int ntiles = (klen + kSlotKeys - 1) / kSlotKeys;
  if (ntiles > 0) issue_tile(0, 0);
  if (AHEAD > 1 && ntiles > 1) issue_tile(1, 1);

  const float c = p.scale_log2e;
  // after the mask term is folded in, the logits already are in the exp2 domain
  const float cs = ADD ? 1.0f : c;
  const bool mask_vec = (p.S & 3) == 0;

  // ST: the ring stage of tile t, a compile-time constant (the loop below is unrolled over
  // the stages)
  auto process_tile = [&](int t, auto masked_tag, auto stage_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    constexpr int ST = decltype(stage_tag)::value;
    // this wave's share of tile t has landed once only tile t+1's four loads are outstanding
    if (AHEAD > 1 && t + 1 < ntiles)
      att_wait_vmcnt<4>();
    else
      att_wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (t + AHEAD < ntiles) issue_tile(t + AHEAD, (ST + AHEAD) % STAGES);
    // a wave whose queries all lie past the sequence, or whose half of the slot lies past
    // the last key, only copies and keeps the barriers
    const int k0 = t * kSlotKeys + grp * kKT;
    if (!wave_live || (KS > 1 && k0 >= klen)) return;
    const half_t *sK = ring + ST * kSlotHalfs + grp * 2 * kTileHalfs;
    const half_t *sV = sK + kTileHalfs;

    // S^T = K . Q^T for this tile: 4 key blocks x QB query blocks
    float4_t s[4][QB];
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const half8_t kf0 = *(const half8_t *)(sK + kb * 16 * kHeadDim + koff[0]);
      const half8_t kf1 = *(const half8_t *)(sK + kb * 16 * kHeadDim + koff[1]);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        s[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf0, qf[qb][0], zero4, 0, 0, 0);
        s[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf1, qf[qb][1], s[kb][qb], 0, 0, 0);
      }
    }
    if (ADD) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int q = min(q0 + (wave * QB + qb) * 16 + lq, p.S - 1);
        const half_t *mrow = mask ? mask + ((size_t)b * p.S + q) * p.S : nullptr;
        const half_t *brow = p.bias ? p.bias + ((size_t)head * p.S + q) * p.S : nullptr;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
          const float4_t bias = add_terms4(mrow, brow, k0 + kb * 16 + lg * 4, p.S, mask_vec);
#pragma unroll
          for (int r = 0; r < 4; ++r) s[kb][qb][r] = __builtin_fmaf(s[kb][qb][r], c, bias[r]);
        }
      }
    }
    if (MASKED) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const bool dead = k0 + kb * 16 + lg * 4 + r >= klen;
#pragma unroll
          for (int qb = 0; qb < QB; ++qb) s[kb][qb][r] = dead ? kNegBig : s[kb][qb][r];
        }
    }

    half8_t pf[2][QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mx = fmaxf(s[0][qb][0], s[0][qb][1]);
      mx = fmaxf(fmaxf(mx, s[0][qb][2]), s[0][qb][3]);
#pragma unroll
      for (int kb = 1; kb < 4; ++kb) {
        mx = fmaxf(fmaxf(mx, s[kb][qb][0]), s[kb][qb][1]);
        mx = fmaxf(fmaxf(mx, s[kb][qb][2]), s[kb][qb][3]);
      }
      mx = rows_max(mx);
      // The reference point of a query's exponentials follows its maximum lazily: it moves
      // only when the maximum has grown by more than kLazyMax binary orders (the first tile
      // always does).  Probabilities then reach at most 2^kLazyMax - far inside fp16, the
      // sums are fp32 - and the quotient O / l does not depend on the reference point, while
      // the rescaling of the running output, a quarter of the vector work of a tile, is
      // left to the few tiles where a maximum jumps.
      const float m_new = (mx - m_run[qb]) * cs > kLazyMax ? mx : m_run[qb];
      const float mc = m_new * cs;
      if (__builtin_amdgcn_ballot_w64(m_new != m_run[qb]) != 0) {
        const float alpha = fast_exp2(m_run[qb] * cs - mc);
#pragma unroll
        for (int db = 0; db < 5; ++db) o[db][qb] *= alpha;
      }
      m_run[qb] = m_new;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        float e[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) e[r] = fast_exp2(__builtin_fmaf(s[kb][qb][r], cs, -mc));
        const half2_t h01 = __builtin_convertvector(float2_t{e[0], e[1]}, half2_t);
        const half2_t h23 = __builtin_convertvector(float2_t{e[2], e[3]}, half2_t);
        pf[kb >> 1][qb][(kb & 1) * 4 + 0] = h01[0];
        pf[kb >> 1][qb][(kb & 1) * 4 + 1] = h01[1];
        pf[kb >> 1][qb][(kb & 1) * 4 + 2] = h23[0];
        pf[kb >> 1][qb][(kb & 1) * 4 + 3] = h23[1];
      }
    }

    // O^T += V^T . P^T ; k-slot (lg, s) <-> key 32*kk + 16*(s>>2) + 4*lg + (s&3)
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const half8_t vf = load_vt_frag_at(sV + kk * 32 * kHeadDim + voff[db]);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          o[db][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[kk][qb], o[db][qb], 0, 0, 0);
      }
#pragma unroll
      for (int qb = 0; qb < QB; ++qb)
        o[4][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pf[kk][qb], o[4][qb], 0, 0, 0);
    }
  };
  // every tile but the last is full: no masking code on the steady-state path
  const bool ragged_end = klen % kSlotKeys != 0;
  auto step = [&](int t, auto stage_tag) {
    if (ragged_end && t == ntiles - 1)
      process_tile(t, std::true_type{}, stage_tag);
    else
      process_tile(t, std::false_type{}, stage_tag);
  };
  // one turn of the ring per iteration: tile t sits in stage t % STAGES
  for (int t = 0; t < ntiles; t += STAGES) {
    step(t, std::integral_constant<int, 0>{});
    if (t + 1 < ntiles) step(t + 1, std::integral_constant<int, 1>{});
    if constexpr (STAGES == 3) {
      if (t + 2 < ntiles) step(t + 2, std::integral_constant<int, 2>{});
    }
  }

  if (KS > 1) {
    // fold the second key half into the first: waves 4-7 hand over maximum, sum and output
    // through the ring (lane-major, one word per lane and item: no bank conflicts)
    float *xch = (float *)ring + (size_t)wave * (21 * QB) * 64 + lane;
    __syncthreads();           // every wave is done reading the ring
    if (grp == 1) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        xch[(qb * 21 + 20) * 64] = m_run[qb];
#pragma unroll
        for (int db = 0; db < 5; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) xch[(qb * 21 + db * 4 + r) * 64] = o[db][qb][r];
      }
    }
    __syncthreads();
    if (grp == 1) {
      prefetch_slice(p);
      return;
    }
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      const float m_other = xch[(qb * 21 + 20) * 64];
      const float m_new = fmaxf(m_run[qb], m_other);
      const float a_mine = fast_exp2((m_run[qb] - m_new) * cs);
      const float a_other = fast_exp2((m_other - m_new) * cs);
#pragma unroll
      for (int db = 0; db < 5; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          o[db][qb][r] = o[db][qb][r] * a_mine + xch[(qb * 21 + db * 4 + r) * 64] * a_other;
    }
  }

  // O / (l + 1e-6) -> fp16, token-major [row][head*64 + d]
  const int H = p.heads * kHeadDim;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float inv = __builtin_amdgcn_rcpf(o[4][qb][0] + 1e-6f);
    const int q = q0 + (wave * QB + qb) * 16 + lq;
    if (q >= nq) continue;
    half_t *dst = p.out + (size_t)(row_start + q) * H + head * kHeadDim + 4 * lg;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      const float4_t v = o[db][qb] * inv;
      *(half4_t *)(dst + 16 * db) = half4_t{(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
    }
  }
  prefetch_slice(p);
}

// The balanced order of a launch of `entries` workgroups as a list: one wave per entry.
template <int BQ>
__global__ __launch_bounds__(kAttThreads) void attention_worklist_kernel(AttArgs p, int4 *list,
                                                                        unsigned entries) {
  const unsigned e = blockIdx.x * (kAttThreads / 64) + (threadIdx.x >> 6);
  if (e >= entries) return;
  const AttWork w = att_work_balanced<BQ>(p, e);
  if ((threadIdx.x & 63) == 0)
    list[e] = w.exists ? int4{w.b, w.head | (w.qb << 16), w.seq_start, w.len} : int4{-1, 0, 0, 0};
}

// ---------------------------------------------------------------------------
// short kernel: K, V resident in LDS, logits of the query tile in registers
// ---------------------------------------------------------------------------
template <int NKB, bool ADD>  // capacity in 16-key blocks (keys <= 16*NKB), NKB even; ADD as above
__global__ __launch_bounds__(kAttThreads) void attention_short_kernel(AttArgs p) {
  constexpr int KEYS = NKB * 16;
  constexpr int BQ = 64;  // 4 waves x 16 queries
  extern __shared__ __attribute__((aligned(1024))) half_t att_smem[];
  half_t *sK = att_smem;                      // [KEYS][64] swizzled
  half_t *sV = att_smem + KEYS * kHeadDim;    // [KEYS][64] swizzled

  const AttItem item = att_item(p);
  if (!item.exists) {
    prefetch_slice(p);
    return;
  }
  const int b = p.seq_order ? p.seq_order[item.rank] : item.rank, head = item.head;
  const int seq_start = p.batch_idx[b];
  const int klen = ADD && p.mask ? p.S : p.batch_idx[b + 1] - seq_start;
  const int row_start = p.padded_rows ? b * p.S : seq_start;
  const int nq = p.padded_rows ? p.S : klen;
  const int q0 = item.qb * BQ;
  if (q0 >= nq) {
    prefetch_slice(p);
    return;
  }

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lq = lane & 15, lg = lane >> 4;
  const int H = p.heads * kHeadDim;
  const int q = q0 + wave * 16 + lq;

  const size_t head_stride = (size_t)p.rows_cap * kHeadDim;
  const half_t *Q = p.qkv + (size_t)head * head_stride + (size_t)row_start * kHeadDim;
  const half_t *K = Q + (size_t)p.heads * head_stride;
  const half_t *V = K + (size_t)p.heads * head_stride;

  // copy K and V rows [0, keys32) into LDS, 8 rows per wave instruction
  const int keys32 = min(((klen + 31) >> 5) << 5, KEYS);
  if (klen > 0) {
    const int ld_row = lane >> 3, ld_slot = lane & 7;
    for (int g8 = wave; g8 < keys32 / 8; g8 += 4) {
      const int row = g8 * 8 + ld_row;
      const int key = min(row, klen - 1);
      lds_dma16(K + (size_t)key * kHeadDim + ((ld_slot ^ swz_k(row)) << 3),
                sK + g8 * 8 * kHeadDim);
      lds_dma16(V + (size_t)key * kHeadDim + ((ld_slot ^ swz_v(row)) << 3),
                sV + g8 * 8 * kHeadDim);
    }
  }
  half8_t qf[2];
#pragma unroll
  for (int dh = 0; dh < 2; ++dh) {
    uint4_t v = {0u, 0u, 0u, 0u};
    if (q < nq) v = *(const uint4_t *)(Q + (size_t)q * kHeadDim + 32 * dh + 8 * lg);
    qf[dh] = __builtin_bit_cast(half8_t, v);
  }
  att_wait_vmcnt<0>();
  asm volatile("" ::: "memory");
  __syncthreads();
  // no barrier follows: a wave whose 16 queries all lie past the sequence is done
  if (q0 + wave * 16 >= nq) {
    prefetch_slice(p);
    return;
  }

  const int nkb = keys32 >> 4;  // even
  float4_t s[NKB];
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb) {
    s[kb] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (kb < nkb) {
#pragma unroll
      for (int dh = 0; dh < 2; ++dh)
        s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(load_k_frag(sK, kb, dh, lq, lg), qf[dh],
                                                       s[kb], 0, 0, 0);
    }
  }

  const float c = p.scale_log2e;
  const float cs = ADD ? 1.0f : c;
  if (ADD) {
    const int qc = min(q, p.S - 1);
    const half_t *mrow = p.mask ? p.mask + ((size_t)b * p.S + qc) * p.S : nullptr;
    const half_t *brow = p.bias ? p.bias + ((size_t)head * p.S + qc) * p.S : nullptr;
    const bool mask_vec = (p.S & 3) == 0;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      const float4_t bias = add_terms4(mrow, brow, kb * 16 + lg * 4, p.S, mask_vec);
#pragma unroll
      for (int r = 0; r < 4; ++r) s[kb][r] = __builtin_fmaf(s[kb][r], c, bias[r]);
    }
  }
  // exact softmax over the row: mask by index, max, exp, sum, normalise, round
  float mx = kNegBig;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (kb * 16 + lg * 4 + r >= klen) s[kb][r] = kNegBig;
      mx = fmaxf(mx, s[kb][r]);
    }
  mx = rows_max(mx);
  const float mc = mx * cs;
  float sum = 0.f;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s[kb][r] = fast_exp2(__builtin_fmaf(s[kb][r], cs, -mc));
      sum += s[kb][r];
    }
  sum = rows_sum(sum);
  const float inv = 1.0f / (sum + 1e-6f);

  float4_t o[4];
#pragma unroll
  for (int db = 0; db < 4; ++db) o[db] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int kk = 0; kk < NKB / 2; ++kk) {
    if (2 * kk < nkb) {
      half8_t pf;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pf[r] = (half_t)(s[2 * kk][r] * inv);
        pf[4 + r] = (half_t)(s[2 * kk + 1][r] * inv);
      }
#pragma unroll
      for (int db = 0; db < 4; ++db)
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(load_vt_frag(sV, kk, db, lq, lg), pf, o[db],
                                                       0, 0, 0);
    }
  }

  if (q < nq) {
    half_t *dst_row = p.out + (size_t)(row_start + q) * H + head * kHeadDim + 4 * lg;
#pragma unroll
    for (int db = 0; db < 4; ++db)
      *(half4_t *)(dst_row + 16 * db) =
          half4_t{(half_t)o[db][0], (half_t)o[db][1], (half_t)o[db][2], (half_t)o[db][3]};
  }
  prefetch_slice(p);
}

// The warm-up pays when the attention kernel runs long enough to hide it: measured
// a gain of 4-6 % per forward with >= 2 workgroups per CU (batch 16 at 512 tokens
// and up) and a loss of 2-3 % with smaller grids, which therefore skip it.  Each
// duty workgroup (last quarter of the issue order; a half measured 0.7 % slower) touches at most four
// lines per thread; the range is cut to that.
static int set_prefetch(AttArgs &a, unsigned grid, const void *const *prefetch,
                        const unsigned long long *bytes, int count) {
  for (int r = 0; r < kPrefetchRanges; ++r) {
    a.pf_base[r] = nullptr;
    a.pf_end[r] = 0;
  }
  BT_REQUIRE(count >= 0 && count <= kPrefetchRanges, BT_ERR_INVALID_ARGUMENT,
             "attention: prefetch_count=%d outside [0, %d]", count, kPrefetchRanges);
  BT_REQUIRE(count == 0 || (prefetch && bytes), BT_ERR_INVALID_ARGUMENT,
             "attention: prefetch ranges need their pointers and sizes");
  if (!count || !option_prefetch()) return BT_OK;
  if (grid < (unsigned)option_prefetch_min_grid()) return BT_OK;
  const unsigned long long duty = grid - (unsigned long long)grid * 3 / 4;
  unsigned long long left = duty * 4 * kAttThreads;   // lines the duty workgroups take on
  unsigned end = 0;
  for (int r = 0; r < kPrefetchRanges; ++r) {
    if (r < count && prefetch[r] && left) {
      // one dword at the start of each 128-byte line; a last line of fewer than four bytes
      // is left alone, so no byte outside the range is read
      unsigned long long lines = (bytes[r] + 124) / 128;
      if (lines > left) lines = left;
      left -= lines;
      a.pf_base[r] = (const char *)prefetch[r];
      end += (unsigned)lines;
    }
    a.pf_end[r] = end;
  }
  return BT_OK;
}

// Size of the 1-D grid for `nqb` query tiles per sequence; fills the mapping fields.
static unsigned att_grid(AttArgs &a, int nqb, bool streaming = false) {
  a.nqb = nqb;
  a.xcd_map = option_attention_xcd_map();
  const unsigned pairs = (unsigned)a.B * a.heads;
  // The balanced list is the streaming kernel's, and pays from the third round of 32
  // workgroups per XCD on: up to two rounds its look-up (vector loads and a wave scan
  // where the plain order needs three scalar loads) cost 0.3-1.5 % per forward.
  // Its look-up takes one pass (two dependent loads) per 64 sequences: beyond 128 the
  // plain order stays, and so many sequences even out by themselves.
  if (a.xcd_map == 2 && ((pairs + 7) / 8 * nqb <= 64 || a.B > 128)) a.xcd_map = 1;
  if (a.xcd_map == 3) a.xcd_map = 2;   // option value 3: the balanced list at any size
  if (a.xcd_map == 2 && !streaming) a.xcd_map = 1;
  if (a.xcd_map == 2) return ((pairs + 7) / 8 * nqb + 31) / 32 * 32 * 8;   // whole rounds of 32 per XCD
  return a.xcd_map ? (pairs + 7) / 8 * 8 * nqb : pairs * nqb;
}

static int check_att_args(const char *who, const void *qkv, const void *out, const int *batch_idx,
                          const void *mask, int padded_rows, int B, int S, int rows_cap,
                          int heads, int d) {
  BT_REQUIRE(!mask || padded_rows, BT_ERR_INVALID_ARGUMENT,
             "%s: atten_mask is only applied on padded rows (padded_rows != 0)", who);
  BT_REQUIRE(qkv && out && batch_idx, BT_ERR_INVALID_ARGUMENT, "%s: null pointer argument", who);
  BT_REQUIRE(aligned16({qkv, out, mask}), BT_ERR_INVALID_ARGUMENT,
             "%s: tensor pointers must be 16-byte aligned", who);
  BT_REQUIRE(B > 0 && S > 0 && heads > 0 && rows_cap > 0, BT_ERR_INVALID_ARGUMENT,
             "%s: batch_size=%d seq_len=%d head_num=%d rows_cap=%d must be positive", who, B, S,
             heads, rows_cap);
  BT_REQUIRE(d == kHeadDim, BT_ERR_UNSUPPORTED, "%s: size_per_head=%d, only 64 is supported", who,
             d);
  BT_REQUIRE(B <= 65535 && heads <= 65535, BT_ERR_UNSUPPORTED, "%s: grid too large", who);
  return BT_OK;
}

template <int NKB, bool ADD>
static int launch_short_impl(const AttArgs &a, hipStream_t s) {
  constexpr size_t smem = (size_t)2 * NKB * 16 * kHeadDim * sizeof(half_t);
  static_assert(smem <= 160 * 1024, "LDS budget");
  static std::atomic<bool> configured[kMaxDevices];
  const int rc = allow_dynamic_lds(attention_short_kernel<NKB, ADD>, smem, configured,
                                   "hipFuncSetAttribute(attention_short_kernel)");
  if (rc != BT_OK) return rc;
  attention_short_kernel<NKB, ADD><<<a.nqb_grid, kAttThreads, smem, s>>>(a);
  BT_CHECK_LAUNCH("attention_short_kernel");
  return BT_OK;
}

template <int NKB>
static int launch_short(const AttArgs &a, hipStream_t s) {
  return a.mask || a.bias ? launch_short_impl<NKB, true>(a, s) : launch_short_impl<NKB, false>(a, s);
}

}  // namespace bt

using namespace bt;

extern "C" int bt_attention_short(const void *qkv_heads, void *attention_output,
                                  const int *batch_idx, const int *seq_order,
                                  const void *atten_mask, const void *attention_bias,
                                  int batch_size, int seq_len, int rows_cap, int head_num,
                                  int size_per_head, float scale, int padded_rows,
                                  const void *const *prefetch,
                                  const unsigned long long *prefetch_bytes, int prefetch_count,
                                  void *stream) {
  int rc = check_att_args("bt_attention_short", qkv_heads, attention_output, batch_idx, atten_mask,
                          padded_rows, batch_size, seq_len, rows_cap, head_num, size_per_head);
  if (rc) return rc;
  BT_REQUIRE(seq_len <= 512, BT_ERR_UNSUPPORTED,
             "bt_attention_short: seq_len=%d exceeds 512, use bt_attention_grouped", seq_len);
  AttArgs a{(const half_t *)qkv_heads, (half_t *)attention_output, batch_idx, seq_order,
            (const half_t *)atten_mask, (const half_t *)attention_bias,
            {}, {}, batch_size, seq_len,
            rows_cap, head_num, scale * kLog2e, padded_rows};
  hipStream_t s = as_stream(stream);
  a.nqb_grid = att_grid(a, (seq_len + 63) / 64);
  rc = set_prefetch(a, a.nqb_grid, prefetch, prefetch_bytes, prefetch_count);
  if (rc) return rc;
  if (seq_len <= 64) return launch_short<4>(a, s);
  if (seq_len <= 128) return launch_short<8>(a, s);
  if (seq_len <= 256) return launch_short<16>(a, s);
  if (seq_len <= 384) return launch_short<24>(a, s);
  return launch_short<32>(a, s);
}

namespace bt {
// Shape of a streaming-attention launch: 128-query tiles with a three-deep ring once there
// is plenty of work (three workgroups per CU); else 64-query tiles with a two-deep ring: 32 KB
// of LDS and ~100 registers let four workgroups share a CU (a build held to 84 registers fits
// five and measures the same), which hides more of the per-tile dependency chain than the
// third stage did (-0.1 to -2.8 % per forward from batch 1 x 256 to batch 16 x 384; with the
// balanced work list also -0.8 to -1.9 % at batch 32 x 256 / 384 and 16 x 768, so the switch
// sits at 1300 workgroups of 128 queries; batch 16 x 512 is within 0.3 % either way).
struct GroupedPlan {
  bool wide;        // 128-query tiles
  unsigned grid;
};
static GroupedPlan plan_grouped(AttArgs &a, int batch_size, int seq_len, int head_num) {
  const long long blocks128 = (long long)((seq_len + 127) / 128) * head_num * batch_size;
  const int qb = option_attention_qb();
  GroupedPlan plan;
  plan.wide = qb == 2 || (qb < 0 && blocks128 >= 1300);
  plan.grid = att_grid(a, plan.wide ? (seq_len + 127) / 128 : (seq_len + 63) / 64, true);
  return plan;
}
AttListPlan att_worklist_plan(int B, int S, int heads) {
  AttListPlan out{0, 64, 0};
  if (B <= 0 || S <= 0 || heads <= 0) return out;
  AttArgs a{};
  a.B = B, a.S = S, a.heads = heads;
  const GroupedPlan plan = plan_grouped(a, B, S, heads);
  out.bq = plan.wide ? 128 : 64;
  out.nqb = a.nqb;
  out.entries = a.xcd_map == 2 ? plan.grid : 0;
  return out;
}
}  // namespace bt

extern "C" unsigned long long bt_attention_worklist_bytes(int batch_size, int seq_len,
                                                          int head_num) {
  return (unsigned long long)att_worklist_plan(batch_size, seq_len, head_num).entries *
         sizeof(int4);
}

extern "C" int bt_attention_worklist(const int *batch_idx, const int *seq_order, int batch_size,
                                     int seq_len, int head_num, int padded_rows, void *work_list,
                                     void *stream) {
  BT_REQUIRE(batch_idx && work_list, BT_ERR_INVALID_ARGUMENT,
             "bt_attention_worklist: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0 && head_num > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_attention_worklist: sizes must be positive");
  BT_REQUIRE(aligned16({work_list}), BT_ERR_INVALID_ARGUMENT,
             "bt_attention_worklist: work_list must be 16-byte aligned");
  AttArgs a{};
  a.batch_idx = batch_idx, a.seq_order = seq_order;
  a.B = batch_size, a.S = seq_len, a.heads = head_num, a.padded_rows = padded_rows;
  const GroupedPlan plan = plan_grouped(a, batch_size, seq_len, head_num);
  BT_REQUIRE(a.xcd_map == 2, BT_ERR_INVALID_ARGUMENT,
             "bt_attention_worklist: launches of this shape take no work list "
             "(bt_attention_worklist_bytes is 0)");
  const unsigned blocks = (plan.grid + kAttThreads / 64 - 1) / (kAttThreads / 64);
  if (plan.wide)
    attention_worklist_kernel<128><<<blocks, kAttThreads, 0, as_stream(stream)>>>(
        a, (int4 *)work_list, plan.grid);
  else
    attention_worklist_kernel<64><<<blocks, kAttThreads, 0, as_stream(stream)>>>(
        a, (int4 *)work_list, plan.grid);
  BT_CHECK_LAUNCH("attention_worklist_kernel");
  return BT_OK;
}

extern "C" int bt_attention_grouped(const void *qkv_heads, void *attention_output,
                                    const int *batch_idx, const int *seq_order,
                                    const void *atten_mask, const void *attention_bias,
                                    int batch_size, int seq_len, int rows_cap, int head_num,
                                    int size_per_head, float scale, int padded_rows,
                                    const void *const *prefetch,
                                    const unsigned long long *prefetch_bytes, int prefetch_count,
                                    const int *mask_prefix_slots, const void *work_list,
                                    void *stream) {
  // without offsets: only where nothing would read them (padded rows, the mask tensor
  // applied element by element, no verdict that could drop it, no balanced order)
  const bool no_offsets = !batch_idx && padded_rows && atten_mask && !mask_prefix_slots;
  int rc = check_att_args("bt_attention_grouped", qkv_heads, attention_output,
                          no_offsets ? (const int *)qkv_heads : batch_idx, atten_mask,
                          padded_rows, batch_size, seq_len, rows_cap, head_num, size_per_head);
  if (rc) return rc;
  BT_REQUIRE(aligned16({work_list}), BT_ERR_INVALID_ARGUMENT,
             "bt_attention_grouped: work_list must be 16-byte aligned");
  if (no_offsets) seq_order = nullptr;
  AttArgs a{(const half_t *)qkv_heads, (half_t *)attention_output, batch_idx, seq_order,
            (const half_t *)atten_mask, (const half_t *)attention_bias,
            {}, {}, batch_size, seq_len,
            rows_cap, head_num, scale * kLog2e, padded_rows};
  a.mask_ok = a.mask ? mask_prefix_slots : nullptr;
  a.work_list = (const int4 *)work_list;   // read only when the launch uses the balanced order
  hipStream_t s = as_stream(stream);
  const bool add = a.mask || a.bias;
  GroupedPlan plan = plan_grouped(a, batch_size, seq_len, head_num);
  if (no_offsets && a.xcd_map == 2) {   // the balanced order ranks the sequences by length
    a.xcd_map = 1;
    plan.grid = ((unsigned)batch_size * head_num + 7) / 8 * 8 * a.nqb;
  }
  const unsigned grid = plan.grid;
  rc = set_prefetch(a, grid, prefetch, prefetch_bytes, prefetch_count);
  if (rc) return rc;
  if (plan.wide) {
    if (add)
      attention_grouped_kernel<2, true, 3><<<grid, kAttThreads, 0, s>>>(a);
    else
      attention_grouped_kernel<2, false, 3><<<grid, kAttThreads, 0, s>>>(a);
  } else {
    // eight waves over two key halves: pays for a few long sequences that leave most CUs
    // with one workgroup or none (batch 1 x 1024: 9.9 -> 8.7 us); with several workgroups
    // per CU the four-wave form is faster (batch 16 x 512: 16.3 against 19.6 us)
    const int ks = option_attention_key_split();
    if (ks == 1 || (ks < 0 && seq_len >= 512 && grid <= 256)) {
      if (add)
        attention_grouped_kernel<1, true, 2, 2><<<grid, 2 * kAttThreads, 0, s>>>(a);
      else
        attention_grouped_kernel<1, false, 2, 2><<<grid, 2 * kAttThreads, 0, s>>>(a);
    } else if (add) {
      attention_grouped_kernel<1, true, 2><<<grid, kAttThreads, 0, s>>>(a);
    } else {
      attention_grouped_kernel<1, false, 2><<<grid, kAttThreads, 0, s>>>(a);
    }
  }
  BT_CHECK_LAUNCH("attention_grouped_kernel");
  return BT_OK;
}
