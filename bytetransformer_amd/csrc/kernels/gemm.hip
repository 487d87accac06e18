// fp16 MFMA GEMM family for gfx950: C[rows, N] = A[rows, K] . W[K, N] with
// fp32 accumulation and three fused epilogues (plain store, +bias+tanh-GELU,
// +bias with the Q/K/V head split).  A is consumed k-contiguous as stored; W either
// as the row-major [K, N] matrix itself (its LDS tile is read with the LDS transpose
// read) or through the k-contiguous [N, K] pre-pack made by bt_transpose_weights.
//
// Structure of one workgroup (tile BM x BN, BK = 64):
//   * global -> LDS copies are 16-byte buffer loads with an LDS destination: no
//     staging registers, no ds_write; each wave instruction lands 1 KB = 8 tile
//     rows back to back in LDS.  Small tiles give this job to dedicated loader
//     waves so the computing waves' instruction streams hold MFMAs and LDS
//     reads only;
//   * the LDS image is XOR-swizzled on 16-byte chunks (slot = chunk ^ (row>>1 & 7));
//     the swizzle is applied by choosing which global chunk each lane fetches,
//     and makes the ds_read_b128 operand fetches conflict-free on the 64 banks;
//   * a ring of STAGES tiles, one barrier per k-step, vmcnt-counted waits so
//     later stages stay in flight across the barrier;
//   * v_mfma_f32_32x32x16_f16 with the weight tile as the MFMA "A" operand and
//     the activation tile as "B": a lane's accumulator quad holds 4 consecutive
//     output columns of one row; operand fragments are double-buffered across
//     the four k-slices of a tile;
//   * epilogue: bias / GELU on the accumulators, then each wave stages 32 rows
//     at a time through a private LDS tile and writes 16-byte, row-contiguous
//     global stores.
//   * workgroup -> tile order is XCD-aware: hardware deals consecutive
//     workgroup ids round-robin to the 8 XCDs, so id%8 selects a contiguous
//     range of the LIVE tiles (live = those below the device-side row count)
//     and the workgroups sharing an XCD's L2 also share operand panels.
//
// Rows are bounded on the device: the live row count is read from
// `valid_rows`; workgroups beyond the live tiles retire at once.
#include "common.h"

#include <type_traits>

namespace bt {


// kEpiPartial: split-k launch (grid y = split): fp32 partial sums to c32[split][rows_cap][N]
// kEpiBias: + bias, row-major store (the QKV projection of layers whose head size is not 64)
enum Epilogue { kEpiPlain = 0, kEpiBiasGelu = 1, kEpiQkvSplit = 2, kEpiPartial = 3, kEpiBias = 4 };

struct GemmArgs {
  const half_t *a;      // [rows_cap, K]
  const half_t *wt;     // [N, K] (pre-packed), or [K, N] as the layer's weights are stored (w_kn)
  const half_t *bias;   // [N] or null
  half_t *c;            // [rows_cap, N]  (or [3][heads][rows_cap][64] for the QKV split)
  const int *valid_rows;
  const int *a_row_index;   // optional gather: A row r is a[a_row_index[r]] (null = identity)
  int rows_cap, N, K;
  int tiles_n;
  int rows_hint;        // host-side estimate of the live rows (0 = unknown); tile choice only
  float *c32;           // kEpiPartial only: [splits][rows_cap][N]
  int w_kn;             // 1: wt is the row-major [K, N] matrix itself
  // Rows taken straight from the attention mask (the QKV projection of a padding-free
  // layer): A is the padded [mask_B * mask_S, K] tensor, the live rows and their order are
  // what the mask's row lengths say, counted by every workgroup for itself - no launch
  // ahead of the product has to build a row index first.  Workgroup 0 leaves the offsets
  // for the kernels that follow (each pointer may be null).
  const void *mask;     // [mask_B, mask_S, mask_S] or null
  int mask_f32;         // element type: 0 half, 1 float
  int mask_B, mask_S;
  int *out_batch_idx;   // [mask_B + 1]
  int *out_word_idx;    // [mask_B * mask_S]: the complete row map (valid positions, then the padded ones)
  int *out_seq_order;   // [mask_B]
  int tile_grid;        // workgroups of the launch (set by the launcher)
};

// ---- rows from the mask ---------------------------------------------------------
constexpr int kMaskRowsMaxBatch = 64;   // one wave scans the lengths

// Per-lane view of the offsets, the same in every wave: lane l < B holds sequence l.
struct MaskRows {
  int len;     // its length
  int excl;    // its first packed row (lanes >= B: M)
  int delta;   // l * S - excl: padded row = packed row + delta
  int M;       // live rows
};

// All `nwaves` waves of the workgroup take part (one barrier inside).  `s_len`: 64 ints of
// LDS that nothing else writes until every wave has left this function.
__device__ __forceinline__ MaskRows mask_rows_setup(const GemmArgs &p, int wave, int nwaves,
                                                    int lane, int *s_len) {
  const int B = p.mask_B, S = p.mask_S;
  const size_t plane = (size_t)S * S;
  // R rows per wave in flight at a time: two for up to 2 * nwaves sequences (their 16-byte
  // loads cover rows of up to 1024 halfs in one round trip), four beyond
  auto count_rows = [&](auto elem_tag, auto r_tag) {
    using T = decltype(elem_tag);
    constexpr int R = decltype(r_tag)::value;
    const T *m = (const T *)p.mask;
    for (int b0 = wave; b0 < B; b0 += R * nwaves) {
      const T *rows[R];
      int count[R];
#pragma unroll
      for (int r = 0; r < R; ++r)
        rows[r] = b0 + r * nwaves < B ? m + (b0 + r * nwaves) * plane : nullptr;
      wave_row_lengths<T, R>(rows, S, lane, count);
      if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
          if (b0 + r * nwaves < B) s_len[b0 + r * nwaves] = count[r];
      }
    }
  };
  using two = std::integral_constant<int, 2>;
  using four = std::integral_constant<int, 4>;
  if (p.mask_f32) {
    if (B <= 2 * nwaves) count_rows(float{}, two{}); else count_rows(float{}, four{});
  } else {
    if (B <= 2 * nwaves) count_rows(half_t{}, two{}); else count_rows(half_t{}, four{});
  }
  __syncthreads();
  MaskRows mr;
  mr.len = lane < B ? s_len[lane] : 0;
  const int incl = wave_inclusive_sum(mr.len);
  mr.excl = incl - mr.len;
  mr.delta = lane * S - mr.excl;
  mr.M = __builtin_amdgcn_readlane(incl, 63);
  return mr;
}

// Which sequences the packed rows [r0, r1] (0 <= r0 <= r1 < M, wave-uniform) belong to: the
// first one and how many more.  The first packed rows rise with the lane, so the lanes whose
// sequence starts at or before a row form a prefix; the last of them holds the row (empty
// sequences in between start at the same row and lose to it).
struct MaskRowSpan {
  int first, more;
};
__device__ __forceinline__ MaskRowSpan mask_rows_span(const MaskRows &mr, int B, int lane, int r0,
                                                      int r1) {
  const int lo = __popcll(__ballot(lane < B && mr.excl <= r0)) - 1;
  const int hi = __popcll(__ballot(lane < B && mr.excl <= r1)) - 1;
  return MaskRowSpan{lo, hi - lo};
}

// Padded row of packed row r inside such a span.  Every lane of the wave must call it (the
// look-ups read the other lanes' registers).
__device__ __forceinline__ int mask_rows_map(const MaskRows &mr, const MaskRowSpan &sp, int r) {
  int b = sp.first;
  for (int k = 1; k <= sp.more; ++k) b += r >= __builtin_amdgcn_readlane(mr.excl, sp.first + k);
  return r + __shfl(mr.delta, b, 64);
}

// The offsets as the stand-alone launch writes them (padding.hip), by `nthreads` threads
// (whole waves, t = thread index among them) of one workgroup.
__device__ __forceinline__ void mask_rows_write(const GemmArgs &p, const MaskRows &mr, int t,
                                                int nthreads, int lane) {
  const int B = p.mask_B, S = p.mask_S;
  if (t < 64) {   // the first of the writing waves
    if (p.out_batch_idx) {
      if (lane < B) p.out_batch_idx[lane] = mr.excl;
      if (lane == 0) p.out_batch_idx[B] = mr.M;
    }
    if (p.out_seq_order) {
      // sequences by descending length (ties by index): rank by counting
      int rank = 0;
      for (int o = 0; o < B; ++o) {
        const int lo = __shfl(mr.len, o, 64);
        rank += (lo > mr.len) || (lo == mr.len && o < lane);
      }
      if (lane < B) p.out_seq_order[rank] = lane;
    }
  }
  if (p.out_word_idx) {
    for (int b = 0; b < B; ++b) {
      const int off = __shfl(mr.excl, b, 64), len = __shfl(mr.len, b, 64);
      const int pad_at = mr.M + b * S - off;   // the padded positions fill the tail from M on
      for (int i = t; i < S; i += nthreads)
        p.out_word_idx[i < len ? off + i : pad_at + i - len] = b * S + i;
    }
  }
}

__device__ __forceinline__ float gelu_tanh_f32(float x) {
  // 0.5 x (1 + tanh(u)) == x / (1 + exp(-2u)),  u = 0.79788456 (x + 0.044715 x^3)
  // exponent folded into one polynomial: -2 u log2(e) = x (c1 + c3 x^2)
  constexpr float c1 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  constexpr float c3 = c1 * 0.044715f;
  const float e = __builtin_amdgcn_exp2f(x * (c1 + c3 * x * x));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// XOR swizzle of the 16-byte chunk slot inside a 128-byte tile row: rows r and r+1
// differ by half of the 256-byte bank window, so 16 consecutive rows need 8 distinct
// slots.  The 16 lanes that one ds_read_b128 pass serves then touch every bank once.
__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

constexpr int kBK = 64;   // k extent of one LDS tile (halfs) = 8 chunks of 16 bytes

// A [K, N] weight tile sits in LDS as 64 k-rows of BN halfs and is read with the LDS
// transpose read: the 32 lanes of one pass fetch 4 consecutive k-rows x 64 bytes.  Rows are
// BN / 32 segments of 64 bytes long; with a multiple of four segments per row the four rows
// start on the same bank and the segment is XORed with row & 3, with an odd multiple of
// two (BN = 64, 192) rows r and r + 2 do and bit 0 of the segment is XORed with bit 1 of the
// row.  Returned in 16-byte chunks (the unit a loading lane moves).
template <int BN>
__device__ __forceinline__ int swz_kn(int k_row) {
  static_assert(BN % 64 == 0, "whole 64-byte segment pairs");
  return (BN / 32) % 4 == 0 ? (k_row & 3) << 2 : ((k_row >> 1) & 1) << 2;
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // s_waitcnt immediate on gfx9: vmcnt[3:0], expcnt[6:4], lgkmcnt[11:8], vmcnt[5:4] in [15:14]
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// Wait until at most `younger` whole stages (NI loads each) are still in flight.
template <int NI, int MAXY>
__device__ __forceinline__ void wait_stages(int younger) {
  if constexpr (MAXY == 0) {
    wait_vmcnt<0>();
  } else {
    if (younger >= MAXY)
      wait_vmcnt<MAXY * NI>();
    else
      wait_stages<NI, MAXY - 1>(younger);
  }
}

// The buffer-descriptor type exists in the device pass only; the host pass sees the
// kernel as an empty stub.
#if defined(__HIP_DEVICE_COMPILE__)
// Untyped buffer descriptor (stride 0) over [base, base + bytes): loads past the end
// return 0.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void *base, size_t bytes) {
  const int recs = bytes > 0x7fffffffull ? 0x7fffffff : (int)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, recs, 0x00020000);
}

// One stage's loads of one wave: instruction i lands 8 tile rows (1 KB) at
// lds + i * lds_step; the first NIA instructions read A, the rest W.
template <int NI, int NIA, int COUNT = NI>
__device__ __forceinline__ void issue_stage_loads(rsrc_t rs_a, rsrc_t rs_w, const int (&voff)[NI],
                                                  half_t *lds, int lds_step, int k_bytes,
                                                  int k_bytes_w) {
#pragma unroll
  for (int i = 0; i < COUNT; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(i < NIA ? rs_a : rs_w,
                                             (__attribute__((address_space(3))) void *)(lds + i * lds_step),
                                             16, voff[i], i < NIA ? k_bytes : k_bytes_w, 0, 0);
}

// Byte offset, from the first element of a [K, N] weight tile (k-step 0, first column of
// the tile), of the 16 bytes that a loading lane moves with the load that fills bytes
// [1024 g, 1024 g + 1024) of the tile's LDS image; the tile has `cols` columns inside the
// matrix, and chunks past them get an offset outside every descriptor (they read as zero).
template <int BN>
__device__ __forceinline__ int kn_load_offset(int g, int lane, int N, int cols) {
  constexpr int CPR = BN / 8;                       // 16-byte chunks per k-row
  const int slot = g * 64 + lane;
  const int k_row = slot / CPR, c = (slot % CPR) ^ swz_kn<BN>(k_row);
  return c * 8 < cols ? (k_row * N + c * 8) * (int)sizeof(half_t) : 0x7ffffff0;
}

// Weight operand of one 32x32x16 MFMA (32 columns from n_base, 16 k-rows from k_base) out
// of the LDS image of a [K, N] tile: lane l holds column n_base + (l & 31) at k-rows
// k_base + 8 (l >> 5) .. + 7, gathered by two transpose reads of 4 k-rows x 16 columns per
// 16 lanes.  `lane_part` = kn_frag_lane_part(lane).
template <int BN>
__device__ __forceinline__ half8_t load_kn_frag(const half_t *sW, int n_base, int k_base, int lane) {
  const int lq = lane & 15, g2 = lane >> 4;
  const int k_row = k_base + 8 * (g2 >> 1) + (lq >> 2);
  const int col = n_base + 16 * (g2 & 1) + 4 * (lq & 3);
  const half_t *p0 = sW + k_row * BN + (((col >> 3) ^ swz_kn<BN>(k_row)) << 3) + (col & 7);
  const fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t *)p0);
  const fp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (__attribute__((address_space(3))) fp16x4_t *)(p0 + 4 * BN));   // rows + 4: same swizzle term
  const half4_t l4 = __builtin_bit_cast(half4_t, lo), h4 = __builtin_bit_cast(half4_t, hi);
  return half8_t{l4[0], l4[1], l4[2], l4[3], h4[0], h4[1], h4[2], h4[3]};
}

// ---- the epilogue's wave-private staging tile -------------------------------------------
// 32 rows of WTN halfs, written 8 bytes per lane straight from the accumulator layout (lane l
// owns row l & 31, the 8-byte half l >> 5 of a 16-byte chunk) and read back 16 bytes per lane,
// row-contiguous, for the global stores.  With 128-byte rows (WTN = 64) the tile is
// swizzled instead of padded: chunk ^= (row >> 1) & 7 and half ^= row >> 4 put the 32 lanes
// of one write pass on 32 distinct bank pairs (a padded pitch leaves rows r and r + 16 on the
// same banks: every write two passes); a reader undoes the half swap in registers.
template <int WTN>
struct Staging {
  static constexpr bool kSwizzled = WTN == 64;
  static constexpr int kPitch = kSwizzled ? WTN : WTN + 8;   // halfs
  // where lane (row, half hf of the chunk) writes the 4 halfs of 16-byte chunk `chunk`
  __device__ static __forceinline__ int write_at(int row, int hf, int chunk) {
    if (kSwizzled) return row * kPitch + ((chunk ^ ((row >> 1) & 7)) << 3) + (((hf ^ (row >> 4)) & 1) << 2);
    return row * kPitch + (chunk << 3) + (hf << 2);
  }
  // the 8 halfs of chunk `chunk` of row `row`, in order
  __device__ static __forceinline__ uint4_t read(const half_t *st, int row, int chunk) {
    if (kSwizzled) {
      const uint4_t v = *(const uint4_t *)(st + row * kPitch + ((chunk ^ ((row >> 1) & 7)) << 3));
      return (row >> 4) & 1 ? uint4_t{v[2], v[3], v[0], v[1]} : v;
    }
    return *(const uint4_t *)(st + row * kPitch + (chunk << 3));
  }
};

// ---- a [K, N] weight tile of 256 columns through registers ----------------------------
// The LDS transpose read runs at half the rate of the 16-byte read, and the 256 x 256 tile
// (eight waves that load and compute, LDS reads ~ 3/4 of its MFMA time) is the one shape
// that cannot hide that.  There the 64 x 256 tile of a row-major [K, N] weight is fetched
// into registers instead - each of the 512 lanes takes a block of 4 k-rows x 8 columns, four
// 16-byte loads - transposed in the lane (16 byte permutes) and written k-contiguous with
// eight 8-byte LDS writes into the very image the pre-packed [N, K] layout lands in, so the
// k loop reads both layouts the same way.  Lane -> block: four consecutive lanes take four
// consecutive column blocks (64 contiguous bytes per k-row), the next lanes the next k-rows.
// Which lanes write odd rows first and which even ones, together with the image's swizzle,
// puts the 32 lanes of one write pass on 32 distinct bank pairs.
struct RegW {
  uint4_t r[4];        // k-rows k_base .. k_base + 3, columns n_base .. n_base + 7
  int voff[4];         // byte offsets of the four loads from the tile's first element
  int woff[8];         // LDS offsets (halfs, from the W image of a stage) of the eight writes
  unsigned sel[2];     // permute selectors of even / odd write instructions
};
__device__ __forceinline__ void regw_setup(RegW &w, int wave, int lane, int N, int cols, int BM) {
  // (eight consecutive lanes on whole 128-byte lines measured slower: their writes then
  // collide two ways, and the memory side does not mind the 64-byte pieces)
  const int kq = lane >> 2, ngl = lane & 3, ng = wave * 4 + ngl;
  const int bit = ngl >> 1;
  const int k_base = 4 * kq, n_base = 8 * ng;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w.voff[i] = n_base < cols ? ((k_base + i) * N + n_base) * (int)sizeof(half_t) : 0x7ffffff0;
  const int c = kq >> 1, h = kq & 1;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int n = n_base + (i ^ bit);
    w.woff[i] = n * kBK + ((c ^ swz(n + BM)) << 3) + h * 4;
  }
  // write i moves column n_base + (i ^ bit): its halfs are the low or the high halves of
  // dword (i >> 1) of the four loads
  w.sel[0] = bit ? 0x07060302u : 0x05040100u;
  w.sel[1] = bit ? 0x05040100u : 0x07060302u;
}
__device__ __forceinline__ void regw_load(RegW &w, rsrc_t rs_w, int k_bytes_w) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w.r[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, w.voff[i], k_bytes_w, 0);
}
__device__ __forceinline__ void regw_store(const RegW &w, half_t *sW) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const unsigned lo = __builtin_amdgcn_perm(w.r[1][i >> 1], w.r[0][i >> 1], w.sel[i & 1]);
    const unsigned hi = __builtin_amdgcn_perm(w.r[3][i >> 1], w.r[2][i >> 1], w.sel[i & 1]);
    *(uint2_t *)(sW + w.woff[i]) = uint2_t{lo, hi};
  }
}

template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI, bool WKN>
__device__ __forceinline__ void gemm_tile(const GemmArgs &p) {
  constexpr int BK = kBK;
  constexpr int NW = WM * WN;                   // waves that run the MFMAs
  constexpr int NL = NP > 0 ? NP : NW;          // waves that issue the global loads
  constexpr int WTM = BM / WM, WTN = BN / WN;   // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;   // 32x32 MFMA blocks per wave
  constexpr int ROWS = BM + BN;                 // A rows then W rows in one stage
  constexpr int NI = ROWS / 8 / NL;             // load instructions per loading wave per stage
  constexpr int NIA = BM / 8 / NL;              // ... of which the first NIA fetch A rows
  constexpr int STAGE_HALFS = ROWS * BK;
  static_assert(BM % (8 * NL) == 0 && BN % (8 * NL) == 0, "tile rows must split evenly over the loading waves");
  static_assert(STAGES >= 2 && STAGES <= 5 && (STAGES - 2) * NI < 64, "pipeline depth");
  constexpr int YOUNG = STAGES - 2;   // stages that may still be in flight at a barrier
  // a [K, N] weight tile goes through registers (see RegW) where every wave loads and computes
  constexpr bool kRegW = WKN && NP == 0 && BN == 256 && NW == 8 && STAGES == 2;

  extern __shared__ __attribute__((aligned(1024))) half_t gemm_smem[];
  half_t *smem = gemm_smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = (int)blockIdx.x;
  int M;
  MaskRows mr{};
  if (p.mask) {
    // the last ring stage is first written after the first barrier of the k loop, which
    // every wave reaches only after it has read the lengths
    mr = mask_rows_setup(p, wave, NW + NP, lane, (int *)(smem + (STAGES - 1) * STAGE_HALFS));
    M = min(mr.M, p.rows_cap);
    if (bid == 0 && blockIdx.y == 0 && wave < NW) mask_rows_write(p, mr, tid, NW * 64, lane);
  } else {
    M = p.valid_rows ? min(*p.valid_rows, p.rows_cap) : p.rows_cap;
  }

  // XCD-aware tile order over the live tiles
  int tile_m, tile_n;
  {
    const int live = ((M + BM - 1) / BM) * p.tiles_n;
    const int per = (live + 7) >> 3;
    const int L = (bid & 7) * per + (bid >> 3);
    if (bid >= per * 8 || L >= live) return;
    tile_m = L / p.tiles_n;
    tile_n = L - tile_m * p.tiles_n;
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  // a split-k launch gives grid row y the k range [y, y+1) * K / gridDim.y
  const int nk = EPI == kEpiPartial ? p.K / BK / (int)gridDim.y : p.K / BK;
  const int k_first = EPI == kEpiPartial ? (int)blockIdx.y * nk * BK : 0;

  // ---- loading side ---------------------------------------------------------
  // Global -> LDS copies are buffer loads with the LDS destination: descriptor and
  // k offset in scalar registers, one fixed 32-bit byte offset per lane and load.
  // (Beside a wave that keeps the MFMA pipe full this form issues at the full
  // 64 B/clk of the vector memory path; the flat-address form drops to half.)
  // Load instruction i of loading wave w fills tile rows [(i*NL + w)*8, +8); a lane
  // fetches the chunk that the swizzle places in its slot.  Rows past the end of
  // either operand fall outside the descriptor and read as zero.
  //
  // With NP == 0 every wave loads its share and then computes.  With NP > 0 the
  // last NP waves only load: the vector-memory unit accepts one 1 KB instruction
  // per 16 clocks, and a wave that has to push its loads through that queue at the
  // top of every k-step cannot feed the MFMA pipe meanwhile; for small tiles
  // (load clocks ~ MFMA clocks) that serialisation costs half of the throughput.
  const bool loader = NP == 0 || wave >= NW;
  const int lw = NP == 0 ? wave : wave - NW;    // index among the loading waves
  const bool gather = p.a_row_index != nullptr || p.mask != nullptr;
  const rsrc_t rs_a =
      gather ? make_rsrc(p.a + k_first, ((size_t)p.rows_cap * p.K - k_first) * sizeof(half_t))
             : make_rsrc(p.a + (size_t)m0 * p.K + k_first,
                         ((size_t)(p.rows_cap - m0) * p.K - k_first) * sizeof(half_t));
  // the weight tile: BN rows of 64 k ([N, K] pre-pack), or 64 k-rows of BN columns ([K, N]);
  // 1 KB per load instruction either way
  const rsrc_t rs_w =
      WKN ? make_rsrc(p.wt + (size_t)k_first * p.N + n0,
                      ((size_t)(p.K - k_first) * p.N - n0) * sizeof(half_t))
          : make_rsrc(p.wt + (size_t)n0 * p.K + k_first,
                      ((size_t)(p.N - n0) * p.K - k_first) * sizeof(half_t));
  int voff[NI];
  if (loader) {
    MaskRowSpan span{};
    if (p.mask) span = mask_rows_span(mr, p.mask_B, lane, m0, min(m0 + BM, M) - 1);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = (i * NL + lw) * 8 + (lane >> 3);
      const int kc = (lane & 7) ^ swz(r);
      int row = i < NIA ? r : r - BM;
      if (i < NIA && gather) {   // live rows only hold valid indices
        const int live_row = min(m0 + r, M - 1);
        row = p.mask ? mask_rows_map(mr, span, live_row) : p.a_row_index[live_row];
      }
      voff[i] = (row * p.K + kc * 8) * (int)sizeof(half_t);
      if (WKN && i >= NIA) voff[i] = kn_load_offset<BN>((i - NIA) * NL + lw, lane, p.N, p.N - n0);
    }
  }
  const int w_step_bytes = (WKN ? BK * p.N : BK) * (int)sizeof(half_t);   // one k-step further
  RegW rw;
  if (kRegW) regw_setup(rw, wave, lane, p.N, p.N - n0, BM);
#define BT_ISSUE_LOADS(kt, stage)                                                              \
  issue_stage_loads<NI, NIA, kRegW ? NIA : NI>(                                                \
      rs_a, rs_w, voff, smem + (stage)*STAGE_HALFS + lw * 8 * BK, NL * 8 * BK,                 \
      (kt)*BK * (int)sizeof(half_t), (kt)*w_step_bytes)
  // Register-staged weight tile: one register set.  The loads of k-step s + 1 go out early in
  // step s - 1 (right after the registers have been emptied into LDS), have the rest of that
  // step and the start of step s to arrive, and are written to LDS early in step s, behind
  // the first quarter of its MFMAs: neither the loads nor the writes are waited for where
  // they were issued.  In vmcnt terms every wait is "at most the NIA youngest outstanding":
  // at the top of a step those are the weight loads (the A tile's direct-to-LDS loads are
  // older), at the write they are the A tile's loads of the next step.
#define BT_LOAD_W(kt) regw_load(rw, rs_w, (kt)*w_step_bytes)
#define BT_STORE_W(stage) regw_store(rw, smem + (stage)*STAGE_HALFS + BM * BK)
  static_assert(!kRegW || NIA == 4, "the weight tile's four loads per lane pair with four A loads");

  if (loader) {
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
      if (s < nk) BT_ISSUE_LOADS(s, s);
    if (kRegW) {
      BT_LOAD_W(0);
      wait_vmcnt<0>();
      BT_STORE_W(0);
      if (nk > 1) BT_LOAD_W(1);
    }
  }

  if (NP > 0 && wave >= NW) {
    // pure loader: one barrier per k-step, in step with the computing waves
    int stage = 0;
    for (int kt = 0; kt < nk; ++kt) {
      wait_stages<NI, YOUNG>(nk - 1 - kt);       // this wave's part of tile kt has landed
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();               // tile kt is complete; stage of tile kt-1 is free
      asm volatile("" ::: "memory");
      if (kt + STAGES - 1 < nk) {
        int ps = stage + STAGES - 1;
        if (ps >= STAGES) ps -= STAGES;
        BT_ISSUE_LOADS(kt + STAGES - 1, ps);
      }
      if (++stage == STAGES) stage = 0;
    }
    __builtin_amdgcn_s_barrier();                 // pairs with the barrier before the epilogue
    return;
  }

  // ---- computing side -------------------------------------------------------
  const int wm = wave / WN, wn = wave % WN;
  // The accumulators start from the bias of their column (element 4q + e of block (i, j)
  // is column n0 + wn*WTN + 32 i + 8 q + 4 (lane >> 5) + e), so the epilogue adds nothing.
  constexpr bool kHasBias = EPI == kEpiBiasGelu || EPI == kEpiQkvSplit || EPI == kEpiBias;
  float16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i) {
    float16_t init;
#pragma unroll
    for (int v = 0; v < 16; ++v) init[v] = 0.f;
    if (kHasBias) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = min(n0 + wn * WTN + i * 32 + q * 8 + (lane >> 5) * 4, p.N - 4);
        const half4_t b = *(const half4_t *)(p.bias + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) init[4 * q + e] = (float)b[e];
      }
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = init;
  }

  const int fr_row = lane & 31, fr_kc = lane >> 5;
  half8_t fw[2][TN], fa[2][TM];
  auto load_frags = [&](int st, int ks, int b) {
    const half_t *sA = smem + st * STAGE_HALFS;
    const half_t *sB = sA + BM * BK;
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      const int r = wn * WTN + i * 32 + fr_row;
      if (WKN && !kRegW)
        fw[b][i] = load_kn_frag<BN>(sB, wn * WTN + i * 32, 16 * ks, lane);
      else
        fw[b][i] = *(const half8_t *)(sB + r * BK + (((2 * ks + fr_kc) ^ swz(r + BM)) * 8));
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int r = wm * WTM + j * 32 + fr_row;
      fa[b][j] = *(const half8_t *)(sA + r * BK + (((2 * ks + fr_kc) ^ swz(r)) * 8));
    }
  };
  int stage = 0;
  for (int kt = 0; kt < nk; ++kt) {
    // tile kt has landed for this wave once only the younger stages' loads are outstanding
    if (kRegW) {
      // this wave's A loads of tile kt and its LDS writes of the W tile; the weight loads of
      // tile kt + 1 stay in flight
      if (kt + 1 < nk)
        __builtin_amdgcn_s_waitcnt(0x0074);   // vmcnt(4) lgkmcnt(0)
      else
        __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0)
    } else if (NP == 0)
      wait_stages<NI, YOUNG>(nk - 1 - kt);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();   // everyone's tile is in LDS; stage (kt-1) is free again
    asm volatile("" ::: "memory");
    if (NP == 0 && kt + STAGES - 1 < nk) {
      int ps = stage + STAGES - 1;
      if (ps >= STAGES) ps -= STAGES;
      BT_ISSUE_LOADS(kt + STAGES - 1, ps);
    }
    load_frags(stage, 0, 0);
    // compiler scheduling strategy that interleaves the LDS reads with the MFMAs
    if (SCHED == 0) __builtin_amdgcn_iglp_opt(0);
    if (SCHED == 1) __builtin_amdgcn_iglp_opt(1);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (ks + 1 < BK / 16) load_frags(stage, ks + 1, (ks + 1) & 1);
      if (kRegW && ks == 1 && kt + 1 < nk) {
        wait_vmcnt<NIA>();            // the weight registers of step kt + 1 (older than its A loads)
        BT_STORE_W(stage ^ 1);
        if (kt + 2 < nk) BT_LOAD_W(kt + 2);
      }
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[ks & 1][i], fa[ks & 1][j],
                                                            acc[i][j], 0, 0, 0);
    }
    if (++stage == STAGES) stage = 0;
  }

#undef BT_ISSUE_LOADS
#undef BT_LOAD_W
#undef BT_STORE_W
  // ---- epilogue -------------------------------------------------------------
  // accumulator block (i, j), quad q: columns n..n+3 of row m with
  //   n = n0 + wn*WTN + i*32 + q*8 + (lane>>5)*4,  m = m0 + wm*WTM + j*32 + (lane&31)
  constexpr int EP = Staging<WTN>::kPitch;   // pitch (halfs) of the wave-private staging tile
  static_assert((size_t)NW * 32 * EP <= (size_t)STAGES * STAGE_HALFS, "staging fits the ring");
  __builtin_amdgcn_s_barrier();   // all waves are done with the last stage
  half_t *st = smem + wave * 32 * EP;
  const int row_in = lane & 31, col_in = (lane >> 5) * 4;
  if (EPI == kEpiPartial) {
    // fp32 partial sums straight from the accumulators: 16 bytes per lane and quad
    float *dst = p.c32 + (size_t)blockIdx.y * p.rows_cap * p.N;
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int m = m0 + wm * WTM + j * 32 + row_in;
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * WTN + i * 32 + q * 8 + col_in;
          if (m < M && n < p.N)
            *(float4_t *)(dst + (size_t)m * p.N + n) =
                float4_t{acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                         acc[i][j][4 * q + 3]};
        }
    }
    return;
  }
  constexpr int CPRW = WTN / 8;   // 16-byte chunks per staged row
  constexpr int RPS = 64 / CPRW;  // rows per store instruction
  const int sr = lane / CPRW, sc = (lane % CPRW) * 8;
#pragma unroll
  for (int j = 0; j < TM; ++j) {
#pragma unroll
    for (int i = 0; i < TN; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v0 = acc[i][j][4 * q + 0], v1 = acc[i][j][4 * q + 1];
        float v2 = acc[i][j][4 * q + 2], v3 = acc[i][j][4 * q + 3];
        if (EPI == kEpiBiasGelu) {
          v0 = gelu_tanh_f32(v0);
          v1 = gelu_tanh_f32(v1);
          v2 = gelu_tanh_f32(v2);
          v3 = gelu_tanh_f32(v3);
        }
        *(half4_t *)(st + Staging<WTN>::write_at(row_in, lane >> 5, i * 4 + q)) =
            half4_t{(half_t)v0, (half_t)v1, (half_t)v2, (half_t)v3};
      }
    }
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += RPS) {
      const int r = r0 + sr;
      if (sr >= RPS || r >= 32) continue;   // lanes left over when 64 % CPRW != 0
      const int m = m0 + wm * WTM + j * 32 + r, n = n0 + wn * WTN + sc;
      const uint4_t v = Staging<WTN>::read(st, r, sc >> 3);
      if (m < M && n < p.N) {
        if (EPI == kEpiQkvSplit) {
          // column n = which*H + g*64 + dd  ->  [which*heads + g][m][dd]
          *(uint4_t *)(p.c + ((size_t)(n >> 6) * p.rows_cap + m) * 64 + (n & 63)) = v;
        } else {
          *(uint4_t *)(p.c + (size_t)m * p.N + n) = v;
        }
      }
    }
  }
}

// ---- persistent form ---------------------------------------------------------------
// The launch has about one workgroup per CU and every workgroup takes SEVERAL tiles of its
// XCD's range, running ONE software pipeline over all their k-steps: the loads of the next
// tile's first stages are in flight while the current tile's accumulators are stored, and
// a tile's stores drain to memory under the next tile's products instead of in one burst of
// the whole launch at its end.  (One tile per workgroup leaves the matrix pipe idle from
// the first store instruction on: with 228 tiles on 256 CUs the last 7 us of the 31 us of
// the FFN1 product at batch 16 x 512 are 29.5 MB of stores.)  The grid no longer depends
// on the row count: a workgroup counts its tiles from the device-side row count.
template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI, bool WKN>
__device__ __forceinline__ void gemm_tiles_flat(const GemmArgs &p) {
  constexpr int BK = kBK;
  constexpr int NW = WM * WN;
  constexpr int NL = NP > 0 ? NP : NW;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int ROWS = BM + BN;
  constexpr int NI = ROWS / 8 / NL;
  constexpr int NIA = BM / 8 / NL;
  constexpr int STAGE_HALFS = ROWS * BK;
  static_assert(BM % (8 * NL) == 0 && BN % (8 * NL) == 0, "tile rows must split evenly over the loading waves");
  static_assert(STAGES >= 2 && STAGES <= 5 && (STAGES - 2) * NI < 64, "pipeline depth");
  static_assert(EPI != kEpiPartial, "split-k launches keep one tile per workgroup");
  constexpr int YOUNG = STAGES - 2;
  constexpr int EP = Staging<WTN>::kPitch;   // pitch (halfs) of the wave-private staging tile
  static_assert((size_t)NW * 32 * EP <= (size_t)STAGE_HALFS, "staging fits one stage of the ring");

  extern __shared__ __attribute__((aligned(1024))) half_t gemm_smem[];
  half_t *smem = gemm_smem;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bid = (int)blockIdx.x;
  int M;
  MaskRows mr{};
  if (p.mask) {
    // (the last ring stage: first written after the first barrier of the k loop)
    mr = mask_rows_setup(p, wave, NW + NP, lane, (int *)(smem + (STAGES - 1) * STAGE_HALFS));
    M = min(mr.M, p.rows_cap);
    if (bid == 0 && wave < NW) mask_rows_write(p, mr, tid, NW * 64, lane);
  } else {
    M = p.valid_rows ? min(*p.valid_rows, p.rows_cap) : p.rows_cap;
  }

  // XCD x owns the contiguous range [x * per, (x + 1) * per) of the live tiles; its
  // workgroups take them round-robin
  const int live = ((M + BM - 1) / BM) * p.tiles_n;
  const int per = (live + 7) >> 3;
  const int wgx = p.tile_grid >> 3;                      // workgroups per XCD
  const int lo = (bid & 7) * per;
  const int hi = min(lo + per, live);
  const int L0 = lo + (bid >> 3);
  if (L0 >= hi) return;
  const int n_my = (hi - L0 + wgx - 1) / wgx;
  const int nk = p.K / BK;
  const int total = n_my * nk;                           // k-steps of this workgroup

  // ---- loading side: a cursor (tile, k-step) STAGES - 1 steps ahead of the products ----
  const bool loader = NP == 0 || wave >= NW;
  const int lw = NP == 0 ? wave : wave - NW;
  const bool gather = p.a_row_index != nullptr || p.mask != nullptr;
  rsrc_t rs_a = make_rsrc(p.a, 0), rs_w = make_rsrc(p.wt, 0);
  constexpr bool kHasBias = EPI == kEpiBiasGelu || EPI == kEpiQkvSplit || EPI == kEpiBias;
  // The bias of a tile's columns reaches the computing waves through LDS, fetched by the
  // first loading wave together with the tile's first k-step: a global load in a computing
  // wave after its stores would wait for every one of them to complete - the very wait this
  // form of the kernel exists to avoid.  (Only the first tile's bias is loaded directly.)
  // It is requested as soon as the cursor moves to the tile, one k-step ahead of the tile's
  // first loads (so that the wait for those loads' predecessors covers it), and the cursor
  // runs STAGES - 1 k-steps ahead of the products: with k = 64 (one k-step per tile) up to
  // STAGES biases are waiting to be read, hence STAGES buffers, taken in turn.
  half_t *s_bias = smem + STAGES * STAGE_HALFS;          // [STAGES][BN]
  const rsrc_t rs_bias = make_rsrc(kHasBias ? p.bias : p.wt, kHasBias ? (size_t)p.N * sizeof(half_t) : 0);
  int voff[NI];
  int idx_next[NIA];   // gathered A rows of the tile after the one being loaded
  int ld_L = L0, ld_kt = 0, ld_left = loader ? total : 0;
  int ld_slot = 0;     // bias buffer of the tile being set up: its position in the sequence mod STAGES
  auto fetch_indices = [&](int Lt) {
    const int m0 = (Lt / p.tiles_n) * BM;
    MaskRowSpan span{};
    if (p.mask) span = mask_rows_span(mr, p.mask_B, lane, m0, min(m0 + BM, M) - 1);
#pragma unroll
    for (int i = 0; i < NIA; ++i) {
      const int r = (i * NL + lw) * 8 + (lane >> 3);
      const int live_row = min(m0 + r, M - 1);   // live rows only hold valid indices
      idx_next[i] = p.mask ? mask_rows_map(mr, span, live_row) : p.a_row_index[live_row];
    }
  };
  auto load_setup = [&](int Lt, bool more, bool bias_to_lds) {
    const int tm = Lt / p.tiles_n, tn = Lt - tm * p.tiles_n;
    const int m0 = tm * BM, n0 = tn * BN;
    if (kHasBias && bias_to_lds && lw == 0) {
      // 4 bytes per lane and instruction: 128 columns each
#pragma unroll
      for (int i = 0; i < BN / 128; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            rs_bias,
            (__attribute__((address_space(3))) void *)(s_bias + ld_slot * BN + i * 128), 4,
            (lane + i * 64) * 4, n0 * (int)sizeof(half_t), 0, 0);
    }
    rs_a = gather ? make_rsrc(p.a, (size_t)p.rows_cap * p.K * sizeof(half_t))
                  : make_rsrc(p.a + (size_t)m0 * p.K, (size_t)(p.rows_cap - m0) * p.K * sizeof(half_t));
    rs_w = WKN ? make_rsrc(p.wt + n0, ((size_t)p.K * p.N - n0) * sizeof(half_t))
               : make_rsrc(p.wt + (size_t)n0 * p.K, (size_t)(p.N - n0) * p.K * sizeof(half_t));
    if (WKN && (p.N % BN) != 0) {
      // the column mask of the weight loads depends on the tile's first column
#pragma unroll
      for (int i = NIA; i < NI; ++i)
        voff[i] = kn_load_offset<BN>((i - NIA) * NL + lw, lane, p.N, p.N - n0);
    }
    if (gather) {
#pragma unroll
      for (int i = 0; i < NIA; ++i) {
        const int r = (i * NL + lw) * 8 + (lane >> 3);
        const int kc = (lane & 7) ^ swz(r);
        voff[i] = (idx_next[i] * p.K + kc * 8) * (int)sizeof(half_t);
      }
      if (more) fetch_indices(Lt + wgx);
    }
  };
  if (loader) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = (i * NL + lw) * 8 + (lane >> 3);
      const int kc = (lane & 7) ^ swz(r);
      const int row = i < NIA ? r : r - BM;
      voff[i] = (row * p.K + kc * 8) * (int)sizeof(half_t);
      if (WKN && i >= NIA) voff[i] = kn_load_offset<BN>((i - NIA) * NL + lw, lane, p.N, BN);
    }
    if (gather) fetch_indices(L0);
    load_setup(L0, n_my > 1, false);
  }
  // issues the loads of the cursor's k-step into `stage` and moves the cursor on
  auto issue_next = [&](int stage) {
    if (ld_left == 0) return;
    issue_stage_loads<NI, NIA>(rs_a, rs_w, voff, smem + stage * STAGE_HALFS + lw * 8 * BK,
                               NL * 8 * BK, ld_kt * BK * (int)sizeof(half_t),
                               ld_kt * (WKN ? BK * p.N : BK) * (int)sizeof(half_t));
    --ld_left;
    if (++ld_kt == nk) {
      ld_kt = 0;
      ld_L += wgx;
      if (++ld_slot == STAGES) ld_slot = 0;
      if (ld_left) load_setup(ld_L, ld_left > nk, true);
    }
  };
  if (loader) {
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue_next(s);
  }

  if (NP > 0 && wave >= NW) {
    // pure loader: one barrier per k-step in step with the computing waves, one more at
    // the end of every tile (the computing waves then overlay the consumed stage)
    int stage = 0, kt = 0;
    for (int g = 0; g < total; ++g) {
      wait_stages<NI, YOUNG>(total - 1 - g);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      int ps = stage + STAGES - 1;
      if (ps >= STAGES) ps -= STAGES;
      issue_next(ps);
      if (++kt == nk) {
        kt = 0;
        __builtin_amdgcn_s_barrier();
      }
      if (++stage == STAGES) stage = 0;
    }
    return;
  }

  // ---- computing side ---------------------------------------------------------------
  const int wm = wave / WN, wn = wave % WN;
  // The accumulators of a tile start from the bias of their columns (element 4q + e of
  // block (i, j) is column n0 + wn*WTN + 32 i + 8 q + 4 (lane >> 5) + e).
  float16_t acc[TN][TM];
  auto init_acc = [&](const half_t *bias_of_tile, int n_limit) {
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      float16_t init;
#pragma unroll
      for (int v = 0; v < 16; ++v) init[v] = 0.f;
      if (kHasBias) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = min(wn * WTN + i * 32 + q * 8 + (lane >> 5) * 4, n_limit);
          const half4_t b = *(const half4_t *)(bias_of_tile + n);
#pragma unroll
          for (int e = 0; e < 4; ++e) init[4 * q + e] = (float)b[e];
        }
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) acc[i][j] = init;
    }
  };
  int cL = L0, c_slot = 0;
  {
    const int n0 = (cL % p.tiles_n) * BN;
    init_acc(kHasBias ? p.bias + n0 : nullptr, p.N - 4 - n0);   // the first tile: straight from memory
  }

  const int fr_row = lane & 31, fr_kc = lane >> 5;
  half8_t fw[2][TN], fa[2][TM];
  auto load_frags = [&](int st, int ks, int b) {
    const half_t *sA = smem + st * STAGE_HALFS;
    const half_t *sB = sA + BM * BK;
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      const int r = wn * WTN + i * 32 + fr_row;
      if (WKN)
        fw[b][i] = load_kn_frag<BN>(sB, wn * WTN + i * 32, 16 * ks, lane);
      else
        fw[b][i] = *(const half8_t *)(sB + r * BK + (((2 * ks + fr_kc) ^ swz(r + BM)) * 8));
    }
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int r = wm * WTM + j * 32 + fr_row;
      fa[b][j] = *(const half8_t *)(sA + r * BK + (((2 * ks + fr_kc) ^ swz(r)) * 8));
    }
  };
  const int row_in = lane & 31, col_in = (lane >> 5) * 4;
  constexpr int CPRW = WTN / 8;   // 16-byte chunks per staged row
  constexpr int RPS = 64 / CPRW;  // rows per store instruction
  const int sr = lane / CPRW, sc = (lane % CPRW) * 8;

  int stage = 0, kt = 0;
  for (int g = 0; g < total; ++g) {
    if (NP == 0) wait_stages<NI, YOUNG>(total - 1 - g);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();   // everyone's k-step g is in LDS; the stage of step g-1 is free again
    asm volatile("" ::: "memory");
    if (NP == 0) {
      int ps = stage + STAGES - 1;
      if (ps >= STAGES) ps -= STAGES;
      issue_next(ps);
    }
    load_frags(stage, 0, 0);
    if (SCHED == 0) __builtin_amdgcn_iglp_opt(0);
    if (SCHED == 1) __builtin_amdgcn_iglp_opt(1);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (ks + 1 < BK / 16) load_frags(stage, ks + 1, (ks + 1) & 1);
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[ks & 1][i], fa[ks & 1][j],
                                                            acc[i][j], 0, 0, 0);
    }
    if (++kt == nk) {
      // ---- this tile is complete: store it, start the next from its bias ----
      kt = 0;
      const int tm = cL / p.tiles_n, tn = cL - tm * p.tiles_n;
      const int m0 = tm * BM, n0 = tn * BN;
      __builtin_amdgcn_s_barrier();   // all waves are done reading this stage: it becomes the staging area
      half_t *st = smem + stage * STAGE_HALFS + wave * 32 * EP;
#pragma unroll
      for (int j = 0; j < TM; ++j) {
#pragma unroll
        for (int i = 0; i < TN; ++i) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float v0 = acc[i][j][4 * q + 0], v1 = acc[i][j][4 * q + 1];
            float v2 = acc[i][j][4 * q + 2], v3 = acc[i][j][4 * q + 3];
            if (EPI == kEpiBiasGelu) {
              v0 = gelu_tanh_f32(v0);
              v1 = gelu_tanh_f32(v1);
              v2 = gelu_tanh_f32(v2);
              v3 = gelu_tanh_f32(v3);
            }
            *(half4_t *)(st + Staging<WTN>::write_at(row_in, lane >> 5, i * 4 + q)) =
                half4_t{(half_t)v0, (half_t)v1, (half_t)v2, (half_t)v3};
          }
        }
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += RPS) {
          const int r = r0 + sr;
          if (sr >= RPS || r >= 32) continue;   // lanes left over when 64 % CPRW != 0
          const int m = m0 + wm * WTM + j * 32 + r, n = n0 + wn * WTN + sc;
          const uint4_t v = Staging<WTN>::read(st, r, sc >> 3);
          if (m < M && n < p.N) {
            if (EPI == kEpiQkvSplit) {
              // column n = which*H + g*64 + dd  ->  [which*heads + g][m][dd]
              *(uint4_t *)(p.c + ((size_t)(n >> 6) * p.rows_cap + m) * 64 + (n & 63)) = v;
            } else {
              *(uint4_t *)(p.c + (size_t)m * p.N + n) = v;
            }
          }
        }
      }
      cL += wgx;
      if (++c_slot == STAGES) c_slot = 0;
      if (g + 1 < total) init_acc(s_bias + c_slot * BN, BN - 4);   // from LDS, where the loading side has put it
    }
    if (++stage == STAGES) stage = 0;
  }
}

#endif  // __HIP_DEVICE_COMPILE__

template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI, bool WKN>
__global__ __launch_bounds__((WM * WN + NP) * 64) void gemm_flat_kernel(GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  gemm_tiles_flat<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, WKN>(p);
#endif
}

template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI, bool WKN>
__global__ __launch_bounds__((WM * WN + NP) * 64) void gemm_kernel(GemmArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  gemm_tile<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, WKN>(p);
#endif
}

// ---- weight pre-pack: wt[n][k] = w[k][n] for up to four matrices in one launch ---
struct TransposeJob {
  const half_t *w;
  half_t *wt;
  int K, N;
  int tiles_n, tile_begin;   // 64x64 tiles: tiles along n, first global tile id
};
struct TransposeArgs {
  TransposeJob job[4];
  int njobs;
};

__global__ __launch_bounds__(256) void transpose_kernel(TransposeArgs a) {
  __shared__ half_t tile[64][kTransposePitch];
  int j = 0;
#pragma unroll
  for (int i = 1; i < 4; ++i)
    if (i < a.njobs && (int)blockIdx.x >= a.job[i].tile_begin) j = i;
  const TransposeJob jb = a.job[j];
  const int t = blockIdx.x - jb.tile_begin;
  transpose_tile_64(jb.w, jb.wt, jb.K, jb.N, (t / jb.tiles_n) * 64, (t % jb.tiles_n) * 64, tile,
                    threadIdx.x, true);
}

template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI, bool WKN>
static int launch_gemm_tile_as(GemmArgs p, hipStream_t s, int splits) {
  constexpr size_t smem = (size_t)STAGES * (BM + BN) * kBK * sizeof(half_t);
  static_assert(smem <= 160 * 1024, "LDS budget");
  static std::atomic<bool> configured[kMaxDevices];
  const int rc = allow_dynamic_lds(gemm_kernel<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, WKN>, smem,
                                   configured, "hipFuncSetAttribute(gemm_kernel)");
  if (rc != BT_OK) return rc;
  const int tiles_m = (p.rows_cap + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  p.tile_grid = (tiles_m * p.tiles_n + 7) / 8 * 8;
  const dim3 grid(p.tile_grid, splits);
  gemm_kernel<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, WKN>
      <<<grid, (WM * WN + NP) * 64, smem, s>>>(p);
  BT_CHECK_LAUNCH("gemm_kernel");
  return BT_OK;
}

template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI>
static int launch_gemm_tile(GemmArgs p, hipStream_t s, int splits = 1) {
  return p.w_kn ? launch_gemm_tile_as<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, true>(p, s, splits)
                : launch_gemm_tile_as<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, false>(p, s, splits);
}

static int cu_count();

// Persistent launch: about one workgroup per CU (a multiple of 8, one share per XCD), each
// looping over its tiles on the device.
template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI, bool WKN>
static int launch_gemm_flat_as(GemmArgs p, hipStream_t s) {
  constexpr size_t smem = (size_t)STAGES * (BM + BN) * kBK * sizeof(half_t) + STAGES * BN * sizeof(half_t);
  static_assert(smem <= 160 * 1024, "LDS budget");
  static std::atomic<bool> configured[kMaxDevices];
  const int rc = allow_dynamic_lds(gemm_flat_kernel<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, WKN>,
                                   smem, configured, "hipFuncSetAttribute(gemm_flat_kernel)");
  if (rc != BT_OK) return rc;
  const int tiles_m = (p.rows_cap + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const long long tiles = (long long)tiles_m * p.tiles_n;
  const int per_cu = smem <= 80 * 1024 ? 2 : 1;          // workgroups that fit one CU's LDS
  long long wgs = (long long)cu_count() * per_cu;
  if (wgs > tiles) wgs = tiles;
  p.tile_grid = (int)((wgs + 7) / 8 * 8);
  const dim3 grid((unsigned)p.tile_grid);
  gemm_flat_kernel<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, WKN>
      <<<grid, (WM * WN + NP) * 64, smem, s>>>(p);
  BT_CHECK_LAUNCH("gemm_flat_kernel");
  return BT_OK;
}

template <int BM, int BN, int STAGES, int WM, int WN, int NP, int SCHED, int EPI>
static int launch_gemm_flat(GemmArgs p, hipStream_t s) {
  return p.w_kn ? launch_gemm_flat_as<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, true>(p, s)
                : launch_gemm_flat_as<BM, BN, STAGES, WM, WN, NP, SCHED, EPI, false>(p, s);
}

static int cu_count() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}

// Live rows the tile choice is made for: the exact count when every row is live, the
// caller's hint when it has one, else 60 % of the capacity (the fill the padding-free
// path is built for).
static long long estimated_rows(const GemmArgs &p) {
  if (!p.valid_rows && !p.mask) return p.rows_cap;
  if (p.rows_hint > 0) return p.rows_hint < p.rows_cap ? p.rows_hint : p.rows_cap;
  return (p.rows_cap * 3LL + 4) / 5;
}

#include "gemm_tuned.inc"

// Measured times of every tile for this weight shape at the first table row of at least m
// rows, or nullptr when the shape is not in the table or m lies outside it (the analytic
// model then decides alone).  The rows are kTunedStep apart, the height of the tallest
// tile, so the row used has the same number of row tiles as m or one more: run time moves
// in steps with the number of rounds of workgroups, and interpolating between two row
// counts on either side of such a step would describe neither.
static const float *tuned_times(long long m, int n, int k, int epi, int kn, int full) {
  if (cu_count() != 256) return nullptr;     // the table was measured on a 256-CU part
  // below about a thousand rows a launch is latency bound and a loop of identical
  // launches says little about the layer sequence
  if (m < 1024 || m > kTunedRows[kTunedPoints - 1]) return nullptr;
  for (const TunedShape &ts : kTunedShapes) {
    if (ts.n != n || ts.k != k || ts.epi != epi || ts.kn != kn || ts.full != full) continue;
    int at = 0;
    while (at < kTunedPoints - 1 && kTunedRows[at] < m) ++at;
    return ts.us[at];
  }
  return nullptr;
}

template <int EPI>
static int launch_gemm(GemmArgs p, hipStream_t s) {
  // Tile table (rows x cols, ring depth, computing wave grid, loader waves):
  //   0: 256x256, 2, 2x4, 0   wide outputs: one tile per CU, every wave loads and computes
  //   1: 128x128, 3, 2x2, 4   narrow outputs (projection, FFN2) and small problems
  //   2: 256x128, 3, 4x2, 4   narrow outputs with enough rows to fill the chip
  //   3: 256x192, 2, 4x2, 4   outputs that split into 192-wide panels but not into a
  //                           full wave of 256-wide ones (QKV at hidden 768); 141 registers
  //                           leave room for the loader waves (-2 to -4 % against unified)
  //   4:  32x64,  4, 1x2, 2   a few hundred rows or fewer: the k loop of one tile is the
  //                           whole run time, and a small tile has the shortest k-step
  //   5: 128x128, 2, 2x2, 4   tile 1 with a two-deep ring: 64 KB of LDS, so two workgroups
  //                           share a CU and one's fill and epilogue hide under the other's
  //                           k loop; pays when tile 1 would need several rounds
  //   6, 7, 8                 tiles 2, 1 and 0 in the persistent form (gemm_tiles_flat); never
  //                           the model's choice, only the measured table's, and there
  //                           within a few per cent of the one-tile-per-workgroup form
  // The choice minimises rounds x (k-steps x time of one k-step + fill and epilogue) with
  // the per-tile constants below, for the estimated live rows; for the weight shapes of
  // BERT-base and BERT-large a table of measured times (gemm_tuned.inc) then overrides it
  // where another tile is clearly faster.
  const int forced = option_gemm_tile();
  int choice = forced;
  if (choice < 0) {
    const int cus = cu_count();
    const long long m_est = estimated_rows(p);
    struct Cand {
      int id, bm, bn;
      float step_us, fixed_us;   // one k-step of one tile; fill + epilogue of one tile
      bool shares_cu;            // several workgroups per CU: time grows with tiles / CUs, not in rounds
    };
    const Cand cands[5] = {{0, 256, 256, 1.29f, 3.4f, false},
                           {3, 256, 192, 1.04f, 2.8f, false},
                           {2, 256, 128, 0.62f, 2.3f, false},
                           {1, 128, 128, 0.43f, 1.8f, false},
                           {4, 32, 64, 0.16f, 2.6f, true}};
    const float nk = (float)(p.K / kBK);
    float best = 0.f;
    for (const Cand &c : cands) {
      const long long tiles = ((m_est + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn);
      float t;
      if (c.shares_cu) {
        const float load = (float)tiles / (float)cus;
        t = c.fixed_us + nk * c.step_us * (load > 1.f ? load : 1.f);
      } else {
        t = (float)((tiles + cus - 1) / cus) * (nk * c.step_us + c.fixed_us);
      }
      if (choice < 0 || t < best) {
        best = t;
        choice = c.id;
      }
    }
  }
  if (forced < 0) {
    // the table overrides the model only for a clear win: the timings come from a loop
    // of identical launches, and differences of a few per cent do not carry over to the
    // layer sequence
    // (a launch whose estimated live rows fill its capacity to within one tile row is looked
    // up among the all-live measurements)
    const long long m_est = estimated_rows(p);
    if (const float *us = tuned_times(m_est, p.N, p.K, EPI, p.w_kn, m_est + kTunedStep > p.rows_cap)) {
      int tuned = -1;
      for (int t = 0; t < kTunedTiles; ++t)
        if (us[t] > 0.f && (tuned < 0 || us[t] < us[tuned])) tuned = t;
      const float t_model = choice < kTunedTiles ? us[choice] : 0.f;
      const float margin = 1.f - 0.01f * (float)option_gemm_table_margin();
      if (tuned >= 0 && tuned != choice && (t_model <= 0.f || us[tuned] < margin * t_model))
        choice = tuned;
    }
  }
  switch (choice) {
    case 0:
      return launch_gemm_tile<256, 256, 2, 2, 4, 0, 1, EPI>(p, s);
    case 2:
      return launch_gemm_tile<256, 128, 3, 4, 2, 4, 1, EPI>(p, s);
    case 3:
      return launch_gemm_tile<256, 192, 2, 4, 2, 4, 1, EPI>(p, s);
    case 4:
      return launch_gemm_tile<32, 64, 4, 1, 2, 2, 0, EPI>(p, s);
    case 5:
      return launch_gemm_tile<128, 128, 2, 2, 2, 4, 0, EPI>(p, s);
    case 6:
      return launch_gemm_flat<256, 128, 3, 4, 2, 4, 1, EPI>(p, s);
    case 7:
      return launch_gemm_flat<128, 128, 3, 2, 2, 4, 0, EPI>(p, s);
    case 8:
      return launch_gemm_flat<256, 256, 2, 2, 4, 0, 1, EPI>(p, s);
    default:
      return launch_gemm_tile<128, 128, 3, 2, 2, 4, 0, EPI>(p, s);
  }
}

static int check_gemm_args(const char *who, const void *a, const void *wt, const void *c,
                           int rows_cap, int n, int k, int weight_kn) {
  BT_REQUIRE(a && wt && c, BT_ERR_INVALID_ARGUMENT, "%s: null pointer argument", who);
  BT_REQUIRE(aligned16({a, wt, c}), BT_ERR_INVALID_ARGUMENT,
             "%s: tensor pointers must be 16-byte aligned", who);
  BT_REQUIRE(rows_cap >= 0 && n > 0 && k > 0, BT_ERR_INVALID_ARGUMENT,
             "%s: rows_cap=%d n=%d k=%d out of range", who, rows_cap, n, k);
  BT_REQUIRE(k % 64 == 0, BT_ERR_UNSUPPORTED, "%s: k=%d must be a multiple of 64", who, k);
  BT_REQUIRE(n % 8 == 0, BT_ERR_UNSUPPORTED, "%s: n=%d must be a multiple of 8", who, n);
  // a 256-row tile is addressed with 32-bit byte offsets from its first row
  BT_REQUIRE(k <= (1 << 21), BT_ERR_UNSUPPORTED, "%s: k=%d is beyond 2^21", who, k);
  BT_REQUIRE(weight_kn == 0 || weight_kn == 1, BT_ERR_INVALID_ARGUMENT,
             "%s: weight_kn=%d must be 0 ([n, k] pre-pack) or 1 ([k, n] as stored)", who, weight_kn);
  // a [k, n] weight is addressed with 32-bit byte offsets from its first row
  BT_REQUIRE(!weight_kn || (long long)n * k * 2 <= 0x7fffffffLL, BT_ERR_UNSUPPORTED,
             "%s: a [k, n] weight of %d x %d halfs is beyond 2 GiB", who, k, n);
  return BT_OK;
}

}  // namespace bt

using namespace bt;

extern "C" int bt_transpose_weights(int count, const void *const *w, void *const *wt,
                                    const int *k, const int *n, void *stream) {
  BT_REQUIRE(count >= 1 && count <= 4, BT_ERR_INVALID_ARGUMENT,
             "bt_transpose_weights: count=%d outside [1, 4]", count);
  BT_REQUIRE(w && wt && k && n, BT_ERR_INVALID_ARGUMENT,
             "bt_transpose_weights: null pointer argument");
  TransposeArgs a;
  a.njobs = count;
  int tiles = 0;
  for (int i = 0; i < count; ++i) {
    BT_REQUIRE(w[i] && wt[i], BT_ERR_INVALID_ARGUMENT,
               "bt_transpose_weights: null matrix pointer #%d", i);
    BT_REQUIRE(k[i] > 0 && n[i] > 0 && k[i] % 8 == 0 && n[i] % 8 == 0, BT_ERR_UNSUPPORTED,
               "bt_transpose_weights: k=%d n=%d must be positive multiples of 8", k[i], n[i]);
    a.job[i] = TransposeJob{(const half_t *)w[i], (half_t *)wt[i], k[i], n[i],
                            (n[i] + 63) / 64, tiles};
    tiles += ((n[i] + 63) / 64) * ((k[i] + 63) / 64);
  }
  for (int i = count; i < 4; ++i) a.job[i] = a.job[0];
  transpose_kernel<<<tiles, 256, 0, as_stream(stream)>>>(a);
  BT_CHECK_LAUNCH("transpose_kernel");
  return BT_OK;
}

extern "C" int bt_transpose_weight(const void *w, void *wt, int k, int n, void *stream) {
  const void *ws[1] = {w};
  void *wts[1] = {wt};
  return bt_transpose_weights(1, ws, wts, &k, &n, stream);
}

extern "C" float bt_gemm_prepack_gain_us(long long rows, int n, int k, int epilogue) {
  const int forced = option_layer_prepack();
  if (forced >= 0) return forced ? 1e9f : -1e9f;
  // (asked for the padded batch: the layer's launches are sized for batch x seq_len rows)
  const float *nk = tuned_times(rows, n, k, epilogue, 0, 0), *kn = tuned_times(rows, n, k, epilogue, 1, 0);
  if (!nk || !kn) return 0.f;
  float best_nk = 0.f, best_kn = 0.f;
  for (int t = 0; t < kTunedTiles; ++t) {
    if (nk[t] > 0.f && (best_nk == 0.f || nk[t] < best_nk)) best_nk = nk[t];
    if (kn[t] > 0.f && (best_kn == 0.f || kn[t] < best_kn)) best_kn = kn[t];
  }
  if (best_nk == 0.f || best_kn == 0.f) return 0.f;
  // the copy is made inside the layer's first launch, beside the offsets: measured in the
  // layer sequence it adds about 0.5 us per megabyte of weight to that launch (2.4 us for
  // FFN1 of BERT-base, 7.4 us for all four matrices)
  const float pack_us = 0.5e-6f * (float)n * (float)k * sizeof(half_t);
  return best_kn - best_nk - pack_us;
}

extern "C" int bt_gemm_prepack_pays(long long rows, int n, int k, int epilogue) {
  return bt_gemm_prepack_gain_us(rows, n, k, epilogue) > 1.0f ? 1 : 0;   // asked to return a microsecond more
}

extern "C" int bt_gemm(const void *a, const void *wt, void *c, const int *valid_rows,
                       int rows_cap, int rows_hint, int n, int k, int weight_kn, void *stream) {
  int rc = check_gemm_args("bt_gemm", a, wt, c, rows_cap, n, k, weight_kn);
  if (rc) return rc;
  if (rows_cap == 0) return BT_OK;
  GemmArgs p{(const half_t *)a, (const half_t *)wt, nullptr, (half_t *)c, valid_rows, nullptr,
             rows_cap,          n,                  k,       0,           rows_hint,
             nullptr,           weight_kn};
  return launch_gemm<kEpiPlain>(p, as_stream(stream));
}

extern "C" int bt_gemm_splitk(const void *a, const void *wt, void *partials, int splits,
                              const int *valid_rows, int rows_cap, int n, int k, int weight_kn,
                              void *stream) {
  int rc = check_gemm_args("bt_gemm_splitk", a, wt, partials, rows_cap, n, k, weight_kn);
  if (rc) return rc;
  BT_REQUIRE(splits >= 1 && splits <= 16 && k % (splits * kBK) == 0, BT_ERR_INVALID_ARGUMENT,
             "bt_gemm_splitk: splits=%d must lie in [1, 16] and divide k / 64 = %d", splits,
             k / kBK);
  if (rows_cap == 0) return BT_OK;
  GemmArgs p{(const half_t *)a, (const half_t *)wt, nullptr, nullptr, valid_rows, nullptr,
             rows_cap,          n,                  k,       0,       0,          (float *)partials,
             weight_kn};
  // the small tile only: splitting k is for launches whose k loop is the whole run time
  return launch_gemm_tile<32, 64, 4, 1, 2, 2, 0, kEpiPartial>(p, as_stream(stream), splits);
}

extern "C" int bt_gemm_bias_gelu(const void *a, const void *wt, const void *bias, void *c,
                                 const int *valid_rows, int rows_cap, int rows_hint, int n, int k,
                                 int weight_kn, void *stream) {
  int rc = check_gemm_args("bt_gemm_bias_gelu", a, wt, c, rows_cap, n, k, weight_kn);
  if (rc) return rc;
  BT_REQUIRE(bias, BT_ERR_INVALID_ARGUMENT, "bt_gemm_bias_gelu: null bias");
  if (rows_cap == 0) return BT_OK;
  GemmArgs p{(const half_t *)a, (const half_t *)wt, (const half_t *)bias, (half_t *)c, valid_rows,
             nullptr,           rows_cap,           n,                    k,           0,
             rows_hint,         nullptr,            weight_kn};
  return launch_gemm<kEpiBiasGelu>(p, as_stream(stream));
}

extern "C" int bt_gemm_qkv_bias_split(const void *a, const int *a_row_index, const void *wt_qkv,
                                      const void *bias_qkv, void *qkv_heads,
                                      const int *valid_rows, int rows_cap, int rows_hint,
                                      int head_num, int size_per_head, int weight_kn,
                                      void *stream) {
  BT_REQUIRE(head_num > 0, BT_ERR_INVALID_ARGUMENT, "bt_gemm_qkv_bias_split: head_num=%d",
             head_num);
  BT_REQUIRE(size_per_head > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_gemm_qkv_bias_split: size_per_head=%d", size_per_head);
  const int H = head_num * size_per_head;
  int rc = check_gemm_args("bt_gemm_qkv_bias_split", a, wt_qkv, qkv_heads, rows_cap, 3 * H, H,
                           weight_kn);
  if (rc) return rc;
  BT_REQUIRE(bias_qkv, BT_ERR_INVALID_ARGUMENT, "bt_gemm_qkv_bias_split: null bias");
  if (rows_cap == 0) return BT_OK;
  BT_REQUIRE(!a_row_index || valid_rows, BT_ERR_INVALID_ARGUMENT,
             "bt_gemm_qkv_bias_split: a_row_index needs valid_rows (only live rows are indexed)");
  // gathered rows are addressed with 32-bit byte offsets from the start of `a`
  BT_REQUIRE(!a_row_index || (long long)rows_cap * H * 2 <= 0x7fffffffLL, BT_ERR_UNSUPPORTED,
             "bt_gemm_qkv_bias_split: a gathered input of %d x %d halfs is beyond 2 GiB", rows_cap, H);
  GemmArgs p{(const half_t *)a, (const half_t *)wt_qkv, (const half_t *)bias_qkv,
             (half_t *)qkv_heads, valid_rows, a_row_index, rows_cap, 3 * H, H, 0, rows_hint,
             nullptr, weight_kn};
  // the head-major split is the layout of the fp16 attention kernels, which are built for
  // 64-wide heads; any other head size keeps the projections token-major [rows_cap, 3H]
  // for bt_attention_generic_f16
  if (size_per_head != 64) return launch_gemm<kEpiBias>(p, as_stream(stream));
  return launch_gemm<kEpiQkvSplit>(p, as_stream(stream));
}

extern "C" int bt_gemm_qkv_mask_rows_supported(int batch_size, int seq_len, int mask_dtype) {
  if (batch_size <= 0 || batch_size > kMaskRowsMaxBatch || seq_len <= 0) return 0;
  if (mask_dtype != BT_F16 && mask_dtype != BT_F32) return 0;
  // every workgroup reads row 0 of every sequence's mask: keep that to 64 KB
  return (long long)batch_size * seq_len * (mask_dtype == BT_F32 ? 4 : 2) <= 64 * 1024;
}

extern "C" int bt_gemm_qkv_bias_split_mask_rows(
    const void *from_tensor, const void *atten_mask, int mask_dtype, int batch_size, int seq_len,
    const void *wt_qkv, const void *bias_qkv, void *qkv_heads, int *batch_idx, int *word_idx,
    int *seq_order, int rows_hint, int head_num, int size_per_head, int weight_kn,
    void *stream) {
  const char *who = "bt_gemm_qkv_bias_split_mask_rows";
  BT_REQUIRE(head_num > 0 && size_per_head > 0, BT_ERR_INVALID_ARGUMENT,
             "%s: head_num=%d size_per_head=%d", who, head_num, size_per_head);
  BT_REQUIRE(batch_size > 0 && seq_len > 0, BT_ERR_INVALID_ARGUMENT,
             "%s: batch_size=%d seq_len=%d must be positive", who, batch_size, seq_len);
  BT_REQUIRE(bt_gemm_qkv_mask_rows_supported(batch_size, seq_len, mask_dtype), BT_ERR_UNSUPPORTED,
             "%s: batch_size=%d seq_len=%d mask_dtype=%d is outside what "
             "bt_gemm_qkv_mask_rows_supported allows", who, batch_size, seq_len, mask_dtype);
  const int H = head_num * size_per_head;
  const int rows_cap = batch_size * seq_len;
  int rc = check_gemm_args(who, from_tensor, wt_qkv, qkv_heads, rows_cap, 3 * H, H, weight_kn);
  if (rc) return rc;
  BT_REQUIRE(bias_qkv && atten_mask && batch_idx, BT_ERR_INVALID_ARGUMENT,
             "%s: null pointer argument", who);
  BT_REQUIRE(aligned16({atten_mask}), BT_ERR_INVALID_ARGUMENT,
             "%s: tensor pointers must be 16-byte aligned", who);
  // gathered rows are addressed with 32-bit byte offsets from the start of the input
  BT_REQUIRE((long long)rows_cap * H * 2 <= 0x7fffffffLL, BT_ERR_UNSUPPORTED,
             "%s: a gathered input of %d x %d halfs is beyond 2 GiB", who, rows_cap, H);
  GemmArgs p{(const half_t *)from_tensor, (const half_t *)wt_qkv, (const half_t *)bias_qkv,
             (half_t *)qkv_heads, nullptr, nullptr, rows_cap, 3 * H, H, 0, rows_hint,
             nullptr, weight_kn};
  p.mask = atten_mask;
  p.mask_f32 = mask_dtype == BT_F32;
  p.mask_B = batch_size, p.mask_S = seq_len;
  p.out_batch_idx = batch_idx, p.out_word_idx = word_idx, p.out_seq_order = seq_order;
  if (size_per_head != 64) return launch_gemm<kEpiBias>(p, as_stream(stream));
  return launch_gemm<kEpiQkvSplit>(p, as_stream(stream));
}
