// fp16 MFMA GEMM family for gfx950: C[rows, N] = A[rows, K] . W[K, N] with
// fp32 accumulation and three fused epilogues (plain store, +bias+tanh-GELU,
// +bias with the Q/K/V head split).  Both operands are consumed k-contiguous:
// A as stored, W through the [N, K] pre-pack made by bt_transpose_weights.
//
// Structure of one workgroup (tile BM x BN, BK = 64):
//   * global -> LDS copies are direct-to-LDS 16-byte loads (global_load_lds):
//     no staging registers, no ds_write; each wave instruction lands 1 KB = 8
//     tile rows back to back in LDS;
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

namespace bt {

constexpr int kBK = 64;   // k extent of one LDS tile (halfs) = 8 chunks of 16 bytes

enum Epilogue { kEpiPlain = 0, kEpiBiasGelu = 1, kEpiQkvSplit = 2 };

struct GemmArgs {
  const half_t *a;      // [rows_cap, K]
  const half_t *wt;     // [N, K]
  const half_t *bias;   // [N] or null
  half_t *c;            // [rows_cap, N]  (or [3][heads][rows_cap][64] for the QKV split)
  const int *valid_rows;
  const int *a_row_index;   // optional gather: A row r is a[a_row_index[r]] (null = identity)
  int rows_cap, N, K;
  int tiles_n;
  int rows_hint;        // host-side estimate of the live rows (0 = unknown); tile choice only
};

__device__ __forceinline__ float gelu_tanh_f32(float x) {
  // 0.5 x (1 + tanh(u)) == x / (1 + exp(-2u)),  u = 0.79788456 (x + 0.044715 x^3)
  // exponent folded into one polynomial: -2 u log2(e) = x (c1 + c3 x^2)
  constexpr float c1 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  constexpr float c3 = c1 * 0.044715f;
  const float e = __builtin_amdgcn_exp2f(x * (c1 + c3 * x * x));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ int swz(int row) { return (row >> 1) & 7; }

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  // s_waitcnt immediate on gfx9: vmcnt[3:0], expcnt[6:4], lgkmcnt[11:8], vmcnt[5:4] in [15:14]
  static_assert(N >= 0 && N < 64, "vmcnt range");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

template <int BM, int BN, int STAGES, int WM, int WN, int SCHED, int EPI>
__global__ __launch_bounds__(WM *WN * 64) void gemm_kernel(GemmArgs p) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;   // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;   // 32x32 MFMA blocks per wave
  constexpr int ROWS = BM + BN;                 // A rows then W rows in one stage
  constexpr int NI = ROWS / 8 / NW;             // load instructions per wave per stage
  constexpr int STAGE_HALFS = ROWS * kBK;
  static_assert(ROWS % (8 * NW) == 0, "tile rows must split evenly over the waves");
  static_assert(STAGES >= 2 && STAGES <= 3, "pipeline depth");

  extern __shared__ __attribute__((aligned(1024))) half_t gemm_smem[];
  half_t *smem = gemm_smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int M = p.valid_rows ? min(*p.valid_rows, p.rows_cap) : p.rows_cap;

  // XCD-aware tile order over the live tiles
  int tile_m, tile_n;
  {
    const int live = ((M + BM - 1) / BM) * p.tiles_n;
    const int per = (live + 7) >> 3;
    const int L = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if ((int)blockIdx.x >= per * 8 || L >= live) return;
    tile_m = L / p.tiles_n;
    tile_n = L - tile_m * p.tiles_n;
  }
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // Per-lane source of each load instruction: instruction i of this wave fills
  // tile rows [(i*NW + wave)*8, +8); lane -> (row, slot), fetching the chunk
  // that the swizzle places in that slot.
  const half_t *gsrc[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int r = (i * NW + wave) * 8 + (lane >> 3);
    const int kc = (lane & 7) ^ swz(r);
    if (r < BM) {
      int ar = min(m0 + r, p.rows_cap - 1);
      if (p.a_row_index) ar = p.a_row_index[min(ar, M - 1)];   // live rows only hold valid indices
      gsrc[i] = p.a + (size_t)ar * p.K + kc * 8;
    } else
      gsrc[i] = p.wt + (size_t)min(n0 + r - BM, p.N - 1) * p.K + kc * 8;
  }
  auto issue_loads = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      half_t *dst = smem + stage * STAGE_HALFS + (i * NW + wave) * 8 * kBK;
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(gsrc[i] + kt * kBK),
          (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
    }
  };

  float16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int nk = p.K / kBK;
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < nk) issue_loads(s, s);

  const int fr_row = lane & 31, fr_kc = lane >> 5;
  int stage = 0;
  for (int kt = 0; kt < nk; ++kt) {
    // tile kt has landed for this wave once only the younger stages' loads are outstanding
    if (STAGES == 3 && kt + 1 < nk)
      wait_vmcnt<NI>();
    else
      wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();   // everyone's tile kt is in LDS; stage (kt-1) is free again
    asm volatile("" ::: "memory");
    if (kt + STAGES - 1 < nk) {
      int ps = stage + STAGES - 1;
      if (ps >= STAGES) ps -= STAGES;
      issue_loads(kt + STAGES - 1, ps);
    }
    const half_t *sA = smem + stage * STAGE_HALFS;
    const half_t *sB = sA + BM * kBK;

    half8_t fw[2][TN], fa[2][TM];
    auto load_frags = [&](int ks, int b) {
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const int r = wn * WTN + i * 32 + fr_row;
        fw[b][i] = *(const half8_t *)(sB + r * kBK + (((2 * ks + fr_kc) ^ swz(r + BM)) * 8));
      }
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        const int r = wm * WTM + j * 32 + fr_row;
        fa[b][j] = *(const half8_t *)(sA + r * kBK + (((2 * ks + fr_kc) ^ swz(r)) * 8));
      }
    };
    load_frags(0, 0);
    // compiler scheduling strategy that interleaves the LDS reads with the MFMAs
    if (SCHED == 0) __builtin_amdgcn_iglp_opt(0);
    if (SCHED == 1) __builtin_amdgcn_iglp_opt(1);
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      if (ks + 1 < kBK / 16) load_frags(ks + 1, (ks + 1) & 1);
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[ks & 1][i], fa[ks & 1][j],
                                                            acc[i][j], 0, 0, 0);
    }
    if (++stage == STAGES) stage = 0;
  }

  // ---- epilogue -------------------------------------------------------------
  // accumulator block (i, j), quad q: columns n..n+3 of row m with
  //   n = n0 + wn*WTN + i*32 + q*8 + (lane>>5)*4,  m = m0 + wm*WTM + j*32 + (lane&31)
  constexpr int EP = WTN + 8;   // pitch (halfs) of the wave-private staging tile
  static_assert((size_t)NW * 32 * EP <= (size_t)STAGES * STAGE_HALFS, "staging fits the ring");
  __syncthreads();              // all waves are done with the last stage
  half_t *st = smem + wave * 32 * EP;
  const int row_in = lane & 31, col_in = (lane >> 5) * 4;
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
        if (EPI != kEpiPlain) {
          const int n = min(n0 + wn * WTN + i * 32 + q * 8 + col_in, p.N - 4);
          const half4_t b = *(const half4_t *)(p.bias + n);
          v0 += (float)b[0];
          v1 += (float)b[1];
          v2 += (float)b[2];
          v3 += (float)b[3];
        }
        if (EPI == kEpiBiasGelu) {
          v0 = gelu_tanh_f32(v0);
          v1 = gelu_tanh_f32(v1);
          v2 = gelu_tanh_f32(v2);
          v3 = gelu_tanh_f32(v3);
        }
        *(half4_t *)(st + row_in * EP + i * 32 + q * 8 + col_in) =
            half4_t{(half_t)v0, (half_t)v1, (half_t)v2, (half_t)v3};
      }
    }
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += RPS) {
      const int r = r0 + sr;
      if (sr >= RPS || r >= 32) continue;   // lanes left over when 64 % CPRW != 0
      const int m = m0 + wm * WTM + j * 32 + r, n = n0 + wn * WTN + sc;
      const uint4_t v = *(const uint4_t *)(st + r * EP + sc);
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
  __shared__ half_t tile[64][64 + 2];
  int j = 0;
#pragma unroll
  for (int i = 1; i < 4; ++i)
    if (i < a.njobs && (int)blockIdx.x >= a.job[i].tile_begin) j = i;
  const TransposeJob jb = a.job[j];
  const int t = blockIdx.x - jb.tile_begin;
  const int k0 = (t / jb.tiles_n) * 64, n0 = (t % jb.tiles_n) * 64;
  // read 64 k-rows x 128 B: thread -> (row = tid/8 + 32*i, 16-byte chunk tid%8)
  const int r = threadIdx.x >> 3, c = (threadIdx.x & 7) * 8;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int k = k0 + r + 32 * i, n = n0 + c;
    uint4_t v = {0u, 0u, 0u, 0u};
    if (k < jb.K && n < jb.N) v = *(const uint4_t *)(jb.w + (size_t)k * jb.N + n);
    const half_t *h = (const half_t *)&v;
#pragma unroll
    for (int e = 0; e < 8; ++e) tile[r + 32 * i][c + e] = h[e];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int n = n0 + r + 32 * i, k = k0 + c;
    if (n < jb.N && k < jb.K) {
      half8_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = tile[c + e][r + 32 * i];
      *(half8_t *)(jb.wt + (size_t)n * jb.K + k) = o;
    }
  }
}

template <int BM, int BN, int STAGES, int WM, int WN, int SCHED, int EPI>
static int launch_gemm_tile(GemmArgs p, hipStream_t s) {
  constexpr size_t smem = (size_t)STAGES * (BM + BN) * kBK * sizeof(half_t);
  static_assert(smem <= 160 * 1024, "LDS budget");
  static bool configured = false;  // benign race: setting the attribute is idempotent
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)gemm_kernel<BM, BN, STAGES, WM, WN, SCHED, EPI>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(gemm_kernel)");
    configured = true;
  }
  const int tiles_m = (p.rows_cap + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int grid = (tiles_m * p.tiles_n + 7) / 8 * 8;
  gemm_kernel<BM, BN, STAGES, WM, WN, SCHED, EPI><<<grid, WM * WN * 64, smem, s>>>(p);
  BT_CHECK_LAUNCH("gemm_kernel");
  return BT_OK;
}

template <int EPI>
static int launch_gemm(GemmArgs p, hipStream_t s) {
  // Tile table (rows x cols, ring depth, wave grid):
  //   0: 256x256, 2, 2x4   wide outputs (FFN1 at hidden 768): one tile per CU
  //   1: 128x128, 2, 2x2   narrow outputs, short k loop (projection)
  //   2: 128x128, 3, 4x2   narrow outputs, long k loop (FFN2)
  //   3: 256x192, 2, 4x2   outputs that split into 192-wide panels but not into a
  //                        full wave of 256-wide ones (QKV at hidden 768)
  // The choice minimises (tiles per CU, rounded up) x (measured time of one tile)
  // for the estimated live rows: the exact count when every row is live, the
  // caller's hint when it has one, else 60 % of the capacity (the fill the
  // padding-free path is built for).
  int choice = option_gemm_tile();
  if (choice < 0) {
    static const int cus = [] {
      int dev = 0, n = 0;
      if (hipGetDevice(&dev) != hipSuccess ||
          hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
          n <= 0)
        n = 256;
      return n;
    }();
    const long long m_est = !p.valid_rows ? p.rows_cap
                            : p.rows_hint > 0 ? (p.rows_hint < p.rows_cap ? p.rows_hint : p.rows_cap)
                                              : (p.rows_cap * 3LL + 4) / 5;
    struct Cand {
      int id, bm, bn;
      float tile_time;   // relative time of one tile of this shape per k-step
    };
    const Cand cands[3] = {{0, 256, 256, 24.0f}, {3, 256, 192, 19.5f},
                           {p.K >= 2048 ? 2 : 1, 128, 128, 7.5f}};
    float best = 0.f;
    for (const Cand &c : cands) {
      const long long tiles = ((m_est + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn);
      const float t = (float)((tiles + cus - 1) / cus) * c.tile_time;
      if (choice < 0 || t < best) {
        best = t;
        choice = c.id;
      }
    }
  }
  switch (choice) {
    case 0:
      return launch_gemm_tile<256, 256, 2, 2, 4, 1, EPI>(p, s);
    case 2:
      return launch_gemm_tile<128, 128, 3, 4, 2, 1, EPI>(p, s);
    case 3:
      return launch_gemm_tile<256, 192, 2, 4, 2, 1, EPI>(p, s);
    default:
      return launch_gemm_tile<128, 128, 2, 2, 2, 0, EPI>(p, s);
  }
}

static int check_gemm_args(const char *who, const void *a, const void *wt, const void *c,
                           int rows_cap, int n, int k) {
  BT_REQUIRE(a && wt && c, BT_ERR_INVALID_ARGUMENT, "%s: null pointer argument", who);
  BT_REQUIRE(rows_cap >= 0 && n > 0 && k > 0, BT_ERR_INVALID_ARGUMENT,
             "%s: rows_cap=%d n=%d k=%d out of range", who, rows_cap, n, k);
  BT_REQUIRE(k % kBK == 0, BT_ERR_UNSUPPORTED, "%s: k=%d must be a multiple of %d", who, k, kBK);
  BT_REQUIRE(n % 8 == 0, BT_ERR_UNSUPPORTED, "%s: n=%d must be a multiple of 8", who, n);
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

extern "C" int bt_gemm(const void *a, const void *wt, void *c, const int *valid_rows,
                       int rows_cap, int rows_hint, int n, int k, void *stream) {
  int rc = check_gemm_args("bt_gemm", a, wt, c, rows_cap, n, k);
  if (rc) return rc;
  if (rows_cap == 0) return BT_OK;
  GemmArgs p{(const half_t *)a, (const half_t *)wt, nullptr, (half_t *)c, valid_rows, nullptr,
             rows_cap,          n,                  k,       0,           rows_hint};
  return launch_gemm<kEpiPlain>(p, as_stream(stream));
}

extern "C" int bt_gemm_bias_gelu(const void *a, const void *wt, const void *bias, void *c,
                                 const int *valid_rows, int rows_cap, int rows_hint, int n, int k,
                                 void *stream) {
  int rc = check_gemm_args("bt_gemm_bias_gelu", a, wt, c, rows_cap, n, k);
  if (rc) return rc;
  BT_REQUIRE(bias, BT_ERR_INVALID_ARGUMENT, "bt_gemm_bias_gelu: null bias");
  if (rows_cap == 0) return BT_OK;
  GemmArgs p{(const half_t *)a, (const half_t *)wt, (const half_t *)bias, (half_t *)c, valid_rows,
             nullptr,           rows_cap,           n,                    k,           0,
             rows_hint};
  return launch_gemm<kEpiBiasGelu>(p, as_stream(stream));
}

extern "C" int bt_gemm_qkv_bias_split(const void *a, const int *a_row_index, const void *wt_qkv,
                                      const void *bias_qkv, void *qkv_heads,
                                      const int *valid_rows, int rows_cap, int rows_hint,
                                      int head_num, int size_per_head, void *stream) {
  BT_REQUIRE(head_num > 0, BT_ERR_INVALID_ARGUMENT, "bt_gemm_qkv_bias_split: head_num=%d",
             head_num);
  BT_REQUIRE(size_per_head == 64, BT_ERR_UNSUPPORTED,
             "bt_gemm_qkv_bias_split: size_per_head=%d, only 64 is supported", size_per_head);
  const int H = head_num * size_per_head;
  int rc = check_gemm_args("bt_gemm_qkv_bias_split", a, wt_qkv, qkv_heads, rows_cap, 3 * H, H);
  if (rc) return rc;
  BT_REQUIRE(bias_qkv, BT_ERR_INVALID_ARGUMENT, "bt_gemm_qkv_bias_split: null bias");
  if (rows_cap == 0) return BT_OK;
  BT_REQUIRE(!a_row_index || valid_rows, BT_ERR_INVALID_ARGUMENT,
             "bt_gemm_qkv_bias_split: a_row_index needs valid_rows (only live rows are indexed)");
  GemmArgs p{(const half_t *)a, (const half_t *)wt_qkv, (const half_t *)bias_qkv,
             (half_t *)qkv_heads, valid_rows, a_row_index, rows_cap, 3 * H, H, 0, rows_hint};
  return launch_gemm<kEpiQkvSplit>(p, as_stream(stream));
}
