// fp16 MFMA GEMM family for gfx950: C[rows, N] = A[rows, K] . W[K, N] with
// fp32 accumulation and three fused epilogues (plain store, +bias+tanh-GELU,
// +bias with the Q/K/V head split).  Both operands are consumed k-contiguous:
// A as stored, W through the [N, K] pre-pack made by bt_transpose_weight.
//
// Tiling: 256 threads = 4 wave64 in a 2x2 grid, v_mfma_f32_32x32x16_f16, BK = 64,
// LDS double buffer with one barrier per k-step, global->register prefetch of
// the next k-tile issued before the MFMAs of the current one.  The MFMA "A"
// operand is the weight tile and the "B" operand the activation tile, so each
// lane's accumulator quad holds 4 consecutive output columns of one row and the
// epilogue stores 8-byte packed fp16.
//
// Rows are bounded on the device: a block whose first row is past the live row
// count (read from `valid_rows`) retires before touching LDS.
#include "common.h"

namespace bt {

constexpr int kBK = 64;        // k extent of one LDS tile (halfs)
constexpr int kLdk = kBK + 8;  // padded LDS row (144 B): conflict-free 16-byte reads
constexpr int kGemmThreads = 256;

enum Epilogue { kEpiPlain = 0, kEpiBiasGelu = 1, kEpiQkvSplit = 2 };

struct GemmArgs {
  const half_t *a;      // [rows_cap, K]
  const half_t *wt;     // [N, K]
  const half_t *bias;   // [N] or null
  half_t *c;            // [rows_cap, N]  (or [3][heads][rows_cap][64] for the QKV split)
  const int *valid_rows;
  int rows_cap, N, K;
  int head_num;         // QKV split only
  int tiles_n;
};

__device__ __forceinline__ float gelu_tanh_f32(float x) {
  // 0.5 x (1 + tanh(u)) == x * sigmoid(2u),  u = 0.79788456 (x + 0.044715 x^3)
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return __fdividef(x, 1.0f + __expf(-2.0f * u));
}

template <int BM, int BN, int EPI>
__global__ __launch_bounds__(kGemmThreads) void gemm_kernel(GemmArgs p) {
  constexpr int WTM = BM / 2, WTN = BN / 2;   // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32; // 32x32 MFMA blocks per wave
  constexpr int PA = BM / 32, PB = BN / 32;   // 16-byte global loads per thread per k-tile

  extern __shared__ __attribute__((aligned(16))) half_t smem[];
  half_t *sA = smem;                       // [2][BM][kLdk]
  half_t *sB = smem + 2 * BM * kLdk;       // [2][BN][kLdk]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  const int tile_m = blockIdx.x / p.tiles_n;
  const int tile_n = blockIdx.x - tile_m * p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int M = p.valid_rows ? min(*p.valid_rows, p.rows_cap) : p.rows_cap;
  if (m0 >= M) return;

  // global -> register staging: thread covers chunk (row = tid/8 + 32*pass, col = tid%8)
  const int ld_row = tid >> 3, ld_col = (tid & 7) * 8;
  const half_t *ga[PA];
  const half_t *gb[PB];
#pragma unroll
  for (int i = 0; i < PA; ++i) {
    int r = min(m0 + ld_row + 32 * i, p.rows_cap - 1);
    ga[i] = p.a + (size_t)r * p.K + ld_col;
  }
#pragma unroll
  for (int i = 0; i < PB; ++i) {
    int r = min(n0 + ld_row + 32 * i, p.N - 1);
    gb[i] = p.wt + (size_t)r * p.K + ld_col;
  }
  uint4_t ra[PA], rb[PB];

  auto load_global = [&](int kt) {
#pragma unroll
    for (int i = 0; i < PA; ++i) ra[i] = *(const uint4_t *)(ga[i] + kt * kBK);
#pragma unroll
    for (int i = 0; i < PB; ++i) rb[i] = *(const uint4_t *)(gb[i] + kt * kBK);
  };
  auto store_lds = [&](int buf) {
    half_t *da = sA + buf * BM * kLdk + ld_row * kLdk + ld_col;
    half_t *db = sB + buf * BN * kLdk + ld_row * kLdk + ld_col;
#pragma unroll
    for (int i = 0; i < PA; ++i) *(uint4_t *)(da + 32 * i * kLdk) = ra[i];
#pragma unroll
    for (int i = 0; i < PB; ++i) *(uint4_t *)(db + 32 * i * kLdk) = rb[i];
  };

  float16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int nk = p.K / kBK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  const int fr_row = lane & 31, fr_k = (lane >> 5) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) load_global(kt + 1);
    const half_t *tA = sA + buf * BM * kLdk + (wm * WTM + fr_row) * kLdk + fr_k;
    const half_t *tB = sB + buf * BN * kLdk + (wn * WTN + fr_row) * kLdk + fr_k;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      half8_t fw[TN], fa[TM];
#pragma unroll
      for (int i = 0; i < TN; ++i) fw[i] = *(const half8_t *)(tB + i * 32 * kLdk + ks * 16);
#pragma unroll
      for (int j = 0; j < TM; ++j) fa[j] = *(const half8_t *)(tA + j * 32 * kLdk + ks * 16);
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[i], fa[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) store_lds(buf ^ 1);
    __syncthreads();
  }

  // epilogue: lane holds, per 32x32 block and quad q, columns n..n+3 of row m
  const int row_in = lane & 31, col_in = (lane >> 5) * 4;
#pragma unroll
  for (int j = 0; j < TM; ++j) {
    const int m = m0 + wm * WTM + j * 32 + row_in;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < TN; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * WTN + i * 32 + q * 8 + col_in;
        if (n >= p.N) continue;
        float v0 = acc[i][j][4 * q + 0], v1 = acc[i][j][4 * q + 1];
        float v2 = acc[i][j][4 * q + 2], v3 = acc[i][j][4 * q + 3];
        if (EPI != kEpiPlain) {
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
        half4_t o = {(half_t)v0, (half_t)v1, (half_t)v2, (half_t)v3};
        if (EPI == kEpiQkvSplit) {
          // column n = which*H + g*64 + dd  ->  [which][g][m][dd]
          const int hg = n >> 6, dd = n & 63;   // hg = which*head_num + g
          *(half4_t *)(p.c + ((size_t)hg * p.rows_cap + m) * 64 + dd) = o;
        } else {
          *(half4_t *)(p.c + (size_t)m * p.N + n) = o;
        }
      }
    }
  }
}

// ---- weight pre-pack: wt[n][k] = w[k][n], 64x64 tiles through LDS ---------
__global__ __launch_bounds__(256) void transpose_kernel(const half_t *__restrict__ w,
                                                        half_t *__restrict__ wt, int K, int N) {
  __shared__ half_t tile[64][64 + 2];
  const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    int k = k0 + r, n = n0 + tx;
    tile[r][tx] = (k < K && n < N) ? w[(size_t)k * N + n] : (half_t)0;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    int n = n0 + r, k = k0 + tx;
    if (n < N && k < K) wt[(size_t)n * K + k] = tile[tx][r];
  }
}

template <int BM, int BN, int EPI>
static int launch_gemm_tile(GemmArgs p, hipStream_t s) {
  constexpr size_t smem = (size_t)2 * (BM + BN) * kLdk * sizeof(half_t);
  static bool configured = false;  // benign race: the attribute is idempotent
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)gemm_kernel<BM, BN, EPI>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(gemm_kernel)");
    configured = true;
  }
  const int tiles_m = (p.rows_cap + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  gemm_kernel<BM, BN, EPI><<<tiles_m * p.tiles_n, kGemmThreads, smem, s>>>(p);
  BT_CHECK_LAUNCH("gemm_kernel");
  return BT_OK;
}

template <int EPI>
static int launch_gemm(GemmArgs p, hipStream_t s) {
  // Tile choice: the largest tile that still gives the 256 CUs about a full
  // wave of workgroups; small problems fall to 128x128.
  int choice = option_gemm_tile();
  if (choice < 0) {
    const long long t256 = (long long)((p.rows_cap + 255) / 256) * ((p.N + 255) / 256);
    const long long t256x128 = (long long)((p.rows_cap + 255) / 256) * ((p.N + 127) / 128);
    if (t256 >= 200)
      choice = 0;
    else if (t256x128 >= 200)
      choice = 1;
    else
      choice = 2;
  }
  switch (choice) {
    case 0:
      return launch_gemm_tile<256, 256, EPI>(p, s);
    case 1:
      return launch_gemm_tile<256, 128, EPI>(p, s);
    default:
      return launch_gemm_tile<128, 128, EPI>(p, s);
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

extern "C" int bt_transpose_weight(const void *w, void *wt, int k, int n, void *stream) {
  BT_REQUIRE(w && wt, BT_ERR_INVALID_ARGUMENT, "bt_transpose_weight: null pointer argument");
  BT_REQUIRE(k > 0 && n > 0, BT_ERR_INVALID_ARGUMENT, "bt_transpose_weight: k=%d n=%d", k, n);
  dim3 grid((n + 63) / 64, (k + 63) / 64);
  transpose_kernel<<<grid, 256, 0, as_stream(stream)>>>((const half_t *)w, (half_t *)wt, k, n);
  BT_CHECK_LAUNCH("transpose_kernel");
  return BT_OK;
}

extern "C" int bt_gemm(const void *a, const void *wt, void *c, const int *valid_rows,
                       int rows_cap, int n, int k, void *stream) {
  int rc = check_gemm_args("bt_gemm", a, wt, c, rows_cap, n, k);
  if (rc) return rc;
  if (rows_cap == 0) return BT_OK;
  GemmArgs p{(const half_t *)a, (const half_t *)wt, nullptr, (half_t *)c, valid_rows,
             rows_cap,          n,                  k,       0,           0};
  return launch_gemm<kEpiPlain>(p, as_stream(stream));
}

extern "C" int bt_gemm_bias_gelu(const void *a, const void *wt, const void *bias, void *c,
                                 const int *valid_rows, int rows_cap, int n, int k,
                                 void *stream) {
  int rc = check_gemm_args("bt_gemm_bias_gelu", a, wt, c, rows_cap, n, k);
  if (rc) return rc;
  BT_REQUIRE(bias, BT_ERR_INVALID_ARGUMENT, "bt_gemm_bias_gelu: null bias");
  if (rows_cap == 0) return BT_OK;
  GemmArgs p{(const half_t *)a, (const half_t *)wt, (const half_t *)bias, (half_t *)c, valid_rows,
             rows_cap,          n,                  k,                    0,           0};
  return launch_gemm<kEpiBiasGelu>(p, as_stream(stream));
}

extern "C" int bt_gemm_qkv_bias_split(const void *a, const void *wt_qkv, const void *bias_qkv,
                                      void *qkv_heads, const int *valid_rows, int rows_cap,
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
  GemmArgs p{(const half_t *)a, (const half_t *)wt_qkv, (const half_t *)bias_qkv,
             (half_t *)qkv_heads, valid_rows, rows_cap, 3 * H, H, head_num, 0};
  return launch_gemm<kEpiQkvSplit>(p, as_stream(stream));
}
