// The OperationType::FP32 flavour of the encoder layer on gfx950: every tensor
// is float, every product runs on v_mfma_f32_32x32x2_f32 (true fp32 operands and
// accumulators).  Three kernels:
//
//   f32_gemm_kernel       C = A[M,K] . W[K,N] (+bias, +tanh-GELU), W row-major as the
//                         caller stores it (no pre-pack: a row-major W tile already is the
//                         MFMA "B" operand), optional row gather on A.  Role of the
//                         reference's cuBLAS calls for float (gemm.cu:32-39) and of
//                         gemm_bias_gelu<float> / add_bias_gelu<float>
//                         (gemm_bias_act.cu:24-75).
//   f32_attention_kernel  fused softmax(scale Q K^T + bias + (mask-1) 10000) V over
//                         token-major [rows, 3H] projections, K / V streamed in 32-key
//                         tiles with an online softmax.  Role of the unfused float path
//                         (attention_nofused.cu:27-114, softmax.h:25-60,103-140) without
//                         its [B,h,S,S] logits buffer and its four transposes.
//   f32_layernorm_kernel  add-bias + residual + LayerNorm, in place on packed rows or
//                         scattered to the padded layout with zero fill
//                         (layernorm.h:20-40, layernorm.cu:89-148 for float).
//
// fp32 MFMA runs at 1/16 of the fp16 rate, so both MFMA kernels are compute bound with
// a trivial memory system: one LDS buffer pair, register-staged global loads, scalar
// ds_read operands (4 LDS reads feed 256 clocks of MFMA).
#include "common.h"

namespace bt {

typedef float float2_t __attribute__((ext_vector_type(2)));

namespace {

constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kDeadLogit = -1.0e30f;

__device__ __forceinline__ float gelu_tanh_exact(float x) {
  // 0.5 x (1 + tanh(u)) == x / (1 + exp(-2u)),  u = 0.79788456 (x + 0.044715 x^3)
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  return x / (1.0f + __expf(-2.0f * u));
}

// ---------------------------------------------------------------------------
// GEMM
// ---------------------------------------------------------------------------
struct F32GemmArgs {
  const float *a;      // [rows_cap or more, K]
  const float *w;      // [K, N]
  const float *bias;   // [N] or null
  float *c;            // [rows_cap, N]
  const int *valid_rows;
  const int *a_row_index;   // optional gather: A row r is a[a_row_index[r]]
  int rows_cap, N, K;
  int gelu;
};

constexpr int kF32BK = 16;

// 256 threads = 2 x 2 waves, each wave a (BM/2) x (BN/2) block of 32x32 MFMA tiles.
// LDS: A tile k-major [16][BM+4] (the gather / transposition happens in the store),
// W tile [16][BN+32]; both strides make the operand reads of one wave conflict free.
template <int BM, int BN>
__global__ __launch_bounds__(256) void f32_gemm_kernel(F32GemmArgs p) {
  constexpr int SA = BM + 4, SW = BN + 32;
  constexpr int WM = BM / 2, WN = BN / 2, MT = WM / 32, NT = WN / 32;
  constexpr int AV = BM / 64;          // float4 of A per thread and k-tile
  constexpr int WV = BN / 64;          // float4 of W per thread and k-tile
  __shared__ float sA[2][kF32BK * SA];
  __shared__ __attribute__((aligned(16))) float sW[2][kF32BK * SW];

  const int M = p.valid_rows ? min(*p.valid_rows, p.rows_cap) : p.rows_cap;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (m0 >= M) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> register staging
  const int a_kq = tid & 3;            // which float4 of the 16 k
  const float *a_src[AV];
#pragma unroll
  for (int i = 0; i < AV; ++i) {
    const int r = m0 + (tid >> 2) + i * 64;
    a_src[i] = nullptr;
    if (r < M) {
      const size_t row = p.a_row_index ? (size_t)p.a_row_index[r] : (size_t)r;
      a_src[i] = p.a + row * p.K + 4 * a_kq;
    }
  }
  constexpr int WPR = BN / 4;          // float4 per W tile row
  constexpr int WROWS = 256 / WPR;     // tile rows covered by one pass of the workgroup
  const int w_k = tid / WPR, w_n = n0 + 4 * (tid % WPR);
  const bool w_ok = w_n < p.N;

  float4_t ra[AV], rw[WV];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < AV; ++i) {
      ra[i] = float4_t{0.f, 0.f, 0.f, 0.f};
      if (a_src[i] && k0 + 4 * a_kq < p.K) ra[i] = *(const float4_t *)(a_src[i] + k0);
    }
#pragma unroll
    for (int i = 0; i < WV; ++i) {
      const int k = k0 + w_k + i * WROWS;
      rw[i] = float4_t{0.f, 0.f, 0.f, 0.f};
      if (w_ok && k < p.K) rw[i] = *(const float4_t *)(p.w + (size_t)k * p.N + w_n);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < AV; ++i) {
      float *d = &sA[buf][(4 * a_kq) * SA + (tid >> 2) + i * 64];
#pragma unroll
      for (int j = 0; j < 4; ++j) d[j * SA] = ra[i][j];
    }
#pragma unroll
    for (int i = 0; i < WV; ++i)
      *(float4_t *)&sW[buf][(w_k + i * WROWS) * SW + 4 * (tid % WPR)] = rw[i];
  };

  float16_t acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.f;

  const int nk = (p.K + kF32BK - 1) / kF32BK;
  fetch(0);
  stash(0);
  __syncthreads();
  int cur = 0;
  for (int kt = 0; kt < nk; ++kt) {
    if (kt + 1 < nk) fetch((kt + 1) * kF32BK);
    const float *a_base = &sA[cur][half * SA + wm * WM + l32];
    const float *w_base = &sW[cur][half * SW + wn * WN + l32];
#pragma unroll
    for (int kk = 0; kk < kF32BK / 2; ++kk) {
      float af[MT], bf[NT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt] = a_base[2 * kk * SA + mt * 32];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) bf[nt] = w_base[2 * kk * SW + nt * 32];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[mt], bf[nt], acc[mt][nt], 0, 0, 0);
    }
    if (kt + 1 < nk) stash(cur ^ 1);
    __syncthreads();
    cur ^= 1;
  }

  // accumulator element i of a 32x32 tile: row 8*(i/4) + 4*half + i%4, column l32
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int col = n0 + wn * WN + nt * 32 + l32;
    if (col >= p.N) continue;
    const float bv = p.bias ? p.bias[col] : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = m0 + wm * WM + mt * 32 + 8 * (i >> 2) + 4 * half + (i & 3);
        if (row >= M) continue;
        float v = acc[mt][nt][i] + bv;
        if (p.gelu) v = gelu_tanh_exact(v);
        p.c[(size_t)row * p.N + col] = v;
      }
  }
}

// ---------------------------------------------------------------------------
// attention
// ---------------------------------------------------------------------------
struct F32AttArgs {
  const float *qkv;    // [rows, 3H], QKV bias already added
  float *out;          // [rows, H]
  const int *batch_idx;
  const float *mask;   // optional [B,S,S]
  const float *bias;   // optional [heads,S,S]
  int B, S, rows_cap, heads;
  float scale;
  int padded_rows;
};

constexpr int kF32KT = 32;   // keys per tile
constexpr int kF32BQ = 128;  // queries per workgroup (32 per wave)

// One workgroup = 128 queries of one (sequence, head).  The logits are computed
// transposed, S^T = K.Q^T (lane = query, 16 keys per lane), so their accumulator is
// directly the "B" operand of O^T = V^T.P^T and the softmax statistics of a query are
// lane-local up to one exchange between the two halves of the wave.  The MFMA's k index
// may be any bijection as long as both operands agree; it is chosen so that Q and K are
// read as float4 (k = half*D/2 + step) and P needs no shuffle (key of step j in half h
// = 8*(j/4) + 4*h + j%4, the accumulator's own row order).
template <int ND>
__global__ __launch_bounds__(256) void f32_attention_kernel(F32AttArgs p) {
  constexpr int D = 32 * ND;
  constexpr int SK = D + 4, SV = D + 8;
  __shared__ __attribute__((aligned(16))) float sK[kF32KT * SK];
  __shared__ __attribute__((aligned(16))) float sV[kF32KT * SV];

  const int b = blockIdx.z, head = blockIdx.y;
  const int seq_start = p.batch_idx[b];
  const int len = p.batch_idx[b + 1] - seq_start;
  const int klen = (p.mask && p.padded_rows) ? p.S : len;
  const int row_start = p.padded_rows ? b * p.S : seq_start;
  const int nq = p.padded_rows ? p.S : len;
  const int q0 = blockIdx.x * kF32BQ;
  if (q0 >= nq || klen <= 0) {
    // padded rows of an empty sequence still get defined output: zeros
    if (q0 < nq) {
      const int H = p.heads * D;
      for (int i = threadIdx.x; i < kF32BQ * D; i += 256) {
        const int q = q0 + i / D;
        if (q < nq) p.out[(size_t)(row_start + q) * H + head * D + i % D] = 0.f;
      }
    }
    return;
  }

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int H = p.heads * D;
  const size_t ld = (size_t)3 * H;
  const float *Q = p.qkv + (size_t)row_start * ld + head * D;
  const float *K = Q + H;
  const float *V = K + H;

  const int q = q0 + wave * 32 + l32;       // this lane's query
  const bool wave_live = q0 + wave * 32 < nq;
  const int qc = min(q, nq - 1);

  // Q^T operand: lane (query, half) holds Q[q][half*D/2 + i]
  float qf[D / 2];
#pragma unroll
  for (int i = 0; i < D / 8; ++i) {
    const float4_t v = *(const float4_t *)(Q + (size_t)qc * ld + half * (D / 2) + 4 * i);
#pragma unroll
    for (int j = 0; j < 4; ++j) qf[4 * i + j] = v[j];
  }

  // tile staging: 32 keys x D floats of K and of V, ND float4 each per thread
  constexpr int CPR = D / 4;   // float4 per row
  float4_t rk[ND], rv[ND];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int idx = tid + 256 * i;
      const int key = min(k0 + idx / CPR, klen - 1);
      const size_t off = (size_t)key * ld + 4 * (idx % CPR);
      rk[i] = *(const float4_t *)(K + off);
      rv[i] = *(const float4_t *)(V + off);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int idx = tid + 256 * i;
      *(float4_t *)&sK[(idx / CPR) * SK + 4 * (idx % CPR)] = rk[i];
      *(float4_t *)&sV[(idx / CPR) * SV + 4 * (idx % CPR)] = rv[i];
    }
  };

  float16_t o[ND];
#pragma unroll
  for (int dt = 0; dt < ND; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m_run = kDeadLogit, l_run = 0.f;

  const float c = p.scale * kLog2eF;
  const float *mrow = p.mask ? p.mask + ((size_t)b * p.S + min(q, p.S - 1)) * p.S : nullptr;
  const float *brow = p.bias ? p.bias + ((size_t)head * p.S + min(q, p.S - 1)) * p.S : nullptr;

  const int ntiles = (klen + kF32KT - 1) / kF32KT;
  fetch(0);
  stash();
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    if (t + 1 < ntiles) fetch((t + 1) * kF32KT);
    if (wave_live) {
      const int k0 = t * kF32KT;
      // S^T = K . Q^T : A operand K[key = l32][k = half*D/2 + i]
      float16_t s;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] = 0.f;
      const float *kp = &sK[l32 * SK + half * (D / 2)];
#pragma unroll
      for (int i4 = 0; i4 < D / 8; ++i4) {
        const float4_t kv = *(const float4_t *)(kp + 4 * i4);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          s = __builtin_amdgcn_mfma_f32_32x32x2f32(kv[j], qf[4 * i4 + j], s, 0, 0, 0);
      }
      // logits in the exp2 domain; accumulator row i is key k0 + 8*(i/4) + 4*half + i%4
      float x[16];
      float tmax = kDeadLogit;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = k0 + 8 * (i >> 2) + 4 * half + (i & 3);
        float v = s[i] * c;
        if (key < klen) {
          if (brow) v += brow[key] * kLog2eF;
          if (mrow) v += (mrow[key] - 1.0f) * (10000.0f * kLog2eF);
        } else {
          v = kDeadLogit;
        }
        x[i] = v;
        tmax = fmaxf(tmax, v);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run, tmax);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = k0 + 8 * (i >> 2) + 4 * half + (i & 3);
        const float pv = key < klen ? __builtin_amdgcn_exp2f(x[i] - m_new) : 0.f;
        x[i] = pv;
        psum += pv;
      }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
      // O^T += V^T . P^T : A operand V[key(j, half)][d = 32*dt + l32], B operand P^T = x[j]
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float *vp = &sV[(8 * (j >> 2) + 4 * half + (j & 3)) * SV + l32];
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[32 * dt], x[j], o[dt], 0, 0, 0);
      }
    }
    __syncthreads();
    if (t + 1 < ntiles) {
      stash();
      __syncthreads();
    }
  }

  if (!wave_live || q >= nq) return;
  const float l_all = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = 1.0f / (l_all + 1e-6f);
  // accumulator element i of d-tile dt: d = 32*dt + 8*(i/4) + 4*half + i%4, query = l32
  float *orow = p.out + (size_t)(row_start + q) * H + head * D;
#pragma unroll
  for (int dt = 0; dt < ND; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float4_t v;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = o[dt][4 * g + r] * inv;
      *(float4_t *)(orow + 32 * dt + 8 * g + 4 * half) = v;
    }
}

// ---------------------------------------------------------------------------
// add-bias + residual + LayerNorm
// ---------------------------------------------------------------------------
constexpr int kF32LnRows = 4;

// One wave per row, float4 per lane, the row in registers between the two passes.
template <int NC, bool RESTORE>
__global__ __launch_bounds__(kF32LnRows *kWave) void f32_layernorm_kernel(
    const float4_t *src, const float4_t *__restrict__ residual, const float4_t *__restrict__ bias,
    const float4_t *__restrict__ gamma, const float4_t *__restrict__ beta, float4_t *dst,
    const int *__restrict__ idx, const int *__restrict__ residual_row_index, int S, int rows_cap,
    int chunks, float inv_n, float eps) {
  const int r = blockIdx.x * kF32LnRows + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows_cap) return;
  size_t src_row;
  if (RESTORE) {
    const int b = r / S, s = r - b * S;
    const int start = idx[b], len = idx[b + 1] - start;
    if (s >= len) {
      const float4_t z = {0.f, 0.f, 0.f, 0.f};
      for (int c = lane; c < chunks; c += kWave) dst[(size_t)r * chunks + c] = z;
      return;
    }
    src_row = (size_t)start + s;
  } else {
    const int M = idx ? *idx : rows_cap;
    if (r >= M) return;
    src_row = r;
  }
  const float4_t *a = src + src_row * chunks;
  const size_t res_row = residual_row_index ? (size_t)residual_row_index[src_row] : src_row;
  const float4_t *rs = residual + res_row * chunks;
  float4_t v[NC];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = lane + i * kWave;
    v[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (c < chunks) {
      v[i] = a[c] + rs[c] + bias[c];
      sum += v[i][0] + v[i][1] + v[i][2] + v[i][3];
    }
  }
  const float mean = wave_sum(sum) * inv_n;
  float sq = 0.f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = lane + i * kWave;
    if (c < chunks) {
      v[i] -= mean;
      sq += v[i][0] * v[i][0] + v[i][1] * v[i][1] + v[i][2] * v[i][2] + v[i][3] * v[i][3];
    }
  }
  const float rstd = rsqrtf(wave_sum(sq) * inv_n + eps);
  float4_t *o = dst + (size_t)r * chunks;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = lane + i * kWave;
    if (c < chunks) o[c] = v[i] * rstd * gamma[c] + beta[c];
  }
}

template <bool RESTORE>
int launch_f32_ln(const void *src, const void *residual, const void *bias, const void *gamma,
                  const void *beta, void *dst, const int *idx, const int *residual_row_index,
                  int S, int rows_cap, int H, float eps, hipStream_t s, const char *who) {
  BT_REQUIRE(H > 0 && H % 4 == 0, BT_ERR_UNSUPPORTED, "%s: hidden_dim %d must be a multiple of 4",
             who, H);
  const int chunks = H / 4;
  const int nc = (chunks + kWave - 1) / kWave;
  BT_REQUIRE(nc <= 16, BT_ERR_UNSUPPORTED, "%s: hidden_dim %d exceeds 4096", who, H);
  if (rows_cap == 0) return BT_OK;
  const int grid = (rows_cap + kF32LnRows - 1) / kF32LnRows;
  const float inv_n = 1.0f / (float)H;
#define BT_F32_LN(NC_)                                                                          \
  f32_layernorm_kernel<NC_, RESTORE><<<grid, kF32LnRows * kWave, 0, s>>>(                       \
      (const float4_t *)src, (const float4_t *)residual, (const float4_t *)bias,                \
      (const float4_t *)gamma, (const float4_t *)beta, (float4_t *)dst, idx, residual_row_index, \
      S, rows_cap, chunks, inv_n, eps)
  if (nc <= 2)
    BT_F32_LN(2);
  else if (nc <= 4)
    BT_F32_LN(4);
  else if (nc <= 8)
    BT_F32_LN(8);
  else
    BT_F32_LN(16);
#undef BT_F32_LN
  BT_CHECK_LAUNCH(who);
  return BT_OK;
}

}  // namespace
}  // namespace bt

using namespace bt;

extern "C" int bt_gemm_f32(const void *a, const int *a_row_index, const void *w, const void *bias,
                           void *c, int gelu, const int *valid_rows, int rows_cap, int n, int k,
                           void *stream) {
  BT_REQUIRE(a && w && c, BT_ERR_INVALID_ARGUMENT, "bt_gemm_f32: null pointer argument");
  BT_REQUIRE(rows_cap >= 0 && n > 0 && k > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_gemm_f32: sizes must be positive");
  BT_REQUIRE(n % 4 == 0 && k % 4 == 0, BT_ERR_UNSUPPORTED,
             "bt_gemm_f32: n (%d) and k (%d) must be multiples of 4", n, k);
  BT_REQUIRE(!a_row_index || valid_rows, BT_ERR_INVALID_ARGUMENT,
             "bt_gemm_f32: a_row_index needs valid_rows");
  BT_REQUIRE(!gelu || bias, BT_ERR_INVALID_ARGUMENT, "bt_gemm_f32: gelu needs a bias");
  BT_REQUIRE((long long)rows_cap * n < (1ll << 40), BT_ERR_UNSUPPORTED, "bt_gemm_f32: too large");
  if (rows_cap == 0) return BT_OK;
  F32GemmArgs p{(const float *)a, (const float *)w, (const float *)bias, (float *)c, valid_rows,
                a_row_index, rows_cap, n, k, gelu ? 1 : 0};
  // 128x128 tiles once they fill the chip; 64x64 below that
  const long long big = (long long)((rows_cap + 127) / 128) * ((n + 127) / 128);
  if (big >= 192) {
    dim3 grid((n + 127) / 128, (rows_cap + 127) / 128);
    BT_REQUIRE(grid.y <= 65535, BT_ERR_UNSUPPORTED, "bt_gemm_f32: too many rows");
    f32_gemm_kernel<128, 128><<<grid, 256, 0, as_stream(stream)>>>(p);
  } else {
    dim3 grid((n + 63) / 64, (rows_cap + 63) / 64);
    BT_REQUIRE(grid.y <= 65535, BT_ERR_UNSUPPORTED, "bt_gemm_f32: too many rows");
    f32_gemm_kernel<64, 64><<<grid, 256, 0, as_stream(stream)>>>(p);
  }
  BT_CHECK_LAUNCH("bt_gemm_f32");
  return BT_OK;
}

extern "C" int bt_attention_f32(const void *qkv, void *out, const int *batch_idx,
                                const void *atten_mask, const void *attention_bias,
                                int batch_size, int seq_len, int rows_cap, int head_num,
                                int size_per_head, float scale, int padded_rows, void *stream) {
  BT_REQUIRE(qkv && out && batch_idx, BT_ERR_INVALID_ARGUMENT,
             "bt_attention_f32: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0 && head_num > 0 && rows_cap >= 0,
             BT_ERR_INVALID_ARGUMENT, "bt_attention_f32: sizes must be positive");
  BT_REQUIRE(size_per_head == 32 || size_per_head == 64 || size_per_head == 128,
             BT_ERR_UNSUPPORTED, "bt_attention_f32: size_per_head %d (supported: 32, 64, 128)",
             size_per_head);
  BT_REQUIRE(batch_size <= 65535 && head_num <= 65535, BT_ERR_UNSUPPORTED,
             "bt_attention_f32: batch_size / head_num exceed the grid limit");
  BT_REQUIRE(!padded_rows || (long long)batch_size * seq_len <= rows_cap, BT_ERR_INVALID_ARGUMENT,
             "bt_attention_f32: padded rows need rows_cap >= batch_size * seq_len");
  F32AttArgs p{(const float *)qkv, (float *)out, batch_idx, (const float *)atten_mask,
               (const float *)attention_bias, batch_size, seq_len, rows_cap, head_num, scale,
               padded_rows ? 1 : 0};
  dim3 grid((seq_len + kF32BQ - 1) / kF32BQ, head_num, batch_size);
  hipStream_t s = as_stream(stream);
  if (size_per_head == 32)
    f32_attention_kernel<1><<<grid, 256, 0, s>>>(p);
  else if (size_per_head == 64)
    f32_attention_kernel<2><<<grid, 256, 0, s>>>(p);
  else
    f32_attention_kernel<4><<<grid, 256, 0, s>>>(p);
  BT_CHECK_LAUNCH("bt_attention_f32");
  return BT_OK;
}

extern "C" int bt_add_bias_residual_layernorm_f32(void *out, const void *residual,
                                                  const int *residual_row_index, const void *bias,
                                                  const void *gamma, const void *beta,
                                                  const int *valid_rows, int rows_cap,
                                                  int hidden_dim, float eps, void *stream) {
  BT_REQUIRE(out && residual && bias && gamma && beta, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm_f32: null pointer argument");
  BT_REQUIRE(rows_cap >= 0, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm_f32: negative rows_cap");
  BT_REQUIRE(!residual_row_index || valid_rows, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm_f32: residual_row_index needs valid_rows");
  return launch_f32_ln<false>(out, residual, bias, gamma, beta, out, valid_rows,
                              residual_row_index, 1, rows_cap, hidden_dim, eps, as_stream(stream),
                              "bt_add_bias_residual_layernorm_f32");
}

extern "C" int bt_add_bias_residual_layernorm_restore_f32(
    const void *out, const void *residual, const void *bias, const void *gamma, const void *beta,
    void *out_padded, const int *batch_idx, int batch_size, int seq_len, int hidden_dim, float eps,
    void *stream) {
  BT_REQUIRE(out && residual && bias && gamma && beta && out_padded && batch_idx,
             BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm_restore_f32: null pointer argument");
  BT_REQUIRE(batch_size > 0 && seq_len > 0, BT_ERR_INVALID_ARGUMENT,
             "bt_add_bias_residual_layernorm_restore_f32: sizes must be positive");
  BT_REQUIRE((long long)batch_size * seq_len < (1ll << 31), BT_ERR_UNSUPPORTED,
             "bt_add_bias_residual_layernorm_restore_f32: too many rows");
  return launch_f32_ln<true>(out, residual, bias, gamma, beta, out_padded, batch_idx, nullptr,
                             seq_len, batch_size * seq_len, hidden_dim, eps, as_stream(stream),
                             "bt_add_bias_residual_layernorm_restore_f32");
}
