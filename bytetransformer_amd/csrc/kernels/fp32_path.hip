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

__device__ __forceinline__ float gelu_tanh(float x) {
  // 0.5 x (1 + tanh(u)) == x / (1 + exp(-2u)),  u = 0.79788456 (x + 0.044715 x^3)
  // exponent folded into one polynomial: -2 u log2(e) = x (c1 + c3 x^2)
  constexpr float c1 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;
  constexpr float c3 = c1 * 0.044715f;
  const float e = __builtin_amdgcn_exp2f(x * (c1 + c3 * x * x));
  return x * __builtin_amdgcn_rcpf(1.0f + e);
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
constexpr int kF32CUs = 256;

// WGM x WGN waves, each a (BM/WGM) x (BN/WGN) block of 32x32 MFMA tiles.
// LDS: A tile k-major [16][BM+4] (the gather / transposition happens in the store),
// W tile [16][BN+32]; both strides make the operand reads of one wave conflict free.
template <int BM, int BN, int WGM, int WGN>
__global__ __launch_bounds__(64 * WGM *WGN) void f32_gemm_kernel(F32GemmArgs p) {
  constexpr int THREADS = 64 * WGM * WGN;
  constexpr int SA = BM + 4, SW = BN + 32;
  constexpr int WM = BM / WGM, WN = BN / WGN, MT = WM / 32, NT = WN / 32;
  constexpr int AV = BM * 4 / THREADS;     // float4 of A per thread and k-tile
  constexpr int WV = BN * 4 / THREADS;     // float4 of W per thread and k-tile
  static_assert(MT >= 1 && NT >= 1 && AV >= 1 && WV >= 1, "tile too small for the wave grid");
  __shared__ float sA[2][kF32BK * SA];
  __shared__ __attribute__((aligned(16))) float sW[2][kF32BK * SW];

  const int M = p.valid_rows ? min(*p.valid_rows, p.rows_cap) : p.rows_cap;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (m0 >= M) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int wm = wave / WGN, wn = wave % WGN;

  // global -> register staging
  const int a_kq = tid & 3;            // which float4 of the 16 k
  constexpr int AROWS = THREADS / 4;   // tile rows covered by one pass of the workgroup
  const float *a_src[AV];
#pragma unroll
  for (int i = 0; i < AV; ++i) {
    const int r = m0 + (tid >> 2) + i * AROWS;
    a_src[i] = nullptr;
    if (r < M) {
      const size_t row = p.a_row_index ? (size_t)p.a_row_index[r] : (size_t)r;
      a_src[i] = p.a + row * p.K + 4 * a_kq;
    }
  }
  constexpr int WPR = BN / 4;            // float4 per W tile row
  constexpr int WROWS = THREADS / WPR;   // tile rows covered by one pass of the workgroup
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
      float *d = &sA[buf][(4 * a_kq) * SA + (tid >> 2) + i * AROWS];
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
    // all operand fetches of the k-tile first, the MFMA chain after them: the fence keeps
    // the compiler from sinking each ds_read next to its MFMA (which exposes the LDS
    // latency once per MFMA pair instead of once per k-tile)
    float af[kF32BK / 2][MT], bf[kF32BK / 2][NT];
#pragma unroll
    for (int kk = 0; kk < kF32BK / 2; ++kk) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[kk][mt] = a_base[2 * kk * SA + mt * 32];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) bf[kk][nt] = w_base[2 * kk * SW + nt * 32];
    }
    asm volatile("" ::: "memory");
#pragma unroll
    for (int kk = 0; kk < kF32BK / 2; ++kk)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[kk][mt], bf[kk][nt], acc[mt][nt],
                                                             0, 0, 0);
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
        if (p.gelu) v = gelu_tanh(v);
        p.c[(size_t)row * p.N + col] = v;
      }
  }
}

// ---------------------------------------------------------------------------
// attention
// ---------------------------------------------------------------------------
// Four consecutive elements of a float or fp16 tensor as floats, and back.
__device__ __forceinline__ float4_t load4(const float *p) { return *(const float4_t *)p; }
__device__ __forceinline__ float4_t load4(const half_t *p) {
  const half4_t h = *(const half4_t *)p;
  return float4_t{(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
}
__device__ __forceinline__ void store4(float *p, float4_t v) { *(float4_t *)p = v; }
__device__ __forceinline__ void store4(half_t *p, float4_t v) {
  *(half4_t *)p = half4_t{(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
}

// T = float for OperationType::FP32; T = half_t serves fp16 layers whose head size the fp16
// attention kernels do not cover (they are built for 64): same kernel, operands widened to
// float on the way into LDS and registers.
template <typename T>
struct F32AttArgs {
  const T *qkv;        // [rows, 3H], QKV bias already added
  T *out;              // [rows, H]
  const int *batch_idx;
  const int *seq_order;   // optional: rank -> sequence, longest first
  const T *mask;       // optional [B,S,S]
  const T *bias;       // optional [heads,S,S]
  int B, S, rows_cap, heads;
  float scale;
  int padded_rows;
  int nqb;             // query tiles per sequence
  int balanced;        // 1: the live query tiles are dealt evenly to the CUs (common.h)
  int d;               // head size (a multiple of 8, <= the kernel's D = 32 * ND; the
                       // columns d..D-1 of Q, K and V read as zero)
};

constexpr int kF32KT = 32;   // keys per tile

// One workgroup = NW waves x 32 queries of one (sequence, head).  The logits are computed
// transposed, S^T = K.Q^T (lane = query, 16 keys per lane), so their accumulator is
// directly the "B" operand of O^T = V^T.P^T and the softmax statistics of a query are
// lane-local up to one exchange between the two halves of the wave.  The MFMA's k index
// may be any bijection as long as both operands agree; it is chosen so that Q and K are
// read as float4 (k = half*D/2 + step) and P needs no shuffle (key of step j in half h
// = 8*(j/4) + 4*h + j%4, the accumulator's own row order).
template <typename T, int ND, int NW>
__global__ __launch_bounds__(64 * NW) void f32_attention_kernel(F32AttArgs<T> p) {
  constexpr int D = 32 * ND;
  constexpr int THREADS = 64 * NW, BQ = 32 * NW;   // 32 queries per wave
  constexpr int SK = D + 4, SV = D + 8;
  __shared__ __attribute__((aligned(16))) float sK[kF32KT * SK];
  __shared__ __attribute__((aligned(16))) float sV[kF32KT * SV];

  // 1-D grid, XCD-aware: the hardware deals consecutive workgroup ids round-robin to the
  // 8 XCDs; XCD x works on the (sequence, head) pairs p = x (mod 8), the query tiles of
  // one pair back to back (its K / V then come from that XCD's L2), so every XCD sees the
  // same mix of sequence lengths however ragged the batch is.
  // Launches of more than two rounds of workgroups per CU take the balanced work list.
  int b, head, seq_start, len, qb_index;
  if (p.balanced) {
    const AttWork w = att_work_balanced<BQ>(p, blockIdx.x);
    if (!w.exists) return;
    b = w.b, head = w.head, seq_start = w.seq_start, len = w.len, qb_index = w.qb;
  } else {
    const unsigned lin = blockIdx.x, slot = lin >> 3;
    const unsigned pair = (slot / p.nqb) * 8 + (lin & 7);
    if (pair >= (unsigned)(p.B * p.heads)) return;
    const int rank = pair / p.heads;
    head = pair % p.heads;
    b = p.seq_order ? p.seq_order[rank] : rank;
    seq_start = p.batch_idx[b];
    len = p.batch_idx[b + 1] - seq_start;
    qb_index = (int)(slot % p.nqb);
  }
  const int klen = (p.mask && p.padded_rows) ? p.S : len;
  const int row_start = p.padded_rows ? b * p.S : seq_start;
  const int nq = p.padded_rows ? p.S : len;
  const int q0 = qb_index * BQ;
  if (q0 >= nq || klen <= 0) {
    // padded rows of an empty sequence still get defined output: zeros
    if (q0 < nq) {
      const int H = p.heads * p.d;
      for (int i = threadIdx.x; i < BQ * p.d; i += THREADS) {
        const int q = q0 + i / p.d;
        if (q < nq) p.out[(size_t)(row_start + q) * H + head * p.d + i % p.d] = (T)0.f;
      }
    }
    return;
  }

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, half = lane >> 5;
  const int d = p.d;
  const int H = p.heads * d;
  const size_t ld = (size_t)3 * H;
  const T *Q = p.qkv + (size_t)row_start * ld + head * d;
  const T *K = Q + H;
  const T *V = K + H;

  const int q = q0 + wave * 32 + l32;       // this lane's query
  const bool wave_live = q0 + wave * 32 < nq;
  const int qc = min(q, nq - 1);

  // Q^T operand: lane (query, half) holds Q[q][half*D/2 + i]
  float qf[D / 2];
#pragma unroll
  for (int i = 0; i < D / 8; ++i) {
    const int e = half * (D / 2) + 4 * i;
    float4_t v = {0.f, 0.f, 0.f, 0.f};
    if (e < d) v = load4(Q + (size_t)qc * ld + e);
#pragma unroll
    for (int j = 0; j < 4; ++j) qf[4 * i + j] = v[j];
  }

  // tile staging: 32 keys x D floats of K and of V, NV float4 each per thread
  constexpr int CPR = D / 4;   // float4 per row
  constexpr int NV = kF32KT * CPR / THREADS;
  float4_t rk[NV], rv[NV];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + THREADS * i;
      const int key = min(k0 + idx / CPR, klen - 1);
      const int e = 4 * (idx % CPR);
      const size_t off = (size_t)key * ld + e;
      rk[i] = rv[i] = float4_t{0.f, 0.f, 0.f, 0.f};
      if (e < d) {
        rk[i] = load4(K + off);
        rv[i] = load4(V + off);
      }
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + THREADS * i;
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
  const T *mrow = p.mask ? p.mask + ((size_t)b * p.S + min(q, p.S - 1)) * p.S : nullptr;
  const T *brow = p.bias ? p.bias + ((size_t)head * p.S + min(q, p.S - 1)) * p.S : nullptr;

  const int ntiles = (klen + kF32KT - 1) / kF32KT;
  fetch(0);
  stash();
  __syncthreads();
  const bool has_add = mrow || brow;
  const bool add_vec = (p.S & 3) == 0;
  for (int t = 0; t < ntiles; ++t) {
    const int k0 = t * kF32KT;
    // additive terms of this tile's 16 keys per lane (4 groups of 4 consecutive keys),
    // in the exp2 domain; issued ahead of the next tile's K / V so that the wait for
    // them does not include those
    float4_t add[4];
    if (has_add && wave_live) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int key = k0 + 8 * g + 4 * half;
        float4_t mv = {1.f, 1.f, 1.f, 1.f}, bv = {0.f, 0.f, 0.f, 0.f};
        if (add_vec && key + 3 < p.S) {
          if (mrow) mv = load4(mrow + key);
          if (brow) bv = load4(brow + key);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (key + r < p.S) {
              if (mrow) mv[r] = (float)mrow[key + r];
              if (brow) bv[r] = (float)brow[key + r];
            }
        }
        add[g] = (mv - 1.0f) * (10000.0f * kLog2eF) + bv * kLog2eF;
      }
    }
    if (t + 1 < ntiles) fetch((t + 1) * kF32KT);
    if (wave_live) {
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
        if (has_add) v += add[i >> 2][i & 3];
        if (key >= klen) v = kDeadLogit;
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
      // the running maximum of most queries settles after a few tiles: skip the rescale
      // of the accumulators when it moved for no query of the wave
      if (__any(alpha != 1.0f)) {
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
      }
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
  T *orow = p.out + (size_t)(row_start + q) * H + head * d;
#pragma unroll
  for (int dt = 0; dt < ND; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float4_t v;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = o[dt][4 * g + r] * inv;
      if (32 * dt + 8 * g + 4 * half < d) store4(orow + 32 * dt + 8 * g + 4 * half, v);
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
  BT_REQUIRE(aligned16({src, residual, bias, gamma, beta, dst}), BT_ERR_INVALID_ARGUMENT,
             "%s: tensor pointers must be 16-byte aligned", who);
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

template <typename T>
static int launch_generic_attention(const char *who, const void *qkv, void *out,
                                    const int *batch_idx, const int *seq_order,
                                    const void *atten_mask, const void *attention_bias,
                                    int batch_size, int seq_len, int rows_cap, int head_num,
                                    int size_per_head, float scale, int padded_rows,
                                    hipStream_t s) {
  BT_REQUIRE(qkv && out && batch_idx, BT_ERR_INVALID_ARGUMENT, "%s: null pointer argument", who);
  BT_REQUIRE(aligned16({qkv, out, atten_mask, attention_bias}), BT_ERR_INVALID_ARGUMENT,
             "%s: tensor pointers must be 16-byte aligned", who);
  BT_REQUIRE(batch_size > 0 && seq_len > 0 && head_num > 0 && rows_cap >= 0,
             BT_ERR_INVALID_ARGUMENT, "%s: sizes must be positive", who);
  BT_REQUIRE(size_per_head > 0 && size_per_head % 8 == 0 && size_per_head <= 128,
             BT_ERR_UNSUPPORTED, "%s: size_per_head %d (supported: multiples of 8 up to 128)",
             who, size_per_head);
  BT_REQUIRE(batch_size <= 65535 && head_num <= 65535, BT_ERR_UNSUPPORTED,
             "%s: batch_size / head_num exceed the grid limit", who);
  BT_REQUIRE(!padded_rows || (long long)batch_size * seq_len <= rows_cap, BT_ERR_INVALID_ARGUMENT,
             "%s: padded rows need rows_cap >= batch_size * seq_len", who);
  F32AttArgs<T> p{(const T *)qkv, (T *)out, batch_idx, seq_order, (const T *)atten_mask,
                  (const T *)attention_bias, batch_size, seq_len, rows_cap, head_num, scale,
                  padded_rows ? 1 : 0};
  p.d = size_per_head;
  constexpr int kWaves = 4;    // 128 queries per workgroup (two-wave workgroups measured slower)
  p.nqb = (seq_len + 32 * kWaves - 1) / (32 * kWaves);
  // the conditions of the fp16 streaming kernel: from the third round of 32 workgroups
  // per XCD on and up to 128 sequences, or always / never by the option
  const unsigned per_xcd = ((unsigned)batch_size * head_num + 7) / 8 * p.nqb;
  const int order = option_attention_xcd_map();
  p.balanced = order == 3 || (order == 2 && per_xcd > 64 && batch_size <= 128);
  const unsigned grid = p.balanced ? (per_xcd + 31) / 32 * 32 * 8 : per_xcd * 8;
#define BT_F32_ATT(ND_) f32_attention_kernel<T, ND_, kWaves><<<grid, 64 * kWaves, 0, s>>>(p)
  switch ((size_per_head + 31) / 32) {
    case 1: BT_F32_ATT(1); break;
    case 2: BT_F32_ATT(2); break;
    case 3: BT_F32_ATT(3); break;
    default: BT_F32_ATT(4); break;
  }
#undef BT_F32_ATT
  BT_CHECK_LAUNCH(who);
  return BT_OK;
}

}  // namespace
}  // namespace bt

using namespace bt;

extern "C" int bt_gemm_f32(const void *a, const int *a_row_index, const void *w, const void *bias,
                           void *c, int gelu, const int *valid_rows, int rows_cap, int rows_hint,
                           int n, int k, void *stream) {
  BT_REQUIRE(a && w && c, BT_ERR_INVALID_ARGUMENT, "bt_gemm_f32: null pointer argument");
  BT_REQUIRE(aligned16({a, w, c}), BT_ERR_INVALID_ARGUMENT,
             "bt_gemm_f32: tensor pointers must be 16-byte aligned");
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
  // Tile table: 0: 128x128, 8 waves | 1: 128x64, 4 waves | 2: 64x64, 4 waves.
  // Choice by a two-term model per k-tile of 16: a workgroup alone on its CU needs
  // `alone` us (latency bound), a CU shared by b workgroups needs b * `shared` us (MFMA
  // bound); b = ceil(workgroups / CUs).  Constants measured on MI355X.
  struct Cand { int id, bm, bn; float alone, shared; };
  static const Cand cands[3] = {{0, 128, 128, 1.20f, 1.15f}, {1, 128, 64, 0.76f, 0.60f},
                                {2, 64, 64, 0.49f, 0.32f}};
  int tile = option_f32_gemm_tile();
  if (tile < 0) {
    // the row count that matters is the live one; the hint is the caller's estimate of it
    const int rows = (valid_rows && rows_hint > 0 && rows_hint < rows_cap) ? rows_hint : rows_cap;
    float best = 0.f;
    for (const Cand &cd : cands) {
      const long long wgs = (long long)((rows + cd.bm - 1) / cd.bm) * ((n + cd.bn - 1) / cd.bn);
      const float b = (float)((wgs + kF32CUs - 1) / kF32CUs);
      const float cost = fmaxf(cd.alone, b * cd.shared);
      if (tile < 0 || cost < best) {
        best = cost;
        tile = cd.id;
      }
    }
  }
  const int bm = cands[tile].bm, bn = cands[tile].bn;
  dim3 grid((n + bn - 1) / bn, (rows_cap + bm - 1) / bm);
  BT_REQUIRE(grid.y <= 65535, BT_ERR_UNSUPPORTED, "bt_gemm_f32: too many rows");
  hipStream_t s = as_stream(stream);
  switch (tile) {
    case 0: f32_gemm_kernel<128, 128, 4, 2><<<grid, 512, 0, s>>>(p); break;
    case 1: f32_gemm_kernel<128, 64, 2, 2><<<grid, 256, 0, s>>>(p); break;
    default: f32_gemm_kernel<64, 64, 2, 2><<<grid, 256, 0, s>>>(p); break;
  }
  BT_CHECK_LAUNCH("bt_gemm_f32");
  return BT_OK;
}

extern "C" int bt_attention_f32(const void *qkv, void *out, const int *batch_idx,
                                const int *seq_order, const void *atten_mask,
                                const void *attention_bias, int batch_size, int seq_len,
                                int rows_cap, int head_num, int size_per_head, float scale,
                                int padded_rows, void *stream) {
  return launch_generic_attention<float>("bt_attention_f32", qkv, out, batch_idx, seq_order,
                                         atten_mask, attention_bias, batch_size, seq_len,
                                         rows_cap, head_num, size_per_head, scale, padded_rows,
                                         as_stream(stream));
}

extern "C" int bt_attention_generic_f16(const void *qkv, void *out, const int *batch_idx,
                                        const int *seq_order, const void *atten_mask,
                                        const void *attention_bias, int batch_size, int seq_len,
                                        int rows_cap, int head_num, int size_per_head,
                                        float scale, int padded_rows, void *stream) {
  return launch_generic_attention<half_t>("bt_attention_generic_f16", qkv, out, batch_idx,
                                          seq_order, atten_mask, attention_bias, batch_size,
                                          seq_len, rows_cap, head_num, size_per_head, scale,
                                          padded_rows, as_stream(stream));
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
