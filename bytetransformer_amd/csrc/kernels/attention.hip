// Fused multi-head attention for gfx950 over head-major Q/K/V
// ([3][heads][rows_cap][64], fp16), one workgroup per (query tile, head,
// sequence), wave64 + v_mfma_f32_16x16x32_f16.
//
// Both kernels compute the logits TRANSPOSED, S^T = K.Q^T, so that the MFMA
// accumulator of a 16-key block (lane = query, 4 consecutive keys per lane) is
// already laid out as the "B" operand of the second product O^T = V^T.P^T: the
// probabilities never leave registers.  V is staged into LDS transposed
// ([d][key]) so the "A" operand of that product is two 8-byte LDS reads.
//
//   attention_short_kernel    whole K / V^T of the sequence resident in LDS,
//                             all logits of a query tile in registers, exact
//                             two-pass softmax: P = exp(s-max)/(sum+1e-6) is
//                             rounded to fp16 before P.V exactly as
//                             attention_fused.cu:348-381 does.
//   attention_grouped_kernel  K / V streamed in 64-key tiles through an LDS
//                             double buffer with an online softmax; handles
//                             any length; the [S, S] logits never exist.
//
// Keys at or past the sequence length are excluded by index (the mask tensor is
// not read), the convention of the reference's remove-padding kernels
// (attention_fused.cu:359, attention_fused_long.cu:254).
#include "common.h"

namespace bt {

constexpr int kAttThreads = 256;
constexpr int kKld = 72;   // K tile row stride (halfs): 64 + 8 pad
constexpr int kHeadDim = 64;
constexpr float kNegBig = -1.0e30f;
constexpr float kLog2e = 1.4426950408889634f;

struct AttArgs {
  const half_t *qkv;   // [3][heads][rows_cap][64]
  half_t *out;         // [rows, heads*64]
  const int *batch_idx;
  int B, S, rows_cap, heads;
  float scale_log2e;   // scale * log2(e)
  int padded_rows;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ uint4_t zero16() { return uint4_t{0u, 0u, 0u, 0u}; }

// Interleave two 8-half rows (keys 2p and 2p+1) into LDS as V^T[d][key pair].
__device__ __forceinline__ void store_vt_pair(half_t *sVt, int vld, int d0, int key, uint4_t v0,
                                              uint4_t v1) {
  const unsigned short *a = (const unsigned short *)&v0;
  const unsigned short *b = (const unsigned short *)&v1;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    unsigned int w = (unsigned int)a[i] | ((unsigned int)b[i] << 16);
    *(unsigned int *)(sVt + (d0 + i) * vld + key) = w;
  }
}

// ---------------------------------------------------------------------------
// grouped / streaming kernel
// ---------------------------------------------------------------------------
constexpr int kKT = 64;          // keys per streamed tile
constexpr int kVldT = kKT + 4;   // V^T tile row stride (halfs), 136 B keeps 8-byte alignment

template <int QB>  // 16-query blocks per wave; workgroup covers 4*QB*16 queries
__global__ __launch_bounds__(kAttThreads) void attention_grouped_kernel(AttArgs p) {
  constexpr int BQ = 4 * QB * 16;
  __shared__ __attribute__((aligned(16))) half_t sK[2][kKT * kKld];
  __shared__ __attribute__((aligned(16))) half_t sVt[2][kHeadDim * kVldT];

  const int b = blockIdx.z, head = blockIdx.y;
  const int seq_start = p.batch_idx[b];
  const int klen = p.batch_idx[b + 1] - seq_start;
  const int row_start = p.padded_rows ? b * p.S : seq_start;
  const int nq = p.padded_rows ? p.S : klen;
  const int q0 = blockIdx.x * BQ;
  if (q0 >= nq) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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
      uint4_t v = zero16();
      if (q < nq) v = *(const uint4_t *)(Q + (size_t)q * kHeadDim + 32 * dh + 8 * lg);
      qf[qb][dh] = __builtin_bit_cast(half8_t, v);
    }
  }

  // staging registers: K 2 chunks/thread (row = tid/8 + 32*i, col = tid%8),
  //                    V 2 chunks/thread (keys 2*kp, 2*kp+1 ; d chunk = tid%8)
  const int k_row = tid >> 3, k_col = (tid & 7) * 8;
  const int v_kp = tid >> 3, v_dc = (tid & 7) * 8;
  uint4_t rk[2], rv[2];

  auto load_tile = [&](int t) {
    const int k0 = t * kKT;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int key = k0 + k_row + 32 * i;
      rk[i] = key < klen ? *(const uint4_t *)(K + (size_t)key * kHeadDim + k_col) : zero16();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int key = k0 + 2 * v_kp + i;
      rv[i] = key < klen ? *(const uint4_t *)(V + (size_t)key * kHeadDim + v_dc) : zero16();
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      *(uint4_t *)(&sK[buf][(k_row + 32 * i) * kKld + k_col]) = rk[i];
    store_vt_pair(sVt[buf], kVldT, v_dc, 2 * v_kp, rv[0], rv[1]);
  };

  float4_t o[4][QB];
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = kNegBig;
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db) o[db][qb] = float4_t{0.f, 0.f, 0.f, 0.f};
  }

  const int ntiles = (klen + kKT - 1) / kKT;
  if (ntiles > 0) {
    load_tile(0);
    store_tile(0);
  }
  __syncthreads();

  const float c = p.scale_log2e;
  for (int t = 0; t < ntiles; ++t) {
    const int buf = t & 1;
    if (t + 1 < ntiles) load_tile(t + 1);

    // S^T = K . Q^T for this tile: 4 key blocks x QB query blocks
    float4_t s[4][QB];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) s[kb][qb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dh = 0; dh < 2; ++dh) {
        const half8_t kf =
            *(const half8_t *)(&sK[buf][(kb * 16 + lq) * kKld + 32 * dh + 8 * lg]);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          s[kb][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[qb][dh], s[kb][qb], 0, 0, 0);
      }
    }
    const int k0 = t * kKT;
    if (k0 + kKT > klen) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (k0 + kb * 16 + lg * 4 + r >= klen)
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) s[kb][qb][r] = kNegBig;
    }

    half8_t pf[2][QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
      float mx = kNegBig;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[kb][qb][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run[qb], mx);
      const float alpha = fast_exp2((m_run[qb] - m_new) * c);
      m_run[qb] = m_new;
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float e = fast_exp2((s[kb][qb][r] - m_new) * c);
          psum += e;
          pf[kb >> 1][qb][(kb & 1) * 4 + r] = (half_t)e;
        }
      l_run[qb] = l_run[qb] * alpha + psum;
#pragma unroll
      for (int db = 0; db < 4; ++db) o[db][qb] *= alpha;
    }

    // O^T += V^T . P^T ; k-slot (lg, s) <-> key 32*kk + 16*(s>>2) + 4*lg + (s&3)
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const half_t *vp = &sVt[buf][(db * 16 + lq) * kVldT + 32 * kk + 4 * lg];
        const half4_t v0 = *(const half4_t *)vp, v1 = *(const half4_t *)(vp + 16);
        const half8_t vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
          o[db][qb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[kk][qb], o[db][qb], 0, 0, 0);
      }

    if (t + 1 < ntiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // O / (l + 1e-6) -> fp16, token-major [row][head*64 + d]
  const int H = p.heads * kHeadDim;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    float l = l_run[qb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const float inv = 1.0f / (l + 1e-6f);
    const int q = q0 + (wave * QB + qb) * 16 + lq;
    if (q >= nq) continue;
    half_t *dst = p.out + (size_t)(row_start + q) * H + head * kHeadDim + 4 * lg;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      const float4_t v = o[db][qb] * inv;
      *(half4_t *)(dst + 16 * db) = half4_t{(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
    }
  }
}

// ---------------------------------------------------------------------------
// short kernel: K, V^T resident in LDS, logits of the query tile in registers
// ---------------------------------------------------------------------------
template <int NKB>  // capacity in 16-key blocks (keys <= 16*NKB), NKB even
__global__ __launch_bounds__(kAttThreads) void attention_short_kernel(AttArgs p) {
  constexpr int KEYS = NKB * 16;
  constexpr int VLD = KEYS + 4;
  constexpr int BQ = 64;  // 4 waves x 16 queries
  extern __shared__ __attribute__((aligned(16))) half_t smem[];
  half_t *sK = smem;                  // [KEYS][kKld]
  half_t *sVt = smem + KEYS * kKld;   // [64][VLD]

  const int b = blockIdx.z, head = blockIdx.y;
  const int seq_start = p.batch_idx[b];
  const int klen = p.batch_idx[b + 1] - seq_start;
  const int row_start = p.padded_rows ? b * p.S : seq_start;
  const int nq = p.padded_rows ? p.S : klen;
  const int q0 = blockIdx.x * BQ;
  if (q0 >= nq) return;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lq = lane & 15, lg = lane >> 4;
  const int H = p.heads * kHeadDim;
  half_t *dst_row = nullptr;
  const int q = q0 + wave * 16 + lq;

  const size_t head_stride = (size_t)p.rows_cap * kHeadDim;
  const half_t *Q = p.qkv + (size_t)head * head_stride + (size_t)row_start * kHeadDim;
  const half_t *K = Q + (size_t)p.heads * head_stride;
  const half_t *V = K + (size_t)p.heads * head_stride;

  half8_t qf[2];
#pragma unroll
  for (int dh = 0; dh < 2; ++dh) {
    uint4_t v = zero16();
    if (q < nq) v = *(const uint4_t *)(Q + (size_t)q * kHeadDim + 32 * dh + 8 * lg);
    qf[dh] = __builtin_bit_cast(half8_t, v);
  }

  // stage K rows and V^T columns for keys [0, keys32), zero past klen
  const int keys32 = min(((klen + 31) >> 5) << 5, KEYS);
  const int col = (tid & 7) * 8;
  for (int key = tid >> 3; key < keys32; key += 32) {
    uint4_t v = key < klen ? *(const uint4_t *)(K + (size_t)key * kHeadDim + col) : zero16();
    *(uint4_t *)(sK + key * kKld + col) = v;
  }
  for (int kp = tid >> 3; kp < keys32 / 2; kp += 32) {
    const int key = 2 * kp;
    uint4_t v0 = key < klen ? *(const uint4_t *)(V + (size_t)key * kHeadDim + col) : zero16();
    uint4_t v1 =
        key + 1 < klen ? *(const uint4_t *)(V + (size_t)(key + 1) * kHeadDim + col) : zero16();
    store_vt_pair(sVt, VLD, col, key, v0, v1);
  }
  __syncthreads();

  const int nkb = keys32 >> 4;  // even
  float4_t s[NKB];
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb) {
    s[kb] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (kb < nkb) {
#pragma unroll
      for (int dh = 0; dh < 2; ++dh) {
        const half8_t kf = *(const half8_t *)(sK + (kb * 16 + lq) * kKld + 32 * dh + 8 * lg);
        s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[dh], s[kb], 0, 0, 0);
      }
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
  mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  const float c = p.scale_log2e;
  float sum = 0.f;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s[kb][r] = fast_exp2((s[kb][r] - mx) * c);
      sum += s[kb][r];
    }
  sum += __shfl_xor(sum, 16, 64);
  sum += __shfl_xor(sum, 32, 64);
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
      for (int db = 0; db < 4; ++db) {
        const half_t *vp = sVt + (db * 16 + lq) * VLD + 32 * kk + 4 * lg;
        const half4_t v0 = *(const half4_t *)vp, v1 = *(const half4_t *)(vp + 16);
        const half8_t vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
        o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, o[db], 0, 0, 0);
      }
    }
  }

  if (q < nq) {
    dst_row = p.out + (size_t)(row_start + q) * H + head * kHeadDim + 4 * lg;
#pragma unroll
    for (int db = 0; db < 4; ++db)
      *(half4_t *)(dst_row + 16 * db) =
          half4_t{(half_t)o[db][0], (half_t)o[db][1], (half_t)o[db][2], (half_t)o[db][3]};
  }
}

static int check_att_args(const char *who, const void *qkv, const void *out, const int *batch_idx,
                          int B, int S, int rows_cap, int heads, int d) {
  BT_REQUIRE(qkv && out && batch_idx, BT_ERR_INVALID_ARGUMENT, "%s: null pointer argument", who);
  BT_REQUIRE(B > 0 && S > 0 && heads > 0 && rows_cap > 0, BT_ERR_INVALID_ARGUMENT,
             "%s: batch_size=%d seq_len=%d head_num=%d rows_cap=%d must be positive", who, B, S,
             heads, rows_cap);
  BT_REQUIRE(d == kHeadDim, BT_ERR_UNSUPPORTED, "%s: size_per_head=%d, only 64 is supported", who,
             d);
  BT_REQUIRE(B <= 65535 && heads <= 65535, BT_ERR_UNSUPPORTED, "%s: grid too large", who);
  return BT_OK;
}

template <int NKB>
static int launch_short(const AttArgs &a, hipStream_t s) {
  constexpr size_t smem = ((size_t)NKB * 16 * kKld + (size_t)kHeadDim * (NKB * 16 + 4)) * 2;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)attention_short_kernel<NKB>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(attention_short_kernel)");
    configured = true;
  }
  dim3 grid((a.S + 63) / 64, a.heads, a.B);
  attention_short_kernel<NKB><<<grid, kAttThreads, smem, s>>>(a);
  BT_CHECK_LAUNCH("attention_short_kernel");
  return BT_OK;
}

}  // namespace bt

using namespace bt;

extern "C" int bt_attention_short(const void *qkv_heads, void *attention_output,
                                  const int *batch_idx, int batch_size, int seq_len, int rows_cap,
                                  int head_num, int size_per_head, float scale, int padded_rows,
                                  void *stream) {
  int rc = check_att_args("bt_attention_short", qkv_heads, attention_output, batch_idx,
                          batch_size, seq_len, rows_cap, head_num, size_per_head);
  if (rc) return rc;
  BT_REQUIRE(seq_len <= 512, BT_ERR_UNSUPPORTED,
             "bt_attention_short: seq_len=%d exceeds 512, use bt_attention_grouped", seq_len);
  AttArgs a{(const half_t *)qkv_heads, (half_t *)attention_output, batch_idx, batch_size, seq_len,
            rows_cap, head_num, scale * kLog2e, padded_rows};
  hipStream_t s = as_stream(stream);
  if (seq_len <= 64) return launch_short<4>(a, s);
  if (seq_len <= 128) return launch_short<8>(a, s);
  if (seq_len <= 256) return launch_short<16>(a, s);
  if (seq_len <= 384) return launch_short<24>(a, s);
  return launch_short<32>(a, s);
}

extern "C" int bt_attention_grouped(const void *qkv_heads, void *attention_output,
                                    const int *batch_idx, int batch_size, int seq_len,
                                    int rows_cap, int head_num, int size_per_head, float scale,
                                    int padded_rows, void *stream) {
  int rc = check_att_args("bt_attention_grouped", qkv_heads, attention_output, batch_idx,
                          batch_size, seq_len, rows_cap, head_num, size_per_head);
  if (rc) return rc;
  AttArgs a{(const half_t *)qkv_heads, (half_t *)attention_output, batch_idx, batch_size, seq_len,
            rows_cap, head_num, scale * kLog2e, padded_rows};
  hipStream_t s = as_stream(stream);
  // 128-query tiles once there is enough work to fill the chip, else 64
  const long long blocks128 = (long long)((seq_len + 127) / 128) * head_num * batch_size;
  const int qb = option_attention_qb();
  if (qb == 2 || (qb < 0 && blocks128 >= 512)) {
    dim3 grid((seq_len + 127) / 128, head_num, batch_size);
    attention_grouped_kernel<2><<<grid, kAttThreads, 0, s>>>(a);
  } else {
    dim3 grid((seq_len + 63) / 64, head_num, batch_size);
    attention_grouped_kernel<1><<<grid, kAttThreads, 0, s>>>(a);
  }
  BT_CHECK_LAUNCH("attention_grouped_kernel");
  return BT_OK;
}
