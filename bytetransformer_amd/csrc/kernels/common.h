// Shared device helpers for the gfx950 kernels: vector types, wave64
// reductions, error plumbing for the C ABI.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <initializer_list>
#include <cstdio>

#include "bt_hip.h"

namespace bt {

constexpr int kWave = 64;

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __fp16 fp16x4_t __attribute__((ext_vector_type(4)));   // element type of the LDS transpose-read builtin
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));

// ---- error plumbing -------------------------------------------------------
void set_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what);

#define BT_REQUIRE(cond, code, ...) \
  do {                              \
    if (!(cond)) {                  \
      ::bt::set_error(__VA_ARGS__); \
      return (code);                \
    }                               \
  } while (0)

#define BT_CHECK_LAUNCH(what)                     \
  do {                                            \
    hipError_t e__ = hipGetLastError();           \
    if (e__ != hipSuccess)                        \
      return ::bt::hip_fail(e__, what);           \
  } while (0)

// ---- tuning options (bt_set_option) ----------------------------------------
// Once-per-device set-up of a kernel's dynamic LDS limit (the attribute belongs to the
// function on one device).  `done` is the kernel's own flag array; a lost race only
// repeats an idempotent call.
constexpr int kMaxDevices = 64;
template <typename Kernel>
inline int allow_dynamic_lds(Kernel kernel, size_t bytes, std::atomic<bool> (&done)[kMaxDevices],
                             const char *what) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) {
    e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)bytes);
    return e == hipSuccess ? BT_OK : hip_fail(e, what);
  }
  if (!done[dev].load(std::memory_order_acquire)) {
    e = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)bytes);
    if (e != hipSuccess) return hip_fail(e, what);
    done[dev].store(true, std::memory_order_release);
  }
  return BT_OK;
}

int option_gemm_tile();      // -1 = heuristic, else index into the tile table
int option_gemm_table_margin();   // per cent by which a measured tile must beat the model's choice
int option_layer_prepack();  // -1 = by the measured table, 0 = never, 1 = always
int option_attention_qb();   // -1 = heuristic, 1 or 2 = query blocks per wave
int option_f32_gemm_tile();  // -1 = heuristic, else index into the float GEMM's tile table
int option_attention_xcd_map();     // workgroup order of the attention kernels: 0 plain, 1 XCD-aware, 2 balanced (default), 3 balanced always
int option_prefetch();       // 1 = honour the prefetch hints of the attention entries (default), 0 = ignore
int option_attention_key_split();  // streaming attention, 64-query tiles: -1 heuristic, 0 four waves, 1 eight waves over two key halves
int option_prefetch_min_grid();   // attention launches of fewer workgroups skip the cache warm-up (default 512)

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// Every kernel moves tensors in 16-byte pieces: all tensor pointers of an entry point must
// be 16-byte aligned (null counts as aligned: nullable arguments are checked elsewhere).
inline bool aligned16(std::initializer_list<const void *> ptrs) {
  for (const void *p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) & 15) return false;
  return true;
}

// ---- wave64 reductions ----------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Inclusive prefix sum across the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int t = __shfl_up(v, o, 64);
    if (lane >= o) v += t;
  }
  return v;
}


// Inclusive prefix sum over the 64 lanes with data-parallel-primitive adds only: four
// shifts inside each row of 16, then lane 15 of rows 0 / 2 into rows 1 / 3 and lane 31
// into the upper half.
__device__ __forceinline__ int wave_inclusive_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 -> rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 -> rows 2, 3
  return v;
}

// Sum over the 64 lanes, as a wave-uniform value.
__device__ __forceinline__ int wave_total(int v) {
  return __builtin_amdgcn_readlane(wave_inclusive_sum(v), 63);
}

// Number of row elements >= 0.5 (the length rule of the offsets, remove_padding.h:36-86),
// counted by one wave for R mask rows at a time (row r may be null: length 0).
// A mask row that has not been touched since the last layer comes from HBM: the wave
// fetches it with 16-byte loads, 4 per lane in flight over the R rows (R rows of up to
// 2048 / R halfs are one round trip; element by element a 512-token row was eight
// dependent ones).
template <typename T, int R>
__device__ __forceinline__ void wave_row_lengths(const T *const *row, int S, int lane,
                                                 int (&count)[R]) {
  constexpr int kVec = 16 / (int)sizeof(T);
  constexpr int kUnroll = 4 / R;
  static_assert(R == 1 || R == 2 || R == 4, "rows per call");
  bool vec = S % kVec == 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    count[r] = 0;
    vec = vec && (reinterpret_cast<uintptr_t>(row[r]) & 15) == 0;
  }
  if (vec) {
    for (int j0 = 0; j0 < S; j0 += kWave * kVec * kUnroll) {
      uint4_t raw[R][kUnroll];
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int j = j0 + (u * kWave + lane) * kVec;
          raw[r][u] = uint4_t{0u, 0u, 0u, 0u};
          if (row[r] && j < S) raw[r][u] = *(const uint4_t *)(row[r] + j);
        }
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const T *e = (const T *)&raw[r][u];
#pragma unroll
          for (int i = 0; i < kVec; ++i) count[r] += (float)e[i] >= 0.5f;
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) count[r] = wave_total(count[r]);
    return;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (!row[r]) continue;
    for (int i0 = 0; i0 < S; i0 += kWave) {
      const int i = i0 + lane;
      const bool on = (i < S) && ((float)row[r][i] >= 0.5f);
      count[r] += __popcll(__ballot(on));
    }
  }
}
template <typename T>
__device__ __forceinline__ int wave_row_length(const T *__restrict__ row, int S, int lane) {
  const T *const rows[1] = {row};
  int count[1];
  wave_row_lengths<T, 1>(rows, S, lane, count);
  return count[0];
}

// ---- 64 x 64 tile of the weight pre-pack: wt[n][k] = w[k][n] ---------------------------
// 256 threads (t = 0..255) move one tile through `tile`; both sides are 16-byte accesses.
// `live` = false keeps a thread group in step (it meets the barrier) without touching memory.
constexpr int kTransposePitch = 64 + 2;
__device__ __forceinline__ void transpose_tile_64(const half_t *__restrict__ w,
                                                  half_t *__restrict__ wt, int K, int N, int k0,
                                                  int n0, half_t (*tile)[kTransposePitch], int t,
                                                  bool live) {
  // read 64 k-rows x 128 B: thread -> (row = t/8 + 32*i, 16-byte chunk t%8)
  const int r = t >> 3, c = (t & 7) * 8;
  if (live) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int k = k0 + r + 32 * i, n = n0 + c;
      uint4_t v = {0u, 0u, 0u, 0u};
      if (k < K && n < N) v = *(const uint4_t *)(w + (size_t)k * N + n);
      const half_t *h = (const half_t *)&v;
#pragma unroll
      for (int e = 0; e < 8; ++e) tile[r + 32 * i][c + e] = h[e];
    }
  }
  __syncthreads();
  if (live) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int n = n0 + r + 32 * i, k = k0 + c;
      if (n < N && k < K) {
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = tile[c + e][r + 32 * i];
        *(half8_t *)(wt + (size_t)n * K + k) = o;
      }
    }
  }
}

// ---- jobs that ride along with a layer's first launch ----------------------------------
// k-contiguous copies [N, K] of up to four [K, N] weight matrices, and ranges whose
// 128-byte lines are touched once so that later launches find them in the memory-side cache.
struct WeightJobs {
  const half_t *w[4];        // [K, N] as the caller stores them
  half_t *wt[4];             // [N, K] copies to make
  int K[4], N[4];
  int tiles_n[4];            // 64 x 64 tiles along n
  int tile_end[4];           // tiles up to and including matrix i
  int count;                 // 0 = none
  // range r holds the 128-byte lines [warm_end[r - 1], warm_end[r]) of the concatenation
  const char *warm[4];
  unsigned warm_end[4];
};
// Fills `out` from the tail arguments of the C entries that take such jobs (checks them and
// reports errors under the name `who`; returns a BT status).  With the `prefetch` option off
// the ranges to warm are dropped.
int make_weight_jobs(const char *who, WeightJobs *out, int weight_count, const void *const *w,
                     void *const *wt, const int *k, const int *n, int warm_count,
                     const void *const *warm, const unsigned long long *warm_bytes);

// U tiles at a time per group of 256 threads (t = thread index in the group): tiles t0 .. t0 +
// U - 1 of the concatenated tile list of the jobs (ids from pw.tile_end[pw.count - 1] on do not
// exist).  All the loads of the U tiles are in flight together, so a group that has several
// tiles to move pays one memory round trip for U of them.  `tiles` holds U consecutive LDS
// tiles of this group.  The whole workgroup must call it together (two barriers inside).
template <int U>
__device__ __forceinline__ void transpose_tiles_64(const WeightJobs &pw, int t0,
                                                   half_t (*tiles)[kTransposePitch], int t) {
  const int r = t >> 3, c = (t & 7) * 8;
  const int t_end = pw.tile_end[pw.count - 1];
  uint4_t v[U][2];
  const half_t *src[U];
  half_t *dst[U];
  int K[U], N[U], k0[U], n0[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int tile = t0 + u;
    int j = 0, first = 0;
#pragma unroll
    for (int q = 1; q < 4; ++q)
      if (q < pw.count && tile >= pw.tile_end[q - 1]) {
        j = q;
        first = pw.tile_end[q - 1];
      }
    const int tl = tile - first;
    src[u] = pw.w[j], dst[u] = pw.wt[j], K[u] = tile < t_end ? pw.K[j] : 0, N[u] = pw.N[j];
    k0[u] = (tl / pw.tiles_n[j]) * 64, n0[u] = (tl % pw.tiles_n[j]) * 64;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int k = k0[u] + r + 32 * i, n = n0[u] + c;
      v[u][i] = uint4_t{0u, 0u, 0u, 0u};
      if (k < K[u] && n < N[u]) v[u][i] = *(const uint4_t *)(src[u] + (size_t)k * N[u] + n);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const half_t *h = (const half_t *)&v[u][i];
#pragma unroll
      for (int e = 0; e < 8; ++e) tiles[u * 64 + r + 32 * i][c + e] = h[e];
    }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int n = n0[u] + r + 32 * i, k = k0[u] + c;
      if (n < N[u] && k < K[u]) {
        half8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = tiles[u * 64 + c + e][r + 32 * i];
        *(half8_t *)(dst[u] + (size_t)n * K[u] + k) = o;
      }
    }
  }
  __syncthreads();
}

// One dword per 128-byte line of the ranges, lines [first, last) in steps of `stride`.
__device__ __forceinline__ void warm_lines(const WeightJobs &pw, unsigned first, unsigned last,
                                           unsigned stride) {
  for (unsigned l = first; l < last; l += stride) {
    const char *base = pw.warm[0];
    unsigned begin = 0;
#pragma unroll
    for (int r = 1; r < 4; ++r)
      if (l >= pw.warm_end[r - 1]) {
        base = pw.warm[r];
        begin = pw.warm_end[r - 1];
      }
    unsigned sink;
    const char *addr = base + (unsigned long long)(l - begin) * 128;
    asm volatile("global_load_dword %0, %1, off" : "=v"(sink) : "v"(addr) : "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---- balanced work list of the streaming attention kernels -------------------------
// Within an XCD the hardware deals consecutive workgroups to its 32 CUs round-robin
// (slot s of the XCD lands on CU s % 32), and a launch of a few workgroups per CU is
// resident at once, so the static order alone decides what each CU gets.  With a fixed
// number of query-tile slots per sequence the tile index is s % 4 at 512 tokens: one CU
// in four received only the last tiles - dead for most sequences - while others held
// three live ones of the longest sequences.  Here the live (pair, query tile) items of
// the XCD - (sequence, head) pairs p = x (mod 8) over the longest-first order, the tiles
// of a pair adjacent, so that one L2 serves a pair's K / V to all of them - are counted
// on the device, and slot s takes item j = s in even rounds of 32 and the mirrored
// position in odd rounds: a CU that drew a long item in one round draws a short one in
// the next.  Every lane of a wave holds one rank: lengths, tile counts and a wave prefix
// sum invert j -> (rank, head, tile) with the two dependent loads a plain look-up needs
// as well.  Args: a kernel argument struct with B, S, heads, nqb, padded_rows, batch_idx
// and seq_order.

struct AttWork {
  int b, head, qb, seq_start, len;
  bool exists;
};
// Shape of the balanced order of a streaming-attention launch over (B, S, heads): entries =
// workgroups of the launch (0: such a launch does not use the balanced order), bq = queries
// per tile (64 or 128), nqb = tile slots per sequence.  One function decides for the
// attention launcher and for whoever builds the list ahead of it.
struct AttListPlan {
  unsigned entries;
  int bq, nqb;
};
AttListPlan att_worklist_plan(int B, int S, int heads);
// Arguments of att_work_balanced when the offsets come from somewhere else than a kernel's
// own argument struct (the layer prologue builds the list from lengths it holds in LDS).
struct AttListArgs {
  int B, S, heads, nqb, padded_rows;
  const int *batch_idx, *seq_order;
};
template <int BQ, typename Args>
__device__ __forceinline__ AttWork att_work_balanced(const Args &p, unsigned int workgroup) {
  AttWork w{0, 0, 0, 0, 0, false};
  const int lane = threadIdx.x & 63;
  const int x = workgroup & 7, s = workgroup >> 3;
  const int round = s >> 5, pos = s & 31;
  const int j = (round << 5) + ((round & 1) ? 31 - pos : pos);
  int carry = 0;
  for (int base = 0; base < p.B; base += 64) {
    const int r = base + lane;
    const bool valid = r < p.B;
    const int seq = valid ? (p.seq_order ? p.seq_order[r] : r) : 0;
    const int start = p.batch_idx[seq];
    const int len = valid ? p.batch_idx[seq + 1] - start : 0;
    const int nq = p.padded_rows ? p.S : len;
    const int nqb = valid ? min((nq + BQ - 1) / BQ, p.nqb) : 0;
    const int first = r * p.heads;   // pairs [first, first + heads) belong to rank r
    const int cnt = ((first + p.heads + 7 - x) >> 3) - ((first + 7 - x) >> 3);
    const int mine = cnt * nqb;
    const int incl = wave_inclusive_sum(mine);
    const int lo = carry + incl - mine;   // first item of this rank
    const unsigned long long hit = __builtin_amdgcn_ballot_w64(mine > 0 && j >= lo && j < lo + mine);
    if (hit) {
      const int src = __builtin_ctzll(hit);
      const int jj = j - __builtin_amdgcn_readlane(lo, src);
      const int nqb_s = __builtin_amdgcn_readlane(nqb, src);
      const int first_s = (base + src) * p.heads;
      w.b = __builtin_amdgcn_readlane(seq, src);
      w.seq_start = __builtin_amdgcn_readlane(start, src);
      w.len = __builtin_amdgcn_readlane(len, src);
      w.qb = jj % nqb_s;
      // the (jj / nqb_s)-th head h of the rank with first_s + h = x (mod 8)
      w.head = ((x - first_s) & 7) + 8 * (jj / nqb_s);
      w.exists = true;
      return w;
    }
    carry += __builtin_amdgcn_readlane(incl, 63);
  }
  return w;
}

}  // namespace bt
