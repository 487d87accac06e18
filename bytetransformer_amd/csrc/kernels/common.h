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
int option_attention_qb();   // -1 = heuristic, 1 or 2 = query blocks per wave
int option_f32_gemm_tile();  // -1 = heuristic, else index into the float GEMM's tile table
int option_attention_xcd_map();     // workgroup order of the fp16 attention: 0 plain, 1 XCD-aware, 2 balanced (default), 3 balanced always
int option_prefetch();       // 1 = honour the prefetch hints of the attention entries (default), 0 = ignore

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

}  // namespace bt
