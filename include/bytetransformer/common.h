// Shared API types of the BERT encoder-layer library, gfx950 build.
//
// Mirrors the public names of the reference's bytetransformer/include/common.h
// (OperationType, Traits, ET_Param, ModelType, ActType, the runtime-error
// convention of common.h:130-138) so that caller code written against the
// reference compiles against this header.  cuBLAS/CUDA types do not exist
// here: streams are hipStream_t and the BLAS-handle slots are opaque pointers
// that the library never dereferences (every GEMM is an in-tree MFMA kernel).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdlib>
#include <stdexcept>
#include <string>

#include "bt_hip.h"

namespace bytetransformer {

enum class OperationType { FP32, HALF };

// Opaque stand-in for the reference's cublasHandle_t members.
typedef void *BlasHandle;

template <OperationType OpType>
class Traits;

template <>
class Traits<OperationType::FP32> {
 public:
  typedef float DataType;
  static const int dtype = BT_F32;
  static const int algo = -1;
};

template <>
class Traits<OperationType::HALF> {
 public:
  typedef __half DataType;
  static const int dtype = BT_F16;
  static const int algo = 99;
};

// Packed-token bookkeeping produced by the mask prefix sum.  valid_word_num is
// only filled in when the caller asked the offsets builder for it; the kernels
// read the count from batch_idx[batch_size] on the device.
typedef struct {
  int *batch_idx;
  int *word_idx;
  int valid_word_num;
} ET_Param;

// FFN2 with few rows and a long k runs as a split-k GEMM whose fp32 partial sums the last
// LayerNorm folds in (bt_gemm_splitk / bt_splitk_layernorm): 4 splits up to 192 expected
// rows, 2 up to 272, none beyond or when the launch is sized for more than kSplitKMaxRows
// rows (the partials live in a scratch area sized for that many).
constexpr int kSplitKMaxRows = 512;
inline int splitk_splits(long long rows_cap, long long rows_expected, int k) {
  static const bool enabled = [] {
    const char *e = std::getenv("BT_SPLITK");     // BT_SPLITK=0 turns the split-k path off
    return !(e && e[0] == '0');
  }();
  if (!enabled || rows_cap > kSplitKMaxRows || k < 2048) return 1;
  if (rows_expected <= 192 && k % (4 * 64) == 0) return 4;
  if (rows_expected <= 272 && k % (2 * 64) == 0) return 2;
  return 1;
}
inline unsigned long long splitk_scratch_bytes(unsigned long long max_rows,
                                               unsigned long long hidden) {
  const unsigned long long rows = max_rows < (unsigned long long)kSplitKMaxRows
                                      ? max_rows
                                      : (unsigned long long)kSplitKMaxRows;
  return 4ull * rows * hidden * sizeof(float);
}

// Which of a padding-free fp16 layer's four products (QKV, projection, FFN1, FFN2; weights
// [k, n] as stored) run on a k-contiguous copy made afresh in the call's first launch.
// `live` = expected valid tokens, `padded_rows` = batch x seq_len, `first_launch_optional` =
// the QKV product could count the mask rows itself, so that a layer without copies goes
// without any launch ahead of it.  There the copies have to return what that launch costs
// (about 3 us beyond the copies themselves with one round of tiles: never copying wins
// 1.5-1.8 % per forward up to 10 k padded rows and loses as much beyond), elsewhere a
// microsecond more than they cost.  Returns the number of copies and sets copy[i].
inline int plan_weight_copies(long long live, long long padded_rows, int hidden, int inter,
                              bool split_heads, bool first_launch_optional, bool copy[4]) {
  const int n[4] = {3 * hidden, hidden, inter, hidden}, k[4] = {hidden, hidden, hidden, inter};
  const int epilogue[4] = {split_heads ? BT_EPILOGUE_QKV_SPLIT : -1, BT_EPILOGUE_PLAIN,
                           BT_EPILOGUE_BIAS_GELU, BT_EPILOGUE_PLAIN};
  float gain[4] = {0.f, 0.f, 0.f, 0.f}, total = 0.f;
  for (int i = 0; i < 4; ++i) {
    if (epilogue[i] < 0) continue;
    gain[i] = bt_gemm_prepack_gain_us(live, n[i], k[i], epilogue[i]);
    if (gain[i] > 1.0f) total += gain[i];
  }
  const bool launch_at_stake = first_launch_optional && padded_rows <= 10240;
  const bool copy_any = !launch_at_stake || total > 1e8f || total >= 4.0f;
  int count = 0;
  for (int i = 0; i < 4; ++i) count += (copy[i] = copy_any && gain[i] > 1.0f);
  return count;
}

enum ModelType { Bert };

enum ActType { Relu, Sigmoid, SoftPlus, No };

// Turns a non-zero C-ABI status into the exception the reference's
// check_cuda_error raises (std::runtime_error, "[BT][ERROR] ..." prefix).
inline void check_status(int status, const char *file, int line) {
  if (status != BT_OK) {
    std::string msg = bt_last_error_string();
    if (msg.rfind("[BT][ERROR]", 0) != 0) msg = "[BT][ERROR] " + msg;
    throw std::runtime_error(msg + " " + file + ":" + std::to_string(line) + " \n");
  }
}

#define check_bt_error(val) ::bytetransformer::check_status((val), __FILE__, __LINE__)

}  // namespace bytetransformer
