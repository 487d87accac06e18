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
// [k, n] as stored) run on a k-contiguous copy made afresh in the call, and by which launch:
// copy[i] - by the launch ahead of the layer (bt_layer_prologue), ln_copy[i] - by the first
// LayerNorm's launch (FFN1 and FFN2 only: the products behind it).  A product gets a copy
// when the measured tile table says it gains more than a microsecond beyond the cost of the
// copy.  `live` = expected valid tokens, `padded_rows` = batch x seq_len,
// `first_launch` = 0: the layer has a launch ahead of it in any case, 1: the QKV product could
// count the mask rows itself, so that a layer with nothing for a prologue to do goes without
// it, 2: it does so in any case; `ln_can_copy` = the LayerNorm's launch may carry copies.  Where the prologue is optional it is kept only if the copies that nothing
// else can make (QKV, projection) return what it costs (about 4 us with one round of tiles) -
// it then makes the others as well; without it the FFN copies ride in the LayerNorm's launch
// (or, if they may not, are dropped unless they pay for a prologue: up to 10 k padded rows
// never copying then wins 1.5-1.8 % per forward and loses as much beyond).
// Returns the number of prologue copies.
inline int plan_weight_copies(long long live, long long padded_rows, int hidden, int inter,
                              bool split_heads, int first_launch, bool ln_can_copy, bool copy[4],
                              bool ln_copy[4]) {
  const int n[4] = {3 * hidden, hidden, inter, hidden}, k[4] = {hidden, hidden, hidden, inter};
  const int epilogue[4] = {split_heads ? BT_EPILOGUE_QKV_SPLIT : -1, BT_EPILOGUE_PLAIN,
                           BT_EPILOGUE_BIAS_GELU, BT_EPILOGUE_PLAIN};
  float gain[4] = {0.f, 0.f, 0.f, 0.f}, early = 0.f, total = 0.f;
  bool want[4];
  for (int i = 0; i < 4; ++i) {
    if (epilogue[i] >= 0) gain[i] = bt_gemm_prepack_gain_us(live, n[i], k[i], epilogue[i]);
    want[i] = gain[i] > 1.0f;
    if (want[i]) total += gain[i];
    if (want[i] && i < 2) early += gain[i];
  }
  bool prologue = true;
  if (first_launch == 1)
    prologue = ln_can_copy ? early >= 4.0f : (padded_rows > 10240 ? total > 0.f : total >= 4.0f);
  if (first_launch == 2) prologue = false;
  int count = 0;
  for (int i = 0; i < 4; ++i) {
    copy[i] = prologue && want[i];
    // (measured where the table's gain is smallest, 1.5 us for FFN1 at batch 16 x 512: kernel time
    // -1 % per forward, wall time -0.5 % on one box and +0.6 % on another; with 4.5 us at
    // 16 x 1024, where the copy also replaces the prologue, -2 %)
    ln_copy[i] = !prologue && ln_can_copy && i >= 2 && want[i];
    count += copy[i];
  }
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
