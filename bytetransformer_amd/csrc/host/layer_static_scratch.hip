// bt_encoder_layer_forward_static: bt_encoder_layer_forward_bias with the layer's
// scratch (`buf`) living in a library-owned device array instead of a caller-owned
// workspace, for callers that cannot allocate device memory.  The only translation
// unit of the host library that holds device code: the array itself.
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <string>

#include "bt_encoder.h"
#include "bt_hip.h"
#include "host_error.h"

namespace {

// Every GPU the library runs on holds its own copy of this array, at its own address,
// until the process ends.  In host code the name is only a handle for
// hipGetSymbolAddress; the address kernels may use is what that call returns.
static __device__ __align__(256) unsigned char scratch[BT_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];
std::mutex g_lookup_mutex;

// Device address of `scratch` on the current device (looked up once per device).
int static_scratch(void **ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    bt_host::set_error(std::string("[BT][ERROR] hipGetDevice: ") + hipGetErrorString(e));
    return BT_ERR_HIP;
  }
  if (device < 0 || device >= kMaxDevices) {
    bt_host::set_error("[BT][ERROR] bt_encoder_layer_forward_static: device ordinal " +
                       std::to_string(device) + " outside [0, " + std::to_string(kMaxDevices) +
                       ")");
    return BT_ERR_UNSUPPORTED;
  }
  void *p = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (!p) {
    std::lock_guard<std::mutex> lock(g_lookup_mutex);
    p = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!p) {
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !p) {
        bt_host::set_error(std::string("[BT][ERROR] hipGetSymbolAddress(static scratch): ") +
                           hipGetErrorString(e));
        return BT_ERR_HIP;
      }
      g_scratch_ptr[device].store(p, std::memory_order_release);
    }
  }
  *ptr = p;
  return BT_OK;
}

}  // namespace

extern "C" int bt_encoder_layer_forward_static(const bt_encoder_config *cfg,
                                               const bt_layer_weights *weights, const void *input,
                                               const void *atten_mask, const void *attention_bias,
                                               void *output, int batch_size, int seq_len,
                                               void *stream) {
  const unsigned long long need = bt_encoder_bufsize(cfg);
  if (need == 0) return BT_ERR_INVALID_ARGUMENT;   // message set by bt_encoder_bufsize
  if (need > BT_STATIC_SCRATCH_BYTES) {
    bt_host::set_error("[BT][ERROR] bt_encoder_layer_forward_static: this configuration needs " +
                       std::to_string(need) + " bytes of scratch, the static scratch holds " +
                       std::to_string((unsigned long long)BT_STATIC_SCRATCH_BYTES) +
                       "; use bt_encoder_layer_forward with a caller-owned buffer");
    return BT_ERR_UNSUPPORTED;
  }
  void *buf = nullptr;
  const int rc = static_scratch(&buf);
  if (rc != BT_OK) return rc;
  // No part of the scratch has to start at zero: every region is written by the launch
  // that precedes its first reader on the stream (offsets, pre-packed weights, Q/K/V,
  // split-k partial sums, prefix-mask slots).
  return bt_encoder_layer_forward_bias(cfg, weights, input, atten_mask, attention_bias, output,
                                       buf, batch_size, seq_len, stream);
}
