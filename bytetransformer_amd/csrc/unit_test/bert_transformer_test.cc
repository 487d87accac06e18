// bert_transformer_test <batch_size> <seq_len> <head_num> <size_per_head> [--data DIR]
//                       [--iters N] [--tol MAX_ABS] [--no-rm] [--no-fused] [--fp32]
//                       [--synthetic [--lens L0,L1,...]]
//
// Stand-alone C++ driver of BertTransformer<OperationType::HALF> or, with --fp32,
// BertTransformer<OperationType::FP32> (the reference picks the type at build time with
// -DDataType and defaults to FP32, unit_test/bert_transformer_test.cc:25-31): loads one layer's
// tensors from text fixtures (one "%f" value per line, flattened row-major; file
// names and shapes as written by the reference's exporter,
// unit_test/python_scripts/bert_transformer_test.py:160-181), runs the layer once,
// reports the running max-abs difference against transformer_out.out, then times
// warm-up + N iterations.  Role of the reference's unit_test/bert_transformer_test.cc
// and helper.h; LayerNorm gamma/beta are kept in fp32 (use_fp32 = true) as there.
// With --tol the exit status is 1 when the difference exceeds it (the reference
// only prints).  --synthetic needs no fixtures: seeded N(0, 0.02) weights, N(0, 1) input, a
// prefix mask of the given lengths (default: every sequence full) - timing only, the
// torch-free per-layer time of the C++ API (the reference's timing loop,
// unit_test/bert_transformer_test.cc:190-202).
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cmath>
#include <random>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "bytetransformer/bert_transformer.h"

using namespace bytetransformer;

#define HIP_OK(x)                                                                   \
  do {                                                                              \
    hipError_t e__ = (x);                                                           \
    if (e__ != hipSuccess) {                                                        \
      fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e__), __FILE__, \
              __LINE__);                                                            \
      exit(2);                                                                      \
    }                                                                               \
  } while (0)

static uint16_t float_to_half_bits(float f) {  // round to nearest even
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  int32_t exp = (int32_t)((x >> 23) & 0xff) - 127 + 15;
  uint32_t man = x & 0x7fffffu;
  if (((x >> 23) & 0xff) == 0xff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));
  if (exp >= 31) return (uint16_t)(sign | 0x7c00u);
  if (exp <= 0) {
    if (exp < -10) return (uint16_t)sign;
    man |= 0x800000u;
    const int shift = 14 - exp;
    uint32_t h = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1))) ++h;
    return (uint16_t)(sign | h);
  }
  uint32_t h = ((uint32_t)exp << 10) | (man >> 13);
  const uint32_t rem = man & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) ++h;
  return (uint16_t)(sign | h);
}

static float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, x;
  if (exp == 0) {
    if (man == 0) {
      x = sign;
    } else {
      int e = -1;
      do {
        ++e;
        man <<= 1;
      } while (!(man & 0x400u));
      x = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    x = sign | 0x7f800000u | (man << 13);
  } else {
    x = sign | ((exp - 15 + 127) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

static bool read_text(const std::string &path, size_t n, std::vector<float> *out) {
  FILE *fd = fopen(path.c_str(), "r");
  if (!fd) {
    printf("FILE %s does not exist.\n", path.c_str());
    return false;
  }
  out->resize(n);
  for (size_t i = 0; i < n; ++i)
    if (fscanf(fd, "%f", &(*out)[i]) != 1) {
      printf("FILE %s holds fewer than %zu values.\n", path.c_str(), n);
      fclose(fd);
      return false;
    }
  fclose(fd);
  return true;
}

static void *upload_half(const std::vector<float> &v) {
  std::vector<uint16_t> h(v.size());
  for (size_t i = 0; i < v.size(); ++i) h[i] = float_to_half_bits(v[i]);
  void *d;
  HIP_OK(hipMalloc(&d, h.size() * 2));
  HIP_OK(hipMemcpy(d, h.data(), h.size() * 2, hipMemcpyHostToDevice));
  return d;
}

static void *upload_float(const std::vector<float> &v) {
  void *d;
  HIP_OK(hipMalloc(&d, v.size() * 4));
  HIP_OK(hipMemcpy(d, v.data(), v.size() * 4, hipMemcpyHostToDevice));
  return d;
}

struct Options {
  int batch_size, seq_len, head_num, size_per_head, iters = 50;
  double tol = -1.0;
  bool is_remove_padding = true, use_fused_attention = true;
  std::string dir = ".";
  bool synthetic = false;
  std::vector<int> lens;
};

// One tensor of the synthetic layer: what the fixture file of that name would hold.
static void synthesize(const Options &o, const char *file, size_t n, std::mt19937 &gen,
                       std::vector<float> *out) {
  out->assign(n, 0.f);
  const std::string name = file;
  if (name == "atten_mask.in") {
    const size_t S = (size_t)o.seq_len;
    for (int b = 0; b < o.batch_size; ++b) {
      const size_t len = b < (int)o.lens.size() ? (size_t)o.lens[(size_t)b] : S;
      for (size_t i = 0; i < S; ++i)
        for (size_t j = 0; j < len && j < S; ++j) (*out)[((size_t)b * S + i) * S + j] = 1.f;
    }
  } else if (name.find("gamma") != std::string::npos) {
    out->assign(n, 1.f);
  } else if (name.find("kernel") != std::string::npos || name == "from_tensor.in") {
    std::normal_distribution<float> dist(0.f, name == "from_tensor.in" ? 1.f : 0.02f);
    for (float &v : *out) v = dist(gen);
  }   // biases and beta stay zero
}

template <OperationType Op>
static int run(const Options &o) {
  typedef typename Traits<Op>::DataType T;
  constexpr bool kHalf = Op == OperationType::HALF;
  const int batch_size = o.batch_size, seq_len = o.seq_len;
  const size_t H = (size_t)o.head_num * o.size_per_head, F = 4 * H;
  const size_t N = (size_t)batch_size * seq_len;   // padded rows

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  struct Item {
    const char *file;
    size_t n;
    bool fp32;   // LayerNorm gamma / beta stay float next to fp16 weights (use_fp32)
  } items[] = {{"qkv_kernel.in", H * 3 * H, false},
               {"qkv_bias.in", 3 * H, false},
               {"attr_output_kernel.in", H * H, false},
               {"attr_output_bias.in", H, false},
               {"attr_output_layernorm_gamma.in", H, true},
               {"attr_output_layernorm_beta.in", H, true},
               {"inter_kernel.in", H * F, false},
               {"inter_bias.in", F, false},
               {"output_kernel.in", F * H, false},
               {"output_bias.in", H, false},
               {"output_layernorm_gamma.in", H, true},
               {"output_layernorm_beta.in", H, true},
               {"from_tensor.in", N * H, false},
               {"atten_mask.in", N * seq_len, false}};
  void *dev[14];
  std::vector<float> host;
  std::mt19937 gen(0);
  for (int i = 0; i < 14; ++i) {
    if (o.synthetic)
      synthesize(o, items[i].file, items[i].n, gen, &host);
    else if (!read_text(o.dir + "/" + items[i].file, items[i].n, &host))
      return 2;
    dev[i] = (items[i].fp32 || !kHalf) ? upload_float(host) : upload_half(host);
  }

  try {
    BertTransformerParam<Op> param;
    param.attr_kernel_QKV = (const T *)dev[0];
    param.attention_param.attr_bias_QKV = (const T *)dev[1];
    param.attr_output_kernel = (const T *)dev[2];
    param.attr_output_bias = (const T *)dev[3];
    param.attr_output_layernorm_gamma = dev[4];
    param.attr_output_layernorm_beta = dev[5];
    param.inter_kernel = (const T *)dev[6];
    param.inter_bias = (const T *)dev[7];
    param.output_kernel = (const T *)dev[8];
    param.output_bias = (const T *)dev[9];
    param.output_layernorm_gamma = dev[10];
    param.output_layernorm_beta = dev[11];

    BertTransformer<Op> layer(batch_size, o.head_num, o.size_per_head, seq_len,
                              o.use_fused_attention, o.is_remove_padding, /*use_fp32=*/true);
    layer.initialize(param);
    const unsigned long long buf_size = layer.cal_bufsize();
    void *buf, *out;
    HIP_OK(hipMalloc(&buf, buf_size));
    HIP_OK(hipMalloc(&out, N * H * sizeof(T)));
    BertTransformerInferParam<T> infer_param{(const T *)dev[12], (const T *)dev[13], (T *)out, buf,
                                             batch_size,         seq_len,            nullptr,  stream};
    layer.infer(infer_param);
    HIP_OK(hipStreamSynchronize(stream));

    // compare valid rows and zero-filled rows alike: the exported expectation is
    // already multiplied by the row mask
    double max_diff = -1.0;
    std::vector<float> expect;
    if (!o.synthetic && read_text(o.dir + "/transformer_out.out", N * H, &expect)) {
      std::vector<float> got(N * H);
      if (kHalf) {
        std::vector<uint16_t> bits(N * H);
        HIP_OK(hipMemcpy(bits.data(), out, bits.size() * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < N * H; ++i) got[i] = half_bits_to_float(bits[i]);
      } else {
        HIP_OK(hipMemcpy(got.data(), out, got.size() * 4, hipMemcpyDeviceToHost));
      }
      std::vector<float> mask_row;
      read_text(o.dir + "/atten_mask.in", N * seq_len, &mask_row);
      for (size_t i = 0; i < N * H; ++i) {
        const size_t row = i / H, b = row / seq_len, s = row % seq_len;
        // padded path: rows past the length are not zeroed, the reference masks them out
        const bool valid = mask_row[(b * seq_len) * seq_len + s] >= 0.5f;
        const float g = (valid || layer.is_remove_padding()) ? got[i] : 0.f;
        const double diff = fabs((double)expect[i] - g);
        if (diff > max_diff) {
          max_diff = diff;
          printf("%zu HIP %f Expect %f diff %f\n", i, g, expect[i], diff);
        }
      }
      printf("Check with transformer_out.out max_diff %f\n", max_diff);
    }

    for (int i = 0; i < o.iters; ++i) layer.infer(infer_param);   // warm-up
    HIP_OK(hipStreamSynchronize(stream));
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < o.iters; ++i) layer.infer(infer_param);
    HIP_OK(hipStreamSynchronize(stream));
    const double ms =
        std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    printf("batch_size %d seq_len %d %s layer time costs %.3f ms (%d iterations, remove_padding %d)\n",
           batch_size, seq_len, kHalf ? "fp16" : "fp32", ms / o.iters, o.iters,
           (int)layer.is_remove_padding());
    if (o.tol >= 0 && (max_diff < 0 || max_diff > o.tol)) {
      printf("FAILED: max_diff %f exceeds %f\n", max_diff, o.tol);
      return 1;
    }
  } catch (const std::exception &e) {
    fprintf(stderr, "%s\n", e.what());
    return 2;
  }
  return 0;
}

int main(int argc, char *argv[]) {
  if (argc < 5) {
    printf("./bert_transformer_test <batch_size> <seq_len> <head_num> <size_per_head> "
           "[--data DIR] [--iters N] [--tol MAX_ABS] [--no-rm] [--no-fused] [--fp32] "
           "[--synthetic [--lens L0,L1,...]] [--option NAME=VALUE ...]\n");
    return 0;
  }
  Options o;
  o.batch_size = atoi(argv[1]);
  o.seq_len = atoi(argv[2]);
  o.head_num = atoi(argv[3]);
  o.size_per_head = atoi(argv[4]);
  o.is_remove_padding = o.batch_size > 2;
  bool fp32 = false;
  for (int i = 5; i < argc; ++i) {
    if (!strcmp(argv[i], "--data") && i + 1 < argc) o.dir = argv[++i];
    else if (!strcmp(argv[i], "--iters") && i + 1 < argc) o.iters = atoi(argv[++i]);
    else if (!strcmp(argv[i], "--tol") && i + 1 < argc) o.tol = atof(argv[++i]);
    else if (!strcmp(argv[i], "--no-rm")) o.is_remove_padding = false;
    else if (!strcmp(argv[i], "--no-fused")) o.use_fused_attention = false;
    else if (!strcmp(argv[i], "--fp32")) fp32 = true;
    else if (!strcmp(argv[i], "--synthetic")) o.synthetic = true;
    else if (!strcmp(argv[i], "--option") && i + 1 < argc) {
      // a tuning knob of the kernel library (bt_set_option), e.g. qkv_mask_rows=0
      const std::string kv = argv[++i];
      const size_t eq = kv.find('=');
      if (eq == std::string::npos ||
          bt_set_option(kv.substr(0, eq).c_str(), atoi(kv.c_str() + eq + 1)) != BT_OK) {
        fprintf(stderr, "bad --option %s: %s\n", kv.c_str(), bt_last_error_string());
        return 2;
      }
    }
    else if (!strcmp(argv[i], "--lens") && i + 1 < argc) {
      for (const char *p = argv[++i]; *p;) {
        o.lens.push_back(atoi(p));
        while (*p && *p != ',') ++p;
        if (*p == ',') ++p;
      }
    }
  }
  hipDeviceProp_t prop;
  HIP_OK(hipGetDeviceProperties(&prop, 0));
  printf("Device %s\n", prop.name);
  return fp32 ? run<OperationType::FP32>(o) : run<OperationType::HALF>(o);
}
