"""bt_encoder_layer_forward_static (the entry point that brings its own scratch and
allocates nothing) against bt_encoder_layer_forward_bias with a caller-owned buffer:
same kernels, same launches, so the outputs must agree bit for bit - and against the CPU
oracle on the same inputs within the fp16 tolerance (max-abs 2e-2, mean-abs 2e-3 over the valid
rows).  Two calls in a row share the library's device array, the second with a smaller input,
so stale contents of the first call would show."""
import ctypes

import numpy as np
import pytest
import torch

from bytetransformer_amd import workload
from bytetransformer_amd._lib import EncoderConfig, LayerWeights, host_lib
from oracle import bert_oracle as O

pytestmark = pytest.mark.gpu

STATIC_SCRATCH_BYTES = 32 << 20     # BT_STATIC_SCRATCH_BYTES of include/bt_encoder.h


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _case(device, batch, seq_len, lens, seed, head_num=12):
    cfg = workload.EncoderConfig("static", batch, seq_len, head_num, layers=1, lens=lens,
                                 seed=seed)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    weights = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
    return wl, weights, _dev(wl.x, device), _dev(wl.mask, device)


def _both(device, batch, seq_len, lens, seed, with_bias=False):
    lib = host_lib()
    wl, weights, x, mask = _case(device, batch, seq_len, lens, seed)
    w = LayerWeights(*[ctypes.c_void_p(t.data_ptr()) for t in weights])
    cfg = EncoderConfig(1, batch, seq_len, wl.cfg.head_num, 64, 4, 1, 1, 0, 1.0, 1e-6)
    need = lib.bt_encoder_bufsize(ctypes.byref(cfg))
    assert 0 < need <= STATIC_SCRATCH_BYTES
    bias = None
    if with_bias:
        rs = np.random.RandomState(seed + 5)
        bias = _dev((rs.standard_normal((wl.cfg.head_num, seq_len, seq_len)) * 0.5)
                    .astype(np.float16), device)
    bias_ptr = ctypes.c_void_p(bias.data_ptr() if bias is not None else None)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    buf = torch.empty(need, dtype=torch.int8, device=device)
    # NaN poison in both outputs: a row that a call fails to write stands out
    ref = torch.full_like(x, float("nan"))
    got = torch.full_like(x, float("nan"))
    torch.cuda.synchronize()
    rc = lib.bt_encoder_layer_forward_bias(
        ctypes.byref(cfg), ctypes.byref(w), ctypes.c_void_p(x.data_ptr()),
        ctypes.c_void_p(mask.data_ptr()), bias_ptr, ctypes.c_void_p(ref.data_ptr()),
        ctypes.c_void_p(buf.data_ptr()), batch, seq_len, stream)
    assert rc == 0, lib.bt_encoder_last_error().decode()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(device)
    rc = lib.bt_encoder_layer_forward_static(
        ctypes.byref(cfg), ctypes.byref(w), ctypes.c_void_p(x.data_ptr()),
        ctypes.c_void_p(mask.data_ptr()), bias_ptr, ctypes.c_void_p(got.data_ptr()),
        batch, seq_len, stream)
    assert rc == 0, lib.bt_encoder_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(device) == before
    ref, got = ref.cpu().numpy(), got.cpu().numpy()
    assert np.isfinite(ref.astype(np.float32)).all()
    assert np.array_equal(ref.view(np.uint16), got.view(np.uint16)), \
        "static-scratch layer differs from the caller-buffer layer"
    # ... and the oracle's layer on the same inputs (valid rows; fp16 tolerance of the path)
    w32 = {k: np.asarray(v, np.float32) for k, v in wl.layers[0].items()}
    kw = {"attention_bias": bias.float().cpu().numpy()} if with_bias else {}
    exp = O.encoder_layer(wl.x.astype(np.float32), wl.mask.astype(np.float32), w32,
                          wl.cfg.head_num, **kw).numpy()
    mx, mean, _ = O.parity_metrics(O.masked_output(got, wl.lens), O.masked_output(exp, wl.lens),
                                   wl.lens)
    print("static scratch against the oracle: max-abs %.3e mean-abs %.3e" % (mx, mean), flush=True)
    assert mx <= 2e-2 and mean <= 2e-3, (mx, mean)
    return got


def test_static_scratch_layer_two_calls_second_smaller(device):
    print("static scratch: 4 x 96 then 3 x 40", flush=True)
    _both(device, 4, 96, (96, 17, 50, 1), seed=11)
    _both(device, 3, 40, (5, 40, 23), seed=12)
    # padded-row path (batch <= 2) with an attention bias, then the split-k FFN2 sizes again
    print("static scratch: 2 x 64 with bias then 1 x 256", flush=True)
    _both(device, 2, 64, (64, 38), seed=13, with_bias=True)
    _both(device, 1, 256, (154,), seed=14)


def test_static_scratch_rejects_oversized_configuration(device):
    lib = host_lib()
    cfg = EncoderConfig(1, 16, 512, 12, 64, 4, 1, 1, 0, 1.0, 1e-6)
    assert lib.bt_encoder_bufsize(ctypes.byref(cfg)) > STATIC_SCRATCH_BYTES
    # the size check comes before any pointer is touched
    w = LayerWeights(*[ctypes.c_void_p(256)] * 12)
    rc = lib.bt_encoder_layer_forward_static(
        ctypes.byref(cfg), ctypes.byref(w), ctypes.c_void_p(256), ctypes.c_void_p(256), None,
        ctypes.c_void_p(256), 16, 512, None)
    assert rc == 2      # BT_ERR_UNSUPPORTED
    msg = lib.bt_encoder_last_error().decode()
    assert "static scratch" in msg and str(STATIC_SCRATCH_BYTES) in msg
