"""CPU-side checks of the boundary: the libraries load, export every symbol the
headers declare, reject bad arguments before touching the GPU, and the PyTorch
operator keeps the reference's schema and error behaviour."""
import ctypes
import os
import re

import pytest
import torch

import bytetransformer_amd as bt
from bytetransformer_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bt_[a-z0-9_]+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    names = _declared("bt_hip.h")
    assert len(names) >= 12
    lib = ctypes.CDLL(os.path.join(bt.lib_dir(), "libbt_hip.so"))
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.KERNEL_ABI) == names       # the ctypes table covers the header
    assert bt.kernel_lib().bt_version() == 1


def test_host_library_exports_every_declared_symbol():
    names = _declared("bt_encoder.h")
    bt.kernel_lib()
    lib = ctypes.CDLL(os.path.join(bt.lib_dir(), "libbytetransformer.so"))
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.HOST_ABI) == names


def test_argument_validation_returns_codes_without_gpu():
    lib = bt.kernel_lib()
    err = lambda: lib.bt_last_error_string().decode()
    assert lib.bt_gemm(None, None, None, None, 4, 0, 8, 64, 0, None) == 1 and "null pointer" in err()
    p = ctypes.c_void_p(256)   # never dereferenced: validation fails first
    assert lib.bt_gemm(p, p, p, None, 4, 0, 8, 100, 0, None) == 2 and "multiple of 64" in err()
    assert lib.bt_gemm(p, p, p, None, 4, 0, 12, 64, 1, None) == 2 and "multiple of 8" in err()
    assert lib.bt_gemm(p, p, p, None, 4, 0, 8, 64, 2, None) == 1 and "weight_kn" in err()
    assert lib.bt_gemm(p, p, p, None, 4, 0, 1 << 20, 1 << 11, 1, None) == 2 and "2 GiB" in err()
    # the layout question: forced answers, and 0 for a shape outside the measured table
    assert lib.bt_gemm_prepack_pays(5000, 520, 64, 0) == 0
    for forced in (1, 0):
        assert lib.bt_set_option(b"layer_prepack", forced) == 0
        assert lib.bt_gemm_prepack_pays(5000, 3072, 768, 1) == forced
    assert lib.bt_set_option(b"layer_prepack", -1) == 0
    assert lib.bt_set_option(b"layer_prepack", 2) == 1
    # rows from the mask inside the QKV product: which shapes the entry takes, its checks
    assert lib.bt_gemm_qkv_mask_rows_supported(16, 512, 1) == 1
    assert lib.bt_gemm_qkv_mask_rows_supported(32, 1024, 1) == 1
    assert lib.bt_gemm_qkv_mask_rows_supported(32, 1024, 0) == 0    # float mask rows: 128 KB
    assert lib.bt_gemm_qkv_mask_rows_supported(65, 8, 1) == 0
    assert lib.bt_gemm_qkv_mask_rows_supported(8, 8, 7) == 0
    assert lib.bt_gemm_qkv_bias_split_mask_rows(p, p, 1, 65, 8, p, p, p, p, None, None, 0, 12,
                                                64, 1, None) == 2
    assert "bt_gemm_qkv_mask_rows_supported" in err()
    assert lib.bt_gemm_qkv_bias_split_mask_rows(p, p, 1, 4, 8, p, p, p, None, None, None, 0, 12,
                                                64, 1, None) == 1 and "null pointer" in err()
    assert lib.bt_gemm_qkv_bias_split_mask_rows(p, None, 1, 4, 8, p, p, p, p, None, None, 0, 12,
                                                64, 1, None) == 1
    for v in (0, 1, -1):
        assert lib.bt_set_option(b"qkv_mask_rows", v) == 0
    assert lib.bt_set_option(b"qkv_mask_rows", 2) == 1
    assert lib.bt_set_option(b"qkv_mask_rows", -1) == 0
    # the margin by which the measured tile table has to beat the cost model's choice
    got = ctypes.c_int(-1)
    assert lib.bt_get_option(b"gemm_table_margin", ctypes.byref(got)) == 0 and got.value == 4
    assert lib.bt_set_option(b"gemm_table_margin", 100) == 0
    assert lib.bt_set_option(b"gemm_table_margin", 101) == 1 and "gemm_table_margin" in err()
    assert lib.bt_set_option(b"gemm_table_margin", 4) == 0
    assert lib.bt_gemm_qkv_bias_split(p, None, p, p, p, None, 4, 0, 1, 32, 0, None) == 2
    assert "multiple of 64" in err()        # hidden = 1 * 32
    assert lib.bt_gemm_qkv_bias_split(p, p, p, p, p, None, 4, 0, 12, 64, 1, None) == 1
    assert "needs valid_rows" in err()
    assert lib.bt_attention_short(p, p, p, None, None, None, 1, 1024, 1024, 12, 64, 0.125, 0, None, None, 0, None) == 2
    assert "exceeds 512" in err()
    assert lib.bt_attention_grouped(p, p, p, None, None, None, 1, 16, 16, 12, 48, 0.125, 0, None, None, 0, None, None, None) == 2
    assert lib.bt_attention_grouped(p, p, p, None, p, None, 1, 16, 16, 12, 64, 0.125, 0, None, None, 0, None, None, None) == 1
    assert "only applied on padded rows" in err()
    assert lib.bt_compress(p, p, p, p, 2, 4, 12, None) == 2 and "multiple of 8" in err()
    assert lib.bt_build_offsets(p, 7, 2, 4, p, p, None, None, None) == 1 and "dtype" in err()
    assert lib.bt_build_offsets(p, 1, 0, 4, p, p, None, None, None) == 1
    assert lib.bt_add_bias_residual_layernorm(p, p, None, p, p, p, 0, None, 4, 12, 1e-6, None) == 2
    assert lib.bt_add_bias_residual_layernorm(p, p, None, p, p, p, 0, None, 4, 8192, 1e-6, None) == 2
    assert lib.bt_add_bias_residual_layernorm_restore(p, p, p, p, p, 0, None, p, None, 2, 4, 64, 1e-6,
                                                      None) == 1
    assert lib.bt_transpose_weight(None, p, 8, 8, None) == 1
    odd = ctypes.c_void_p(264)   # 8-byte aligned only
    assert lib.bt_gemm(odd, p, p, None, 4, 0, 8, 64, 0, None) == 1 and "16-byte aligned" in err()
    assert lib.bt_add_bias_residual_layernorm(p, odd, None, p, p, p, 0, None, 4, 64, 1e-6, None) == 1
    assert "16-byte aligned" in err()
    # float entry points
    assert lib.bt_gemm_f32(p, None, p, None, p, 0, None, 4, 0, 6, 8, None) == 2 and "multiples of 4" in err()
    assert lib.bt_gemm_f32(p, None, p, None, p, 1, None, 4, 0, 8, 8, None) == 1 and "gelu needs a bias" in err()
    assert lib.bt_gemm_f32(p, p, p, None, p, 0, None, 4, 0, 8, 8, None) == 1 and "needs valid_rows" in err()
    assert lib.bt_attention_f32(p, p, p, None, None, None, 1, 16, 16, 12, 44, 0.125, 0, None) == 2
    assert lib.bt_attention_f32(p, p, p, None, None, None, 2, 16, 16, 12, 64, 0.125, 1, None) == 1
    assert lib.bt_add_bias_residual_layernorm_f32(p, p, None, p, p, p, None, 4, 6, 1e-6, None) == 2
    assert lib.bt_add_bias_residual_layernorm_restore_f32(p, p, p, p, p, None, p, 2, 4, 64, 1e-6,
                                                          None) == 1


def test_encoder_c_api_validation_and_bufsize():
    lib = bt.host_lib()
    cfg = _lib.EncoderConfig(1, 16, 512, 12, 64, 4, 1, 1, 0, 1.0, 1e-6)
    need = lib.bt_encoder_bufsize(ctypes.byref(cfg))
    T = 16 * 512 * 768
    # nine activation tensors + two index arrays + the pre-packed weights + the split-k area
    # + the attention's work list (16 bytes per workgroup of its largest launch)
    splitk = 4 * 512 * 768 * 4
    work_list = (16 * 12 // 8) * (512 // 64) * 8 * 16
    assert need >= 9 * T * 2 + 2 * 16 * 512 * 4 + 12 * 768 * 768 * 2 + splitk + work_list
    assert need < 9 * T * 2 + 2 * 16 * 512 * 4 + 12 * 768 * 768 * 2 + splitk + work_list + 8192
    f32 = _lib.EncoderConfig(0, 16, 512, 12, 64, 4, 1, 1, 0, 1.0, 1e-6)   # float: twice the bytes
    need32 = lib.bt_encoder_bufsize(ctypes.byref(f32))
    assert 2 * need - 4 * 16 * 512 * 4 - splitk - 8192 < need32 < 2 * need
    bad = _lib.EncoderConfig(7, 16, 512, 12, 64, 4, 1, 1, 0, 1.0, 1e-6)
    assert lib.bt_encoder_bufsize(ctypes.byref(bad)) == 0
    assert b"BT_F16 or BT_F32" in lib.bt_encoder_last_error()
    w = _lib.LayerWeights()
    rc = lib.bt_encoder_layer_forward(ctypes.byref(cfg), ctypes.byref(w), None, None, None, None,
                                      1, 1, None)
    assert rc != 0 and b"null weight pointer" in lib.bt_encoder_last_error()


def _cpu_args(H=128, B=2, S=8, dtype=torch.float16):
    w = [torch.zeros(H, 3 * H), torch.zeros(3 * H), torch.zeros(H, H), torch.zeros(H),
         torch.ones(H), torch.zeros(H), torch.zeros(H, 4 * H), torch.zeros(4 * H),
         torch.zeros(4 * H, H), torch.zeros(H), torch.ones(H), torch.zeros(H)]
    w = [t.to(dtype) for t in w]
    return w, torch.zeros(B, S, H, dtype=dtype), torch.ones(B, S, S, dtype=dtype)


def test_th_op_schema_matches_reference():
    bt.load_th_op()
    schema = str(torch.ops.ByteTransformer.BertTransformer.default._schema)
    assert schema.startswith("ByteTransformer::BertTransformer(int head_num, int head_size, "
                             "Tensor qkv_kernel, Tensor qkv_bias, Tensor attr_output_kernel")
    assert "Tensor input, Tensor attr_mask, bool is_remove_padding=True, " \
           "bool use_fused_attention=True) -> Tensor" in schema


def test_th_op_rejects_host_tensors_like_the_reference():
    bt.load_th_op()
    w, x, m = _cpu_args()
    with pytest.raises(RuntimeError, match="qkv_kernel must be a CUDA tensor"):
        torch.ops.ByteTransformer.BertTransformer(2, 64, *w, x, m, True, True)


def test_torchscript_class_is_registered_and_checks_arguments():
    bt.load_th_op()
    w, _, _ = _cpu_args()
    cls = torch.classes.ByteTransformer.BertTransformer
    with pytest.raises(RuntimeError, match="qkv_kernel must be a CUDA tensor"):
        cls(2, 64, *w)


def test_missing_library_raises(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_DIR", str(tmp_path))
    with pytest.raises(bt.LibraryMissing, match="no fallback"):
        _lib._path("libbt_hip.so")


def test_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "bytetransformer_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cc", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)


def test_layer_plan_is_a_host_side_decision():
    """bt_encoder_layer_plan answers without a GPU: at the headline shape and with several
    rounds of tiles the layer starts with the QKV product that counts the mask rows and lets
    its first LayerNorm's launch make FFN1's copy (2) - without that option no copy at the
    headline shape and the prologue with its copy (1) at the larger one, as for a layer that
    may not start with the QKV product; beyond 32 sequences the prologue makes the copies; a
    short batch of one goes without offsets."""
    import ctypes
    from bytetransformer_amd._lib import EncoderConfig, host_lib, kernel_lib
    lib = host_lib()

    def plan(batch, seq, hint, rm=1):
        cfg = EncoderConfig(1, batch, seq, 12, 64, 4, 1, rm, 0, 1.0, 1e-6)
        out = (ctypes.c_int * 6)()
        assert lib.bt_encoder_layer_plan(ctypes.byref(cfg), batch, seq, hint, out) == 0
        return list(out)

    assert plan(16, 512, 4809) == [0, 0, 2, 0, 1, 0]
    assert plan(16, 1024, 9800) == [0, 0, 2, 0, 1, 0]
    big = plan(64, 256, 9800)
    assert big[4] == 0 and big[2] == 1
    assert plan(1, 64, 0) == [0, 0, 0, 0, 0, 1]
    kl = kernel_lib()
    try:
        assert kl.bt_set_option(b"ln_weight_copy", 0) == 0
        assert plan(16, 512, 4809) == [0, 0, 0, 0, 1, 0]
        big = plan(16, 1024, 9800)
        assert big[4] == 0 and big[5] == 0 and big[2] == 1
        assert kl.bt_set_option(b"ln_weight_copy", 2) == 1
    finally:
        assert kl.bt_set_option(b"ln_weight_copy", 1) == 0
    try:
        assert kl.bt_set_option(b"qkv_mask_rows", 0) == 0
        assert plan(16, 1024, 9800)[:5] == [0, 0, 1, 0, 0]
    finally:
        assert kl.bt_set_option(b"qkv_mask_rows", -1) == 0
    assert lib.bt_encoder_layer_plan(None, 1, 1, 0, (ctypes.c_int * 6)()) != 0
