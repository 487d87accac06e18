"""ctypes bindings of libbt_hip.so / libbytetransformer.so and the loader of the
PyTorch operator library.  Nothing is built here: run
`python -m bytetransformer_amd.build` first."""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_longlong, c_ulonglong, c_void_p

_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")


class LibraryMissing(RuntimeError):
    pass


def lib_dir():
    return _DIR


def _path(name):
    p = os.path.join(_DIR, name)
    if not os.path.exists(p):
        raise LibraryMissing(
            "%s is not built; run `python -m bytetransformer_amd.build` "
            "(there is no fallback implementation)" % p)
    return p


_P = c_void_p
_IP = c_void_p  # int* device pointers travel as raw addresses

# name -> (restype, argtypes); mirrors include/bt_hip.h declaration by declaration
KERNEL_ABI = {
    "bt_version": (c_int, []),
    "bt_last_error_string": (c_char_p, []),
    "bt_set_option": (c_int, [c_char_p, c_int]),
    "bt_get_option": (c_int, [c_char_p, POINTER(c_int)]),
    "bt_build_offsets": (c_int, [_P, c_int, c_int, c_int, _IP, _IP, _IP, POINTER(c_int), _P]),
    "bt_mask_prefix_slots": (c_int, [_P, c_int, c_int, c_int, _IP, _IP, _P]),
    "bt_mask_is_prefix": (c_int, [_P, c_int, c_int, c_int, _IP, _IP, POINTER(c_int), _P]),
    "bt_layer_prologue": (c_int, [_P, c_int, c_int, c_int, _IP, _IP, _IP, _IP, _P, c_int, c_int,
                                  c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int),
                                  POINTER(c_int), c_int, POINTER(c_void_p), POINTER(c_ulonglong),
                                  _P]),
    "bt_gemm_prepack_pays": (c_int, [c_longlong, c_int, c_int, c_int]),
    "bt_gemm_prepack_gain_us": (c_float, [c_longlong, c_int, c_int, c_int]),
    "bt_publish_int": (c_int, [_IP, _IP, _P]),
    "bt_compress": (c_int, [_P, _P, _IP, _IP, c_int, c_int, c_int, _P]),
    "bt_transpose_weight": (c_int, [_P, _P, c_int, c_int, _P]),
    "bt_transpose_weights": (c_int, [c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int),
                                     POINTER(c_int), _P]),
    "bt_gemm": (c_int, [_P, _P, _P, _IP, c_int, c_int, c_int, c_int, c_int, _P]),
    "bt_gemm_bias_gelu": (c_int, [_P, _P, _P, _P, _IP, c_int, c_int, c_int, c_int, c_int, _P]),
    "bt_gemm_qkv_bias_split": (c_int, [_P, _IP, _P, _P, _P, _IP, c_int, c_int, c_int, c_int,
                                       c_int, _P]),
    "bt_gemm_qkv_mask_rows_supported": (c_int, [c_int, c_int, c_int]),
    "bt_gemm_qkv_bias_split_mask_rows": (c_int, [_P, _P, c_int, c_int, c_int, _P, _P, _P, _IP, _IP,
                                                 _IP, c_int, c_int, c_int, c_int, _P]),
    "bt_attention_short": (c_int, [_P, _P, _IP, _IP, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                   c_float, c_int, POINTER(c_void_p), POINTER(c_ulonglong), c_int,
                                   _P]),
    "bt_attention_grouped": (c_int, [_P, _P, _IP, _IP, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                     c_float, c_int, POINTER(c_void_p), POINTER(c_ulonglong),
                                     c_int, _IP, _P, _P]),
    "bt_attention_worklist_bytes": (c_ulonglong, [c_int, c_int, c_int]),
    "bt_attention_worklist": (c_int, [_IP, _IP, c_int, c_int, c_int, c_int, _P, _P]),
    "bt_add_bias_residual_layernorm": (c_int, [_P, _P, _IP, _P, _P, _P, c_int, _IP, c_int, c_int,
                                               c_float, _P]),
    "bt_add_bias_residual_layernorm_copy": (c_int, [_P, _P, _IP, _P, _P, _P, c_int, _IP, c_int,
                                                    c_int, c_float, c_int, POINTER(c_void_p),
                                                    POINTER(c_void_p), POINTER(c_int),
                                                    POINTER(c_int), _P]),
    "bt_add_bias_residual_layernorm_restore": (c_int, [_P, _P, _P, _P, _P, c_int, _P, _IP, _IP,
                                                       c_int, c_int, c_int, c_float, _P]),
    "bt_gemm_splitk": (c_int, [_P, _P, _P, c_int, _IP, c_int, c_int, c_int, c_int, _P]),
    "bt_splitk_layernorm": (c_int, [_P, c_int, _P, _IP, _P, _P, _P, c_int, _P, _IP, _IP, c_int,
                                    c_int, c_int, c_int, c_float, _P]),
    "bt_gemm_f32": (c_int, [_P, _IP, _P, _P, _P, c_int, _IP, c_int, c_int, c_int, c_int, _P]),
    "bt_attention_generic_f16": (c_int, [_P, _P, _IP, _IP, _P, _P, c_int, c_int, c_int, c_int, c_int,
                                         c_float, c_int, _P]),
    "bt_attention_f32": (c_int, [_P, _P, _IP, _IP, _P, _P, c_int, c_int, c_int, c_int, c_int, c_float,
                                 c_int, _P]),
    "bt_add_bias_residual_layernorm_f32": (c_int, [_P, _P, _IP, _P, _P, _P, _IP, c_int, c_int,
                                                   c_float, _P]),
    "bt_add_bias_residual_layernorm_restore_f32": (c_int, [_P, _P, _P, _P, _P, _P, _IP, c_int,
                                                           c_int, c_int, c_float, _P]),
}


class LayerWeights(ctypes.Structure):
    """struct bt_layer_weights of include/bt_encoder.h."""
    _fields_ = [(n, c_void_p) for n in (
        "qkv_kernel", "qkv_bias", "attr_output_kernel", "attr_output_bias",
        "attr_output_layernorm_gamma", "attr_output_layernorm_beta", "inter_kernel",
        "inter_bias", "output_kernel", "output_bias", "output_layernorm_gamma",
        "output_layernorm_beta")]


class EncoderConfig(ctypes.Structure):
    """struct bt_encoder_config of include/bt_encoder.h."""
    _fields_ = [("dtype", c_int), ("max_batch_size", c_int), ("max_seq_len", c_int),
                ("head_num", c_int), ("size_per_head", c_int), ("intermediate_size", c_int),
                ("use_fused_attention", c_int), ("is_remove_padding", c_int),
                ("gamma_beta_fp32", c_int), ("tao", c_float), ("layernorm_eps", c_float)]


HOST_ABI = {
    "bt_encoder_bufsize": (c_ulonglong, [POINTER(EncoderConfig)]),
    "bt_encoder_layer_plan": (c_int, [POINTER(EncoderConfig), c_int, c_int, c_int, POINTER(c_int)]),
    "bt_encoder_layer_forward": (c_int, [POINTER(EncoderConfig), POINTER(LayerWeights), _P, _P,
                                         _P, _P, c_int, c_int, _P]),
    "bt_encoder_layer_forward_bias": (c_int, [POINTER(EncoderConfig), POINTER(LayerWeights), _P,
                                              _P, _P, _P, _P, c_int, c_int, _P]),
    "bt_encoder_layer_forward_static": (c_int, [POINTER(EncoderConfig), POINTER(LayerWeights), _P,
                                                _P, _P, _P, c_int, c_int, _P]),
    "bt_encoder_forward_bufsize": (c_ulonglong, [POINTER(EncoderConfig)]),
    "bt_encoder_prepack_bytes": (c_ulonglong, [POINTER(EncoderConfig), c_int]),
    "bt_encoder_prepack": (c_int, [POINTER(EncoderConfig), c_int, POINTER(LayerWeights), _P, _P]),
    "bt_encoder_forward": (c_int, [POINTER(EncoderConfig), c_int, POINTER(LayerWeights), _P, _P, _P,
                                   _P, _P, _P, c_int, c_int, c_int, _P]),
    "bt_encoder_last_error": (c_char_p, []),
}

_kernel = None
_host = None
_th_op_loaded = False


def _bind(lib, abi):
    for name, (res, args) in abi.items():
        fn = getattr(lib, name)  # AttributeError here = the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


def kernel_lib():
    """libbt_hip.so with every include/bt_hip.h symbol bound."""
    global _kernel
    if _kernel is None:
        _kernel = _bind(ctypes.CDLL(_path("libbt_hip.so"), mode=ctypes.RTLD_GLOBAL), KERNEL_ABI)
    return _kernel


def host_lib():
    """libbytetransformer.so with every include/bt_encoder.h symbol bound."""
    global _host
    if _host is None:
        kernel_lib()
        _host = _bind(ctypes.CDLL(_path("libbytetransformer.so"), mode=ctypes.RTLD_GLOBAL),
                      HOST_ABI)
    return _host


def th_op_path():
    return _path("libths_bytetransformer.so")


def load_th_op():
    """Registers torch.ops.ByteTransformer.BertTransformer (and the TorchScript class)."""
    global _th_op_loaded
    if not _th_op_loaded:
        import torch
        host_lib()
        torch.ops.load_library(th_op_path())
        _th_op_loaded = True
