"""Host-side mirror of the reference's per-layer interface for Python callers
that do not go through torch.ops: BertEncoderLayer wraps
bt_encoder_layer_forward (include/bt_encoder.h), i.e. the C++
BertTransformer<HALF>::infer, with torch tensors providing device memory and
the current stream."""
import ctypes

import torch

from ._lib import EncoderConfig, LayerWeights, host_lib
from .workload import WEIGHT_NAMES


class BertEncoderLayer:
    """One encoder layer bound to twelve GPU weight tensors (dict by
    WEIGHT_NAMES or a 12-sequence in operator-argument order)."""

    def __init__(self, head_num, head_size, weights, is_remove_padding=True,
                 use_fused_attention=True, layernorm_eps=1e-6, tao=1.0):
        if isinstance(weights, dict):
            weights = [weights[n] for n in WEIGHT_NAMES]
        if len(weights) != 12:
            raise ValueError("expected 12 weight tensors")
        for w in weights:
            if not (w.is_cuda and w.is_contiguous()):
                raise ValueError("weights must be contiguous GPU tensors")
        self.weights = list(weights)
        self.head_num, self.head_size = head_num, head_size
        self.hidden = head_num * head_size
        self.is_remove_padding = is_remove_padding
        self.use_fused_attention = use_fused_attention
        self.layernorm_eps, self.tao = layernorm_eps, tao
        self._w = LayerWeights(*[ctypes.c_void_p(w.data_ptr()) for w in self.weights])
        self._buf = None

    def _config(self, B, S):
        return EncoderConfig(1, B, S, self.head_num, self.head_size,
                             self.weights[6].shape[1] // self.hidden,
                             int(self.use_fused_attention), int(self.is_remove_padding),
                             int(self.weights[10].dtype == torch.float32), self.tao,
                             self.layernorm_eps)

    def __call__(self, x, mask, out=None, attention_bias=None):
        lib = host_lib()
        if x.dtype != torch.float16:
            raise RuntimeError("only fp16 activations are implemented")
        B, S, H = x.shape
        cfg = self._config(B, S)
        need = lib.bt_encoder_bufsize(ctypes.byref(cfg))
        if need == 0:
            raise RuntimeError(lib.bt_encoder_last_error().decode())
        if self._buf is None or self._buf.numel() < need or self._buf.device != x.device:
            self._buf = torch.empty(need, dtype=torch.int8, device=x.device)
        if out is None:
            out = torch.empty_like(x)
        if attention_bias is not None:
            if (attention_bias.dtype != x.dtype or not attention_bias.is_contiguous()
                    or tuple(attention_bias.shape) != (self.head_num, S, S)):
                raise ValueError("attention_bias must be a contiguous [head_num, S, S] tensor "
                                 "of the activation dtype")
        rc = lib.bt_encoder_layer_forward_bias(
            ctypes.byref(cfg), ctypes.byref(self._w), ctypes.c_void_p(x.data_ptr()),
            ctypes.c_void_p(mask.data_ptr()),
            ctypes.c_void_p(attention_bias.data_ptr() if attention_bias is not None else None),
            ctypes.c_void_p(out.data_ptr()),
            ctypes.c_void_p(self._buf.data_ptr()), B, S,
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc != 0:
            raise RuntimeError(lib.bt_encoder_last_error().decode())
        return out


def encoder_forward(layers, x, mask):
    """Runs a list of BertEncoderLayer back to back (ping-pong outputs)."""
    h = x
    bufs = [torch.empty_like(x), torch.empty_like(x)]
    for i, layer in enumerate(layers):
        h = layer(h, mask, out=bufs[i & 1])
    return h
