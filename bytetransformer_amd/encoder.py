"""Host-side mirror of the reference's per-layer interface for Python callers
that do not go through torch.ops: BertEncoderLayer wraps
bt_encoder_layer_forward (include/bt_encoder.h), i.e. the C++
BertTransformer<HALF or FP32>::infer, with torch tensors providing device memory and
the current stream."""
import ctypes

import torch

from ._lib import EncoderConfig, LayerWeights, host_lib
from .workload import WEIGHT_NAMES


_DTYPE_CODE = {torch.float32: 0, torch.float16: 1}   # BT_F32, BT_F16


def _activation_dtype(weights):
    """The layer's OperationType follows the QKV weight, as in the PyTorch operator."""
    dt = weights[0].dtype
    if dt not in _DTYPE_CODE:
        raise ValueError("weights must be float16 or float32, got %s" % dt)
    for i, w in enumerate(weights):
        loose = i in (4, 5, 10, 11)      # gamma / beta of fp16 layers may be float
        if w.dtype != dt and not (loose and dt == torch.float16 and w.dtype == torch.float32):
            raise ValueError("weight #%d has dtype %s, expected %s" % (i, w.dtype, dt))
    return dt


def _check_io(dtype, x, mask):
    if x.dtype != dtype or mask.dtype != dtype:
        raise RuntimeError("input and mask must have the weights' dtype %s" % dtype)
    if not (x.is_cuda and x.is_contiguous() and mask.is_cuda and mask.is_contiguous()):
        raise RuntimeError("input and mask must be contiguous GPU tensors")


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
        self.dtype = _activation_dtype(self.weights)

    def _config(self, B, S):
        return EncoderConfig(_DTYPE_CODE[self.dtype], B, S, self.head_num, self.head_size,
                             self.weights[6].shape[1] // self.hidden,
                             int(self.use_fused_attention), int(self.is_remove_padding),
                             int(self.weights[10].dtype == torch.float32), self.tao,
                             self.layernorm_eps)

    def plan(self, batch_size, seq_len, rows_hint=0):
        """bt_encoder_layer_plan for a call of this size: ([copy] * 4 for the QKV, projection,
        FFN1 and FFN2 weights - 0 read as stored, 1 copied by the launch ahead of the layer, 2 by
        the first LayerNorm's launch -, starts_with_qkv, mask_direct): what the layer will
        launch, for benchmarks that time the kernels one by one."""
        lib = host_lib()
        cfg = self._config(batch_size, seq_len)
        out = (ctypes.c_int * 6)()
        if lib.bt_encoder_layer_plan(ctypes.byref(cfg), batch_size, seq_len, int(rows_hint), out) != 0:
            raise RuntimeError(lib.bt_encoder_last_error().decode())
        return [int(v) for v in out[:4]], bool(out[4]), bool(out[5])

    def __call__(self, x, mask, out=None, attention_bias=None):
        lib = host_lib()
        _check_io(self.dtype, x, mask)
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


class BertEncoder:
    """Every layer of an encoder in one call (bt_encoder_forward): the hidden
    state stays on the packed rows between layers, the weights are pre-packed
    once at construction.  The reference has no such interface (one layer per
    call); the result equals running the layers one by one.

    `layers` is a list of 12-tensor weight sets (dicts by WEIGHT_NAMES or
    sequences in operator-argument order)."""

    def __init__(self, head_num, head_size, layers, is_remove_padding=True,
                 use_fused_attention=True, layernorm_eps=1e-6, tao=1.0):
        sets = []
        for w in layers:
            if isinstance(w, dict):
                w = [w[n] for n in WEIGHT_NAMES]
            if len(w) != 12:
                raise ValueError("expected 12 weight tensors per layer")
            for t in w:
                if not (t.is_cuda and t.is_contiguous()):
                    raise ValueError("weights must be contiguous GPU tensors")
            sets.append(list(w))
        if not sets:
            raise ValueError("expected at least one layer")
        self.weights = sets
        self.head_num, self.head_size = head_num, head_size
        self.hidden = head_num * head_size
        self.is_remove_padding = is_remove_padding
        self.use_fused_attention = use_fused_attention
        self.layernorm_eps, self.tao = layernorm_eps, tao
        self._w = (LayerWeights * len(sets))(
            *[LayerWeights(*[ctypes.c_void_p(t.data_ptr()) for t in w]) for w in sets])
        self._prepacked = None
        self._buf = None
        self.dtype = _activation_dtype(sets[0])
        for w in sets[1:]:
            if _activation_dtype(w) != self.dtype:
                raise ValueError("all layers must share one weight dtype")

    def _config(self, B, S):
        w0 = self.weights[0]
        return EncoderConfig(_DTYPE_CODE[self.dtype], B, S, self.head_num, self.head_size,
                             w0[6].shape[1] // self.hidden, int(self.use_fused_attention),
                             int(self.is_remove_padding), int(w0[10].dtype == torch.float32),
                             self.tao, self.layernorm_eps)

    def prepack(self):
        """(Re)builds the k-contiguous weight copies; call again after changing weights."""
        lib = host_lib()
        cfg = self._config(1, 1)
        n = lib.bt_encoder_prepack_bytes(ctypes.byref(cfg), len(self.weights))
        dev = self.weights[0][0].device
        with torch.cuda.device(dev):
            buf = torch.empty(n, dtype=torch.int8, device=dev)
            rc = lib.bt_encoder_prepack(ctypes.byref(cfg), len(self.weights), self._w,
                                        ctypes.c_void_p(buf.data_ptr()),
                                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc != 0:
            raise RuntimeError(lib.bt_encoder_last_error().decode())
        self._prepacked = buf

    def __call__(self, x, mask, out=None, attention_bias=None, valid_rows_hint=0):
        lib = host_lib()
        _check_io(self.dtype, x, mask)
        B, S, H = x.shape
        if attention_bias is not None and (
                attention_bias.dtype != x.dtype or not attention_bias.is_contiguous()
                or tuple(attention_bias.shape) != (self.head_num, S, S)):
            raise ValueError("attention_bias must be a contiguous [head_num, S, S] tensor "
                             "of the activation dtype")
        if self._prepacked is None:
            self.prepack()
        cfg = self._config(B, S)
        need = lib.bt_encoder_forward_bufsize(ctypes.byref(cfg))
        if need == 0:
            raise RuntimeError(lib.bt_encoder_last_error().decode())
        if self._buf is None or self._buf.numel() < need or self._buf.device != x.device:
            self._buf = torch.empty(need, dtype=torch.int8, device=x.device)
        if out is None:
            out = torch.empty_like(x)
        rc = lib.bt_encoder_forward(
            ctypes.byref(cfg), len(self.weights), self._w,
            ctypes.c_void_p(self._prepacked.data_ptr()), ctypes.c_void_p(x.data_ptr()),
            ctypes.c_void_p(mask.data_ptr()),
            ctypes.c_void_p(attention_bias.data_ptr() if attention_bias is not None else None),
            ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(self._buf.data_ptr()), B, S,
            int(valid_rows_hint), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        if rc != 0:
            raise RuntimeError(lib.bt_encoder_last_error().decode())
        return out

    def graph(self, batch_size, seq_len, valid_rows_hint=0):
        """Captures one forward for a fixed [batch_size, seq_len] into a HIP graph."""
        return GraphedBertEncoder(self, batch_size, seq_len, valid_rows_hint)


class GraphedBertEncoder:
    """A captured BertEncoder forward.  `input`, `mask` and `output` are the
    static tensors the graph reads and writes: fill input / mask (any lengths -
    the offsets are rebuilt on the device inside the graph), call replay(), read
    output.  Calling the object copies its arguments in and returns `output`."""

    def __init__(self, encoder, batch_size, seq_len, valid_rows_hint=0):
        dev = encoder.weights[0][0].device
        self.encoder = encoder
        with torch.cuda.device(dev):
            self.input = torch.zeros(batch_size, seq_len, encoder.hidden, dtype=encoder.dtype,
                                     device=dev)
            self.mask = torch.ones(batch_size, seq_len, seq_len, dtype=encoder.dtype, device=dev)
            self.output = torch.empty_like(self.input)
            # first call outside the capture: one-time kernel attribute set-up, pre-pack, scratch
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                encoder(self.input, self.mask, out=self.output, valid_rows_hint=valid_rows_hint)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize(dev)
            self._graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self._graph):
                encoder(self.input, self.mask, out=self.output, valid_rows_hint=valid_rows_hint)
            # the graph holds raw pointers into these: keep them alive with it
            self._buf, self._prepacked = encoder._buf, encoder._prepacked

    def replay(self):
        self._graph.replay()
        return self.output

    def __call__(self, x, mask):
        self.input.copy_(x)
        self.mask.copy_(mask)
        return self.replay()
