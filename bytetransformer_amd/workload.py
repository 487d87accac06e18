"""Deterministic synthetic BERT-encoder workloads.

Shapes, weight layouts and the mask construction follow the reference's test
script (unit_test/python_scripts/bert_transformer_test.py:93-114): weights are
[in, out] row-major, the QKV weight is [H, 3H], the mask is [B, S, S] with
mask[b, i, j] = (j < len_b) for every row i, in the activation dtype.

Values use numpy's legacy RandomState (MT19937 + polar Box-Muller), whose
stream is frozen across numpy releases, so the same seed gives the same bits on
any machine.  Everything is drawn in float32 and rounded to the requested
dtype afterwards.
"""
from dataclasses import dataclass, field

import numpy as np

WEIGHT_NAMES = (
    "qkv_kernel", "qkv_bias",
    "attr_output_kernel", "attr_output_bias",
    "attr_output_layernorm_gamma", "attr_output_layernorm_beta",
    "inter_kernel", "inter_bias",
    "output_kernel", "output_bias",
    "output_layernorm_gamma", "output_layernorm_beta",
)


@dataclass
class EncoderConfig:
    name: str
    batch: int
    seq_len: int
    head_num: int
    head_size: int = 64
    layers: int = 12
    ffn_mult: int = 4
    dtype: str = "fp16"
    lens: tuple = ()          # explicit lengths; empty -> drawn uniformly on [low, seq_len]
    low_frac: float = 0.2
    seed: int = 0

    @property
    def hidden(self):
        return self.head_num * self.head_size


# The five named configurations: a single CPU-runnable fp32 layer, the batch-1
# short-sequence case, the headline padding-free shape, the long-sequence
# shape, and BERT-large with a fixed-length twin.
CONFIGS = {
    "cfg0": EncoderConfig("cfg0", 2, 64, 12, layers=1, dtype="fp32", lens=(64, 38)),
    "cfg1": EncoderConfig("cfg1", 1, 256, 12, lens=(154,)),
    "cfg2": EncoderConfig("cfg2", 16, 512, 12),
    "cfg3": EncoderConfig("cfg3", 16, 1024, 12),
    "cfg4": EncoderConfig("cfg4", 32, 384, 16, layers=24),
    "cfg4_fixed": EncoderConfig("cfg4_fixed", 32, 384, 16, layers=24, lens=(384,) * 32),
}


def draw_lengths(cfg: EncoderConfig):
    """Integer-uniform valid lengths on [ceil(low_frac*S), S] (mean ~0.6 S)."""
    if cfg.lens:
        return np.asarray(cfg.lens, dtype=np.int32)
    rs = np.random.RandomState(cfg.seed + 1000003)
    low = int(np.ceil(cfg.low_frac * cfg.seq_len))
    return rs.randint(low, cfg.seq_len + 1, size=cfg.batch).astype(np.int32)


def make_mask(lens, seq_len, np_dtype):
    """mask[b, i, j] = 1 if j < len_b else 0, for all i (bert_transformer_test.py:41-47,114)."""
    lens = np.asarray(lens)
    row = (np.arange(seq_len)[None, :] < lens[:, None]).astype(np_dtype)      # [B, S]
    return np.ascontiguousarray(np.broadcast_to(row[:, None, :], (len(lens), seq_len, seq_len)))


def make_layer_weights(hidden, ffn, rs, np_dtype, weight_std=0.02, bias_std=0.0,
                       random_affine=False):
    """One layer's 12 tensors.  Defaults: weights N(0, 0.02), biases 0, gamma 1,
    beta 0.  random_affine / bias_std > 0 draw non-trivial biases, gamma and
    beta so that tests exercise those operands."""
    def nrm(shape, std):
        return (rs.standard_normal(shape).astype(np.float32) * np.float32(std)).astype(np_dtype)

    def bias(n):
        return nrm((n,), bias_std) if bias_std > 0 else np.zeros(n, np_dtype)

    w = {}
    w["qkv_kernel"] = nrm((hidden, 3 * hidden), weight_std)
    w["qkv_bias"] = bias(3 * hidden)
    w["attr_output_kernel"] = nrm((hidden, hidden), weight_std)
    w["attr_output_bias"] = bias(hidden)
    if random_affine:
        w["attr_output_layernorm_gamma"] = (1 + nrm((hidden,), 0.1).astype(np.float32)).astype(np_dtype)
        w["attr_output_layernorm_beta"] = nrm((hidden,), 0.1)
    else:
        w["attr_output_layernorm_gamma"] = np.ones(hidden, np_dtype)
        w["attr_output_layernorm_beta"] = np.zeros(hidden, np_dtype)
    w["inter_kernel"] = nrm((hidden, ffn), weight_std)
    w["inter_bias"] = bias(ffn)
    w["output_kernel"] = nrm((ffn, hidden), weight_std)
    w["output_bias"] = bias(hidden)
    if random_affine:
        w["output_layernorm_gamma"] = (1 + nrm((hidden,), 0.1).astype(np.float32)).astype(np_dtype)
        w["output_layernorm_beta"] = nrm((hidden,), 0.1)
    else:
        w["output_layernorm_gamma"] = np.ones(hidden, np_dtype)
        w["output_layernorm_beta"] = np.zeros(hidden, np_dtype)
    return w


@dataclass
class Workload:
    cfg: EncoderConfig
    lens: np.ndarray
    x: np.ndarray                 # [B, S, H]
    mask: np.ndarray              # [B, S, S]
    layers: list = field(default_factory=list)   # list of dicts name -> array

    @property
    def valid_tokens(self):
        return int(self.lens.sum())


def make_workload(cfg, layers=None, bias_std=0.0, random_affine=False) -> Workload:
    """Seeded inputs and weights for a configuration (name or EncoderConfig)."""
    if isinstance(cfg, str):
        cfg = CONFIGS[cfg]
    np_dtype = np.float16 if cfg.dtype == "fp16" else np.float32
    n_layers = cfg.layers if layers is None else layers
    lens = draw_lengths(cfg)
    rs = np.random.RandomState(cfg.seed)
    x = rs.standard_normal((cfg.batch, cfg.seq_len, cfg.hidden)).astype(np.float32).astype(np_dtype)
    mask = make_mask(lens, cfg.seq_len, np_dtype)
    ws = [make_layer_weights(cfg.hidden, cfg.ffn_mult * cfg.hidden, rs, np_dtype,
                             bias_std=bias_std, random_affine=random_affine)
          for _ in range(n_layers)]
    return Workload(cfg, lens, x, mask, ws)


def make_reference_test_workload(batch, seq_len, head_num, head_size=64, avg_seqlen=0, layers=1,
                                 dtype="fp16", seed=0) -> Workload:
    """The data of the reference's own test script
    (unit_test/python_scripts/bert_transformer_test.py:93-114): every one of the 12
    tensors of a layer and the input drawn from U(-0.4, 0.4) (gamma and beta included),
    lengths integer-uniform on [2*avg - S, S] when 2*avg > S else on [0, 2*avg]
    (avg_seqlen 0 = every sequence full)."""
    np_dtype = np.float16 if dtype == "fp16" else np.float32
    hidden, ffn = head_num * head_size, 4 * head_num * head_size
    rs = np.random.RandomState(seed)
    avg = avg_seqlen if avg_seqlen > 0 else seq_len
    low, high = (2 * avg - seq_len, seq_len + 1) if 2 * avg > seq_len else (0, 2 * avg + 1)
    lens = rs.randint(low, high, size=batch).astype(np.int32)

    def uni(*shape):
        return rs.uniform(-0.4, 0.4, size=shape).astype(np.float32).astype(np_dtype)

    shapes = {"qkv_kernel": (hidden, 3 * hidden), "qkv_bias": (3 * hidden,),
              "attr_output_kernel": (hidden, hidden), "attr_output_bias": (hidden,),
              "attr_output_layernorm_gamma": (hidden,), "attr_output_layernorm_beta": (hidden,),
              "inter_kernel": (hidden, ffn), "inter_bias": (ffn,),
              "output_kernel": (ffn, hidden), "output_bias": (hidden,),
              "output_layernorm_gamma": (hidden,), "output_layernorm_beta": (hidden,)}
    ws = [{n: uni(*shapes[n]) for n in WEIGHT_NAMES} for _ in range(layers)]
    x = uni(batch, seq_len, hidden)
    cfg = EncoderConfig("reference-test-data", batch, seq_len, head_num, head_size, layers,
                        dtype=dtype, lens=tuple(int(v) for v in lens), seed=seed)
    return Workload(cfg, lens, x, make_mask(lens, seq_len, np_dtype), ws)


def layer_flops(cfg: EncoderConfig, lens):
    """Algorithmic flops of one layer: the four dense GEMMs on the M valid
    tokens plus unpadded, non-causal attention (QK^T and PV)."""
    H, F = cfg.hidden, cfg.ffn_mult * cfg.hidden
    M = int(np.sum(lens))
    gemm = 2 * M * H * (3 * H + H + 2 * F)
    attn = 4 * H * int(np.sum(np.asarray(lens, np.int64) ** 2))
    return gemm, attn
