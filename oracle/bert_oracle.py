"""CPU restatement of the reference's BERT encoder-layer forward.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The shipped package never imports it.

What each function follows in the reference (paths relative to the reference
tree) and how it is pinned (tests/test_oracle.py):

* seq_lens_from_mask / build_offsets   bytetransformer/include/remove_padding.h:36-86
      pinned: brute-force pure-Python walk over every length vector for tiny
      (B, S); closed form cumsum/arange.
* compress / restore                   remove_padding.h:104-121, layernorm.h:334-373
      pinned: restore(compress(x)) == x * rowmask bit-exactly; permutation check.
* gelu_tanh / gelu_erf                 gemm_bias_act.h:80-87 (tanh constants),
                                       unit_test/python_scripts/bert_transformer_test.py:151 (erf)
      pinned: math.erf / math.tanh scalar closed forms, special values,
      torch.nn.functional.gelu for both approximations.
* layer_norm                           layernorm.h:114-159 (two-pass, biased variance)
      pinned: zero-mean/unit-variance invariant, shift invariance,
      torch.nn.functional.layer_norm.
* attention_packed                     attention_fused.cu:220-260,348-381
      pinned: rows of P sum to S/(S+eps); padded keys contribute exactly 0;
      torch.nn.functional.scaled_dot_product_attention per sequence.
* encoder_layer                        bert_transformer_test.py:120-158
      pinned: torch.nn.TransformerEncoderLayer (post-norm, gelu) loaded with
      the same weights and a key-padding mask; independent float64 NumPy
      per-sequence/per-head loop (encoder_layer_packed_f64).
* gemm                                 gemm.cu:27-39 (row-major C = A.W)
      The reference's own tests pin nothing at the GEMM boundary beyond the
      end-to-end max-diff print; here numpy.matmul in float64 is the routine.

No function here is "parity unpinned".
"""
import math

import numpy as np
import torch
import torch.nn.functional as F

WEIGHT_NAMES = (
    "qkv_kernel", "qkv_bias",
    "attr_output_kernel", "attr_output_bias",
    "attr_output_layernorm_gamma", "attr_output_layernorm_beta",
    "inter_kernel", "inter_bias",
    "output_kernel", "output_bias",
    "output_layernorm_gamma", "output_layernorm_beta",
)


# ----------------------------------------------------------------------------
# padding removal / restoration (integer work: must be bit-exact)
# ----------------------------------------------------------------------------
def seq_lens_from_mask(mask):
    """len_b = #{i < S : mask[b, 0, i] >= 0.5}  (remove_padding.h:49-57).

    Only row 0 of each batch's [S, S] mask is consulted."""
    mask = np.asarray(mask)
    return (mask[:, 0, :].astype(np.float32) >= 0.5).sum(axis=1).astype(np.int32)


def build_offsets(mask):
    """batch_idx[B+1], word_idx[M], M  (remove_padding.h:36-86).

    batch_idx is the exclusive prefix sum of the lengths with the total
    appended; word_idx lists b*S+i for i < len_b in (b, i) order - valid
    tokens are taken to be a prefix of each row (remove_padding.h:81-85)."""
    mask = np.asarray(mask)
    B, S = mask.shape[0], mask.shape[2]
    lens = seq_lens_from_mask(mask)
    batch_idx = np.zeros(B + 1, dtype=np.int32)
    np.cumsum(lens, out=batch_idx[1:])
    word_idx = np.concatenate(
        [b * S + np.arange(lens[b], dtype=np.int32) for b in range(B)]
        + [np.zeros(0, dtype=np.int32)]).astype(np.int32)
    return batch_idx, word_idx, int(batch_idx[B])


def compress(x, word_idx):
    """packed[t, :] = x.reshape(B*S, H)[word_idx[t], :]  (remove_padding.h:104-121)."""
    x = np.asarray(x)
    return x.reshape(-1, x.shape[-1])[np.asarray(word_idx)]


def restore(packed, batch_idx, B, S):
    """out[b, s, :] = packed[batch_idx[b]+s] if s < len_b else 0  (layernorm.h:334-373)."""
    packed = np.asarray(packed)
    out = np.zeros((B, S, packed.shape[-1]), dtype=packed.dtype)
    for b in range(B):
        n = int(batch_idx[b + 1] - batch_idx[b])
        out[b, :n] = packed[batch_idx[b]:batch_idx[b] + n]
    return out


# ----------------------------------------------------------------------------
# elementwise pieces
# ----------------------------------------------------------------------------
def gelu_tanh(x):
    """0.5 x (1 + tanh(0.7978845608 (x + 0.044715 x^3)))  (gemm_bias_act.h:80-87)."""
    x = np.asarray(x, dtype=np.float64)
    return 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)))


def gelu_erf(x):
    """0.5 x (1 + erf(x / sqrt 2)) - F.gelu default used by the reference's
    PyTorch script (bert_transformer_test.py:151)."""
    x = np.asarray(x, dtype=np.float64)
    erf = np.vectorize(math.erf, otypes=[np.float64])
    return 0.5 * x * (1.0 + erf(x / math.sqrt(2.0)))


def layer_norm(v, gamma, beta, eps):
    """(v - mean) * rsqrt(mean((v - mean)^2) + eps) * gamma + beta, float64,
    two-pass biased variance (layernorm.h:114-159)."""
    v = np.asarray(v, dtype=np.float64)
    mean = v.mean(axis=-1, keepdims=True)
    c = v - mean
    var = (c * c).mean(axis=-1, keepdims=True)
    return c / np.sqrt(var + eps) * np.asarray(gamma, np.float64) + np.asarray(beta, np.float64)


def f16(a):
    """Round to fp16 and come back as float64 (the precision the kernels store)."""
    return np.asarray(a).astype(np.float16).astype(np.float64)


def add_bias_residual_layernorm(out, residual, bias, gamma, beta, eps=1e-6, fp16_adds=True):
    """LN((out + residual) + bias) with both adds rounded to fp16 as the CUDA
    kernel does with __hadd2 twice (layernorm.h:289-290); statistics in
    float64 here, fp32 on the device."""
    if fp16_adds:
        s = (np.asarray(out, np.float16) + np.asarray(residual, np.float16)).astype(np.float16)
        s = (s + np.asarray(bias, np.float16)).astype(np.float16)
    else:
        s = np.asarray(out, np.float64) + np.asarray(residual, np.float64) + np.asarray(bias, np.float64)
    return layer_norm(s, gamma, beta, eps)


# ----------------------------------------------------------------------------
# GEMM family (float64 on whatever precision the inputs carry)
# ----------------------------------------------------------------------------
def gemm(a, w, bias=None, act=None):
    """C[M,N] = A[M,K] . W[K,N] (+ bias) (then activation); weights are
    [in, out] row-major (gemm.cu:27-39, bert_transformer_test.py:100,124)."""
    c = np.asarray(a, np.float64) @ np.asarray(w, np.float64)
    if bias is not None:
        c = c + np.asarray(bias, np.float64)
    if act == "gelu_tanh":
        c = gelu_tanh(c)
    elif act == "gelu_erf":
        c = gelu_erf(c)
    elif act is not None:
        raise ValueError(act)
    return c


def split_heads(qkv, head_num, head_size):
    """[M, 3H] -> [3, head_num, M, head_size]; thirds are Q, K, V and head g is
    columns [g*d, (g+1)*d) of each third (attention_fused.cu:183-197)."""
    qkv = np.asarray(qkv)
    M = qkv.shape[0]
    return qkv.reshape(M, 3, head_num, head_size).transpose(1, 2, 0, 3)


def attention_packed(q, k, v, batch_idx, scale, softmax_eps=1e-6, round_p_fp16=True):
    """Per sequence b and head g over the packed rows of that sequence:
    P = exp(scale*QK^T - rowmax) / (rowsum + eps), optionally rounded to fp16
    (attention_fused.cu:348-381), O = P.V.  q, k, v: [heads, M, d].
    Returns token-major [M, heads*d] with head g at columns [g*d, (g+1)*d)."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    heads, M, d = q.shape
    out = np.zeros((M, heads * d), dtype=np.float64)
    for b in range(len(batch_idx) - 1):
        t0, t1 = int(batch_idx[b]), int(batch_idx[b + 1])
        if t1 == t0:
            continue
        for g in range(heads):
            s = (q[g, t0:t1] @ k[g, t0:t1].T) * scale
            e = np.exp(s - s.max(axis=-1, keepdims=True))
            p = e / (e.sum(axis=-1, keepdims=True) + softmax_eps)
            if round_p_fp16:
                p = f16(p)
            out[t0:t1, g * d:(g + 1) * d] = p @ v[g, t0:t1]
    return out


# ----------------------------------------------------------------------------
# the whole layer, padded, as the reference's PyTorch script computes it
# ----------------------------------------------------------------------------
def _t(a, dtype):
    return torch.as_tensor(np.asarray(a)).to(dtype)


def encoder_layer(x, mask, w, head_num, eps=1e-6, gelu="tanh", softmax_eps=1e-6, tao=1.0,
                  dtype=torch.float32, attention_bias=None):
    """One post-LN encoder layer on the PADDED [B, S, H] batch, on CPU torch
    (bert_transformer_test.py:120-158).  `w` maps WEIGHT_NAMES to arrays.

    eps / gelu / softmax_eps select between the three conventions the
    reference itself mixes: CUDA kernels (1e-6, tanh, 1e-6), its PyTorch
    script (1e-5, erf, 0) and the stated config (1e-12).

    attention_bias [head_num, S, S] is added to the scaled logits before the
    mask term (softmax.h:41-46; the reference's script has no such input)."""
    x = _t(x, dtype)
    mask = _t(mask, dtype)
    W = {n: _t(w[n], dtype) for n in WEIGHT_NAMES}
    B, S, H = x.shape
    d = H // head_num

    def heads(t):  # (B,S,H) -> (B,h,S,d)   bert_transformer_test.py:34-38
        return t.view(B, S, head_num, d).permute(0, 2, 1, 3)

    qkv = x @ W["qkv_kernel"] + W["qkv_bias"]
    q, k, v = qkv.chunk(3, dim=-1)
    scores = heads(q) @ heads(k).transpose(-2, -1) / (d ** 0.5) / tao
    if attention_bias is not None:
        scores = scores + _t(attention_bias, dtype).unsqueeze(0)
    scores = scores - 10000.0 * (1.0 - mask.unsqueeze(1))
    if softmax_eps == 0.0:
        probs = F.softmax(scores, dim=-1)
    else:
        e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
        probs = e / (e.sum(dim=-1, keepdim=True) + softmax_eps)
    ctx = (probs @ heads(v)).permute(0, 2, 1, 3).reshape(B, S, H)
    h1 = ctx @ W["attr_output_kernel"] + W["attr_output_bias"] + x
    h1 = F.layer_norm(h1, (H,), W["attr_output_layernorm_gamma"],
                      W["attr_output_layernorm_beta"], eps)
    inter = h1 @ W["inter_kernel"] + W["inter_bias"]
    inter = F.gelu(inter, approximate="tanh" if gelu == "tanh" else "none")
    h2 = inter @ W["output_kernel"] + W["output_bias"] + h1
    h2 = F.layer_norm(h2, (H,), W["output_layernorm_gamma"],
                      W["output_layernorm_beta"], eps)
    return h2


def encoder(x, mask, layers, head_num, **kw):
    """L stacked layers; returns the padded torch tensor of the last one
    (bert_transformer_test.py:118-158 loop)."""
    h = x
    for w in layers:
        h = encoder_layer(h, mask, w, head_num, **kw)
    return h


def masked_output(out, lens):
    """out * rowmask - what the reference compares (bert_transformer_test.py:160-162,205-207)."""
    out = np.array(out, copy=True)
    for b, n in enumerate(lens):
        out[b, int(n):] = 0
    return out


def encoder_layer_packed_f64(x, mask, w, head_num, eps=1e-6, gelu="tanh", softmax_eps=1e-6,
                             tao=1.0):
    """Independent float64 NumPy statement of the same layer on the PACKED
    rows (bert_transformer.cu:28-130 op order), used to cross-check
    encoder_layer and as the kernel-level composition.  Returns padded
    [B, S, H] with zero rows past each length."""
    x = np.asarray(x, np.float64)
    B, S, H = x.shape
    d = H // head_num
    batch_idx, word_idx, _ = build_offsets(mask)
    X = compress(x, word_idx)
    qkv = gemm(X, w["qkv_kernel"], w["qkv_bias"])
    q, k, v = split_heads(qkv, head_num, d)
    ctx = attention_packed(q, k, v, batch_idx, 1.0 / math.sqrt(d) / tao, softmax_eps,
                           round_p_fp16=False)
    a = gemm(ctx, w["attr_output_kernel"])
    y1 = add_bias_residual_layernorm(a, X, w["attr_output_bias"],
                                     w["attr_output_layernorm_gamma"],
                                     w["attr_output_layernorm_beta"], eps, fp16_adds=False)
    inter = gemm(y1, w["inter_kernel"], w["inter_bias"],
                 "gelu_tanh" if gelu == "tanh" else "gelu_erf")
    z = gemm(inter, w["output_kernel"])
    y2 = add_bias_residual_layernorm(z, y1, w["output_bias"], w["output_layernorm_gamma"],
                                     w["output_layernorm_beta"], eps, fp16_adds=False)
    return restore(y2, batch_idx, B, S)


def parity_metrics(ours, ref, lens):
    """(max-abs, mean-abs) over valid rows only, and whether every padded row
    of `ours` is exactly zero."""
    ours = np.asarray(ours, np.float64)
    ref = np.asarray(ref, np.float64)
    diffs = []
    pads_zero = True
    for b, n in enumerate(lens):
        n = int(n)
        diffs.append(np.abs(ours[b, :n] - ref[b, :n]).ravel())
        if n < ours.shape[1] and np.any(ours[b, n:] != 0):
            pads_zero = False
    dd = np.concatenate(diffs) if diffs else np.zeros(1)
    if dd.size == 0:
        dd = np.zeros(1)
    return float(dd.max()), float(dd.mean()), pads_zero
