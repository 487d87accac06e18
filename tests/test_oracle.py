"""Pins the CPU oracle (oracle/bert_oracle.py) against things it did not write
itself: brute force, closed forms, invariants and PyTorch library routines."""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from bytetransformer_amd import workload
from oracle import bert_oracle as O


# ---- offsets: brute force over every length vector for tiny (B, S) ----------
def _walk_offsets(lens, S):
    """Independent pure-Python walk in (b, i) order."""
    batch_idx, word_idx, t = [0], [], 0
    for b, n in enumerate(lens):
        for i in range(S):
            if i < n:
                word_idx.append(b * S + i)
                t += 1
        batch_idx.append(t)
    return batch_idx, word_idx, t


@pytest.mark.parametrize("B,S", [(1, 5), (2, 4), (3, 3)])
def test_offsets_brute_force(B, S):
    for lens in itertools.product(range(S + 1), repeat=B):
        mask = workload.make_mask(np.array(lens), S, np.float16)
        bi, wi, M = O.build_offsets(mask)
        ebi, ewi, eM = _walk_offsets(lens, S)
        assert bi.dtype == np.int32 and wi.dtype == np.int32
        assert bi.tolist() == ebi and wi.tolist() == ewi and M == eM


def test_offsets_only_row0_and_threshold():
    S = 6
    mask = np.zeros((2, S, S), np.float32)
    mask[0, 0, :] = [1, 0.5, 0.49, 0.9, 0, 0]   # three elements >= 0.5
    mask[0, 1:, :] = 1                            # other rows must be ignored
    mask[1, 0, :2] = 1
    assert O.seq_lens_from_mask(mask).tolist() == [3, 2]
    bi, wi, M = O.build_offsets(mask)
    assert bi.tolist() == [0, 3, 5] and wi.tolist() == [0, 1, 2, 6, 7] and M == 5


def test_compress_restore_roundtrip():
    rs = np.random.RandomState(1)
    B, S, H = 4, 9, 16
    lens = np.array([9, 0, 4, 1])
    x = rs.standard_normal((B, S, H)).astype(np.float16)
    bi, wi, M = O.build_offsets(workload.make_mask(lens, S, np.float16))
    packed = O.compress(x, wi)
    assert packed.shape == (M, H)
    # permutation check against flat indexing, and exact round trip
    assert np.array_equal(packed, x.reshape(B * S, H)[wi])
    assert np.array_equal(O.restore(packed, bi, B, S), O.masked_output(x, lens))


# ---- elementwise ------------------------------------------------------------
def test_gelu_closed_forms_and_library():
    xs = np.array([-10.0, -3.0, -1.0, -0.0, 0.0, 0.5, 1.0, 2.7, 10.0])
    for x, t, e in zip(xs, O.gelu_tanh(xs), O.gelu_erf(xs)):
        assert t == pytest.approx(0.5 * x * (1 + math.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x ** 3))), abs=1e-12)
        assert e == pytest.approx(0.5 * x * (1 + math.erf(x / math.sqrt(2))), abs=1e-12)
    assert O.gelu_tanh(0.0) == 0 and O.gelu_erf(0.0) == 0
    assert O.gelu_tanh(30.0) == pytest.approx(30.0) and abs(O.gelu_tanh(-30.0)) < 1e-12
    grid = np.linspace(-6, 6, 2001)
    tg = torch.tensor(grid, dtype=torch.float64)
    assert np.abs(O.gelu_tanh(grid) - F.gelu(tg, approximate="tanh").numpy()).max() < 1e-12
    assert np.abs(O.gelu_erf(grid) - F.gelu(tg).numpy()).max() < 1e-12
    # the two forms differ by at most ~4.7e-4 (tolerance budget of the build)
    assert 3e-4 < np.abs(O.gelu_tanh(grid) - O.gelu_erf(grid)).max() < 6e-4


def test_layer_norm_invariants_and_library():
    rs = np.random.RandomState(2)
    v = rs.standard_normal((7, 96)) * 3 + 1.5
    g, b = rs.standard_normal(96), rs.standard_normal(96)
    y = O.layer_norm(v, np.ones(96), np.zeros(96), 0.0)
    assert np.abs(y.mean(-1)).max() < 1e-12 and np.abs(y.var(-1) - 1).max() < 1e-12
    assert np.abs(O.layer_norm(v + 123.0, g, b, 1e-6) - O.layer_norm(v, g, b, 1e-6)).max() < 1e-9
    ref = F.layer_norm(torch.tensor(v), (96,), torch.tensor(g), torch.tensor(b), 1e-6).numpy()
    assert np.abs(O.layer_norm(v, g, b, 1e-6) - ref).max() < 1e-12


def test_add_bias_residual_layernorm_fp16_add_order():
    # (out + residual) rounded to fp16, then + bias rounded to fp16: pick values
    # where the order of the two roundings changes the fp16 sum
    out = np.array([[2048.0, 1.0, 0.5, 3.0]], np.float16)
    res = np.array([[1.0, 2048.0, 0.25, 1.0]], np.float16)
    bias = np.array([1.0, 1.0, 0.125, -4.0], np.float16)
    s = ((out + res).astype(np.float16) + bias).astype(np.float16)
    assert s[0, 0] == 2048.0 + 2.0 or s[0, 0] == 2048.0   # 2049 is not representable
    y = O.add_bias_residual_layernorm(out, res, bias, np.ones(4), np.zeros(4), 1e-6)
    assert np.allclose(y, O.layer_norm(s, np.ones(4), np.zeros(4), 1e-6))


# ---- attention ----------------------------------------------------------------
def test_attention_packed_invariants_and_sdpa():
    rs = np.random.RandomState(3)
    heads, d = 3, 64
    lens = [5, 0, 17, 1]
    bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    M = int(bi[-1])
    q, k, v = (rs.standard_normal((heads, M, d)) for _ in range(3))
    scale = 1 / math.sqrt(d)
    out = O.attention_packed(q, k, v, bi, scale, softmax_eps=0.0, round_p_fp16=False)
    for b, n in enumerate(lens):
        if n == 0:
            continue
        t0 = int(bi[b])
        ref = F.scaled_dot_product_attention(torch.tensor(q[:, t0:t0 + n]),
                                             torch.tensor(k[:, t0:t0 + n]),
                                             torch.tensor(v[:, t0:t0 + n]))
        ref = ref.permute(1, 0, 2).reshape(n, heads * d).numpy()
        assert np.abs(out[t0:t0 + n] - ref).max() < 1e-12
    # rows of P sum to S/(S+eps): V = ones -> output = that factor
    ones = np.ones_like(v)
    o1 = O.attention_packed(q, k, ones, bi, scale, softmax_eps=1e-6, round_p_fp16=False)
    assert np.all(o1 < 1.0) and np.all(o1 > 1.0 - 1.1e-6)
    # other sequences' rows do not leak in: perturb sequence 0, sequence 2 unchanged
    k2 = k.copy()
    k2[:, :5] += 100.0
    o2 = O.attention_packed(q, k2, v, bi, scale, softmax_eps=0.0, round_p_fp16=False)
    assert np.array_equal(o2[5:], out[5:])


def test_split_heads_layout():
    M, heads, d = 3, 2, 4
    H = heads * d
    qkv = np.arange(M * 3 * H).reshape(M, 3 * H)
    s = O.split_heads(qkv, heads, d)
    assert s.shape == (3, heads, M, d)
    for which in range(3):
        for g in range(heads):
            for t in range(M):
                assert s[which, g, t].tolist() == qkv[t, which * H + g * d: which * H + (g + 1) * d].tolist()


# ---- whole layer ----------------------------------------------------------------
def _small_workload(dtype="fp32", lens=(16, 7, 11), S=16, heads=2, seed=5):
    cfg = workload.EncoderConfig("t", len(lens), S, heads, layers=1, dtype=dtype, lens=tuple(lens),
                                 seed=seed)
    return workload.make_workload(cfg, bias_std=0.05, random_affine=True)


def test_encoder_layer_matches_torch_transformer_encoder_layer():
    """Post-LN, GELU(erf), softmax without eps is exactly nn.TransformerEncoderLayer."""
    wl = _small_workload()
    H, heads = wl.cfg.hidden, wl.cfg.head_num
    w = wl.layers[0]
    ours = O.encoder_layer(wl.x, wl.mask, w, heads, eps=1e-5, gelu="erf", softmax_eps=0.0,
                           dtype=torch.float64).numpy()
    layer = torch.nn.TransformerEncoderLayer(H, heads, dim_feedforward=4 * H, dropout=0.0,
                                             activation="gelu", layer_norm_eps=1e-5,
                                             batch_first=True, norm_first=False).double().eval()
    t = lambda a: torch.tensor(np.asarray(a, np.float64))
    with torch.no_grad():
        layer.self_attn.in_proj_weight.copy_(t(w["qkv_kernel"]).T)
        layer.self_attn.in_proj_bias.copy_(t(w["qkv_bias"]))
        layer.self_attn.out_proj.weight.copy_(t(w["attr_output_kernel"]).T)
        layer.self_attn.out_proj.bias.copy_(t(w["attr_output_bias"]))
        layer.norm1.weight.copy_(t(w["attr_output_layernorm_gamma"]))
        layer.norm1.bias.copy_(t(w["attr_output_layernorm_beta"]))
        layer.linear1.weight.copy_(t(w["inter_kernel"]).T)
        layer.linear1.bias.copy_(t(w["inter_bias"]))
        layer.linear2.weight.copy_(t(w["output_kernel"]).T)
        layer.linear2.bias.copy_(t(w["output_bias"]))
        layer.norm2.weight.copy_(t(w["output_layernorm_gamma"]))
        layer.norm2.bias.copy_(t(w["output_layernorm_beta"]))
        pad = torch.tensor(np.arange(wl.cfg.seq_len)[None, :] >= wl.lens[:, None])
        # train(False) + fast path off so the plain math path runs
        torch.backends.mha.set_fastpath_enabled(False)
        ref = layer(t(wl.x), src_key_padding_mask=pad).numpy()
    mx, mean, _ = O.parity_metrics(O.masked_output(ours, wl.lens), ref, wl.lens)
    assert mx < 1e-9, mx


def test_encoder_layer_attention_bias_and_arbitrary_mask_match_torch_float_mask():
    """Bias and a non-prefix 0/1 mask enter as additive terms: the same layer through
    nn.TransformerEncoderLayer with the float attention mask bias - 10000 (1 - mask)."""
    wl = _small_workload(lens=(16, 16), S=16)
    rs = np.random.RandomState(8)
    H, heads, S, B = wl.cfg.hidden, wl.cfg.head_num, wl.cfg.seq_len, wl.cfg.batch
    w = wl.layers[0]
    mask = (rs.rand(B, S, S) < 0.7).astype(np.float64)
    mask[:, :, 0] = 1
    bias = rs.standard_normal((heads, S, S))
    ours = O.encoder_layer(wl.x, mask, w, heads, eps=1e-5, gelu="erf", softmax_eps=0.0,
                           dtype=torch.float64, attention_bias=bias).numpy()
    layer = torch.nn.TransformerEncoderLayer(H, heads, dim_feedforward=4 * H, dropout=0.0,
                                             activation="gelu", layer_norm_eps=1e-5,
                                             batch_first=True, norm_first=False).double().eval()
    t = lambda a: torch.tensor(np.asarray(a, np.float64))
    with torch.no_grad():
        layer.self_attn.in_proj_weight.copy_(t(w["qkv_kernel"]).T)
        layer.self_attn.in_proj_bias.copy_(t(w["qkv_bias"]))
        layer.self_attn.out_proj.weight.copy_(t(w["attr_output_kernel"]).T)
        layer.self_attn.out_proj.bias.copy_(t(w["attr_output_bias"]))
        layer.norm1.weight.copy_(t(w["attr_output_layernorm_gamma"]))
        layer.norm1.bias.copy_(t(w["attr_output_layernorm_beta"]))
        layer.linear1.weight.copy_(t(w["inter_kernel"]).T)
        layer.linear1.bias.copy_(t(w["inter_bias"]))
        layer.linear2.weight.copy_(t(w["output_kernel"]).T)
        layer.linear2.bias.copy_(t(w["output_bias"]))
        layer.norm2.weight.copy_(t(w["output_layernorm_gamma"]))
        layer.norm2.bias.copy_(t(w["output_layernorm_beta"]))
        add = bias[None] - 10000.0 * (1.0 - mask[:, None])          # [B, heads, S, S]
        torch.backends.mha.set_fastpath_enabled(False)
        ref = layer(t(wl.x), src_mask=t(add.reshape(B * heads, S, S))).numpy()
    assert np.abs(ours - ref).max() < 1e-9
    # and the bias is not a no-op
    plain = O.encoder_layer(wl.x, mask, w, heads, eps=1e-5, gelu="erf", softmax_eps=0.0,
                            dtype=torch.float64).numpy()
    assert np.abs(ours - plain).max() > 1e-3


def test_encoder_layer_padded_torch_vs_packed_numpy_f64():
    wl = _small_workload()
    for eps, gelu, seps in [(1e-6, "tanh", 1e-6), (1e-5, "erf", 0.0), (1e-12, "tanh", 0.0)]:
        a = O.encoder_layer(wl.x, wl.mask, wl.layers[0], wl.cfg.head_num, eps=eps, gelu=gelu,
                            softmax_eps=seps, dtype=torch.float64).numpy()
        b = O.encoder_layer_packed_f64(wl.x, wl.mask, wl.layers[0], wl.cfg.head_num, eps=eps,
                                       gelu=gelu, softmax_eps=seps)
        mx, _, pads_zero = O.parity_metrics(b, a, wl.lens)
        assert mx < 1e-9 and pads_zero


def test_output_independent_of_padded_input_rows():
    wl = _small_workload()
    x2 = wl.x.copy()
    for b, n in enumerate(wl.lens):
        x2[b, n:] = 1e3
    a = O.encoder_layer(wl.x, wl.mask, wl.layers[0], wl.cfg.head_num).numpy()
    b = O.encoder_layer(x2, wl.mask, wl.layers[0], wl.cfg.head_num).numpy()
    mx, _, _ = O.parity_metrics(b, a, wl.lens)
    assert mx < 1e-4


def test_convention_spread_on_cfg0_is_inside_tolerance():
    """eps in {1e-6,1e-5,1e-12} x gelu in {tanh,erf} x softmax eps in {0,1e-6}
    all agree to < 1e-3 on the stated single-layer fp32 configuration."""
    wl = workload.make_workload("cfg0")
    base = O.encoder_layer(wl.x, wl.mask, wl.layers[0], 12).numpy()
    worst = 0.0
    for eps in (1e-6, 1e-5, 1e-12):
        for gelu in ("tanh", "erf"):
            for seps in (0.0, 1e-6):
                o = O.encoder_layer(wl.x, wl.mask, wl.layers[0], 12, eps=eps, gelu=gelu,
                                    softmax_eps=seps).numpy()
                mx, _, _ = O.parity_metrics(o, base, wl.lens)
                worst = max(worst, mx)
    assert worst < 1e-3, worst


def test_cfg0_golden_fixture():
    """The committed cfg0 output (tests/golden/cfg0_out.npy, written by
    tests/golden/make_golden.py) is reproduced bit-for-bit-ish by the oracle on
    the regenerated seeded workload, which also pins the workload generator."""
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "cfg0_out.npy")
    gold = np.load(path)
    wl = workload.make_workload("cfg0")
    assert wl.lens.tolist() == [64, 38]
    out = O.masked_output(O.encoder_layer(wl.x, wl.mask, wl.layers[0], 12).numpy(), wl.lens)
    assert np.abs(out - gold).max() < 2e-5
    chk = np.load(os.path.join(os.path.dirname(__file__), "golden", "workload_checksums.npz"))
    assert float(chk["cfg0_x_sum"]) == pytest.approx(float(wl.x.astype(np.float64).sum()), abs=1e-6)
    assert chk["cfg2_lens"].tolist() == workload.draw_lengths(workload.CONFIGS["cfg2"]).tolist()
