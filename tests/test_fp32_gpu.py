"""OperationType::FP32 on the GPU: the float kernels one by one against float64
NumPy statements of the same arithmetic, then the whole layer (C++ API through
bt_encoder_layer_forward, the PyTorch operator, the whole-encoder entry) against the
CPU oracle.

Tolerances (float): kernels carry a bound derived from fp32 rounding written in each
test; the whole layer must agree with the fp32 oracle within max-abs 2e-4 and mean-abs
2e-5 over the valid rows (outputs are O(1) after the last LayerNorm; both sides round
in fp32, in different orders)."""
import math
import os

import numpy as np
import pytest
import torch

import bytetransformer_amd as bt
from bytetransformer_amd import ops, workload
from oracle import bert_oracle as O

pytestmark = pytest.mark.gpu

F32_MAX_ABS, F32_MEAN_ABS = 2e-4, 2e-5
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _say(*a):
    print(*a, flush=True)


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


@pytest.fixture(params=[2, 3], ids=["default-order", "balanced-order"])
def att_order(request):
    """Runs a test under the default workgroup order and with the balanced work list
    forced on (small launches would not use it by themselves)."""
    ops.set_option("attention_xcd_map", request.param)
    yield request.param
    ops.set_option("attention_xcd_map", 2)


# ---- GEMM ------------------------------------------------------------------------
@pytest.mark.parametrize("rows,M,N,K", [(300, 300, 768, 768), (1000, 777, 2304, 768),
                                        (4920, 4920, 3072, 768), (640, 513, 768, 3072),
                                        (70, 70, 136, 200), (5, 3, 8, 4), (129, 129, 132, 20)])
def test_gemm_f32_plain_and_bias(device, rows, M, N, K):
    _say("gemm_f32", rows, M, N, K)
    rs = np.random.RandomState(rows + N)
    a = rs.standard_normal((rows, K)).astype(np.float32)
    a[M:] = np.nan                                   # rows past the live count are never read
    w = (rs.standard_normal((K, N)) * 0.05).astype(np.float32)
    bias = rs.standard_normal(N).astype(np.float32)
    vr = torch.tensor([M], dtype=torch.int32, device=device)
    # |error| <= K * 2^-24 * sum|a||w| is the textbook bound; sqrt(K) of it is generous
    bound = 4 * math.sqrt(K) * 2.0 ** -24 * (np.abs(a[:M]).astype(np.float64) @ np.abs(w)) + 1e-7
    for b in (None, bias):
        exp = O.gemm(a[:M], w, b)
        sentinel = torch.full((rows, N), 7.0, dtype=torch.float32, device=device)
        g = ops.gemm_f32(_dev(a, device), _dev(w, device), None if b is None else _dev(b, device),
                         valid_rows=vr, out=sentinel).cpu().numpy()
        assert np.all(np.abs(g[:M] - exp) <= bound), np.abs(g[:M] - exp).max()
        assert np.all(g[M:] == 7.0)


def test_gemm_f32_detects_transposed_or_shifted_operands(device):
    """Identity-like weights pin the operand orientation: A . P with P a cyclic column
    shift must shift the columns of A, exactly."""
    rs = np.random.RandomState(3)
    a = rs.standard_normal((200, 64)).astype(np.float32)
    p = np.roll(np.eye(64, dtype=np.float32), 5, axis=1)      # column j of A lands in j + 5
    g = ops.gemm_f32(_dev(a, device), _dev(p, device)).cpu().numpy()
    assert np.array_equal(g, np.roll(a, 5, axis=1))


def test_gemm_f32_bias_gelu_and_gather(device):
    _say("gemm_f32 gelu + gather")
    rs = np.random.RandomState(11)
    B, S, H, F = 4, 50, 128, 512
    lens = np.array([50, 0, 17, 33])
    x = rs.standard_normal((B, S, H)).astype(np.float32)
    mask = workload.make_mask(lens, S, np.float32)
    w = (rs.standard_normal((H, F)) * 0.2).astype(np.float32)
    bias = rs.standard_normal(F).astype(np.float32)
    g_bi, g_wi, M = ops.build_offsets(_dev(mask, device), want_count=True)
    packed = O.compress(x, g_wi.cpu().numpy()[:M])
    exp = O.gemm(packed, w, bias, "gelu_tanh")
    # the product's fp32 rounding (as in the plain test) passes through a slope <= 1.13,
    # then the activation adds a few ulp of its own
    bound = 1.13 * 4 * math.sqrt(H) * 2.0 ** -24 * (np.abs(packed).astype(np.float64) @ np.abs(w)) \
        + 4e-6 * np.abs(exp) + 2e-6
    g = ops.gemm_f32(_dev(x, device).view(B * S, H), _dev(w, device), _dev(bias, device),
                     gelu=True, valid_rows=g_bi[B:], a_row_index=g_wi).cpu().numpy()
    assert np.all(np.abs(g[:M] - exp) <= bound), np.abs(g[:M] - exp).max()
    assert np.all(g[M:] == 0)
    # special values of the activation: 0 -> 0, large |x| -> x or 0
    z = np.zeros((4, 4), np.float32)
    for v, want in ((0.0, 0.0), (30.0, 30.0), (-30.0, 0.0), (1e4, 1e4), (-1e4, 0.0)):
        b4 = np.full(4, v, np.float32)
        got = ops.gemm_f32(_dev(z, device), _dev(z, device), _dev(b4, device), gelu=True)
        assert np.all(got.cpu().numpy() == want), (v, got)


# ---- LayerNorm -------------------------------------------------------------------
@pytest.mark.parametrize("H", [768, 1024, 64, 4096, 260])
def test_layernorm_f32(device, H):
    _say("layernorm_f32", H)
    rs = np.random.RandomState(H)
    rows, M = 37, 30
    out = rs.standard_normal((rows, H)).astype(np.float32)
    res = (rs.standard_normal((rows, H)) + 3.0).astype(np.float32)
    bias = rs.standard_normal(H).astype(np.float32)
    gamma = (1 + 0.2 * rs.standard_normal(H)).astype(np.float32)
    beta = (0.3 * rs.standard_normal(H)).astype(np.float32)
    exp = O.add_bias_residual_layernorm(out[:M], res[:M], bias, gamma, beta, 1e-6, fp16_adds=False)
    vr = torch.tensor([M], dtype=torch.int32, device=device)
    g = ops.add_bias_residual_layernorm_f32(_dev(out, device), _dev(res, device), _dev(bias, device),
                                            _dev(gamma, device), _dev(beta, device), 1e-6,
                                            valid_rows=vr).cpu().numpy()
    assert np.all(np.abs(g[:M] - exp) <= 4e-6 * np.abs(exp) + 4e-6), np.abs(g[:M] - exp).max()
    assert np.array_equal(g[M:], out[M:])            # rows past M untouched
    # gamma = 1, beta = 0: every row has mean 0 and variance 1 / (1 + eps / var)
    one, zero = np.ones(H, np.float32), np.zeros(H, np.float32)
    g = ops.add_bias_residual_layernorm_f32(_dev(out, device), _dev(res, device), _dev(zero, device),
                                            _dev(one, device), _dev(zero, device), 1e-6).cpu().numpy()
    assert np.all(np.abs(g.mean(-1)) < 1e-5) and np.all(np.abs(g.var(-1) - 1) < 1e-4)


def test_layernorm_restore_f32_zero_fills(device):
    rs = np.random.RandomState(5)
    B, S, H = 5, 33, 768
    lens = np.array([33, 0, 20, 1, 32])
    mask = workload.make_mask(lens, S, np.float32)
    bi, wi, M = O.build_offsets(mask)
    out = rs.standard_normal((B * S, H)).astype(np.float32)
    res = rs.standard_normal((B * S, H)).astype(np.float32)
    bias = rs.standard_normal(H).astype(np.float32)
    gamma = (1 + 0.2 * rs.standard_normal(H)).astype(np.float32)
    beta = (0.3 * rs.standard_normal(H)).astype(np.float32)
    exp = O.restore(O.add_bias_residual_layernorm(out[:M], res[:M], bias, gamma, beta, 1e-6,
                                                  fp16_adds=False), bi, B, S)
    g_bi, _, _ = ops.build_offsets(_dev(mask, device))
    target = torch.full((B, S, H), float("nan"), dtype=torch.float32, device=device)
    g = ops.add_bias_residual_layernorm_restore_f32(
        _dev(out, device), _dev(res, device), _dev(bias, device), _dev(gamma, device),
        _dev(beta, device), g_bi, B, S, 1e-6, out_padded=target).cpu().numpy()
    for b in range(B):
        assert np.all(g[b, lens[b]:].view(np.uint32) == 0)
    assert np.all(np.abs(g - exp) <= 4e-6 * np.abs(exp) + 4e-6)


# ---- attention -------------------------------------------------------------------
def _naive_attention(qkv, lens, S, heads, d, scale, padded, mask=None, bias=None):
    """float64, one (sequence, head) at a time, logits + bias + (mask - 1) * 10000."""
    H = heads * d
    out = np.zeros((qkv.shape[0], H))
    start = 0
    for b, n in enumerate(lens):
        r0 = b * S if padded else start
        nq = S if padded else n
        nk = S if (padded and mask is not None) else n
        start += n
        if nk == 0:
            continue
        rows = qkv[r0:r0 + max(nq, nk)].astype(np.float64)
        for g in range(heads):
            q = rows[:nq, g * d:(g + 1) * d]
            k = rows[:nk, H + g * d:H + (g + 1) * d]
            v = rows[:nk, 2 * H + g * d:2 * H + (g + 1) * d]
            s = q @ k.T * scale
            if bias is not None:
                s = s + bias[g, :nq, :nk]
            if mask is not None:
                s = s + (mask[b, :nq, :nk].astype(np.float64) - 1.0) * 10000.0
            e = np.exp(s - s.max(-1, keepdims=True))
            p = e / (e.sum(-1, keepdims=True) + 1e-6)
            out[r0:r0 + nq, g * d:(g + 1) * d] = p @ v
    return out


F32_ATT_CASES = [
    ([64, 38], 64, 12, 64), ([154], 256, 12, 64), ([1, 16, 17, 0, 100, 128, 129], 160, 3, 64),
    ([300, 77, 5], 320, 2, 64), ([40, 33], 40, 4, 32), ([70, 9], 72, 2, 128),
    ([50, 31], 50, 2, 48), ([50, 31], 50, 3, 104),
]


@pytest.mark.parametrize("padded", [False, True])
@pytest.mark.parametrize("lens,S,heads,d", F32_ATT_CASES)
def test_attention_f32(device, lens, S, heads, d, padded, att_order):
    _say("attention_f32", lens, S, heads, d, padded)
    rs = np.random.RandomState(S + heads + d)
    B, H = len(lens), heads * d
    rows_cap = B * S
    bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    qkv = np.full((rows_cap, 3 * H), np.nan, np.float32)
    if padded:
        qkv[:] = rs.standard_normal(qkv.shape).astype(np.float32)   # padded rows hold finite junk
    else:
        qkv[:bi[-1]] = rs.standard_normal((bi[-1], 3 * H)).astype(np.float32)
    qkv[:, :H] *= 2.0
    scale = 1 / math.sqrt(d)
    exp = _naive_attention(qkv, lens, S, heads, d, scale, padded)
    # the issue order (longest first) must not change anything
    order = np.argsort(-np.asarray(lens), kind="stable").astype(np.int32)
    g = ops.attention_f32(_dev(qkv, device), _dev(bi, device), B, S, heads, scale,
                          padded_rows=padded, seq_order=_dev(order, device)).cpu().numpy()
    g0 = ops.attention_f32(_dev(qkv, device), _dev(bi, device), B, S, heads, scale,
                           padded_rows=padded).cpu().numpy()
    live = ~np.isnan(g0)
    assert np.array_equal(np.isnan(g), ~live) and np.array_equal(g[live], g0[live])
    for b, n in enumerate(lens):
        r0 = b * S if padded else bi[b]
        # padded rows: queries past the length attend the valid keys too (defined output)
        nq = S if padded else n
        if n == 0:
            continue
        err = np.abs(g[r0:r0 + nq] - exp[r0:r0 + nq])
        assert err.max() <= 2e-5, (b, err.max())


@pytest.mark.parametrize("padded", [False, True])
def test_attention_f32_mask_and_bias(device, padded, att_order):
    """An arbitrary 0/1 mask (every query keeps at least one key) and a bias: the kernel
    must apply both per (query, key), on both row layouts."""
    _say("attention_f32 mask+bias", padded)
    rs = np.random.RandomState(9)
    lens, S, heads, d = [72, 30, 50], 72, 3, 64
    B, H = len(lens), heads * d
    bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    qkv = rs.standard_normal((B * S, 3 * H)).astype(np.float32)
    mask = (rs.rand(B, S, S) < 0.6).astype(np.float32)
    mask[:, :, 0] = 1
    if not padded:
        for b, n in enumerate(lens):
            mask[b, :, n:] = 0
    bias = rs.standard_normal((heads, S, S)).astype(np.float32)
    scale = 0.125
    exp = _naive_attention(qkv, lens, S, heads, d, scale, padded, mask, bias)
    g = ops.attention_f32(_dev(qkv, device), _dev(bi, device), B, S, heads, scale,
                          padded_rows=padded, mask=_dev(mask, device),
                          bias=_dev(bias, device)).cpu().numpy()
    for b, n in enumerate(lens):
        r0, nq = (b * S, S) if padded else (bi[b], n)
        err = np.abs(g[r0:r0 + nq] - exp[r0:r0 + nq])
        assert err.max() <= 2e-5, (b, err.max())


@pytest.mark.parametrize("padded", [False, True])
@pytest.mark.parametrize("lens,S,heads,d", [([70, 9, 33], 72, 2, 128), ([40, 33], 40, 4, 32),
                                            ([150, 64, 1], 160, 2, 96), ([64, 38], 64, 3, 64),
                                            ([33, 70], 70, 4, 16), ([100, 5], 100, 2, 80),
                                            ([64, 64], 64, 3, 8)])
def test_attention_generic_f16(device, lens, S, heads, d, padded, att_order):
    """The same kernel on fp16 tensors (head sizes the fp16 attention kernels do not take):
    inputs rounded to fp16, arithmetic in float, one fp16 rounding of the output."""
    _say("attention_generic_f16", lens, S, heads, d, padded)
    rs = np.random.RandomState(S + heads + d)
    B, H = len(lens), heads * d
    bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    qkv = rs.standard_normal((B * S, 3 * H)).astype(np.float16)
    if not padded:
        qkv[bi[-1]:] = np.float16("nan")
    mask = None
    bias = (0.5 * rs.standard_normal((heads, S, S))).astype(np.float16)
    if padded:
        mask = (rs.rand(B, S, S) < 0.7).astype(np.float16)
        mask[:, :, 0] = 1
    scale = 1 / math.sqrt(d)
    exp = _naive_attention(qkv.astype(np.float32), lens, S, heads, d, scale, padded,
                           None if mask is None else mask.astype(np.float32),
                           bias.astype(np.float32))
    g = ops.attention_generic_f16(_dev(qkv, device), _dev(bi, device), B, S, heads, scale,
                                  padded_rows=padded,
                                  mask=None if mask is None else _dev(mask, device),
                                  bias=_dev(bias, device)).cpu().numpy()
    assert g.dtype == np.float16
    for b, n in enumerate(lens):
        r0, nq = (b * S, S) if padded else (bi[b], n)
        err = np.abs(g[r0:r0 + nq].astype(np.float64) - exp[r0:r0 + nq])
        assert np.all(err <= 2.0 ** -10 * np.abs(exp[r0:r0 + nq]) + 1e-4), (b, err.max())


def test_attention_f32_rows_sum_and_uniform_keys(device):
    """V = const per column: the output is that constant times sum(P) = 1 / (1 + 1e-6 / sum e),
    whatever Q and K are; identical keys give a uniform P."""
    rs = np.random.RandomState(2)
    S, heads, d = 96, 2, 64
    H = heads * d
    lens = [96, 41]
    bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    qkv = rs.standard_normal((2 * S, 3 * H)).astype(np.float32)
    qkv[:, 2 * H:] = np.arange(H, dtype=np.float32)[None, :]
    g = ops.attention_f32(_dev(qkv, device), _dev(bi, device), 2, S, heads, 0.125).cpu().numpy()
    M = bi[-1]
    assert np.all(np.abs(g[:M] - np.arange(H)[None, :]) <= 2e-5 * (1 + np.arange(H))[None, :])


# ---- the whole layer -------------------------------------------------------------
def _f32_check(got, exp, lens, tag, pads_zero_required):
    mx, mean, pads_zero = O.parity_metrics(got, exp, lens)
    _say("parity %s: max-abs %.3e mean-abs %.3e pads_zero %s" % (tag, mx, mean, pads_zero))
    assert np.isfinite(got).all()
    assert mx <= F32_MAX_ABS and mean <= F32_MEAN_ABS, (mx, mean)
    if pads_zero_required:
        assert pads_zero


def _oracle32(wl, **kw):
    out = O.encoder(wl.x, wl.mask, wl.layers, wl.cfg.head_num, **kw)
    return O.masked_output(out.numpy(), wl.lens)


def _layers(wl, device, **kw):
    return [bt.BertEncoderLayer(wl.cfg.head_num, wl.cfg.head_size,
                                {k: _dev(v, device) for k, v in w.items()}, **kw)
            for w in wl.layers]


def test_cfg0_fp32_matches_the_committed_golden_output(device):
    """The stated fp32 configuration: B = 2 (padded path as in the reference), lengths
    [64, 38], against the oracle and the committed golden output of the same seed."""
    wl = workload.make_workload("cfg0")
    assert wl.x.dtype == np.float32
    got = bt.encoder_forward(_layers(wl, device), _dev(wl.x, device), _dev(wl.mask, device))
    got = O.masked_output(got.cpu().numpy(), wl.lens)
    _f32_check(got, _oracle32(wl), wl.lens, "cfg0/fp32/oracle", False)
    _f32_check(got, np.load(os.path.join(GOLDEN, "cfg0_out.npy")), wl.lens, "cfg0/fp32/golden", False)


@pytest.mark.parametrize("path", ["c_api", "th_op", "whole"])
@pytest.mark.parametrize("rm", [True, False])
def test_fp32_layers_all_paths(device, path, rm):
    _say("fp32 layers", path, rm)
    cfg = workload.EncoderConfig("f32", 5, 80, 4, layers=2, dtype="fp32", lens=(80, 3, 41, 0, 64))
    wl = workload.make_workload(cfg, bias_std=0.1, random_affine=True)
    exp = _oracle32(wl)
    x, m = _dev(wl.x, device), _dev(wl.mask, device)
    if path == "c_api":
        got = bt.encoder_forward(_layers(wl, device, is_remove_padding=rm), x, m)
    elif path == "th_op":
        bt.load_th_op()
        got = x
        for w in wl.layers:
            got = torch.ops.ByteTransformer.BertTransformer(
                cfg.head_num, cfg.head_size, *[_dev(w[n], device) for n in workload.WEIGHT_NAMES],
                got, m, rm, True)
    else:
        enc = bt.BertEncoder(cfg.head_num, cfg.head_size,
                             [{k: _dev(v, device) for k, v in w.items()} for w in wl.layers],
                             is_remove_padding=rm)
        got = enc(x, m)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert got.dtype == np.float32
    if rm:
        _f32_check(got, exp, wl.lens, "f32/%s/rm" % path, True)
    else:
        # an empty sequence has no defined rows on the padded path; compare the rest
        _f32_check(O.masked_output(got, wl.lens), exp, wl.lens, "f32/%s/padded" % path, False)


def test_fp32_attention_bias_tao_and_ffn_width(device):
    """attention_bias, a softmax temperature and intermediate_size = 2 through the float layer."""
    cfg = workload.EncoderConfig("f32b", 3, 48, 2, layers=1, ffn_mult=2, dtype="fp32",
                                 lens=(48, 20, 33))
    wl = workload.make_workload(cfg, bias_std=0.1, random_affine=True)
    bias = np.random.RandomState(4).standard_normal((2, 48, 48)).astype(np.float32)
    exp = O.masked_output(O.encoder_layer(wl.x, wl.mask, wl.layers[0], 2, tao=1.7,
                                          attention_bias=bias).numpy(), wl.lens)
    layer = bt.BertEncoderLayer(2, 64, {k: _dev(v, device) for k, v in wl.layers[0].items()},
                                tao=1.7)
    got = layer(_dev(wl.x, device), _dev(wl.mask, device), attention_bias=_dev(bias, device))
    _f32_check(got.cpu().numpy(), exp, wl.lens, "f32/bias+tao+ffn2", True)


def test_fp32_bert_base_shape_one_layer(device):
    """A BERT-base layer at batch 8 x 256 in float: big enough for the 128x128 GEMM tiles and
    several key tiles, small enough for the CPU oracle."""
    cfg = workload.EncoderConfig("f32base", 8, 256, 12, layers=1, dtype="fp32")
    wl = workload.make_workload(cfg)
    got = bt.encoder_forward(_layers(wl, device), _dev(wl.x, device), _dev(wl.mask, device))
    _f32_check(got.cpu().numpy(), _oracle32(wl), wl.lens, "f32/bert-base", True)


def test_fp32_dtype_mismatches_are_rejected(device):
    cfg = workload.EncoderConfig("e32", 3, 16, 2, layers=1, dtype="fp32", lens=(16, 3, 9))
    wl = workload.make_workload(cfg)
    layer = bt.BertEncoderLayer(2, 64, {k: _dev(v, device) for k, v in wl.layers[0].items()})
    with pytest.raises(RuntimeError, match="weights' dtype"):
        layer(_dev(wl.x, device).half(), _dev(wl.mask, device).half())
    mixed = {k: _dev(v, device) for k, v in wl.layers[0].items()}
    mixed["inter_bias"] = mixed["inter_bias"].half()
    with pytest.raises(ValueError, match="has dtype"):
        bt.BertEncoderLayer(2, 64, mixed)
