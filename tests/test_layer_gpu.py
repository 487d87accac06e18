"""Whole-layer parity on the GPU: the C++ BertTransformer (through
bt_encoder_layer_forward) and the PyTorch operator against the CPU oracle on
identical seeded inputs and weights.

Tolerance (fp16 configurations): max-abs <= 2e-2 and mean-abs <= 2e-3 over the
valid rows, padded rows exactly zero on the remove-padding path.  The oracle is
the fp32 CPU encoder fed the same fp16-rounded inputs and weights."""
import os

import numpy as np
import pytest
import torch

import bytetransformer_amd as bt
from bytetransformer_amd import workload
from oracle import bert_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _say(*a):
    print(*a, flush=True)


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


_ORACLE_CACHE = {}


def _oracle(wl, n_layers=None, **kw):
    """The CPU oracle's masked output; memoised on the bytes of every operand, because
    each test runs once per attention dispatch and the oracle does not depend on it."""
    import zlib
    layers = wl.layers if n_layers is None else wl.layers[:n_layers]
    crc = zlib.crc32(np.ascontiguousarray(wl.x).tobytes())
    crc = zlib.crc32(np.ascontiguousarray(wl.mask).tobytes(), crc)
    for w in layers:
        for name in workload.WEIGHT_NAMES:
            crc = zlib.crc32(np.ascontiguousarray(w[name]).tobytes(), crc)
    key = (crc, wl.x.shape, wl.cfg.head_num, len(layers), tuple(int(v) for v in wl.lens),
           repr(sorted(kw.items())))
    if key not in _ORACLE_CACHE:
        layers32 = [{k: np.asarray(v, np.float32) for k, v in w.items()} for w in layers]
        out = O.encoder(wl.x.astype(np.float32), wl.mask.astype(np.float32), layers32,
                        wl.cfg.head_num, **kw)
        if len(_ORACLE_CACHE) > 8:
            _ORACLE_CACHE.clear()
        _ORACLE_CACHE[key] = O.masked_output(out.numpy(), wl.lens)
    return _ORACLE_CACHE[key]


def _gpu_layers(wl, device, n_layers=None, **kw):
    layers = wl.layers if n_layers is None else wl.layers[:n_layers]
    return [bt.BertEncoderLayer(wl.cfg.head_num, wl.cfg.head_size,
                                {k: _dev(v, device) for k, v in w.items()}, **kw)
            for w in layers]


def _run_c_api(wl, device, n_layers=None, **kw):
    layers = _gpu_layers(wl, device, n_layers, **kw)
    out = bt.encoder_forward(layers, _dev(wl.x, device), _dev(wl.mask, device))
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.fixture(autouse=True, params=[0, 512], ids=["default-dispatch", "short-kernel"])
def attention_short_limit(request):
    """Every test of this file runs twice.  "default-dispatch": the library as shipped and
    as the benchmark times it - every length goes to the streaming attention kernel, with
    its balanced work list and cache warm-up duty on large launches.  "short-kernel":
    use_fused_attention = True selects the LDS-resident short kernel up to its capacity of
    512 tokens again, so that both kernels are covered through the layer."""
    from bytetransformer_amd import ops
    ops.set_option("attention_short_limit", request.param)
    yield request.param
    ops.set_option("attention_short_limit", 0)


def _run_th_op(wl, device, n_layers=None, rm=True, fused=True):
    bt.load_th_op()
    layers = wl.layers if n_layers is None else wl.layers[:n_layers]
    h, mask = _dev(wl.x, device), _dev(wl.mask, device)
    for w in layers:
        h = torch.ops.ByteTransformer.BertTransformer(
            wl.cfg.head_num, wl.cfg.head_size,
            *[_dev(w[n], device) for n in workload.WEIGHT_NAMES], h, mask, rm, fused)
    torch.cuda.synchronize()
    return h.cpu().numpy()


def _check(got, exp, lens, pads_must_be_zero=True, tag=""):
    mx, mean, pads_zero = O.parity_metrics(got, exp, lens)
    _say("parity %s: max-abs %.3e mean-abs %.3e pads_zero %s" % (tag, mx, mean, pads_zero))
    assert np.isfinite(np.asarray(got, np.float32)).all()
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    if pads_must_be_zero:
        assert pads_zero


# ---- committed golden case -------------------------------------------------------
@pytest.mark.parametrize("path", ["c_api", "th_op"])
@pytest.mark.parametrize("fused", [True, False])
def test_small_golden_case(device, path, fused):
    _say("golden small", path, fused)
    z = np.load(os.path.join(GOLDEN, "small_fp16_case.npz"))
    lens = z["lens"]
    cfg = workload.EncoderConfig("small", 3, 48, 2, layers=1, lens=tuple(int(v) for v in lens))
    wl = workload.Workload(cfg, lens, z["x"], workload.make_mask(lens, 48, np.float16),
                           [{n: z[n] for n in workload.WEIGHT_NAMES}])
    if path == "c_api":
        got = _run_c_api(wl, device, use_fused_attention=fused)
    else:
        got = _run_th_op(wl, device, fused=fused)
    _check(got, z["expected"], lens, tag="small/%s/fused=%s" % (path, fused))


# ---- the named configurations ------------------------------------------------------
def test_cfg0_shape_fp16_runs_padded_path(device):
    """B = 2 silently disables remove-padding (as in the reference); padded rows
    are then not zero, only valid rows are compared, against the committed cfg0
    golden output (fp32 oracle) with the fp16-rounded inputs of the same seed."""
    _say("cfg0 fp16")
    wl32 = workload.make_workload("cfg0")
    cfg = workload.EncoderConfig("cfg0h", 2, 64, 12, layers=1, dtype="fp16", lens=(64, 38))
    wl = workload.Workload(cfg, wl32.lens, wl32.x.astype(np.float16),
                           wl32.mask.astype(np.float16),
                           [{k: v.astype(np.float16) for k, v in wl32.layers[0].items()}])
    got = O.masked_output(_run_c_api(wl, device), wl.lens)
    _check(got, _oracle(wl), wl.lens, tag="cfg0/fp16-inputs")
    gold = np.load(os.path.join(GOLDEN, "cfg0_out.npy"))
    _check(got, gold, wl.lens, tag="cfg0/golden-fp32")


def test_cfg1_twelve_layers_short_kernel(device):
    _say("cfg1")
    wl = workload.make_workload("cfg1")
    exp = _oracle(wl)
    got = O.masked_output(_run_th_op(wl, device), wl.lens)   # B = 1: padded path
    _check(got, exp, wl.lens, tag="cfg1/th_op")
    got = O.masked_output(_run_c_api(wl, device, use_fused_attention=False), wl.lens)
    _check(got, exp, wl.lens, tag="cfg1/c_api/grouped")


def test_cfg2_one_layer_and_invariants(device):
    _say("cfg2 one layer")
    wl = workload.make_workload("cfg2", layers=1, bias_std=0.02, random_affine=True)
    exp = _oracle(wl)
    got = _run_c_api(wl, device)
    _check(got, exp, wl.lens, tag="cfg2/L1/rm")
    got_op = _run_th_op(wl, device)
    assert np.array_equal(got_op.view(np.uint16), got.view(np.uint16))   # same kernels, same bits
    # the result must not depend on what the padded input rows hold
    x2 = wl.x.copy()
    for b, n in enumerate(wl.lens):
        x2[b, n:] = np.float16(300.0)
    wl2 = workload.Workload(wl.cfg, wl.lens, x2, wl.mask, wl.layers)
    assert np.array_equal(_run_c_api(wl2, device).view(np.uint16), got.view(np.uint16))
    # padded path on the same data: valid rows agree with the packed path
    got_pad = O.masked_output(_run_c_api(wl, device, is_remove_padding=False), wl.lens)
    _check(got_pad, exp, wl.lens, tag="cfg2/L1/padded")
    mx, _, _ = O.parity_metrics(got_pad, got, wl.lens)
    assert mx <= 4e-3, mx


def test_cfg2_twelve_layers_headline(device):
    _say("cfg2 twelve layers")
    wl = workload.make_workload("cfg2")
    assert abs(wl.valid_tokens / (16 * 512) - 0.6) < 0.1
    exp = _oracle(wl)
    got = _run_th_op(wl, device)
    _check(got, exp, wl.lens, tag="cfg2/L12/th_op")


def test_cfg3_long_sequences_grouped_kernel(device):
    _say("cfg3 two layers")
    wl = workload.make_workload("cfg3", layers=2)
    exp = _oracle(wl)
    got = _run_c_api(wl, device)
    _check(got, exp, wl.lens, tag="cfg3/L2")


def test_cfg3_full_depth_twelve_layers(device):
    """cfg3 at its full depth through the operator (the path the benchmark times)."""
    _say("cfg3 twelve layers")
    wl = workload.make_workload("cfg3")
    assert len(wl.layers) == 12
    _check(_run_th_op(wl, device), _oracle(wl), wl.lens, tag="cfg3/L12/th_op")


def test_cfg4_bert_large_variable_and_fixed(device):
    _say("cfg4")
    wl = workload.make_workload("cfg4", layers=2)
    _check(_run_c_api(wl, device), _oracle(wl), wl.lens, tag="cfg4/var/L2")
    # fixed-length twin: the padding-free path must match the padded path
    wf = workload.make_workload("cfg4_fixed", layers=2)
    rm = _run_c_api(wf, device, is_remove_padding=True)
    pad = _run_c_api(wf, device, is_remove_padding=False)
    _check(rm, _oracle(wf), wf.lens, tag="cfg4/fixed/L2")
    # two roundings of the same math (mask term folded before / after the scale): a few
    # fp16 ulps at |y| in [2, 4) after two layers, far inside the parity budget
    assert np.abs(rm.astype(np.float32) - pad.astype(np.float32)).max() <= 8e-3


@pytest.mark.parametrize("name", ["cfg4", "cfg4_fixed"])
def test_cfg4_full_depth_twenty_four_layers(device, name):
    """BERT-large at all 24 layers, ragged lengths and the fixed-length twin, through the
    operator; the fixed-length twin also on the padded rows."""
    _say(name, "twenty-four layers")
    wl = workload.make_workload(name)
    assert len(wl.layers) == 24
    exp = _oracle(wl)
    got = _run_th_op(wl, device)
    _check(got, exp, wl.lens, tag=name + "/L24/th_op")
    if name == "cfg4_fixed":
        pad = _run_th_op(wl, device, rm=False)
        _check(pad, exp, wl.lens, pads_must_be_zero=False, tag=name + "/L24/th_op/padded rows")


# ---- the reference's own test distribution -----------------------------------------
@pytest.mark.parametrize("B,S,heads,avg,layers", [(4, 64, 2, 40, 1), (8, 128, 4, 77, 3),
                                                  (16, 512, 12, 307, 1), (16, 512, 12, 307, 12)],
                         ids=["small", "medium-3-layers", "cfg2-shape-1-layer",
                              "cfg2-shape-12-layers"])
def test_reference_test_distribution(device, B, S, heads, avg, layers):
    """The only data the reference's own script ever tests with
    (unit_test/python_scripts/bert_transformer_test.py:93-114): every weight, bias, gamma,
    beta and the input drawn from U(-0.4, 0.4), lengths uniform on [2*avg - S, S].
    Activations there are ~50x larger than with N(0, 0.02) weights (|FFN2 output| ~ 50
    before the last LayerNorm), so fp16 storage of the intermediates is what is tested."""
    _say("reference distribution", B, S, heads, avg, layers)
    wl = workload.make_reference_test_workload(B, S, heads, avg_seqlen=avg, layers=layers, seed=2)
    exp = _oracle(wl)
    _check(_run_th_op(wl, device), exp, wl.lens, tag="ref-dist/th_op B%d S%d L%d" % (B, S, layers))
    if layers == 1:
        _check(_run_c_api(wl, device), exp, wl.lens, tag="ref-dist/c_api B%d S%d" % (B, S))


def test_padded_path_applies_arbitrary_masks(device):
    """Batch <= 2 (or is_remove_padding = False) runs on the padded rows and must
    honour any 0/1 mask pattern, not only prefixes - every row is compared."""
    _say("padded path, arbitrary mask")
    rs = np.random.RandomState(12)
    cfg = workload.EncoderConfig("am", 2, 72, 4, layers=2, lens=(72, 72), seed=9)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    mask = (rs.rand(2, 72, 72) < 0.7).astype(np.float16)
    i, j = np.indices((72, 72))
    mask[1] = (j <= i).astype(np.float16)                       # causal
    wl = workload.Workload(cfg, wl.lens, wl.x, mask, wl.layers)
    exp = _oracle(wl)
    _check(_run_th_op(wl, device), exp, wl.lens, pads_must_be_zero=False, tag="mask/th_op")
    _check(_run_c_api(wl, device, use_fused_attention=False), exp, wl.lens,
           pads_must_be_zero=False, tag="mask/c_api/grouped")
    cfg5 = workload.EncoderConfig("am5", 5, 40, 2, layers=1, lens=(40,) * 5, seed=10)
    wl5 = workload.make_workload(cfg5, bias_std=0.05, random_affine=True)
    m5 = (rs.rand(5, 40, 40) < 0.5).astype(np.float16)
    m5[:, :, 0] = 1
    wl5 = workload.Workload(cfg5, wl5.lens, wl5.x, m5, wl5.layers)
    _check(_run_c_api(wl5, device, is_remove_padding=False), _oracle(wl5), wl5.lens,
           pads_must_be_zero=False, tag="mask/c_api/no-rm")


@pytest.mark.parametrize("rm,S,lens", [(True, 48, (48, 20, 33, 7)), (False, 40, (40, 12, 40)),
                                       (True, 300, (300, 120, 211))])
def test_attention_bias_through_the_layer(device, rm, S, lens):
    """The optional [head_num, S, S] bias of the infer parameters reaches the logits
    on the packed path, the padded path and the streaming kernel."""
    _say("attention bias, layer", rm, S)
    rs = np.random.RandomState(21)
    cfg = workload.EncoderConfig("ab", len(lens), S, 2, layers=1, lens=tuple(lens), seed=13)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    bias = (0.5 * rs.standard_normal((2, S, S))).astype(np.float16)
    w32 = {k: np.asarray(v, np.float32) for k, v in wl.layers[0].items()}
    exp = O.encoder_layer(wl.x.astype(np.float32), wl.mask.astype(np.float32), w32, 2,
                          attention_bias=bias.astype(np.float32)).numpy()
    layer = _gpu_layers(wl, device, is_remove_padding=rm)[0]
    got = layer(_dev(wl.x, device), _dev(wl.mask, device), attention_bias=_dev(bias, device))
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    if rm:
        exp = O.masked_output(exp, wl.lens)
    _check(got, exp, wl.lens, pads_must_be_zero=rm, tag="bias rm=%s S=%d" % (rm, S))
    plain = layer(_dev(wl.x, device), _dev(wl.mask, device)).cpu().numpy()
    assert np.abs(plain.astype(np.float32) - got.astype(np.float32)).max() > 1e-2   # not a no-op
    with pytest.raises(ValueError):
        layer(_dev(wl.x, device), _dev(wl.mask, device), attention_bias=_dev(bias[:, :-1], device))


# ---- whole encoder in one call ---------------------------------------------------
def _whole_encoder(wl, device, **kw):
    return bt.BertEncoder(wl.cfg.head_num, wl.cfg.head_size,
                          [{k: _dev(v, device) for k, v in w.items()} for w in wl.layers], **kw)


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg4"])
def test_whole_encoder_matches_oracle_and_layer_by_layer(device, name):
    """bt_encoder_forward (hidden state packed between layers) against the oracle and
    against the per-layer entry point on the same inputs."""
    _say("whole encoder", name)
    wl = workload.make_workload(name)
    n = min(wl.cfg.layers, 4)
    wl4 = workload.Workload(wl.cfg, wl.lens, wl.x, wl.mask, wl.layers[:n])
    enc = _whole_encoder(wl4, device)
    got = enc(_dev(wl.x, device), _dev(wl.mask, device), valid_rows_hint=wl.valid_tokens)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    rm = wl.cfg.batch > 2
    _check(got, _oracle(wl4), wl.lens, pads_must_be_zero=rm, tag="whole/" + name)
    per_layer = _run_c_api(wl4, device)
    d = np.abs(got.astype(np.float32) - per_layer.astype(np.float32))
    for b, ln in enumerate(wl.lens):
        assert d[b, :int(ln)].max() <= 2e-3, d[b, :int(ln)].max()     # same kernels, same order


def test_whole_encoder_graph_replays_with_changing_lengths(device):
    """One captured graph serves any lengths: the offsets are rebuilt on the device
    inside it.  Replays alternate with eager work and are checked every time."""
    _say("whole encoder graph")
    cfg = workload.EncoderConfig("g", 6, 96, 4, layers=3, lens=(96, 40, 77, 5, 60, 31), seed=3)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    enc = _whole_encoder(wl, device)
    g = enc.graph(cfg.batch, cfg.seq_len)
    rs = np.random.RandomState(0)
    for it in range(4):
        lens = np.array(cfg.lens) if it == 0 else rs.randint(1, cfg.seq_len + 1, cfg.batch)
        mask = workload.make_mask(lens, cfg.seq_len, np.float16)
        x = (wl.x if it == 0 else rs.standard_normal(wl.x.shape)).astype(np.float16)
        cur = workload.Workload(cfg, lens, x, mask, wl.layers)
        out = g(_dev(x, device), _dev(mask, device))
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        eager = enc(_dev(x, device), _dev(mask, device))         # eager work between replays
        torch.cuda.synchronize()
        _check(got, _oracle(cur), lens, tag="graph replay %d" % it)
        assert np.array_equal(got, eager.cpu().numpy())


def test_whole_encoder_padded_path_bias_and_errors(device):
    _say("whole encoder padded / bias / errors")
    rs = np.random.RandomState(4)
    cfg = workload.EncoderConfig("p", 2, 40, 2, layers=2, lens=(40, 17), seed=5)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    bias = (0.5 * rs.standard_normal((2, 40, 40))).astype(np.float16)
    enc = _whole_encoder(wl, device)
    got = enc(_dev(wl.x, device), _dev(wl.mask, device), attention_bias=_dev(bias, device))
    torch.cuda.synchronize()
    layers32 = [{k: np.asarray(v, np.float32) for k, v in w.items()} for w in wl.layers]
    exp = O.encoder(wl.x.astype(np.float32), wl.mask.astype(np.float32), layers32, 2,
                    attention_bias=bias.astype(np.float32)).numpy()
    _check(got.cpu().numpy(), exp, wl.lens, pads_must_be_zero=False, tag="whole/padded+bias")
    with pytest.raises(ValueError):
        bt.BertEncoder(2, 64, [])
    with pytest.raises(RuntimeError):
        enc(_dev(wl.x, device).float(), _dev(wl.mask, device))


def test_fp32_gamma_beta_next_to_fp16_weights(device):
    _say("fp32 gamma/beta")
    cfg = workload.EncoderConfig("g32", 4, 96, 4, layers=1, lens=(96, 5, 50, 77), seed=21)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    exp = _oracle(wl)
    for n in workload.WEIGHT_NAMES:
        if "layernorm" in n:
            wl.layers[0][n] = wl.layers[0][n].astype(np.float32)
    _check(_run_th_op(wl, device), exp, wl.lens, tag="g32/th_op")
    _check(_run_c_api(wl, device), exp, wl.lens, tag="g32/c_api")


@pytest.mark.parametrize("tao", [0.5, 3.0])
def test_fp16_softmax_temperature(device, tao):
    """tao != 1 on the fp16 kernels (attention.h:32 of the reference: scale = 1/sqrt(d)/tao),
    packed rows and padded rows."""
    _say("fp16 tao", tao)
    cfg = workload.EncoderConfig("tao", 4, 130, 3, layers=2, lens=(130, 9, 64, 77), seed=17)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    for w in wl.layers:     # logits of a few units, so that the temperature matters
        w["qkv_kernel"] = (w["qkv_kernel"].astype(np.float32) * 6).astype(np.float16)
    exp = _oracle(wl, tao=tao)
    assert np.abs(exp - _oracle(wl)).max() > 1e-2        # the temperature is not a no-op
    _check(_run_c_api(wl, device, tao=tao), exp, wl.lens, tag="tao %.1f/packed" % tao)
    got = O.masked_output(_run_c_api(wl, device, tao=tao, is_remove_padding=False), wl.lens)
    _check(got, exp, wl.lens, tag="tao %.1f/padded rows" % tao)


def test_ragged_edge_cases(device):
    """Zero-length sequences, length 1, odd seq_len, non-default FFN multiple."""
    _say("ragged")
    cfg = workload.EncoderConfig("rag", 5, 37, 3, layers=2, ffn_mult=2, lens=(0, 1, 37, 36, 0),
                                 seed=33)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    _check(_run_c_api(wl, device), _oracle(wl), wl.lens, tag="ragged")
    _check(_run_th_op(wl, device), _oracle(wl), wl.lens, tag="ragged/th_op")


@pytest.mark.parametrize("seed", range(48))
def test_random_small_configurations(device, seed):
    """Seeded random shapes - batch, sequence length, head count, lengths with zeros and
    full ones, both dtypes, both row layouts, both attention kernels - one layer each
    through the C API against the oracle."""
    rs = np.random.RandomState(1000 + seed)
    B = int(rs.randint(1, 10))
    S = int(rs.choice([1, 2, 7, 16, 31, 64, 65, 100, 129, 200, 257, 300]))
    heads = int(rs.choice([1, 2, 3, 5, 12]))
    lens = rs.randint(0, S + 1, size=B)
    lens[rs.randint(B)] = S
    rm = bool(rs.randint(2))
    fused = bool(rs.randint(2))
    dtype = "fp32" if seed % 4 == 3 else "fp16"
    _say("random", seed, B, S, heads, lens.tolist(), rm, fused, dtype)
    cfg = workload.EncoderConfig("rnd%d" % seed, B, S, heads, layers=1, dtype=dtype,
                                 lens=tuple(int(v) for v in lens), seed=seed)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    if dtype == "fp32":
        exp = O.masked_output(O.encoder(wl.x, wl.mask, wl.layers, heads).numpy(), wl.lens)
    else:
        exp = _oracle(wl)
    got = _run_c_api(wl, device, is_remove_padding=rm, use_fused_attention=fused)
    packed = rm and B > 2          # batches of one or two run on the padded rows
    if not packed:
        got = O.masked_output(got, wl.lens)
    mx, mean, pads_zero = O.parity_metrics(got, exp, wl.lens)
    _say("parity random/%d: max-abs %.3e mean-abs %.3e" % (seed, mx, mean))
    assert np.isfinite(np.asarray(got, np.float32)).all()
    if dtype == "fp32":
        assert mx <= 2e-4 and mean <= 2e-5, (mx, mean)
    else:
        assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    assert pads_zero


@pytest.mark.parametrize("lens", [(90, 17, 64, 1, 33), (90, 0, 64, 1, 33), (40, 90)])
def test_operator_on_padded_rows_with_a_prefix_mask(device, lens):
    """On the padded rows the operator checks once per mask whether it is the plain prefix
    mask; then the attention stops at each length instead of reading the tensor (not with
    an empty sequence, whose all-masked softmax is not "no keys").  Valid rows match the
    oracle and the path that always applies the tensor."""
    cfg = workload.EncoderConfig("pp", len(lens), 90, 3, layers=2, lens=lens)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    exp = _oracle(wl)
    got = O.masked_output(_run_th_op(wl, device, rm=False), wl.lens)
    _check(got, exp, wl.lens, tag="padded rows/prefix mask/th_op")
    ref = O.masked_output(_run_c_api(wl, device, is_remove_padding=False), wl.lens)
    mx, _, _ = O.parity_metrics(got, ref, wl.lens)
    assert mx <= 8e-3, mx


@pytest.mark.parametrize("rm", [True, False])
def test_balanced_workgroup_order_through_the_layer(device, rm):
    """The streaming attention kernel with its balanced work list forced on (small launches
    keep the plain order by themselves): ragged and empty sequences, with and without
    remove-padding, bit-identical to the default order."""
    from bytetransformer_amd import ops
    cfg = workload.EncoderConfig("bal", 7, 200, 3, layers=2, lens=(200, 0, 77, 1, 130, 64, 199))
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    exp = _oracle(wl)
    ops.set_option("attention_short_limit", 0)
    try:
        ops.set_option("attention_xcd_map", 3)
        got = _run_c_api(wl, device, is_remove_padding=rm)
        ops.set_option("attention_xcd_map", 1)
        ref = _run_c_api(wl, device, is_remove_padding=rm)
    finally:
        ops.set_option("attention_xcd_map", 2)
    assert np.array_equal(got, ref)
    if not rm:
        got = O.masked_output(got, wl.lens)
    _check(got, exp, wl.lens, tag="balanced order rm=%s" % rm)


@pytest.mark.parametrize("seed", range(24))
def test_random_whole_encoder_bias_masks_and_operator(device, seed):
    """Seeded random stacks of 1-3 layers through the whole-encoder entry and the PyTorch
    operator: FFN widths 1-4x, optional attention bias, arbitrary 0/1 masks on the padded
    rows, both dtypes."""
    rs = np.random.RandomState(5000 + seed)
    B = int(rs.randint(1, 8))
    S = int(rs.choice([3, 8, 33, 64, 72, 130, 260]))
    heads = int(rs.choice([1, 2, 4]))
    layers = int(rs.randint(1, 4))
    mult = int(rs.choice([1, 2, 4]))
    rm = bool(rs.randint(2))
    fused = bool(rs.randint(2))
    with_bias = bool(rs.randint(2))
    dtype = "fp32" if seed % 3 == 2 else "fp16"
    npdt = np.float32 if dtype == "fp32" else np.float16
    packed = rm and B > 2
    lens = rs.randint(0, S + 1, size=B)
    lens[rs.randint(B)] = S
    if not packed:
        lens[:] = S                      # arbitrary masks below: every row is a valid row
    _say("random stack", seed, B, S, heads, layers, mult, rm, fused, with_bias, dtype, lens.tolist())
    cfg = workload.EncoderConfig("rs%d" % seed, B, S, heads, layers=layers, ffn_mult=mult,
                                 dtype=dtype, lens=tuple(int(v) for v in lens), seed=seed)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    mask = wl.mask
    if not packed:
        mask = (rs.rand(B, S, S) < 0.7).astype(npdt)
        mask[:, :, 0] = 1                # every query keeps a key
    bias = (0.5 * rs.standard_normal((heads, S, S))).astype(npdt) if with_bias else None
    h = torch.from_numpy(wl.x.astype(np.float32))
    for w in wl.layers:
        h = O.encoder_layer(h, mask.astype(np.float32),
                            {k: np.asarray(v, np.float32) for k, v in w.items()}, heads,
                            attention_bias=None if bias is None else bias.astype(np.float32))
    exp = O.masked_output(h.numpy(), wl.lens)
    x, m = _dev(wl.x, device), _dev(mask, device)
    bd = None if bias is None else _dev(bias, device)
    enc = bt.BertEncoder(heads, 64, [{k: _dev(v, device) for k, v in w.items()} for w in wl.layers],
                         is_remove_padding=rm, use_fused_attention=fused)
    got = enc(x, m, attention_bias=bd).cpu().numpy()
    tol = (2e-4, 2e-5) if dtype == "fp32" else (MAX_ABS, MEAN_ABS)
    for tag, g in (("whole", got),):
        mx, mean, pads_zero = O.parity_metrics(g if packed else O.masked_output(g, wl.lens), exp, wl.lens)
        _say("parity random stack/%d/%s: max-abs %.3e mean-abs %.3e" % (seed, tag, mx, mean))
        assert np.isfinite(np.asarray(g, np.float32)).all()
        assert mx <= tol[0] and mean <= tol[1], (tag, mx, mean)
        assert pads_zero
    if bias is None:                     # the operator's schema has no attention_bias argument
        bt.load_th_op()
        g = x
        for w in wl.layers:
            g = torch.ops.ByteTransformer.BertTransformer(
                heads, 64, *[_dev(w[n], device) for n in workload.WEIGHT_NAMES], g, m, rm, fused)
        g = g.cpu().numpy()
        mx, mean, _ = O.parity_metrics(g if packed else O.masked_output(g, wl.lens), exp, wl.lens)
        _say("parity random stack/%d/th_op: max-abs %.3e mean-abs %.3e" % (seed, mx, mean))
        assert mx <= tol[0] and mean <= tol[1], ("th_op", mx, mean)


@pytest.mark.parametrize("dtype,head_size,heads", [("fp16", 128, 2), ("fp16", 32, 4),
                                                   ("fp16", 96, 2), ("fp32", 128, 2),
                                                   ("fp32", 32, 6), ("fp32", 96, 2),
                                                   ("fp16", 16, 4), ("fp16", 80, 4),
                                                   ("fp32", 48, 4)])
@pytest.mark.parametrize("rm", [True, False])
def test_head_sizes_other_than_64(device, dtype, head_size, heads, rm):
    """Head sizes other than 64 (multiples of 8 up to 128): the QKV projection stays token-major and the generic
    attention kernel takes over (the reference's unfused path for them)."""
    _say("head size", dtype, head_size, heads, rm)
    cfg = workload.EncoderConfig("hs", 4, 70, heads, head_size=head_size, layers=2, dtype=dtype,
                                 lens=(70, 12, 0, 45), seed=head_size)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    layers32 = [{k: np.asarray(v, np.float32) for k, v in w.items()} for w in wl.layers]
    exp = O.masked_output(O.encoder(wl.x.astype(np.float32), wl.mask.astype(np.float32), layers32,
                                    heads).numpy(), wl.lens)
    tol = (2e-4, 2e-5) if dtype == "fp32" else (MAX_ABS, MEAN_ABS)
    for tag, got in (("c_api", _run_c_api(wl, device, is_remove_padding=rm)),
                     ("th_op", _run_th_op(wl, device, rm=rm)),
                     ("whole", _whole_encoder(wl, device, is_remove_padding=rm)(
                         _dev(wl.x, device), _dev(wl.mask, device)).cpu().numpy())):
        g = got if rm else O.masked_output(got, wl.lens)
        mx, mean, pads_zero = O.parity_metrics(g, exp, wl.lens)
        _say("parity head size %d/%s/%s: max-abs %.3e mean-abs %.3e" % (head_size, dtype, tag, mx, mean))
        assert mx <= tol[0] and mean <= tol[1] and pads_zero, (tag, mx, mean, pads_zero)


def test_hidden_size_rule_of_the_fp16_layer(device):
    """head_num * head_size must be a multiple of 64 on fp16 (the MFMA products step
    through k in tiles of 64); the float layer takes 12 x 40 = 480."""
    bt.load_th_op()
    cfg = workload.EncoderConfig("h480", 3, 33, 12, head_size=40, layers=1, lens=(33, 7, 20))
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        _run_th_op(wl, device)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        _run_c_api(wl, device)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        _whole_encoder(wl, device)(_dev(wl.x, device), _dev(wl.mask, device))
    cfg32 = workload.EncoderConfig("h480f", 3, 33, 12, head_size=40, layers=1, dtype="fp32",
                                   lens=(33, 7, 20))
    wl32 = workload.make_workload(cfg32, bias_std=0.05, random_affine=True)
    exp = O.masked_output(O.encoder(wl32.x, wl32.mask, wl32.layers, 12).numpy(), wl32.lens)
    mx, mean, pads_zero = O.parity_metrics(_run_th_op(wl32, device), exp, wl32.lens)
    assert mx <= 2e-4 and mean <= 2e-5 and pads_zero, (mx, mean)


@pytest.mark.parametrize("dtype", ["fp16", "fp32"])
def test_seq_len_one(device, dtype):
    """seq_len 1: batch_idx has one entry more than there are rows (the scratch carve once
    let the sequence order overwrite its last entry, the live-row count)."""
    cfg = workload.EncoderConfig("s1", 6, 1, 12, layers=1, dtype=dtype, lens=(0, 1, 0, 0, 1, 0))
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    exp = O.masked_output(O.encoder(wl.x.astype(np.float32), wl.mask.astype(np.float32),
                                    [{k: np.asarray(v, np.float32) for k, v in wl.layers[0].items()}],
                                    12).numpy(), wl.lens)
    _check(_run_c_api(wl, device), exp, wl.lens, tag="seq_len 1/" + dtype)
    _check(_run_th_op(wl, device), exp, wl.lens, tag="seq_len 1/th_op/" + dtype)


@pytest.mark.parametrize("B,S,lens,heads", [
    # (remove-padding needs a batch of three or more, as in the reference)
    (3, 1024, (200, 0, 0), 12),         # split-k FFN2 although batch * seq_len is beyond its limit
    (3, 640, (0, 333, 0), 12),          # the same shape without split-k
    (4, 256, (256, 1, 100, 17), 4),     # several sequences, one of them full
    (3, 128, (0, 128, 0), 2),           # empty sequences around a full one
])
def test_operator_sizes_packed_launches_for_the_live_rows(device, B, S, lens, heads):
    """The operator knows the exact number of live rows (its mask plan reads it back) and
    sizes the launches after the attention for it; the per-layer C entry does not and sizes
    them for batch * seq_len.  Both must give the oracle's layer, padded rows zero."""
    ffn = 4 if heads * 64 * 4 >= 2048 else 16    # split-k needs k >= 2048
    cfg = workload.EncoderConfig("tight", B, S, heads, layers=2, lens=lens, ffn_mult=ffn)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    exp = _oracle(wl)
    _check(_run_th_op(wl, device), exp, wl.lens, tag="live-row capacity/th_op")
    _check(_run_c_api(wl, device), exp, wl.lens, tag="live-row capacity/c_api")


def test_default_dispatch_is_the_streaming_kernel(device):
    """attention_short_limit defaults to 0: with it the fused flag changes nothing, and the
    result still matches the oracle."""
    from bytetransformer_amd import ops
    ops.set_option("attention_short_limit", 0)
    assert ops.get_option("attention_short_limit") == 0
    wl = workload.make_workload(workload.EncoderConfig("dd", 4, 100, 2, layers=1,
                                                       lens=(100, 30, 64, 7)))
    a = _run_c_api(wl, device, use_fused_attention=True)
    b = _run_c_api(wl, device, use_fused_attention=False)
    assert np.array_equal(a, b)
    _check(a, _oracle(wl), wl.lens, tag="default dispatch")
    ops.set_option("attention_short_limit", 512)
    c = _run_c_api(wl, device, use_fused_attention=True)
    assert not np.array_equal(a, c)          # another kernel, another rounding
    _check(c, _oracle(wl), wl.lens, tag="short kernel")


def test_two_threads_two_streams_share_nothing(device):
    """The operator from two host threads at once, each on its own stream and its own
    batch: the caches are keyed per stream and every call owns its scratch, so each thread
    must get exactly what it gets alone."""
    import threading
    bt.load_th_op()
    op = torch.ops.ByteTransformer.BertTransformer
    jobs = []
    for seed, (B, S) in enumerate([(4, 96), (6, 130)]):
        cfg = workload.EncoderConfig("mt%d" % seed, B, S, 2, layers=3, seed=40 + seed)
        wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
        ws = [[_dev(w[n], device) for n in workload.WEIGHT_NAMES] for w in wl.layers]
        jobs.append((ws, _dev(wl.x, device), _dev(wl.mask, device)))

    def forward(job):
        ws, x, m = job
        h = x
        for w in ws:
            h = op(2, 64, *w, h, m, True, True)
        return h

    alone = [forward(j).clone() for j in jobs]
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def worker(i):
        try:
            stream = torch.cuda.Stream(device=device)
            with torch.cuda.stream(stream):
                for _ in range(30):
                    out = forward(jobs[i])
                stream.synchronize()
            results[i] = out
        except Exception as exc:   # noqa: BLE001 - reported by the assertion below
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i in range(2):
        assert results[i] is not None and torch.equal(results[i], alone[i])


def test_th_op_tracks_weight_and_mask_updates(device):
    """The operator reads weights and mask as they are at each call: an in-place update
    of a weight or of the mask is picked up, and new tensors at recycled addresses are
    simply other tensors."""
    _say("weight and mask updates")
    bt.load_th_op()
    cfg = workload.EncoderConfig("pc", 4, 64, 2, layers=1, lens=(64, 20, 33, 50), seed=3)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
    x, m = _dev(wl.x, device), _dev(wl.mask, device)
    op = torch.ops.ByteTransformer.BertTransformer
    a = op(2, 64, *w, x, m, True, True)
    b = op(2, 64, *w, x, m, True, True)
    assert torch.equal(a, b)
    _check(a.cpu().numpy(), _oracle(wl), wl.lens, tag="cache/first")
    # in-place update of FFN2's weight
    w[8].mul_(0.5)
    wl.layers[0]["output_kernel"] = (wl.layers[0]["output_kernel"].astype(np.float32) * 0.5).astype(np.float16)
    c = op(2, 64, *w, x, m, True, True)
    assert not torch.equal(a, c)
    _check(c.cpu().numpy(), _oracle(wl), wl.lens, tag="cache/after-inplace-update")
    # in-place change of the mask: the token count kept for that mask tensor must go
    new_lens = np.array([30, 64, 10, 50])
    m.copy_(_dev(workload.make_mask(new_lens, 64, np.float16), device))
    wl_m = workload.Workload(wl.cfg, new_lens, wl.x, workload.make_mask(new_lens, 64, np.float16),
                             wl.layers)
    e = op(2, 64, *w, x, m, True, True)
    _check(e.cpu().numpy(), _oracle(wl_m), new_lens, tag="cache/after-mask-update")
    m.copy_(_dev(wl.mask, device))
    # brand-new tensors (old ones freed, addresses may be recycled)
    for _ in range(3):
        wl2 = workload.make_workload(workload.EncoderConfig("pc2", 4, 64, 2, layers=1,
                                                            lens=(64, 20, 33, 50), seed=4 + _),
                                     bias_std=0.05, random_affine=True)
        del w
        w = [_dev(wl2.layers[0][n], device) for n in workload.WEIGHT_NAMES]
        d = op(2, 64, *w, _dev(wl2.x, device), m, True, True)
        _check(d.cpu().numpy(), _oracle(wl2), wl2.lens, tag="cache/new-tensors")


def test_th_op_caches_cannot_change_results(device):
    """Writes that go around the version counter (`t.data.copy_()`, the way DLPack consumers
    and raw-pointer kernels write too) between two operator calls: weights, the mask on the
    packed rows and the mask on the padded rows.  The second result must be what the operator
    gives with its caches switched off."""
    _say("caches vs raw writes")
    bt.load_th_op()
    op = torch.ops.ByteTransformer.BertTransformer
    for B, S, lens, lens2 in [(4, 64, (64, 20, 33, 50), (30, 64, 64, 50)),
                              (2, 72, (72, 31), (40, 72))]:
        cfg = workload.EncoderConfig("raw", B, S, 2, layers=1, lens=lens, seed=3)
        wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
        w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
        x, m = _dev(wl.x, device), _dev(wl.mask, device)
        first = op(2, 64, *w, x, m, True, True)
        versions = [t._version for t in w] + [m._version]
        # every matrix and the mask rewritten behind the operator's back
        other = workload.make_workload(workload.EncoderConfig("raw2", B, S, 2, layers=1, lens=lens2,
                                                              seed=4),
                                       bias_std=0.05, random_affine=True)
        for i in (0, 2, 6, 8):
            w[i].data.copy_(_dev(other.layers[0][workload.WEIGHT_NAMES[i]], device))
        m.data.copy_(_dev(other.mask, device))
        assert [t._version for t in w] + [m._version] == versions       # nothing the host can see
        second = op(2, 64, *w, x, m, True, True)
        torch.ops.ByteTransformer.set_caches_enabled(False)
        try:
            plain = op(2, 64, *w, x, m, True, True)
        finally:
            torch.ops.ByteTransformer.set_caches_enabled(True)
        assert not torch.equal(first, second)
        assert torch.equal(second, plain)
        mixed = {n: (other.layers[0][n] if i in (0, 2, 6, 8) else wl.layers[0][n])
                 for i, n in enumerate(workload.WEIGHT_NAMES)}
        wl2 = workload.Workload(cfg, np.array(lens2), wl.x, other.mask, [mixed])
        got = second.cpu().numpy()
        _check(got if B > 2 else O.masked_output(got, wl2.lens), _oracle(wl2), wl2.lens,
               tag="raw writes B=%d" % B)
        # one element of one weight
        w[8].data[5, 7] += 0.5
        third = op(2, 64, *w, x, m, True, True)
        torch.ops.ByteTransformer.set_caches_enabled(False)
        try:
            plain = op(2, 64, *w, x, m, True, True)
        finally:
            torch.ops.ByteTransformer.set_caches_enabled(True)
        assert torch.equal(third, plain) and not torch.equal(third, second)
    torch.ops.ByteTransformer.clear_caches()


def test_layer_prepack_choice_never_changes_the_result(device):
    """Which products run on a per-call k-contiguous copy of their weight is a matter of
    time only: never, always and the measured table's choice give the same bits, on
    packed and on padded rows."""
    _say("layer_prepack")
    from bytetransformer_amd import ops
    bt.load_th_op()
    op = torch.ops.ByteTransformer.BertTransformer
    for cfg in (workload.EncoderConfig("pp", 6, 200, 12, layers=1, lens=(200, 20, 133, 50, 64, 7), seed=8),
                workload.EncoderConfig("pp2", 2, 72, 2, layers=1, lens=(72, 31), seed=9)):
        wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
        w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
        x, m = _dev(wl.x, device), _dev(wl.mask, device)
        got = {}
        try:
            for choice in (0, 1, -1):
                ops.set_option("layer_prepack", choice)
                got[choice] = op(cfg.head_num, 64, *w, x, m, True, True)
        finally:
            ops.set_option("layer_prepack", -1)
        assert torch.equal(got[0], got[1]) and torch.equal(got[0], got[-1])
        out = got[1].cpu().numpy()
        _check(out if cfg.batch > 2 else O.masked_output(out, wl.lens), _oracle(wl), wl.lens,
               tag="layer_prepack " + cfg.name)


def test_qkv_rows_from_the_mask_never_change_the_result(device):
    """A padding-free layer may start with the QKV product that counts the mask rows itself
    instead of the prologue launch: never, wherever the entry takes the shape (without the
    per-call weight copies), and the automatic choice give the same bits - ragged lengths
    with an empty sequence, the headline shape with 4 and with 12 heads, and a batch beyond
    the entry's 64 sequences (which falls back by itself).  (A fourth choice, workgroups of
    that launch making the copies and the attention's work list, was taken out of the
    library after one unexplained GPU fault under the C++ driver.)"""
    _say("qkv_mask_rows")
    from bytetransformer_amd import ops
    bt.load_th_op()
    op = torch.ops.ByteTransformer.BertTransformer
    assert ops.get_option("qkv_mask_rows") == -1
    cases = (workload.EncoderConfig("mr", 6, 200, 12, layers=1, lens=(200, 0, 133, 50, 64, 7), seed=18),
             workload.EncoderConfig("mr2", 16, 512, 4, layers=1, seed=19),
             workload.EncoderConfig("mr4", 16, 512, 12, layers=1, seed=21),
             workload.EncoderConfig("mr3", 70, 16, 2, layers=1, seed=20))
    for cfg in cases:
        wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
        w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
        x, m = _dev(wl.x, device), _dev(wl.mask, device)
        got = {}
        try:
            for choice in (0, 1, -1):
                ops.set_option("qkv_mask_rows", choice)
                got[choice] = op(cfg.head_num, 64, *w, x, m, True, True)
        finally:
            ops.set_option("qkv_mask_rows", -1)
        assert torch.equal(got[0], got[1]) and torch.equal(got[0], got[-1])
        _check(got[1].cpu().numpy(), _oracle(wl), wl.lens, tag="qkv_mask_rows " + cfg.name)


def test_weight_copies_in_the_layernorm_launch_never_change_the_result(device):
    """FFN1's (and FFN2's) k-contiguous copy may be made by the first LayerNorm's launch instead
    of a prologue, or not at all: the same bits with the option on and off, on the headline
    shape, with several rounds of tiles, on BERT-large shapes, with the fused start forced and
    with the prologue forced - and within tolerance of the oracle."""
    _say("ln_weight_copy")
    from bytetransformer_amd import ops
    bt.load_th_op()
    op = torch.ops.ByteTransformer.BertTransformer
    assert ops.get_option("ln_weight_copy") == 1
    cases = (workload.EncoderConfig("lc", 16, 512, 12, layers=1, seed=31),
             workload.EncoderConfig("lc2", 16, 1024, 12, layers=1, seed=32),
             workload.EncoderConfig("lc3", 32, 384, 16, layers=1, seed=33),
             workload.EncoderConfig("lc4", 6, 200, 12, layers=1, lens=(200, 0, 133, 50, 64, 7), seed=34))
    for cfg in cases:
        wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
        w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
        x, m = _dev(wl.x, device), _dev(wl.mask, device)
        got = {}
        try:
            for ln_copy, start, prepack in ((1, -1, -1), (0, -1, -1), (1, 1, -1), (1, 0, -1), (1, 1, 1), (0, 1, 1)):
                ops.set_option("ln_weight_copy", ln_copy)
                ops.set_option("qkv_mask_rows", start)
                ops.set_option("layer_prepack", prepack)
                got[(ln_copy, start, prepack)] = op(cfg.head_num, 64, *w, x, m, True, True)
        finally:
            ops.set_option("ln_weight_copy", 1)
            ops.set_option("qkv_mask_rows", -1)
            ops.set_option("layer_prepack", -1)
        ref = got[(0, -1, -1)]
        for key, val in got.items():
            assert torch.equal(val, ref), (cfg.name, key)
        _check(ref.cpu().numpy(), _oracle(wl), wl.lens, tag="ln_weight_copy " + cfg.name)


def test_short_padded_layers_go_without_the_prologue(device):
    """Batches of one and two with up to padded_mask_direct tokens per sequence skip the
    prologue launch and let the attention apply the mask tensor: same results as with the
    prologue (lengths + prefix verdict), for the prefix mask, for a mask of another shape and
    with an attention bias."""
    _say("padded_mask_direct")
    from bytetransformer_amd import ops
    bt.load_th_op()
    op = torch.ops.ByteTransformer.BertTransformer
    assert ops.get_option("padded_mask_direct") == 320
    for B, S, lens in ((1, 64, (38,)), (2, 72, (72, 31)), (2, 256, (154, 256)), (1, 320, (257,))):
        cfg = workload.EncoderConfig("direct", B, S, 3, layers=1, lens=lens, seed=B * S)
        wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
        w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
        x = _dev(wl.x, device)
        banded = np.tril(np.ones((S, S), np.float16), 3) * np.triu(np.ones((S, S), np.float16), -5)
        for mask_np in (wl.mask, np.broadcast_to(banded, (B, S, S)).copy()):
            m = _dev(mask_np, device)
            got = {}
            try:
                for limit in (320, 0):
                    ops.set_option("padded_mask_direct", limit)
                    got[limit] = op(3, 64, *w, x, m, True, True)
            finally:
                ops.set_option("padded_mask_direct", 320)
            assert torch.equal(got[320], got[0]), (B, S)
        
        ref = op(3, 64, *w, x, _dev(wl.mask, device), True, True).cpu().numpy()
        _check(O.masked_output(ref, wl.lens), _oracle(wl), wl.lens, tag="mask direct %dx%d" % (B, S))


def test_th_op_under_graph_capture(device):
    """Two operator layers captured with torch.cuda.graph (the host keeps out of a capture:
    no token count is read back, the layer builds its offsets inside the graph), replayed
    with other lengths and inputs written into the same buffers, eager work in between."""
    _say("operator under capture")
    bt.load_th_op()
    op = torch.ops.ByteTransformer.BertTransformer
    cfg = workload.EncoderConfig("cap", 5, 80, 2, layers=2, lens=(80, 20, 33, 50, 7), seed=6)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    ws = [[_dev(w[n], device) for n in workload.WEIGHT_NAMES] for w in wl.layers]
    x, m = _dev(wl.x, device), _dev(wl.mask, device)

    def forward():
        h = x
        for w in ws:
            h = op(2, 64, *w, h, m, True, True)
        return h

    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream, as torch asks for
        forward()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = forward()
    rs = np.random.RandomState(1)
    for it in range(3):
        lens = np.array(cfg.lens) if it == 0 else rs.randint(1, cfg.seq_len + 1, cfg.batch)
        xn = (wl.x if it == 0 else rs.standard_normal(wl.x.shape)).astype(np.float16)
        mask = workload.make_mask(lens, cfg.seq_len, np.float16)
        x.copy_(_dev(xn, device))
        m.copy_(_dev(mask, device))
        graph.replay()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        eager = forward()                   # eager work (cached copies) between the replays
        torch.cuda.synchronize()
        cur = workload.Workload(cfg, lens, xn, mask, wl.layers)
        _check(got, _oracle(cur), lens, tag="captured operator, replay %d" % it)
        assert np.array_equal(got, eager.cpu().numpy())


def test_torchscript_class_forward_and_pickle(device):
    """torch.classes.ByteTransformer.BertTransformer: forward == functional
    operator, forwardv2 flags, TorchScript save/load round trip (pickle state =
    12 tensors + head_info)."""
    _say("torchscript class")
    import io
    bt.load_th_op()
    cfg = workload.EncoderConfig("ts", 4, 80, 2, layers=1, lens=(80, 20, 33, 50), seed=8)
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
    x, m = _dev(wl.x, device), _dev(wl.mask, device)
    layer = torch.classes.ByteTransformer.BertTransformer(2, 64, *w)
    ref = torch.ops.ByteTransformer.BertTransformer(2, 64, *w, x, m, True, True)
    out = layer.forward(x, m)
    assert torch.equal(out, ref)
    _check(out.cpu().numpy(), _oracle(wl), wl.lens, tag="class/forward")
    padded = layer.forwardv2(x, m, False, False)
    _check(O.masked_output(padded.cpu().numpy(), wl.lens), _oracle(wl), wl.lens,
           tag="class/forwardv2-padded")

    class Wrap(torch.nn.Module):
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, a, b):
            return self.inner.forward(a, b)

    scripted = torch.jit.script(Wrap(layer))
    buf = io.BytesIO()
    torch.jit.save(scripted, buf)
    buf.seek(0)
    loaded = torch.jit.load(buf, map_location=device)
    assert torch.equal(loaded(x, m), ref)
    with pytest.raises(RuntimeError, match="Inconsistency of Tensor type"):
        layer.forward(x.float(), m)


def test_th_op_error_paths_on_gpu(device):
    bt.load_th_op()
    cfg = workload.EncoderConfig("e", 3, 16, 2, layers=1, lens=(16, 3, 9))
    wl = workload.make_workload(cfg)
    w = [_dev(wl.layers[0][n], device) for n in workload.WEIGHT_NAMES]
    x, m = _dev(wl.x, device), _dev(wl.mask, device)
    op = torch.ops.ByteTransformer.BertTransformer
    with pytest.raises(RuntimeError, match="must be contiguous"):
        op(2, 64, *w, x.transpose(0, 1), m, True, True)
    with pytest.raises(RuntimeError, match="Inconsistency of Tensor type"):
        op(2, 64, *w, x.float(), m, True, True)
    with pytest.raises(RuntimeError, match="Wrong Tensor type"):
        op(2, 64, *[t.to(torch.bfloat16) for t in w], x.to(torch.bfloat16),
           m.to(torch.bfloat16), True, True)
    with pytest.raises(RuntimeError, match="seq_len too long"):
        op(2, 64, *w, torch.zeros(1, 1025, 128, dtype=torch.float16, device=device),
           torch.zeros(1, 1025, 1025, dtype=torch.float16, device=device), True, True)
    # float weights select the float kernels (covered by test_fp32_gpu.py), they are no error
    out = op(2, 64, *[t.float() for t in w], x.float(), m.float(), True, True)
    assert out.dtype == torch.float32
