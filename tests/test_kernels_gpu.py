"""Per-kernel parity: every C-ABI entry point of libbt_hip.so against the CPU
oracle on the same seeded inputs.  Integer outputs and copies are bit-exact;
fp16 results carry the tolerance written in each test."""
import math

import numpy as np
import pytest
import torch

from bytetransformer_amd import ops, workload
from oracle import bert_oracle as O

pytestmark = pytest.mark.gpu


def _dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def _say(*a):
    print(*a, flush=True)


# ---- offsets (bit-exact) -------------------------------------------------------
@pytest.mark.parametrize("B,S,dtype", [(1, 256, np.float16), (16, 512, np.float16),
                                       (3, 7, np.float32), (70, 33, np.float16),
                                       (130, 100, np.float16), (32, 384, np.float16),
                                       (16, 1024, np.float32)])
def test_build_offsets_bit_exact(device, B, S, dtype):
    _say("offsets", B, S, dtype)
    rs = np.random.RandomState(B * 1000 + S)
    lens = rs.randint(0, S + 1, size=B)
    lens[0] = S
    if B > 2:
        lens[1] = 0
    mask = workload.make_mask(lens, S, dtype)
    mask[:, 1:, :] = 1 - mask[:, 1:, :]          # rows other than 0 must be ignored
    bi, wi, M = O.build_offsets(mask)
    order = torch.full((B,), -1, dtype=torch.int32, device=device)
    g_bi, g_wi, g_M = ops.build_offsets(_dev(mask, device), want_count=True, seq_order=order)
    assert g_M == M
    # longest first, ties by index: the stable argsort of the negated lengths
    assert order.cpu().numpy().tolist() == np.argsort(-lens.astype(np.int64), kind="stable").tolist()
    assert g_bi.dtype == torch.int32 and g_wi.dtype == torch.int32
    assert np.array_equal(g_bi.cpu().numpy(), bi)
    assert np.array_equal(g_wi.cpu().numpy()[:M], wi)


def test_valid_token_count_published_into_pinned_memory(device):
    """The count the reference reads back with a blocking copy (remove_padding.h:99-100) is
    stored into pinned host memory by a one-wave launch behind the offsets: after the stream
    has drained the host finds the exact count there, for two masks in a row in the same slot."""
    slot = torch.full((4,), -1, dtype=torch.int32, pin_memory=True)
    for B, S, seed in ((16, 512, 1), (5, 33, 2)):
        _say("publish count", B, S)
        rs = np.random.RandomState(seed)
        lens = rs.randint(0, S + 1, size=B)
        mask = workload.make_mask(lens, S, np.float16)
        bi, _, _ = ops.build_offsets(_dev(mask, device))
        ops.publish_int(bi[B:], slot[1:2])
        torch.cuda.synchronize()
        assert slot.tolist() == [-1, int(lens.sum()), -1, -1]
    with pytest.raises(ValueError):
        ops.publish_int(bi[B:], torch.zeros(1, dtype=torch.int32))      # not pinned


# Every product test runs with the weight in both layouts: the [n, k] pre-pack and the
# [k, n] matrix as the layer stores it.
_KN = [False]


@pytest.fixture(autouse=True)
def weight_layout(request):
    _KN[0] = getattr(request, "param", "nk") == "kn"
    yield
    _KN[0] = False


def pytest_generate_tests(metafunc):
    name = metafunc.function.__name__
    if ("gemm" in name or "splitk" in name) and "weight_layout" in metafunc.fixturenames:
        metafunc.parametrize("weight_layout", ["nk", "kn"], indirect=True)


def _prep(w):
    return w if _KN[0] else ops.transpose_weight(w)


def _gemm(*a, **k):
    return ops.gemm(*a, w_kn=_KN[0], **k)


def _gemm_bias_gelu(*a, **k):
    return ops.gemm_bias_gelu(*a, w_kn=_KN[0], **k)


def _gemm_qkv_bias_split(*a, **k):
    return ops.gemm_qkv_bias_split(*a, w_kn=_KN[0], **k)


def _gemm_splitk(*a, **k):
    return ops.gemm_splitk(*a, w_kn=_KN[0], **k)


@pytest.mark.parametrize("B,S,dtype", [(1, 256, np.float16), (16, 512, np.float16),
                                       (3, 7, np.float32), (70, 33, np.float16),
                                       (130, 100, np.float16), (2, 1024, np.float16)])
@pytest.mark.parametrize("kind", ["prefix", "ragged-rows", "empty-sequence"])
def test_layer_prologue_offsets_and_prefix_verdict(device, B, S, dtype, kind):
    """bt_layer_prologue = bt_build_offsets + bt_mask_prefix_slots in one launch: offsets
    bit-exact with the oracle, the verdict equal to the stand-alone check's."""
    _say("prologue", B, S, dtype, kind)
    rs = np.random.RandomState(B * 1000 + S)
    lens = rs.randint(1, S + 1, size=B)
    lens[0] = S
    if kind == "empty-sequence" and B > 1:
        lens[B - 1] = 0
    mask = workload.make_mask(lens, S, dtype).copy()
    if kind == "ragged-rows" and S > 1:
        mask[B // 2, S - 1, 0] = 1 - mask[B // 2, S - 1, 0]      # one element off in the last row
    bi, wi, M = O.build_offsets(mask)
    m = _dev(mask, device)
    g_bi, g_wi, order, slots = ops.layer_prologue(m, want_slots=True)
    assert np.array_equal(g_bi.cpu().numpy(), bi)
    assert np.array_equal(g_wi.cpu().numpy()[:M], wi)
    assert order.cpu().numpy().tolist() == np.argsort(-lens.astype(np.int64), kind="stable").tolist()
    sl = slots.cpu().numpy()
    assert set(np.unique(sl).tolist()) <= {0, 1}              # every slot was written
    expect = kind == "prefix" or (kind == "empty-sequence" and B == 1) or \
        (kind == "ragged-rows" and S == 1)
    assert bool(sl.all()) == expect
    assert ops.mask_is_prefix(m, g_bi) == expect
    # without the slots (packed rows): the small grid, same offsets
    g_bi2, g_wi2, order2, none = ops.layer_prologue(m)
    assert none is None and torch.equal(g_bi2, g_bi) and torch.equal(order2, order)
    assert torch.equal(g_wi2[:M], g_wi[:M])
    # the tail of word_idx: the padded positions, as bt_build_offsets writes them
    ref_wi = ops.build_offsets(m)[1]
    assert torch.equal(g_wi, ref_wi) and torch.equal(g_wi2, ref_wi)
    assert sorted(g_wi.cpu().tolist()) == list(range(g_wi.numel()))


def test_layer_prologue_packs_weights_afresh_in_every_call(device):
    """The prologue's weight job: [n, k] copies of up to four [k, n] matrices, made in the
    same launch as the offsets and from the weights as they are at that call - a weight
    overwritten between two calls (with or without any host-side bookkeeping) is simply
    packed again."""
    _say("prologue pre-pack")
    rs = np.random.RandomState(5)
    shapes = [(128, 384), (128, 128), (128, 512), (512, 128)]
    ws = [_dev(rs.standard_normal(s).astype(np.float16), device) for s in shapes]
    packed = [torch.full((s[1], s[0]), 7, dtype=torch.float16, device=device) for s in shapes]
    mask_np = workload.make_mask([5, 9, 3], 9, np.float16)
    mask = _dev(mask_np, device)
    bi, wi, order, _ = ops.layer_prologue(mask, weights=ws, packed=packed)
    r_bi, r_wi, M = O.build_offsets(mask_np)
    assert np.array_equal(bi.cpu().numpy(), r_bi) and np.array_equal(wi.cpu().numpy()[:M], r_wi[:M])
    assert all(torch.equal(p, w.t().contiguous()) for p, w in zip(packed, ws))
    ws[2].data.copy_(_dev(rs.standard_normal(shapes[2]).astype(np.float16), device))
    ws[3].data[511, 127] += 1
    ops.layer_prologue(mask, weights=ws, packed=packed)
    assert all(torch.equal(p, w.t().contiguous()) for p, w in zip(packed, ws))
    # a subset, and shapes that do not fill their last 64 x 64 tiles
    odd = [_dev(rs.standard_normal(sh).astype(np.float16), device) for sh in [(72, 200), (200, 72)]]
    guard = [torch.full((sh[1] * sh[0] + 64,), 3, dtype=torch.float16, device=device)
             for sh in [(72, 200), (200, 72)]]
    odd_packed = [g[:w.numel()].view(w.shape[1], w.shape[0]) for g, w in zip(guard, odd)]
    ops.layer_prologue(mask, weights=odd, packed=odd_packed)
    assert all(torch.equal(p, w.t().contiguous()) for p, w in zip(odd_packed, odd))
    assert all(bool((g[w.numel():] == 3).all()) for g, w in zip(guard, odd))
    with pytest.raises(ValueError):
        ops.layer_prologue(mask, weights=ws[:1], packed=[ws[0]])
    # ranges to warm are only read (guard bytes on both sides, odd sizes, up to four of them),
    # alone and beside a pack job, and change nothing else
    guard = 4096
    wholes = [torch.full((guard + n + guard,), 7, dtype=torch.uint8, device=device)
              for n in (131, 3, 1 << 20, 70001)]
    for count in (1, 2, 4):
        ranges = [w[guard:w.numel() - guard] for w in wholes[:count]]
        for with_pack in (False, True):
            bi2, wi2, _, _ = ops.layer_prologue(mask, weights=ws[:2] if with_pack else None,
                                                packed=packed[:2] if with_pack else None, warm=ranges)
            torch.cuda.synchronize()
            assert torch.equal(bi2, bi) and torch.equal(wi2[:M], wi[:M])
            assert all(bool((w == 7).all()) for w in wholes)
    with pytest.raises(ops.BtError):
        ops.layer_prologue(mask, warm=[w[guard:-guard] for w in wholes] + [wholes[0][guard:-guard]])


def test_build_offsets_threshold(device):
    S = 70
    mask = np.zeros((2, S, S), np.float16)
    mask[0, 0, :] = np.linspace(0, 1, S)          # crosses 0.5 somewhere in the row
    mask[1, 0, :5] = [0.5, 0.4999, 1, 0.51, 0]
    bi, wi, M = O.build_offsets(mask)
    g_bi, g_wi, g_M = ops.build_offsets(_dev(mask, device), want_count=True)
    assert g_M == M and np.array_equal(g_bi.cpu().numpy(), bi)
    assert np.array_equal(g_wi.cpu().numpy()[:M], wi)


# ---- compress / restore (bit-exact copies) -------------------------------------
@pytest.mark.parametrize("B,S,H", [(4, 50, 768), (16, 512, 768), (3, 9, 1024), (2, 5, 8)])
def test_compress_bit_exact(device, B, S, H):
    _say("compress", B, S, H)
    rs = np.random.RandomState(7)
    lens = rs.randint(0, S + 1, size=B)
    lens[-1] = S
    x = rs.standard_normal((B, S, H)).astype(np.float16)
    mask = workload.make_mask(lens, S, np.float16)
    bi, wi, M = O.build_offsets(mask)
    g_bi, g_wi, _ = ops.build_offsets(_dev(mask, device))
    sentinel = torch.full((B * S, H), 7.0, dtype=torch.float16, device=device)
    packed = ops.compress(_dev(x, device), g_bi, g_wi, out=sentinel).cpu().numpy()
    assert np.array_equal(packed[:M].view(np.uint16), O.compress(x, wi).view(np.uint16))
    assert np.all(packed[M:] == 7.0)               # rows past M are never written


# ---- LayerNorm ----------------------------------------------------------------
@pytest.mark.parametrize("H,gb32", [(768, False), (1024, True), (64, False), (2048, False),
                                    (4096, True), (264, False)])
def test_add_bias_residual_layernorm(device, H, gb32):
    _say("layernorm", H, gb32)
    rs = np.random.RandomState(H)
    rows, M = 37, 29
    out = rs.standard_normal((rows, H)).astype(np.float16)
    res = (rs.standard_normal((rows, H)) * 2).astype(np.float16)
    bias = (rs.standard_normal(H) * 0.5).astype(np.float16)
    gdt = np.float32 if gb32 else np.float16
    gamma = (1 + 0.2 * rs.standard_normal(H)).astype(gdt)
    beta = (0.3 * rs.standard_normal(H)).astype(gdt)
    exp = O.add_bias_residual_layernorm(out, res, bias, gamma, beta, 1e-6)
    vr = torch.tensor([M], dtype=torch.int32, device=device)
    g = ops.add_bias_residual_layernorm(_dev(out, device), _dev(res, device), _dev(bias, device),
                                        _dev(gamma, device), _dev(beta, device), 1e-6,
                                        valid_rows=vr).cpu().numpy()
    # rounding of the fp16 result: half an ulp (2^-11 relative) plus fp32 statistics noise
    err = np.abs(g[:M].astype(np.float64) - exp[:M])
    assert np.all(err <= 2.0 ** -10 * np.abs(exp[:M]) + 1e-4), err.max()
    assert np.array_equal(g[M:], out[M:])          # rows past M untouched
    # all rows live when valid_rows is null
    g2 = ops.add_bias_residual_layernorm(_dev(out, device), _dev(res, device), _dev(bias, device),
                                         _dev(gamma, device), _dev(beta, device), 1e-6).cpu().numpy()
    err = np.abs(g2.astype(np.float64) - exp)
    assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 1e-4)


@pytest.mark.parametrize("H,gb32,rows,M", [(768, False, 300, 211), (1024, True, 37, 37),
                                           (64, False, 5, 0), (2048, False, 130, 129)])
def test_layernorm_with_weight_copies_riding_along(device, H, gb32, rows, M):
    """The LayerNorm launch that also makes k-contiguous weight copies: the rows are the bits of
    the plain launch (gathered residual, live-row count), the copies are the transposed
    matrices - tiles that are partial in either direction, four matrices, guard bytes on both
    sides of every copy, none at all."""
    _say("layernorm + copies", H, gb32, rows, M)
    rs = np.random.RandomState(H + rows)
    out = rs.standard_normal((rows, H)).astype(np.float16)
    res = (rs.standard_normal((rows + 9, H)) * 2).astype(np.float16)
    ridx = rs.permutation(rows + 9)[:rows].astype(np.int32)
    bias = (rs.standard_normal(H) * 0.5).astype(np.float16)
    gdt = np.float32 if gb32 else np.float16
    gamma = (1 + 0.2 * rs.standard_normal(H)).astype(gdt)
    beta = (0.3 * rs.standard_normal(H)).astype(gdt)
    vr = torch.tensor([M], dtype=torch.int32, device=device)
    args = [_dev(a, device) for a in (res, bias, gamma, beta)]
    ri = _dev(ridx, device)
    plain = ops.add_bias_residual_layernorm(_dev(out, device), *args, 1e-6, valid_rows=vr,
                                            residual_row_index=ri)
    for shapes in (((H, 4 * H),), ((H, 4 * H), (4 * H, H), (72, 200), (8, 8)), ()):
        ws = [_dev((rs.standard_normal(sh) * 0.1).astype(np.float16), device) for sh in shapes]
        # each copy sits inside a larger buffer of sevens: nothing beside it may change
        bufs = [torch.full((w.numel() + 256,), 7.0, dtype=torch.float16, device=device) for w in ws]
        packed = [b[128:128 + w.numel()].view(w.shape[1], w.shape[0]) for b, w in zip(bufs, ws)]
        got = ops.add_bias_residual_layernorm_copy(_dev(out, device), *args, ws, packed, 1e-6,
                                                   valid_rows=vr, residual_row_index=ri)
        assert torch.equal(got, plain), shapes
        for w, t, b in zip(ws, packed, bufs):
            assert torch.equal(t, w.t().contiguous()), tuple(w.shape)
            assert bool((b[:128] == 7).all()) and bool((b[128 + w.numel():] == 7).all())
    if M:
        exp = O.add_bias_residual_layernorm(out[:M], res[ridx[:M]], bias, gamma, beta, 1e-6)
        err = np.abs(plain.cpu().numpy()[:M].astype(np.float64) - exp)
        assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 1e-4), err.max()
    assert np.array_equal(plain.cpu().numpy()[M:], out[M:])


@pytest.mark.parametrize("B,S,H", [(4, 33, 768), (16, 128, 1024)])
def test_layernorm_restore_zero_fills_padding(device, B, S, H):
    _say("layernorm_restore", B, S, H)
    rs = np.random.RandomState(B + S)
    lens = rs.randint(0, S + 1, size=B)
    lens[0], lens[-1] = S, 0
    mask = workload.make_mask(lens, S, np.float16)
    bi, wi, M = O.build_offsets(mask)
    out = rs.standard_normal((B * S, H)).astype(np.float16)
    res = rs.standard_normal((B * S, H)).astype(np.float16)
    bias = (rs.standard_normal(H) * 0.5).astype(np.float16)
    gamma = (1 + 0.2 * rs.standard_normal(H)).astype(np.float16)
    beta = (0.3 * rs.standard_normal(H)).astype(np.float16)
    exp = O.restore(O.add_bias_residual_layernorm(out[:M], res[:M], bias, gamma, beta, 1e-6), bi,
                    B, S)
    g_bi, g_wi, _ = ops.build_offsets(_dev(mask, device))
    # word_idx lists the valid positions first and the padded ones after them: a permutation
    wi_all = g_wi.cpu().numpy()
    assert np.array_equal(wi_all[:M], wi[:M])
    pads = np.concatenate([b * S + np.arange(lens[b], S) for b in range(B)]) if M < B * S else []
    assert np.array_equal(np.sort(wi_all[M:]), np.sort(pads))
    results = []
    for row_map in (None, g_wi):        # look-up through batch_idx, and through the row map
        target = torch.full((B, S, H), float("nan"), dtype=torch.float16, device=device)
        g = ops.add_bias_residual_layernorm_restore(
            _dev(out, device), _dev(res, device), _dev(bias, device), _dev(gamma, device),
            _dev(beta, device), g_bi, B, S, 1e-6, out_padded=target, word_idx=row_map).cpu().numpy()
        for b in range(B):
            assert np.all(g[b, lens[b]:].view(np.uint16) == 0)      # exact +0 fill
        err = np.abs(g.astype(np.float64) - exp)
        assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 1e-4), err.max()
        results.append(g)
    assert np.array_equal(results[0].view(np.uint16), results[1].view(np.uint16))


# ---- weight pre-pack -----------------------------------------------------------
@pytest.mark.parametrize("K,N", [(768, 2304), (3072, 768), (64, 8), (200, 136)])
def test_transpose_weight_bit_exact(device, K, N):
    w = np.random.RandomState(K + N).standard_normal((K, N)).astype(np.float16)
    wt = ops.transpose_weight(_dev(w, device)).cpu().numpy()
    assert np.array_equal(wt.view(np.uint16), np.ascontiguousarray(w.T).view(np.uint16))


def test_transpose_weights_fused_launch(device):
    rs = np.random.RandomState(5)
    shapes = [(768, 2304), (768, 768), (768, 3072), (3072, 768)]
    ws = [rs.standard_normal(sh).astype(np.float16) for sh in shapes]
    wts = ops.transpose_weights([_dev(w, device) for w in ws])
    for w, wt in zip(ws, wts):
        assert np.array_equal(wt.cpu().numpy().view(np.uint16),
                              np.ascontiguousarray(w.T).view(np.uint16))


# ---- GEMM family ---------------------------------------------------------------
def _gemm_tol(exp, K, amax, wmax):
    # one fp16 rounding of the result plus fp32 accumulation noise
    return 2.0 ** -10 * np.abs(exp) + 4 * K * 2.0 ** -24 * amax * wmax + 1e-6


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("rows,M,N,K", [(300, 300, 768, 768), (1000, 777, 2304, 768),
                                        (520, 513, 768, 3072), (64, 1, 136, 64),
                                        (257, 257, 3072, 768)])
def test_gemm_plain(device, tile, rows, M, N, K):
    _say("gemm", tile, rows, M, N, K)
    rs = np.random.RandomState(rows + N)
    a = rs.standard_normal((rows, K)).astype(np.float16)
    w = (rs.standard_normal((K, N)) * 0.05).astype(np.float16)
    exp = O.gemm(a[:M], w)
    ops.set_option("gemm_tile", tile)
    try:
        wt = _prep(_dev(w, device))
        vr = torch.tensor([M], dtype=torch.int32, device=device)
        out = torch.full((rows, N), 3.0, dtype=torch.float16, device=device)
        g = _gemm(_dev(a, device), wt, valid_rows=vr, out=out).cpu().numpy()
    finally:
        ops.set_option("gemm_tile", -1)
    err = np.abs(g[:M].astype(np.float64) - exp)
    tol = _gemm_tol(exp, K, np.abs(a).max(), np.abs(w).max())
    assert np.all(err <= tol), (err.max(), np.unravel_index(err.argmax(), err.shape))
    assert np.all(g[M:] == 3.0)


@pytest.mark.parametrize("seed", range(12))
def test_gemm_random_shapes_all_tiles_and_auto(device, seed):
    """Random row counts and n / k at the granularity the entry point accepts (8 and 64),
    every tile shape and the automatic choice."""
    rs = np.random.RandomState(300 + seed)
    rows = int(rs.randint(1, 700))
    M = int(rs.randint(0, rows + 1))
    N = 8 * int(rs.randint(1, 130))
    K = 64 * int(rs.randint(1, 17))
    _say("gemm random", seed, rows, M, N, K)
    a = rs.standard_normal((rows, K)).astype(np.float16)
    a[M:] = np.float16("nan")                       # rows past the live count are never used
    w = (rs.standard_normal((K, N)) * 0.05).astype(np.float16)
    exp = O.gemm(a[:M], w)
    tol = _gemm_tol(exp, K, np.abs(a[:M]).max() if M else 0.0, np.abs(w).max())
    wt = _prep(_dev(w, device))
    vr = torch.tensor([M], dtype=torch.int32, device=device)
    try:
        for tile in (-1, 0, 1, 2, 3, 4, 5, 6, 7, 8):
            ops.set_option("gemm_tile", tile)
            out = torch.full((rows, N), 3.0, dtype=torch.float16, device=device)
            g = _gemm(_dev(a, device), wt, valid_rows=vr, out=out, rows_hint=M).cpu().numpy()
            err = np.abs(g[:M].astype(np.float64) - exp)
            assert np.all(err <= tol), (tile, err.max())
            assert np.all(g[M:] == 3.0), tile
    finally:
        ops.set_option("gemm_tile", -1)


@pytest.mark.parametrize("seed", range(6))
def test_gemm_row_hint_never_changes_the_result(device, seed):
    """rows_hint only steers the launch (tile shape): with the tile pinned, hints from far
    too small to too large give the bits of a launch without a hint, for every tile shape
    and the three epilogues; with the automatic choice the oracle's values."""
    rs = np.random.RandomState(900 + seed)
    rows = int(rs.randint(300, 1500))
    M = int(rs.randint(rows // 2, rows + 1))
    heads = int(rs.randint(1, 4))
    H = 64 * heads
    F = 64 * int(rs.randint(2, 9))
    _say("gemm hint", seed, rows, M, H, F)
    a = rs.standard_normal((rows, H)).astype(np.float16)
    a[M:] = np.float16("nan")
    w1 = (rs.standard_normal((H, F)) * 0.05).astype(np.float16)
    wq = (rs.standard_normal((H, 3 * H)) * 0.05).astype(np.float16)
    b1 = (rs.standard_normal(F) * 0.1).astype(np.float16)
    bq = (rs.standard_normal(3 * H) * 0.1).astype(np.float16)
    ad, vr = _dev(a, device), torch.tensor([M], dtype=torch.int32, device=device)
    wt1, wtq = _prep(_dev(w1, device)), _prep(_dev(wq, device))
    b1d, bqd = _dev(b1, device), _dev(bq, device)
    exp = O.gemm(a[:M], w1)
    tol = _gemm_tol(exp, H, np.abs(a[:M]).max(), np.abs(w1).max())

    def run(hint):
        o1 = torch.full((rows, F), 3.0, dtype=torch.float16, device=device)
        o2 = torch.full((rows, F), 3.0, dtype=torch.float16, device=device)
        o3 = torch.full((3, heads, rows, 64), 3.0, dtype=torch.float16, device=device)
        _gemm(ad, wt1, valid_rows=vr, out=o1, rows_hint=hint)
        _gemm_bias_gelu(ad, wt1, b1d, valid_rows=vr, out=o2, rows_hint=hint)
        _gemm_qkv_bias_split(ad, wtq, bqd, heads, valid_rows=vr, out=o3, rows_hint=hint)
        return o1, o2, o3

    try:
        for tile in (0, 1, 2, 3, 4, 5):
            ops.set_option("gemm_tile", tile)
            ref = run(0)
            g = ref[0].cpu().numpy()
            assert np.all(np.abs(g[:M].astype(np.float64) - exp) <= tol), tile
            assert np.all(g[M:] == 3.0), tile
            for hint in (1, 33, M // 3, M - 1, M, rows):
                for got, want in zip(run(hint), ref):
                    assert torch.equal(got, want), (tile, hint)
        ops.set_option("gemm_tile", -1)
        for hint in (1, M // 3, M, rows):
            g = run(hint)[0].cpu().numpy()
            assert np.all(np.abs(g[:M].astype(np.float64) - exp) <= tol), hint
            assert np.all(g[M:] == 3.0), hint
    finally:
        ops.set_option("gemm_tile", -1)


@pytest.mark.parametrize("splits,restore,tight", [(2, False, False), (4, False, False),
                                                  (4, True, False), (2, True, False),
                                                  (4, True, True), (2, False, True)])
def test_splitk_gemm_and_layernorm(device, splits, restore, tight):
    """FFN2 as split-k partial sums + the LayerNorm that folds them: same result as the
    plain GEMM followed by the plain LayerNorm (one fp16 rounding of the product, then the
    fp16 adds), against the oracle and bit-for-bit against the unsplit pair up to the
    summation order of the fp32 partials."""
    _say("splitk", splits, restore, tight)
    rs = np.random.RandomState(40 + splits)
    B, S, H, F = 3, 50, 128, 1024
    lens = np.array([50, 7, 31])
    mask = workload.make_mask(lens, S, np.float16)
    bi, wi, M = O.build_offsets(mask)
    rows = B * S
    a = np.zeros((rows, F), np.float16)
    a[:M] = rs.standard_normal((M, F)).astype(np.float16)
    a[M:] = np.float16("nan")
    w = (rs.standard_normal((F, H)) * 0.05).astype(np.float16)
    res = rs.standard_normal((rows, H)).astype(np.float16)
    bias = (rs.standard_normal(H) * 0.5).astype(np.float16)
    gamma = (1 + 0.2 * rs.standard_normal(H)).astype(np.float16)
    beta = (0.3 * rs.standard_normal(H)).astype(np.float16)
    prod = O.f16(O.gemm(a[:M], w))
    exp = O.add_bias_residual_layernorm(prod, res[:M], bias, gamma, beta, 1e-6)
    g_bi, _, _ = ops.build_offsets(_dev(mask, device))
    vr = g_bi[B:]
    wt = _prep(_dev(w, device))
    # tight: the launches are sized for exactly the live rows (the padded output of the
    # restore flavour still has batch * seq_len rows)
    cap = M if tight else rows
    a, res = a[:cap], res[:cap]
    parts = _gemm_splitk(_dev(a, device), wt, splits, valid_rows=vr)
    assert tuple(parts.shape) == (splits, cap, H)
    # the partial sums add up to the product
    total = parts.sum(0).cpu().numpy()[:M]
    assert np.all(np.abs(total - O.gemm(a[:M], w)) <= 1e-3 + 1e-4 * np.abs(total))
    args = (_dev(res, device), _dev(bias, device), _dev(gamma, device), _dev(beta, device))
    if restore:
        dst = torch.full((B, S, H), float("nan"), dtype=torch.float16, device=device)
        g = ops.splitk_layernorm(parts, *args, dst, batch_idx=g_bi, batch_size=B, seq_len=S)
        g = g.cpu().numpy()
        exp_pad = O.restore(exp, bi, B, S)
        for b in range(B):
            assert np.all(g[b, lens[b]:].view(np.uint16) == 0)
        err = np.abs(g.astype(np.float64) - exp_pad)
        assert np.all(err <= 2.0 ** -9 * np.abs(exp_pad) + 4e-3), err.max()
    else:
        dst = torch.full((cap, H), 5.0, dtype=torch.float16, device=device)
        g = ops.splitk_layernorm(parts, *args, dst, valid_rows=vr).cpu().numpy()
        err = np.abs(g[:M].astype(np.float64) - exp)
        assert np.all(err <= 2.0 ** -9 * np.abs(exp) + 4e-3), err.max()
        assert np.all(g[M:] == 5.0)
        # and the unsplit pair gives the same numbers except where the fp16 rounding of the
        # product flips on the last bit of the fp32 sum
        plain = _gemm(_dev(a, device), wt, valid_rows=vr)
        ref = ops.add_bias_residual_layernorm(plain, *args, valid_rows=vr).cpu().numpy()
        assert np.mean(ref[:M] == g[:M]) > 0.97
        assert np.abs(ref[:M].astype(np.float32) - g[:M].astype(np.float32)).max() <= 2e-2


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7, 8])
def test_gemm_bias_gelu(device, tile):
    _say("gemm_bias_gelu", tile)
    rs = np.random.RandomState(tile)
    rows, M, N, K = 700, 650, 3072, 768
    a = rs.standard_normal((rows, K)).astype(np.float16)
    w = (rs.standard_normal((K, N)) * 0.06).astype(np.float16)
    bias = (rs.standard_normal(N) * 0.5).astype(np.float16)
    exp = O.gemm(a[:M], w, bias, "gelu_tanh")
    ops.set_option("gemm_tile", tile)
    try:
        vr = torch.tensor([M], dtype=torch.int32, device=device)
        g = _gemm_bias_gelu(_dev(a, device), _prep(_dev(w, device)),
                               _dev(bias, device), valid_rows=vr).cpu().numpy()
    finally:
        ops.set_option("gemm_tile", -1)
    err = np.abs(g[:M].astype(np.float64) - exp)
    # gelu' <= 1.13; fast exp / divide add a few fp32 ulps
    assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 2e-4), err.max()
    assert np.all(g[M:] == 0)


@pytest.mark.parametrize("K", [64, 128, 192, 768])
@pytest.mark.parametrize("tile", [6, 7, 8])
def test_gemm_persistent_workgroups_take_several_tiles_with_a_bias(device, tile, K):
    """The persistent forms with more tiles than workgroups, a column count that the tile does
    not divide, a bias epilogue and k loops shorter than the load pipeline is deep (the next
    tile's bias is then fetched while the current tile's is still unread: two buffers)."""
    _say("gemm persistent several tiles", tile, K)
    rs = np.random.RandomState(tile * 1000 + K)
    rows, M, N = 4100, 4001, 4232
    a = rs.standard_normal((rows, K)).astype(np.float16)
    w = (rs.standard_normal((K, N)) * 0.06).astype(np.float16)
    bias = (rs.standard_normal(N) * 0.5).astype(np.float16)
    exp = O.gemm(a[:M], w, bias, "gelu_tanh")
    heads = K // 64
    rows_q, Mq = 30000, 29000
    aq = rs.standard_normal((rows_q, K)).astype(np.float16)
    wq = (rs.standard_normal((K, 3 * K)) * 0.05).astype(np.float16)
    bq = (rs.standard_normal(3 * K) * 0.5).astype(np.float16)
    expq = O.split_heads(O.gemm(aq[:Mq], wq, bq), heads, 64)
    ops.set_option("gemm_tile", tile)
    try:
        vr = torch.tensor([M], dtype=torch.int32, device=device)
        g = _gemm_bias_gelu(_dev(a, device), _prep(_dev(w, device)), _dev(bias, device),
                            valid_rows=vr).cpu().numpy()
        vq = torch.tensor([Mq], dtype=torch.int32, device=device)
        gq = _gemm_qkv_bias_split(_dev(aq, device), _prep(_dev(wq, device)), _dev(bq, device),
                                  heads, valid_rows=vq).cpu().numpy()
    finally:
        ops.set_option("gemm_tile", -1)
    err = np.abs(g[:M].astype(np.float64) - exp)
    assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 2e-4), err.max()
    assert np.all(g[M:] == 0)
    errq = np.abs(gq[:, :, :Mq].astype(np.float64) - expq)
    assert np.all(errq <= 2.0 ** -10 * np.abs(expq) + 2e-4), errq.max()
    assert np.all(gq[:, :, Mq:] == 0)


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("heads", [12, 16])
def test_gemm_qkv_bias_split(device, tile, heads):
    _say("gemm_qkv", tile, heads)
    rs = np.random.RandomState(heads)
    H = heads * 64
    rows, M = 400, 333
    a = rs.standard_normal((rows, H)).astype(np.float16)
    w = (rs.standard_normal((H, 3 * H)) * 0.05).astype(np.float16)
    bias = (rs.standard_normal(3 * H) * 0.5).astype(np.float16)
    exp = O.split_heads(O.gemm(a[:M], w, bias), heads, 64)           # [3, heads, M, 64]
    ops.set_option("gemm_tile", tile)
    try:
        vr = torch.tensor([M], dtype=torch.int32, device=device)
        g = _gemm_qkv_bias_split(_dev(a, device), _prep(_dev(w, device)),
                                    _dev(bias, device), heads, valid_rows=vr).cpu().numpy()
    finally:
        ops.set_option("gemm_tile", -1)
    assert g.shape == (3, heads, rows, 64)
    err = np.abs(g[:, :, :M].astype(np.float64) - exp)
    assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 2e-4), err.max()
    assert np.all(g[:, :, M:] == 0)


@pytest.mark.parametrize("tile", [-1, 0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("case", ["ragged", "cfg2", "full", "empty-ends", "one", "f32-mask", "wide"])
def test_gemm_qkv_rows_from_the_mask(device, tile, case):
    """The QKV product that counts the mask rows itself: offsets bit-exact with the
    stand-alone launch (and the oracle), projections bit-identical to offsets -> gather."""
    _say("gemm_qkv mask rows", tile, case)
    rs = np.random.RandomState(len(case) + 3 * (tile + 1))
    heads, mdt = 2, np.float16
    if case == "ragged":
        B, S, lens = 5, 70, np.array([70, 0, 33, 1, 64])
    elif case == "cfg2":
        B, S = 16, 512
        lens = rs.randint(100, 513, B)
    elif case == "full":
        B, S, lens = 3, 128, np.array([128, 128, 128])
    elif case == "empty-ends":
        B, S, lens = 6, 48, np.array([0, 0, 17, 48, 0, 0])
    elif case == "one":
        B, S, lens = 1, 200, np.array([77])
    elif case == "f32-mask":
        B, S, mdt, lens = 7, 36, np.float32, np.array([36, 5, 5, 0, 20, 1, 36])
    else:
        B, S, lens = 64, 64, rs.randint(0, 65, 64)
    H = heads * 64
    x = rs.standard_normal((B, S, H)).astype(np.float16)
    mask = workload.make_mask(lens, S, mdt)
    w = (rs.standard_normal((H, 3 * H)) * 0.05).astype(np.float16)
    bias = (rs.standard_normal(3 * H) * 0.5).astype(np.float16)
    md, xd, wt, bd = _dev(mask, device), _dev(x, device), _prep(_dev(w, device)), _dev(bias, device)
    assert ops.gemm_qkv_mask_rows_supported(B, S, md.dtype)
    e_bi, e_wi, e_so, _ = ops.layer_prologue(md)
    M = int(lens.sum())
    ops.set_option("gemm_tile", tile)
    try:
        ref = _gemm_qkv_bias_split(xd.view(B * S, H), wt, bd, heads, valid_rows=e_bi[B:],
                                   a_row_index=e_wi)
        sentinel = lambda n: torch.full((n,), -7, dtype=torch.int32, device=device)
        outs = (sentinel(B + 1), sentinel(B * S), sentinel(B))
        got, g_bi, g_wi, g_so = ops.gemm_qkv_bias_split_mask_rows(
            xd, md, wt, bd, heads, offsets_out=outs, rows_hint=M, w_kn=_KN[0])
    finally:
        ops.set_option("gemm_tile", -1)
    o_bi, o_wi, _ = O.build_offsets(mask)
    assert np.array_equal(g_bi.cpu().numpy(), o_bi)
    assert np.array_equal(g_wi.cpu().numpy()[:M], o_wi[:M])
    assert torch.equal(g_bi, e_bi) and torch.equal(g_wi, e_wi) and torch.equal(g_so, e_so)
    assert torch.equal(ref[:, :, :M], got[:, :, :M])
    assert torch.all(got[:, :, M:] == 0)
    if M:
        exp = O.split_heads(O.gemm(O.compress(x, o_wi[:M]), w, bias), heads, 64)
        err = np.abs(got.cpu().numpy()[:, :, :M].astype(np.float64) - exp)
        assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 2e-4)
    # without the optional outputs
    got2, _, _, _ = ops.gemm_qkv_bias_split_mask_rows(
        xd, md, wt, bd, heads, offsets_out=(sentinel(B + 1), None, None), w_kn=_KN[0])
    assert torch.equal(got2[:, :, :M], got[:, :, :M])


@pytest.mark.skip(reason="the side workgroups of the QKV launch were taken out of the library: a "
                         "layer that used them by default left the GPU faulted once under the "
                         "stand-alone C++ driver (batch 16 x 512) and no cause was found; the "
                         "entry no longer takes work_list / weights / packed / warm")
@pytest.mark.parametrize("tile", [-1, 0, 3, 4, 7])
@pytest.mark.parametrize("case", ["cfg2-like", "many-short", "f32-mask"])
def test_gemm_qkv_rows_from_the_mask_side_jobs(device, case, tile):
    """The jobs that ride along with the launch (the attention's work list, k-contiguous
    weight copies, cache warm-up) are done by workgroups of their own: the list equals the
    stand-alone builder's, the copies equal the transposed weights, and the projections and
    offsets are what the launch gives without any job."""
    rs = np.random.RandomState(len(case) + 10 * (tile + 1))
    mdt = np.float16
    if case == "cfg2-like":
        B, S, heads = 16, 512, 2
        lens = rs.randint(100, 513, B)
    elif case == "many-short":
        B, S, heads = 40, 96, 3
        lens = rs.randint(0, 97, B)
    else:
        B, S, heads, mdt = 9, 160, 1, np.float32
        lens = rs.randint(1, 161, B)
    _say("gemm_qkv mask rows side jobs", case, tile, B, S, heads, int(lens.sum()))
    H = heads * 64
    x = rs.standard_normal((B, S, H)).astype(np.float16)
    mask = workload.make_mask(lens, S, mdt)
    w = (rs.standard_normal((H, 3 * H)) * 0.05).astype(np.float16)
    bias = (rs.standard_normal(3 * H) * 0.5).astype(np.float16)
    md, xd, wt, bd = _dev(mask, device), _dev(x, device), _prep(_dev(w, device)), _dev(bias, device)
    M = int(lens.sum())
    # weights to copy: shapes with partial 64 x 64 tiles too
    ws = [_dev((rs.standard_normal(shape) * 0.1).astype(np.float16), device)
          for shape in ((H, 4 * H), (4 * H, H), (72, 200))]
    packed = [torch.full((v.shape[1], v.shape[0]), 7.0, dtype=torch.float16, device=device) for v in ws]
    warm = [torch.zeros(1000, dtype=torch.float16, device=device), ws[0]]
    ops.set_option("gemm_tile", tile)
    ops.set_option("attention_xcd_map", 3)          # the balanced order at any size
    try:
        plain, p_bi, p_wi, p_so = ops.gemm_qkv_bias_split_mask_rows(xd, md, wt, bd, heads, rows_hint=M,
                                                                    w_kn=_KN[0])
        want_list = ops.attention_worklist(p_bi, B, S, heads, False, seq_order=p_so)
        assert want_list is not None
        got_list = torch.full_like(want_list, -7)
        got, g_bi, g_wi, g_so = ops.gemm_qkv_bias_split_mask_rows(
            xd, md, wt, bd, heads, rows_hint=M, w_kn=_KN[0], work_list=got_list, weights=ws,
            packed=packed, warm=warm)
        # the jobs one at a time
        only_list = torch.full_like(want_list, -7)
        ops.gemm_qkv_bias_split_mask_rows(xd, md, wt, bd, heads, w_kn=_KN[0], work_list=only_list)
        only_packed = [torch.zeros_like(v) for v in packed[:1]]
        ops.gemm_qkv_bias_split_mask_rows(xd, md, wt, bd, heads, w_kn=_KN[0], weights=ws[:1],
                                          packed=only_packed, warm=warm[:1])
    finally:
        ops.set_option("gemm_tile", -1)
        ops.set_option("attention_xcd_map", 2)
    assert torch.equal(got_list, want_list) and torch.equal(only_list, want_list)
    for v, t in zip(ws, packed):
        assert torch.equal(t, v.t().contiguous())
    assert torch.equal(only_packed[0], ws[0].t().contiguous())
    assert torch.equal(g_bi, p_bi) and torch.equal(g_wi, p_wi) and torch.equal(g_so, p_so)
    assert torch.equal(got[:, :, :M], plain[:, :, :M])
    assert torch.all(got[:, :, M:] == 0)


@pytest.mark.parametrize("seed", range(12))
def test_gemm_qkv_rows_from_the_mask_random_shapes(device, seed):
    """Seeded random batch sizes, sequence lengths (odd ones too: the scalar mask-row path),
    head counts and lengths with empty sequences: offsets and projections bit-identical to
    the offsets launch followed by the gathered product."""
    rs = np.random.RandomState(1000 + seed)
    B = int(rs.randint(1, 65))
    S = int(rs.randint(1, min(512, 32768 // B) + 1))
    heads = int(rs.randint(1, 4))
    lens = rs.randint(0, S + 1, B)
    lens[rs.rand(B) < 0.15] = 0
    _say("gemm_qkv mask rows random", seed, B, S, heads, int(lens.sum()))
    H = heads * 64
    mdt = np.float32 if seed % 4 == 3 and B * S * 4 <= 65536 else np.float16
    x = rs.standard_normal((B, S, H)).astype(np.float16)
    mask = workload.make_mask(lens, S, mdt)
    w = (rs.standard_normal((H, 3 * H)) * 0.05).astype(np.float16)
    bias = (rs.standard_normal(3 * H) * 0.5).astype(np.float16)
    md, xd, wt, bd = _dev(mask, device), _dev(x, device), _prep(_dev(w, device)), _dev(bias, device)
    assert ops.gemm_qkv_mask_rows_supported(B, S, md.dtype)
    e_bi, e_wi, e_so, _ = ops.layer_prologue(md)
    M = int(lens.sum())
    ref = _gemm_qkv_bias_split(xd.view(B * S, H), wt, bd, heads, valid_rows=e_bi[B:],
                               a_row_index=e_wi, rows_hint=M)
    got, g_bi, g_wi, g_so = ops.gemm_qkv_bias_split_mask_rows(xd, md, wt, bd, heads, rows_hint=M,
                                                              w_kn=_KN[0])
    assert torch.equal(g_bi, e_bi) and torch.equal(g_wi, e_wi) and torch.equal(g_so, e_so)
    assert torch.equal(ref[:, :, :M], got[:, :, :M])
    assert torch.all(got[:, :, M:] == 0)


def test_gemm_qkv_rows_from_the_mask_limits(device):
    assert ops.gemm_qkv_mask_rows_supported(16, 512) and ops.gemm_qkv_mask_rows_supported(32, 1024)
    assert ops.gemm_qkv_mask_rows_supported(16, 1024, torch.float32)
    assert not ops.gemm_qkv_mask_rows_supported(65, 16)
    assert not ops.gemm_qkv_mask_rows_supported(64, 1024)
    assert not ops.gemm_qkv_mask_rows_supported(16, 2048, torch.float32)
    assert not ops.gemm_qkv_mask_rows_supported(4, 64, torch.float64)
    B, S, H = 65, 16, 64
    with pytest.raises(ops.BtError, match="bt_gemm_qkv_mask_rows_supported"):
        ops.gemm_qkv_bias_split_mask_rows(
            torch.zeros(B, S, H, dtype=torch.float16, device=device),
            torch.ones(B, S, S, dtype=torch.float16, device=device),
            torch.zeros(3 * H, H, dtype=torch.float16, device=device),
            torch.zeros(3 * H, dtype=torch.float16, device=device), 1)


def test_gather_fused_into_qkv_gemm_and_layernorm(device):
    """a_row_index / residual_row_index = word_idx reads the valid tokens straight from
    the padded input: bit-identical to compress followed by the plain call."""
    _say("gather fusion")
    rs = np.random.RandomState(17)
    B, S, heads = 5, 70, 2
    H = heads * 64
    lens = np.array([70, 0, 33, 1, 64])
    x = rs.standard_normal((B, S, H)).astype(np.float16)
    mask = workload.make_mask(lens, S, np.float16)
    w = (rs.standard_normal((H, 3 * H)) * 0.05).astype(np.float16)
    bias = (rs.standard_normal(3 * H) * 0.5).astype(np.float16)
    g_bi, g_wi, M = ops.build_offsets(_dev(mask, device), want_count=True)
    vr = g_bi[B:]
    xd, wt = _dev(x, device), _prep(_dev(w, device))
    packed = ops.compress(xd, g_bi, g_wi)
    ref = _gemm_qkv_bias_split(packed, wt, _dev(bias, device), heads, valid_rows=vr)
    got = _gemm_qkv_bias_split(xd.view(B * S, H), wt, _dev(bias, device), heads, valid_rows=vr,
                                  a_row_index=g_wi)
    assert torch.equal(ref[:, :, :M], got[:, :, :M])
    exp = O.split_heads(O.gemm(O.compress(x, g_wi.cpu().numpy()[:M]), w, bias), heads, 64)
    err = np.abs(got.cpu().numpy()[:, :, :M].astype(np.float64) - exp)
    assert np.all(err <= 2.0 ** -10 * np.abs(exp) + 2e-4)
    # LayerNorm with the residual gathered from the padded input
    out = rs.standard_normal((B * S, H)).astype(np.float16)
    b2 = (rs.standard_normal(H) * 0.5).astype(np.float16)
    gamma = (1 + 0.2 * rs.standard_normal(H)).astype(np.float16)
    beta = (0.3 * rs.standard_normal(H)).astype(np.float16)
    a = ops.add_bias_residual_layernorm(_dev(out, device), packed, _dev(b2, device),
                                        _dev(gamma, device), _dev(beta, device), valid_rows=vr)
    b = ops.add_bias_residual_layernorm(_dev(out, device), xd.view(B * S, H), _dev(b2, device),
                                        _dev(gamma, device), _dev(beta, device), valid_rows=vr,
                                        residual_row_index=g_wi)
    assert torch.equal(a, b)


@pytest.mark.parametrize("np_dtype", [np.float16, np.float32])
def test_mask_is_prefix(device, np_dtype):
    """The verdict is True only for masks that are exactly 1 for j < len_b and exactly 0
    beyond in EVERY row, with no empty sequence; one flipped element anywhere - on past
    the length, off inside it, in a row other than the first - makes it False."""
    _say("mask_is_prefix", np_dtype.__name__)
    rs = np.random.RandomState(5)
    for B, S in ((1, 1), (1, 154), (2, 64), (3, 257), (5, 1024)):
        lens = rs.randint(1, S + 1, size=B)
        lens[rs.randint(B)] = S
        mask = workload.make_mask(lens, S, np_dtype)
        md = _dev(mask, device)
        bi, _, _ = ops.build_offsets(md)
        assert ops.mask_is_prefix(md, bi) is True, (B, S)
        for trial in range(6):
            b, i = int(rs.randint(B)), int(rs.randint(1, S)) if S > 1 else 0
            j = int(rs.randint(S))
            bad = mask.copy()
            bad[b, i, j] = 1 - bad[b, i, j]
            if i == 0:
                continue        # row 0 defines the lengths: flipping there may give another prefix mask
            assert ops.mask_is_prefix(_dev(bad, device), bi) is False, (B, S, b, i, j)
        # only exact ones and zeros qualify: the tensor path shifts a logit by
        # (mask - 1) * 10000, so 0.75 is not "on" and 0.25 is not certainly "off"
        soft = (mask * 0.75 + (1 - mask) * 0.25).astype(np_dtype)
        assert ops.mask_is_prefix(_dev(soft, device), bi) is False
        if S > 1:
            almost = mask.copy()
            almost[0, S - 1, 0] = np_dtype(0.75)
            assert ops.mask_is_prefix(_dev(almost, device), bi) is False
    # an empty sequence: the reference's softmax over an all-masked row is not "no keys"
    lens = np.array([7, 0, 3])
    md = _dev(workload.make_mask(lens, 9, np_dtype), device)
    bi, _, _ = ops.build_offsets(md)
    assert ops.mask_is_prefix(md, bi) is False
    # a causal mask is not a prefix mask
    causal = np.tril(np.ones((2, 16, 16), np_dtype))
    cd = _dev(causal, device)
    bi, _, _ = ops.build_offsets(cd)
    assert ops.mask_is_prefix(cd, bi) is False


# ---- attention -----------------------------------------------------------------
@pytest.fixture(autouse=True, params=[0, 1], ids=["four-waves", "key-split"])
def attention_key_split(request):
    """The streaming attention kernel's 64-query variant exists with four waves and with
    eight (two key halves merged at the end); every test of this file runs under both
    (the option does not touch the other kernels)."""
    ops.set_option("attention_key_split", request.param)
    yield request.param
    ops.set_option("attention_key_split", -1)


def _attention_case(rs, lens, S, heads, scale_q=1.0):
    B = len(lens)
    bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    M = int(bi[-1])
    rows_cap = B * S
    qkv = np.zeros((3, heads, rows_cap, 64), np.float16)
    qkv[:, :, :M] = rs.standard_normal((3, heads, M, 64)).astype(np.float16)
    qkv[0] *= scale_q
    qkv[:, :, M:] = np.float16("nan")        # rows past M must never be consumed
    return bi, M, qkv


ATT_CASES = [
    ("short", [154], 256, 12),
    ("short", [64, 38], 64, 12),
    ("short", [1, 16, 17, 0, 100, 128], 128, 3),
    ("short", [300, 384, 77, 5], 384, 4),
    ("short", [512, 103, 257], 512, 2),
    ("grouped", [512, 103, 257, 64, 65, 1, 0, 300], 512, 3),
    ("grouped", [1024, 205, 700], 1024, 2),
    ("grouped", [154], 256, 12),
    ("grouped", [33, 2, 47], 47, 5),
]


@pytest.mark.parametrize("qb", [-1, 1, 2])
@pytest.mark.parametrize("kind,lens,S,heads", ATT_CASES)
def test_attention_packed(device, kind, lens, S, heads, qb):
    if kind == "short" and qb != -1:
        pytest.skip("option only affects the grouped kernel")
    _say("attention", kind, lens, S, heads, qb)
    rs = np.random.RandomState(S + heads)
    bi, M, qkv = _attention_case(rs, lens, S, heads, scale_q=2.0)
    scale = 1 / math.sqrt(64)
    exp = O.attention_packed(qkv[0, :, :M], qkv[1, :, :M], qkv[2, :, :M], bi, scale, 1e-6,
                             round_p_fp16=True)
    fn = ops.attention_short if kind == "short" else ops.attention_grouped
    ops.set_option("attention_qb", qb)
    try:
        out = torch.full((len(lens) * S, heads * 64), 5.0, dtype=torch.float16, device=device)
        g = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, scale, False, out=out)
        # issuing the workgroups longest-sequence-first must not change a bit
        order = _dev(np.argsort(-np.asarray(lens), kind="stable").astype(np.int32), device)
        g2 = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, scale, False, seq_order=order)
        assert torch.equal(g[:M], g2[:M])
        g = g.cpu().numpy()
    finally:
        ops.set_option("attention_qb", -1)
    err = np.abs(g[:M].astype(np.float64) - exp)
    # P is rounded to fp16 (2^-11 relative per term, |V| ~ N(0,1)) and O once more
    assert err.max() <= 4e-3 and err.mean() <= 4e-4, (err.max(), err.mean())
    assert np.all(g[M:] == 5.0)


@pytest.fixture(params=[2, 3], ids=["default-order", "balanced-order"])
def att_order(request):
    """Runs a test under the default workgroup order and with the balanced work list
    forced on (small launches would not use it by themselves)."""
    ops.set_option("attention_xcd_map", request.param)
    yield request.param
    ops.set_option("attention_xcd_map", 2)


ORDER_CASES = [
    ([512, 103, 257, 64, 65, 1, 0, 300], 512, 3),
    ([33, 2, 47], 47, 5),
    ([154], 256, 12),
    (list(np.random.RandomState(7).randint(0, 97, size=70)), 96, 2),    # more sequences than lanes
    (list(np.random.RandomState(8).randint(1, 193, size=131)), 192, 1),  # three passes of 64 ranks
]


@pytest.mark.parametrize("qb", [1, 2])
@pytest.mark.parametrize("lens,S,heads", ORDER_CASES)
def test_attention_workgroup_orders_agree(device, lens, S, heads, qb):
    """Plain, XCD-aware and balanced workgroup orders (and the identity or longest-first
    sequence order under each) visit every live query tile exactly once: same bits out,
    rows past the last token untouched, and the oracle's values."""
    lens = [int(v) for v in lens]
    _say("attention orders", len(lens), S, heads, qb)
    rs = np.random.RandomState(S * 7 + heads)
    bi, M, qkv = _attention_case(rs, lens, S, heads)
    scale = 1 / math.sqrt(64)
    exp = O.attention_packed(qkv[0, :, :M], qkv[1, :, :M], qkv[2, :, :M], bi, scale, 1e-6,
                             round_p_fp16=True)
    order = _dev(np.argsort(-np.asarray(lens), kind="stable").astype(np.int32), device)
    outs = []
    ops.set_option("attention_qb", qb)
    try:
        for mode in (0, 1, 2, 3):
            ops.set_option("attention_xcd_map", mode)
            for so in (None, order):
                out = torch.full((len(lens) * S, heads * 64), 5.0, dtype=torch.float16, device=device)
                ops.attention_grouped(_dev(qkv, device), _dev(bi, device), len(lens), S, scale, False,
                                      out=out, seq_order=so)
                outs.append(out)
    finally:
        ops.set_option("attention_qb", -1)
        ops.set_option("attention_xcd_map", 2)
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    g = outs[-1].cpu().numpy()
    err = np.abs(g[:M].astype(np.float64) - exp)
    assert err.max() <= 4e-3 and err.mean() <= 4e-4, (err.max(), err.mean())
    assert np.all(g[M:] == 5.0)


@pytest.mark.parametrize("kind", ["short", "grouped"])
def test_attention_padded_rows_mode(device, kind, att_order):
    """Padded layout: sequence b owns rows [b*S, (b+1)*S); every query row is
    computed against the len_b valid keys."""
    _say("attention padded", kind)
    rs = np.random.RandomState(3)
    lens, S, heads = [40, 64, 7], 64, 4
    B = len(lens)
    bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    qkv = rs.standard_normal((3, heads, B * S, 64)).astype(np.float16)
    scale = 1 / math.sqrt(64)
    fn = ops.attention_short if kind == "short" else ops.attention_grouped
    g = fn(_dev(qkv, device), _dev(bi, device), B, S, scale, True).cpu().numpy()
    for b in range(B):
        n = lens[b]
        q = qkv[0, :, b * S:(b + 1) * S].astype(np.float64)
        k = qkv[1, :, b * S:b * S + n].astype(np.float64)
        v = qkv[2, :, b * S:b * S + n].astype(np.float64)
        s = np.einsum("hqd,hkd->hqk", q, k) * scale
        e = np.exp(s - s.max(-1, keepdims=True))
        p = O.f16(e / (e.sum(-1, keepdims=True) + 1e-6))
        exp = np.einsum("hqk,hkd->qhd", p, v).reshape(S, heads * 64)
        err = np.abs(g[b * S:(b + 1) * S].astype(np.float64) - exp)
        assert err.max() <= 4e-3, (b, err.max())


@pytest.mark.parametrize("kind,S", [("short", 64), ("short", 200), ("grouped", 200),
                                     ("grouped", 70), ("short", 37), ("grouped", 640)])
def test_attention_arbitrary_mask_on_padded_rows(device, kind, S, att_order):
    """With the mask tensor given, every (query, key) pair follows mask[b,q,k]:
    logits are shifted by (mask-1)*10000 as in the reference's non-remove-padding
    kernels - banded, random and fully-masked rows included."""
    _say("attention full mask", kind, S)
    rs = np.random.RandomState(S)
    B, heads = 3, 2
    qkv = rs.standard_normal((3, heads, B * S, 64)).astype(np.float16)
    mask = (rs.rand(B, S, S) < 0.6).astype(np.float16)
    i, j = np.indices((S, S))
    mask[1] = (np.abs(i - j) <= 5).astype(np.float16)          # banded
    mask[2, 3, :] = 0                                          # a fully masked query row
    mask[2, :, S // 2:] = 0                                    # a prefix-style block
    bi = np.arange(B + 1, dtype=np.int32) * S                  # lengths are not used here
    scale = 1 / math.sqrt(64)
    fn = ops.attention_short if kind == "short" else ops.attention_grouped
    g = fn(_dev(qkv, device), _dev(bi, device), B, S, scale, True, mask=_dev(mask, device))
    if kind != "short":
        # the streaming kernel reads no offsets under a mask tensor: none given, or an array
        # of sentinels, gives the same bits
        for offsets in (None, torch.full((B + 1,), -12345, dtype=torch.int32, device=device)):
            g2 = fn(_dev(qkv, device), offsets, B, S, scale, True, mask=_dev(mask, device))
            assert torch.equal(g, g2)
    g = g.cpu().numpy().astype(np.float64)
    for b in range(B):
        q = qkv[0, :, b * S:(b + 1) * S].astype(np.float64)
        k = qkv[1, :, b * S:(b + 1) * S].astype(np.float64)
        v = qkv[2, :, b * S:(b + 1) * S].astype(np.float64)
        sc = np.einsum("hqd,hkd->hqk", q, k) * scale - 10000.0 * (1.0 - mask[b].astype(np.float64))
        e = np.exp(sc - sc.max(-1, keepdims=True))
        p = O.f16(e / (e.sum(-1, keepdims=True) + 1e-6))
        exp = np.einsum("hqk,hkd->qhd", p, v).reshape(S, heads * 64)
        err = np.abs(g[b * S:(b + 1) * S] - exp)
        assert err.max() <= 4e-3, (b, err.max())


@pytest.mark.parametrize("qb", [1, 2])
@pytest.mark.parametrize("lens,S,heads,padded", [
    ([512, 103, 257, 64, 65, 1, 0, 300], 512, 3, False),
    (list(np.random.RandomState(7).randint(0, 97, size=70)), 96, 2, False),
    ([200, 77, 130, 5], 200, 12, True),
])
def test_attention_work_list(device, lens, S, heads, padded, qb):
    """The balanced order as a list: the stand-alone builder and the layer prologue write
    the same entries, every live query tile appears exactly once, and the kernel gives the
    same bits with the list as with its own look-up."""
    lens = [int(v) for v in lens]
    _say("attention work list", len(lens), S, heads, padded, qb)
    rs = np.random.RandomState(S + heads)
    B = len(lens)
    mask = _dev(workload.make_mask(lens, S, np.float16), device)
    ops.set_option("attention_qb", qb)
    ops.set_option("attention_xcd_map", 3)          # the balanced order at any size
    try:
        order = torch.empty(B, dtype=torch.int32, device=device)
        bi, wi, _ = ops.build_offsets(mask, seq_order=order)
        wl = ops.attention_worklist(bi, B, S, heads, padded, seq_order=order)
        assert wl is not None
        wl2 = torch.full_like(wl, -7)
        ops.layer_prologue(mask, work_list=wl2, head_num=heads, padded_rows=padded)
        assert torch.equal(wl, wl2)
        e = wl.cpu().numpy()
        live = e[e[:, 0] >= 0]
        bq = 64 * qb
        want = set()
        for b, n in enumerate(lens):
            nq = S if padded else n
            for h in range(heads):
                for t in range((nq + bq - 1) // bq):
                    want.add((b, h, t))
        got = [(int(r[0]), int(r[1]) & 0xffff, int(r[1]) >> 16) for r in live]
        assert len(got) == len(set(got)) and set(got) == want
        starts = np.concatenate([[0], np.cumsum(lens)])
        assert all(int(r[2]) == starts[int(r[0])] and int(r[3]) == lens[int(r[0])] for r in live)
        qkv = _dev(rs.standard_normal((3, heads, B * S, 64)).astype(np.float16), device)
        a = ops.attention_grouped(qkv, bi, B, S, 0.125, padded, seq_order=order)
        b_ = ops.attention_grouped(qkv, bi, B, S, 0.125, padded, seq_order=order, work_list=wl)
        rows = B * S if padded else int(starts[-1])
        assert torch.equal(a[:rows], b_[:rows])
    finally:
        ops.set_option("attention_qb", -1)
        ops.set_option("attention_xcd_map", 2)
    # a shape whose launches keep the plain order takes no list
    assert ops.attention_worklist(bi, 1, 64, 2, False) is None


@pytest.mark.parametrize("qb", [1, 2])
def test_attention_drops_a_prefix_mask_on_the_device(device, qb, att_order):
    """The streaming kernel with the verdict slots of the device-side mask check: a plain
    prefix mask is ignored (keys stop at the lengths: the values of the padded rows'
    attention over the valid keys, as with the tensor applied); any other mask - one
    element flipped - is applied exactly as without the slots."""
    _say("attention mask slots", qb)
    rs = np.random.RandomState(77 + qb)
    B, S, heads = 3, 150, 2
    lens = np.array([150, 40, 97])
    qkv = rs.standard_normal((3, heads, B * S, 64)).astype(np.float16)
    mask = workload.make_mask(lens, S, np.float16)
    qd, md = _dev(qkv, device), _dev(mask, device)
    bi, _, _ = ops.build_offsets(md)
    scale = 1 / math.sqrt(64)
    ops.set_option("attention_qb", qb)
    try:
        slots = ops.mask_prefix_slots(md, bi)
        assert int(slots.min()) == 1
        with_tensor = ops.attention_grouped(qd, bi, B, S, scale, True, mask=md)
        dropped = ops.attention_grouped(qd, bi, B, S, scale, True, mask=md, mask_prefix_slots=slots)
        by_length = ops.attention_grouped(qd, bi, B, S, scale, True)
        # ignoring the tensor: the mask-free instantiation's values up to the last bits
        # of the fp32 logits (the additive path folds the scale in another order)
        d1 = (dropped.float() - by_length.float()).abs().max().item()
        d2 = (dropped.float() - with_tensor.float()).abs().max().item()
        assert d1 <= 2e-3 and d2 <= 2e-3, (d1, d2)
        # a mask that is not a prefix mask: slots say so, and the tensor is applied
        bad = mask.copy()
        bad[1, 7, 3] = 0
        bd = _dev(bad, device)
        bad_slots = ops.mask_prefix_slots(bd, bi)
        assert int(bad_slots.min()) == 0
        a = ops.attention_grouped(qd, bi, B, S, scale, True, mask=bd)
        b = ops.attention_grouped(qd, bi, B, S, scale, True, mask=bd, mask_prefix_slots=bad_slots)
        assert torch.equal(a, b)
        assert not torch.equal(a, with_tensor)
    finally:
        ops.set_option("attention_qb", -1)


@pytest.mark.parametrize("kind,S,padded,with_mask", [("short", 64, True, True), ("grouped", 200, True, True),
                                                    ("short", 100, False, False), ("grouped", 300, False, False),
                                                    ("grouped", 130, True, False)])
def test_attention_bias(device, kind, S, padded, with_mask, att_order):
    """attention_bias[h, q, k] is added to the scaled logits (positions relative to
    the sequence start) in the packed and the padded row layout, with and without
    the mask tensor."""
    _say("attention bias", kind, S, padded, with_mask)
    rs = np.random.RandomState(S + 7)
    B, heads = 3, 2
    lens = np.array([S, max(1, S // 3), S - 5])
    bias = rs.standard_normal((heads, S, S)).astype(np.float16)
    scale = 1 / math.sqrt(64)
    if padded:
        T = B * S
        starts = np.arange(B) * S
        bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    else:
        T = int(lens.sum())
        bi = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        starts = bi[:-1]
    qkv = rs.standard_normal((3, heads, T, 64)).astype(np.float16)
    mask = None
    if with_mask:
        mask = (rs.rand(B, S, S) < 0.6).astype(np.float16)
        mask[:, :, 0] = 1
    fn = ops.attention_short if kind == "short" else ops.attention_grouped
    g = fn(_dev(qkv, device), _dev(bi, device), B, S, scale, padded,
           mask=_dev(mask, device) if with_mask else None, bias=_dev(bias, device))
    g = g.cpu().numpy().astype(np.float64)
    for b in range(B):
        n = int(lens[b])
        nq = S if padded else n
        nk = S if with_mask else n
        t0 = int(starts[b])
        q = qkv[0, :, t0:t0 + nq].astype(np.float64)
        k = qkv[1, :, t0:t0 + nk].astype(np.float64)
        v = qkv[2, :, t0:t0 + nk].astype(np.float64)
        sc = np.einsum("hqd,hkd->hqk", q, k) * scale + bias[:, :nq, :nk].astype(np.float64)
        if with_mask:
            sc = sc - 10000.0 * (1.0 - mask[b, :nq, :nk].astype(np.float64))
        e = np.exp(sc - sc.max(-1, keepdims=True))
        p = O.f16(e / (e.sum(-1, keepdims=True) + 1e-6))
        exp = np.einsum("hqk,hkd->qhd", p, v).reshape(nq, heads * 64)
        err = np.abs(g[t0:t0 + nq] - exp)
        assert err.max() <= 4e-3, (b, err.max())


@pytest.mark.parametrize("kind,lens,S", [("short", [100, 7, 64], 128), ("grouped", [300, 40, 129, 5], 320),
                                        ("grouped", [77], 96)])
def test_attention_prefetch_hint_changes_nothing(device, kind, lens, S):
    """The cache warm-up range is only read: same output bits with and without it, for
    sizes that are not multiples of a line and for a single-sequence grid."""
    _say("attention prefetch", kind, lens, S)
    rs = np.random.RandomState(len(lens) + S)
    bi, M, qkv = _attention_case(rs, lens, S, 2, scale_q=1.0)
    fn = ops.attention_short if kind == "short" else ops.attention_grouped
    base = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, 0.125, False)
    for nbytes in (1, 127, 128, 1000003, 8 << 20):
        warm = torch.full((nbytes,), 7, dtype=torch.uint8, device=device)
        got = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, 0.125, False, prefetch=warm)
        torch.cuda.synchronize()
        assert torch.equal(got[:M], base[:M])
        assert bool((warm == 7).all())
    ops.set_option("prefetch", 0)
    try:
        got = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, 0.125, False, prefetch=warm)
        assert torch.equal(got[:M], base[:M])
    finally:
        ops.set_option("prefetch", 1)
    # Small launches skip the warm-up by themselves; force it on so that the duty
    # workgroups really run here.  The range sits inside a larger allocation (guard bytes on
    # both sides, so a stray line would still land in owned memory), starts on a line
    # boundary or 16 bytes into one, and ends 0-5 bytes into a line: the last touched dword
    # must lie inside the range.
    assert ops.get_option("prefetch_min_grid") == 512
    ops.set_option("prefetch_min_grid", 1)
    try:
        guard = 4096
        for nbytes in (1, 2, 3, 4, 5, 127, 128, 129, 130, 131, 132, 4099, 1000003, (8 << 20) + 2):
            for lead in (0, 16):
                whole = torch.full((guard + lead + nbytes + guard,), 7, dtype=torch.uint8,
                                   device=device)
                warm = whole[guard + lead:guard + lead + nbytes]
                got = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, 0.125, False,
                         prefetch=warm)
                torch.cuda.synchronize()
                assert torch.equal(got[:M], base[:M]), (nbytes, lead)
                assert bool((whole == 7).all())
        # several ranges (a layer's weights are separate tensors), empty ones among them
        wholes = [torch.full((guard + n + guard,), 7, dtype=torch.uint8, device=device)
                  for n in (131, 1, 70001, 4)]
        for count in (2, 3, 4):
            ranges = [w[guard:w.numel() - guard] for w in wholes[:count]]
            got = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, 0.125, False,
                     prefetch=ranges)
            torch.cuda.synchronize()
            assert torch.equal(got[:M], base[:M]), count
            assert all(bool((w == 7).all()) for w in wholes)
        with pytest.raises(ops.BtError):
            fn(_dev(qkv, device), _dev(bi, device), len(lens), S, 0.125, False,
               prefetch=[w[guard:-guard] for w in wholes] + [wholes[0][guard:-guard]])
    finally:
        ops.set_option("prefetch_min_grid", 512)


def test_attention_large_logits_do_not_overflow(device):
    """Logits of a few hundred in magnitude (fp16 Q.K would overflow at 65504)."""
    rs = np.random.RandomState(9)
    lens, S, heads = [96, 200], 256, 2
    bi, M, qkv = _attention_case(rs, lens, S, heads, scale_q=30.0)
    qkv[1, :, :M] *= 8
    scale = 1 / math.sqrt(64)
    exp = O.attention_packed(qkv[0, :, :M], qkv[1, :, :M], qkv[2, :, :M], bi, scale, 1e-6,
                             round_p_fp16=True)
    for fn in (ops.attention_short, ops.attention_grouped):
        g = fn(_dev(qkv, device), _dev(bi, device), len(lens), S, scale, False).cpu().numpy()
        assert np.isfinite(g[:M]).all()
        err = np.abs(g[:M].astype(np.float64) - exp)
        assert err.max() <= 2e-2, err.max()
