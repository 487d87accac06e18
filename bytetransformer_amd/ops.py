"""Tensor-level wrappers over the C ABI: each function takes torch tensors that
already live on the GPU, passes their addresses and the current stream to one
bt_* entry point and raises on a non-zero status.  Used by the tests and the
benchmark; no arithmetic happens in Python."""
import ctypes

import torch

from ._lib import kernel_lib

BT_F32, BT_F16 = 0, 1


class BtError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise BtError("bt status %d: %s" % (rc, kernel_lib().bt_last_error_string().decode()))


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise BtError("tensor must live on the GPU")
    if not t.is_contiguous():
        raise BtError("tensor must be contiguous")
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dtype_code(t):
    if t.dtype == torch.float16:
        return BT_F16
    if t.dtype == torch.float32:
        return BT_F32
    raise BtError("unsupported dtype %s" % t.dtype)


def set_option(name, value):
    _check(kernel_lib().bt_set_option(name.encode(), int(value)))


def get_option(name):
    v = ctypes.c_int(0)
    _check(kernel_lib().bt_get_option(name.encode(), ctypes.byref(v)))
    return v.value


def build_offsets(mask, want_count=False, out=None, seq_order=None):
    """mask [B,S,S] -> (batch_idx int32[B+1], word_idx int32[B*S], M or None)."""
    B, S = mask.shape[0], mask.shape[1]
    if out is None:
        batch_idx = torch.empty(B + 1, dtype=torch.int32, device=mask.device)
        word_idx = torch.empty(B * S, dtype=torch.int32, device=mask.device)
    else:
        batch_idx, word_idx = out
    cnt = ctypes.c_int(-1)
    _check(kernel_lib().bt_build_offsets(_ptr(mask), _dtype_code(mask), B, S, _ptr(batch_idx),
                                         _ptr(word_idx), _ptr(seq_order),
                                         ctypes.byref(cnt) if want_count else None, _stream()))
    return batch_idx, word_idx, (cnt.value if want_count else None)


def publish_int(src, dst):
    """*dst = *src on the current stream without any host wait: src is a device int32 (a view of
    one element, e.g. batch_idx[B:]), dst a pinned host int32 tensor the device can write."""
    if src.dtype != torch.int32 or dst.dtype != torch.int32 or not dst.is_pinned():
        raise ValueError("publish_int: int32 device source and pinned int32 host destination expected")
    _check(kernel_lib().bt_publish_int(_ptr(src), ctypes.c_void_p(dst.data_ptr()), _stream()))


def mask_is_prefix(mask, batch_idx):
    """True when mask [B,S,S] is exactly (j < len_b) in every row and no sequence is empty."""
    B, S = mask.shape[0], mask.shape[1]
    scratch = torch.empty(256, dtype=torch.int32, device=mask.device)
    verdict = ctypes.c_int(-1)
    _check(kernel_lib().bt_mask_is_prefix(_ptr(mask), _dtype_code(mask), B, S, _ptr(batch_idx),
                                          _ptr(scratch), ctypes.byref(verdict), _stream()))
    return bool(verdict.value)


def _weight_jobs(weights, packed, warm):
    """ctypes arguments (count, w, wt, k, n, warm_count, warm, warm_bytes) of the entries that
    make k-contiguous weight copies and touch ranges on behalf of later launches."""
    n = len(weights) if weights else 0
    if n:
        for w, t in zip(weights, packed):
            if tuple(t.shape) != tuple(w.shape[::-1]) or t.dtype != w.dtype:
                raise ValueError("packed copies must be the [n, k] counterparts of the weights")
        src = (ctypes.c_void_p * n)(*[_ptr(w).value for w in weights])
        dst = (ctypes.c_void_p * n)(*[_ptr(w).value for w in packed])
        ks = (ctypes.c_int * n)(*[w.shape[0] for w in weights])
        ns = (ctypes.c_int * n)(*[w.shape[1] for w in weights])
    else:
        src = dst = ks = ns = None
    warm = list(warm)
    nw = len(warm)
    wp = (ctypes.c_void_p * max(nw, 1))(*[_ptr(t).value for t in warm])
    wb = (ctypes.c_ulonglong * max(nw, 1))(*[t.numel() * t.element_size() for t in warm])
    return n, src, dst, ks, ns, nw, wp, wb


def layer_prologue(mask, want_slots=False, weights=None, packed=None, out=None,
                   work_list=None, head_num=0, padded_rows=False, warm=()):
    """bt_layer_prologue: offsets of `mask`, optionally the prefix-mask verdict slots and the
    [n, k] copies `packed` of the [k, n] `weights` (up to four).  Returns (batch_idx,
    word_idx, seq_order, slots or None); `out` = such a tuple to write into.  work_list
    (int32[entries, 4], with head_num and padded_rows): also filled with the attention's
    balanced order, as attention_worklist would.  warm: up to four tensors that later launches
    will read, touched line by line (a cache hint)."""
    B, S = mask.shape[0], mask.shape[1]
    dev = mask.device
    if out is not None:
        batch_idx, word_idx, seq_order, slots = out
    else:
        batch_idx = torch.empty(B + 1, dtype=torch.int32, device=dev)
        word_idx = torch.empty(B * S, dtype=torch.int32, device=dev)
        seq_order = torch.empty(B, dtype=torch.int32, device=dev)
        slots = torch.full((256,), -1, dtype=torch.int32, device=dev) if want_slots else None
    jobs = _weight_jobs(weights, packed, warm)
    _check(kernel_lib().bt_layer_prologue(
        _ptr(mask), _dtype_code(mask), B, S, _ptr(batch_idx), _ptr(word_idx), _ptr(seq_order),
        _ptr(slots), _ptr(work_list), int(head_num), int(padded_rows), *jobs, _stream()))
    return batch_idx, word_idx, seq_order, slots


def gemm_prepack_pays(rows, n, k, epilogue):
    """bt_gemm_prepack_pays; epilogue: 0 plain, 1 bias + GELU, 2 QKV split."""
    return bool(kernel_lib().bt_gemm_prepack_pays(int(rows), int(n), int(k), int(epilogue)))


def gemm_prepack_gain_us(rows, n, k, epilogue):
    """bt_gemm_prepack_gain_us: microseconds per launch that a per-call [n, k] copy returns."""
    return float(kernel_lib().bt_gemm_prepack_gain_us(int(rows), int(n), int(k), int(epilogue)))


def compress(x, batch_idx, word_idx, out=None):
    B, S, H = x.shape
    if out is None:
        out = torch.zeros(B * S, H, dtype=x.dtype, device=x.device)
    _check(kernel_lib().bt_compress(_ptr(x), _ptr(out), _ptr(batch_idx), _ptr(word_idx), B, S, H,
                                    _stream()))
    return out


def transpose_weight(w):
    K, N = w.shape
    wt = torch.empty(N, K, dtype=w.dtype, device=w.device)
    _check(kernel_lib().bt_transpose_weight(_ptr(w), _ptr(wt), K, N, _stream()))
    return wt


def transpose_weights(ws, out=None):
    """Pre-pack up to four [K, N] weights in one launch; returns the [N, K] copies."""
    n = len(ws)
    wts = out if out is not None else [
        torch.empty(w.shape[1], w.shape[0], dtype=w.dtype, device=w.device) for w in ws]
    src = (ctypes.c_void_p * n)(*[w.data_ptr() for w in ws])
    dst = (ctypes.c_void_p * n)(*[w.data_ptr() for w in wts])
    ks = (ctypes.c_int * n)(*[w.shape[0] for w in ws])
    ns = (ctypes.c_int * n)(*[w.shape[1] for w in ws])
    for w in ws:
        _ptr(w)
    _check(kernel_lib().bt_transpose_weights(n, src, dst, ks, ns, _stream()))
    return wts


def _gemm_shapes(who, a, w, w_kn, out, out_elems_per_row=None):
    """Shapes the launch is derived from must agree before anything is launched: a weight
    passed in the wrong layout would otherwise make the kernel write past `out`."""
    rows, K = a.shape
    wk, N = w.shape if w_kn else w.shape[::-1]
    if wk != K:
        raise ValueError("%s: the weight must be %s with k = %d, got %s"
                         % (who, "[k, n]" if w_kn else "the [n, k] pre-pack", K, tuple(w.shape)))
    if out is not None and out.numel() < rows * (out_elems_per_row or N):
        raise ValueError("%s: out holds %d elements, the launch writes up to %d"
                         % (who, out.numel(), rows * (out_elems_per_row or N)))
    return rows, N, K


def gemm(a, wt, valid_rows=None, out=None, rows_hint=0, w_kn=False):
    """a . w; `wt` is the [n, k] pre-pack, or with w_kn the [k, n] weight itself."""
    rows, N, K = _gemm_shapes("gemm", a, wt, w_kn, out)
    if out is None:
        out = torch.zeros(rows, N, dtype=a.dtype, device=a.device)
    _check(kernel_lib().bt_gemm(_ptr(a), _ptr(wt), _ptr(out), _ptr(valid_rows), rows,
                                int(rows_hint), N, K, int(w_kn), _stream()))
    return out


def gemm_bias_gelu(a, wt, bias, valid_rows=None, out=None, rows_hint=0, w_kn=False):
    rows, N, K = _gemm_shapes("gemm_bias_gelu", a, wt, w_kn, out)
    if bias.numel() != N:
        raise ValueError("gemm_bias_gelu: bias must have %d elements" % N)
    if out is None:
        out = torch.zeros(rows, N, dtype=a.dtype, device=a.device)
    _check(kernel_lib().bt_gemm_bias_gelu(_ptr(a), _ptr(wt), _ptr(bias), _ptr(out),
                                          _ptr(valid_rows), rows, int(rows_hint), N, K,
                                          int(w_kn), _stream()))
    return out


def gemm_qkv_bias_split(a, wt_qkv, bias_qkv, head_num, size_per_head=64, valid_rows=None,
                        out=None, a_row_index=None, rows_cap=None, rows_hint=0, w_kn=False):
    rows = a.shape[0] if rows_cap is None else rows_cap
    H = head_num * size_per_head
    want = (H, 3 * H) if w_kn else (3 * H, H)
    if tuple(wt_qkv.shape) != want or a.shape[1] != H or bias_qkv.numel() != 3 * H:
        raise ValueError("gemm_qkv_bias_split: a [*, %d], weight %s and bias [%d] expected"
                         % (H, list(want), 3 * H))
    if a_row_index is None and a.shape[0] < rows:
        raise ValueError("gemm_qkv_bias_split: a has fewer rows than rows_cap")
    if out is not None and out.numel() < rows * 3 * H:
        raise ValueError("gemm_qkv_bias_split: out holds %d elements, the launch writes up to %d"
                         % (out.numel(), rows * 3 * H))
    if out is None:
        out = torch.zeros(3, head_num, rows, size_per_head, dtype=a.dtype, device=a.device)
    _check(kernel_lib().bt_gemm_qkv_bias_split(_ptr(a), _ptr(a_row_index), _ptr(wt_qkv),
                                               _ptr(bias_qkv), _ptr(out),
                                               _ptr(valid_rows), rows, int(rows_hint), head_num,
                                               size_per_head, int(w_kn), _stream()))
    return out


def gemm_qkv_mask_rows_supported(batch_size, seq_len, mask_dtype=torch.float16):
    code = BT_F16 if mask_dtype == torch.float16 else BT_F32 if mask_dtype == torch.float32 else -1
    return bool(kernel_lib().bt_gemm_qkv_mask_rows_supported(batch_size, seq_len, code))


def gemm_qkv_bias_split_mask_rows(x, mask, wt_qkv, bias_qkv, head_num, size_per_head=64, out=None,
                                  offsets_out=None, rows_hint=0, w_kn=False):
    """QKV projection of the padded x [B, S, H] whose live rows come from the mask inside the
    launch; returns (qkv_heads, batch_idx, word_idx, seq_order)."""
    B, S = mask.shape[0], mask.shape[1]
    H = head_num * size_per_head
    rows = B * S
    want = (H, 3 * H) if w_kn else (3 * H, H)
    if tuple(wt_qkv.shape) != want or x.numel() != rows * H or bias_qkv.numel() != 3 * H:
        raise ValueError("gemm_qkv_bias_split_mask_rows: x [%d, %d, %d], weight %s and bias [%d] "
                         "expected" % (B, S, H, list(want), 3 * H))
    if tuple(mask.shape) != (B, S, S):
        raise ValueError("gemm_qkv_bias_split_mask_rows: mask must be [B, S, S]")
    if out is not None and out.numel() < rows * 3 * H:
        raise ValueError("gemm_qkv_bias_split_mask_rows: out holds %d elements, the launch "
                         "writes up to %d" % (out.numel(), rows * 3 * H))
    if out is None:
        out = torch.zeros(3, head_num, rows, size_per_head, dtype=x.dtype, device=x.device)
    if offsets_out is None:
        offsets_out = (torch.empty(B + 1, dtype=torch.int32, device=x.device),
                       torch.empty(rows, dtype=torch.int32, device=x.device),
                       torch.empty(B, dtype=torch.int32, device=x.device))
    batch_idx, word_idx, seq_order = offsets_out
    if batch_idx.numel() < B + 1 or (word_idx is not None and word_idx.numel() < rows) or \
            (seq_order is not None and seq_order.numel() < B):
        raise ValueError("gemm_qkv_bias_split_mask_rows: offset outputs too small")
    _check(kernel_lib().bt_gemm_qkv_bias_split_mask_rows(
        _ptr(x), _ptr(mask), _dtype_code(mask), B, S, _ptr(wt_qkv), _ptr(bias_qkv), _ptr(out),
        _ptr(batch_idx), _ptr(word_idx), _ptr(seq_order), int(rows_hint), head_num, size_per_head,
        int(w_kn), _stream()))
    return out, batch_idx, word_idx, seq_order


def _attention(fn, qkv_heads, batch_idx, batch_size, seq_len, scale, padded_rows, out,
               seq_order=None, mask=None, bias=None, prefetch=None, extra=()):
    _, head_num, rows_cap, d = qkv_heads.shape
    if out is None:
        out = torch.zeros(rows_cap, head_num * d, dtype=qkv_heads.dtype, device=qkv_heads.device)
    if bias is not None and tuple(bias.shape) != (head_num, seq_len, seq_len):
        raise ValueError("attention bias must be [head_num, seq_len, seq_len]")
    # prefetch: one tensor or up to four, the ranges later kernels will read
    ranges = [] if prefetch is None else ([prefetch] if torch.is_tensor(prefetch) else list(prefetch))
    n = len(ranges)
    ptrs = (ctypes.c_void_p * max(n, 1))(*[t.data_ptr() for t in ranges])
    sizes = (ctypes.c_ulonglong * max(n, 1))(*[t.numel() * t.element_size() for t in ranges])
    for t in ranges:
        _ptr(t)
    _check(fn(_ptr(qkv_heads), _ptr(out), _ptr(batch_idx), _ptr(seq_order), _ptr(mask), _ptr(bias),
              batch_size, seq_len, rows_cap, head_num, d, float(scale), int(padded_rows),
              ptrs, sizes, n, *extra, _stream()))
    return out


def attention_short(qkv_heads, batch_idx, batch_size, seq_len, scale, padded_rows=False, out=None,
                    seq_order=None, mask=None, bias=None, prefetch=None):
    return _attention(kernel_lib().bt_attention_short, qkv_heads, batch_idx, batch_size, seq_len,
                      scale, padded_rows, out, seq_order, mask, bias, prefetch)


def attention_grouped(qkv_heads, batch_idx, batch_size, seq_len, scale, padded_rows=False,
                      out=None, seq_order=None, mask=None, bias=None, prefetch=None,
                      mask_prefix_slots=None, work_list=None):
    return _attention(kernel_lib().bt_attention_grouped, qkv_heads, batch_idx, batch_size,
                      seq_len, scale, padded_rows, out, seq_order, mask, bias, prefetch,
                      extra=(_ptr(mask_prefix_slots), _ptr(work_list)))


def attention_worklist(batch_idx, batch_size, seq_len, head_num, padded_rows=False, seq_order=None):
    """The balanced workgroup order of attention_grouped for this shape and these offsets as
    a list (int32[entries, 4]) to pass as work_list, or None when launches of this shape do
    not use that order."""
    lib = kernel_lib()
    nbytes = lib.bt_attention_worklist_bytes(batch_size, seq_len, head_num)
    if nbytes == 0:
        return None
    wl = torch.empty(nbytes // 16, 4, dtype=torch.int32, device=batch_idx.device)
    _check(lib.bt_attention_worklist(_ptr(batch_idx), _ptr(seq_order), batch_size, seq_len,
                                     head_num, int(padded_rows), _ptr(wl), _stream()))
    return wl


def mask_prefix_slots(mask, batch_idx, out=None):
    """int32[256] on the device, all ones when mask [B,S,S] is the plain prefix mask of the
    lengths in batch_idx (asynchronous; attention_grouped takes the array)."""
    B, S = mask.shape[0], mask.shape[1]
    if out is None:
        out = torch.empty(256, dtype=torch.int32, device=mask.device)
    _check(kernel_lib().bt_mask_prefix_slots(_ptr(mask), _dtype_code(mask), B, S, _ptr(batch_idx),
                                             _ptr(out), _stream()))
    return out


def add_bias_residual_layernorm(out, residual, bias, gamma, beta, eps=1e-6, valid_rows=None,
                                residual_row_index=None):
    rows, H = out.shape
    _check(kernel_lib().bt_add_bias_residual_layernorm(
        _ptr(out), _ptr(residual), _ptr(residual_row_index), _ptr(bias), _ptr(gamma), _ptr(beta),
        int(gamma.dtype == torch.float32), _ptr(valid_rows), rows, H, float(eps), _stream()))
    return out


def add_bias_residual_layernorm_copy(out, residual, bias, gamma, beta, weights, packed, eps=1e-6,
                                     valid_rows=None, residual_row_index=None):
    """add_bias_residual_layernorm whose launch also fills `packed` with the [n, k] copies of the
    [k, n] `weights` (up to four)."""
    rows, H = out.shape
    n, src, dst, ks, ns = _weight_jobs(weights, packed, ())[:5]
    _check(kernel_lib().bt_add_bias_residual_layernorm_copy(
        _ptr(out), _ptr(residual), _ptr(residual_row_index), _ptr(bias), _ptr(gamma), _ptr(beta),
        int(gamma.dtype == torch.float32), _ptr(valid_rows), rows, H, float(eps), n, src, dst, ks,
        ns, _stream()))
    return out


def add_bias_residual_layernorm_restore(out, residual, bias, gamma, beta, batch_idx, batch_size,
                                        seq_len, eps=1e-6, out_padded=None, word_idx=None):
    """word_idx: the complete word_idx of the same offsets (the row map); `out` and `residual`
    must then hold batch_size * seq_len rows."""
    H = out.shape[-1]
    if word_idx is not None:
        rows = batch_size * seq_len
        if word_idx.numel() < rows or out.numel() < rows * H or residual.numel() < rows * H:
            raise ValueError("restore through word_idx needs batch_size * seq_len rows of out, "
                             "residual and word_idx")
    if out_padded is None:
        out_padded = torch.empty(batch_size, seq_len, H, dtype=out.dtype, device=out.device)
    _check(kernel_lib().bt_add_bias_residual_layernorm_restore(
        _ptr(out), _ptr(residual), _ptr(bias), _ptr(gamma), _ptr(beta),
        int(gamma.dtype == torch.float32), _ptr(out_padded), _ptr(batch_idx), _ptr(word_idx),
        batch_size, seq_len, H, float(eps), _stream()))
    return out_padded


def gemm_splitk(a, wt, splits, valid_rows=None, out=None, w_kn=False):
    """fp32 partial sums [splits, rows, N] of a . w over `splits` k ranges."""
    rows, N, K = _gemm_shapes("gemm_splitk", a, wt, w_kn, None)
    if out is not None and out.numel() < splits * rows * N:
        raise ValueError("gemm_splitk: out holds %d elements, the launch writes up to %d"
                         % (out.numel(), splits * rows * N))
    if out is None:
        out = torch.zeros(splits, rows, N, dtype=torch.float32, device=a.device)
    _check(kernel_lib().bt_gemm_splitk(_ptr(a), _ptr(wt), _ptr(out), int(splits), _ptr(valid_rows),
                                       rows, N, K, int(w_kn), _stream()))
    return out


def splitk_layernorm(partials, residual, bias, gamma, beta, dst, eps=1e-6, valid_rows=None,
                     residual_row_index=None, batch_idx=None, batch_size=0, seq_len=1):
    splits, rows, H = partials.shape
    _check(kernel_lib().bt_splitk_layernorm(
        _ptr(partials), splits, _ptr(residual), _ptr(residual_row_index), _ptr(bias), _ptr(gamma),
        _ptr(beta), int(gamma.dtype == torch.float32), _ptr(dst), _ptr(batch_idx),
        _ptr(valid_rows), batch_size, seq_len, rows, H, float(eps), _stream()))
    return dst


# ---- float (OperationType::FP32) entry points ---------------------------------
def _need_f32(*ts):
    for t in ts:
        if t is not None and t.dtype != torch.float32:
            raise BtError("the *_f32 entry points take float tensors only")


def gemm_f32(a, w, bias=None, gelu=False, valid_rows=None, a_row_index=None, rows_cap=None,
             out=None, rows_hint=0):
    """c = a . w (+ bias) (+ tanh-GELU); w is [K, N] as stored."""
    _need_f32(a, w, bias, out)
    rows = a.shape[0] if rows_cap is None else rows_cap
    K, N = w.shape
    if out is None:
        out = torch.zeros(rows, N, dtype=a.dtype, device=a.device)
    _check(kernel_lib().bt_gemm_f32(_ptr(a), _ptr(a_row_index), _ptr(w), _ptr(bias), _ptr(out),
                                    int(gelu), _ptr(valid_rows), rows, int(rows_hint), N, K,
                                    _stream()))
    return out


def attention_f32(qkv, batch_idx, batch_size, seq_len, head_num, scale, padded_rows=False,
                  mask=None, bias=None, out=None, seq_order=None):
    """qkv [rows, 3 * hidden] (bias added) -> [rows, hidden]."""
    _need_f32(qkv, mask, bias, out)
    rows_cap, three_h = qkv.shape
    hidden = three_h // 3
    if out is None:
        out = torch.zeros(rows_cap, hidden, dtype=qkv.dtype, device=qkv.device)
    if bias is not None and tuple(bias.shape) != (head_num, seq_len, seq_len):
        raise ValueError("attention bias must be [head_num, seq_len, seq_len]")
    _check(kernel_lib().bt_attention_f32(_ptr(qkv), _ptr(out), _ptr(batch_idx), _ptr(seq_order),
                                         _ptr(mask),
                                         _ptr(bias), batch_size, seq_len, rows_cap, head_num,
                                         hidden // head_num, float(scale), int(padded_rows),
                                         _stream()))
    return out


def attention_generic_f16(qkv, batch_idx, batch_size, seq_len, head_num, scale, padded_rows=False,
                          mask=None, bias=None, out=None, seq_order=None):
    """fp16 qkv [rows, 3 * hidden] (bias added) -> [rows, hidden]; head sizes 32, 64, 96, 128."""
    rows_cap, three_h = qkv.shape
    hidden = three_h // 3
    if out is None:
        out = torch.zeros(rows_cap, hidden, dtype=qkv.dtype, device=qkv.device)
    _check(kernel_lib().bt_attention_generic_f16(
        _ptr(qkv), _ptr(out), _ptr(batch_idx), _ptr(seq_order), _ptr(mask), _ptr(bias), batch_size,
        seq_len, rows_cap, head_num, hidden // head_num, float(scale), int(padded_rows),
        _stream()))
    return out


def add_bias_residual_layernorm_f32(out, residual, bias, gamma, beta, eps=1e-6, valid_rows=None,
                                    residual_row_index=None):
    _need_f32(out, residual, bias, gamma, beta)
    rows, H = out.shape
    _check(kernel_lib().bt_add_bias_residual_layernorm_f32(
        _ptr(out), _ptr(residual), _ptr(residual_row_index), _ptr(bias), _ptr(gamma), _ptr(beta),
        _ptr(valid_rows), rows, H, float(eps), _stream()))
    return out


def add_bias_residual_layernorm_restore_f32(out, residual, bias, gamma, beta, batch_idx,
                                            batch_size, seq_len, eps=1e-6, out_padded=None):
    _need_f32(out, residual, bias, gamma, beta, out_padded)
    H = out.shape[-1]
    if out_padded is None:
        out_padded = torch.empty(batch_size, seq_len, H, dtype=out.dtype, device=out.device)
    _check(kernel_lib().bt_add_bias_residual_layernorm_restore_f32(
        _ptr(out), _ptr(residual), _ptr(bias), _ptr(gamma), _ptr(beta), _ptr(out_padded),
        _ptr(batch_idx), batch_size, seq_len, H, float(eps), _stream()))
    return out_padded
