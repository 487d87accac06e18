#!/usr/bin/env python3
"""Headline benchmark: ms per 12-layer BERT-base forward, fp16, batch 16,
max seq 512, valid lengths uniform on [103, 512] (mean ~0.6 * max), through the
PyTorch operator torch.ops.ByteTransformer.BertTransformer - one operator call
per layer, as the reference's benchmark script drives it
(unit_test/python_scripts/bert_transformer_test.py:184-208,
benchmark/bert_bench.sh:21-57).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2]

Prints ONE JSON line.  A "step" is one full L-layer forward over the synthetic
batch; inputs and weights are resident in HBM before the timed region; the
timed region is bracketed by torch.cuda.synchronize().  The same line carries
the roofline of the dominant kernel (live HIP-event timing of that kernel at
the workload's shape), the CPU baseline (the oracle's PyTorch fp32 encoder on
the host cores, bounded sample), the parity of the last timed forward against one
complete forward of that oracle (the run fails outside max-abs 2e-2 / mean-abs 2e-3),
the vendor GEMM library on the same shapes and the torch-free per-layer time of the
C++ API (the stand-alone driver as a child process).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PUBLISHED_A100_MS = {"cfg1": 1.43, "cfg2": 9.22, "cfg3": 24.70}   # reference README.md:37,63,71
MFMA_F16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg2",
                    choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg4_fixed"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-cpp-driver", action="store_true",
                    help="skip the child process that times the C++ API (profilers that "
                         "initialise the GPU before this program starts forbid spawning it)")
    ap.add_argument("--kernel-iters", type=int, default=50)
    ap.add_argument("--vendor-compare", action="store_true",
                    help="counter mode: only the FFN1 shape and 8192^3 through the vendor library "
                         "and through the in-tree product (see vendor_compare)")
    return ap.parse_args()


def time_kernel(fn, iters):
    """Average duration (ms) of `fn`, which enqueues exactly one kernel on the
    current stream and allocates nothing.  The launches are captured once into a
    HIP graph and the replay is bracketed by HIP events on its stream, so the
    figure is GPU time per launch without the Python call overhead (which exceeds
    the run time of the small kernels).  Falls back to an eager loop if capture
    is unavailable."""
    import torch
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(iters):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        beg.record()
        graph.replay()
        end.record()
    except Exception as exc:   # noqa: BLE001 - any capture problem -> eager timing
        print("bench: graph capture failed (%s), timing eagerly" % exc, file=sys.stderr)
        torch.cuda.synchronize()
        beg.record()
        for _ in range(iters):
            fn()
        end.record()
    end.synchronize()
    return beg.elapsed_time(end) / iters


def kernel_table(wl, dev, iters):
    """Live per-kernel timings at the workload's shape, each against its own
    roofline: algorithmic flops (GEMMs, attention) or bytes (padding, LN)."""
    import numpy as np
    import torch
    from bytetransformer_amd import ops
    cfg = wl.cfg
    B, S, H, F, heads = cfg.batch, cfg.seq_len, cfg.hidden, cfg.ffn_mult * cfg.hidden, cfg.head_num
    T, M = B * S, wl.valid_tokens
    sq = int((wl.lens.astype(np.int64) ** 2).sum())
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    w = {k: t(v) for k, v in wl.layers[0].items()}
    x, mask = t(wl.x), t(wl.mask)
    seq_order = torch.empty(B, dtype=torch.int32, device=dev)
    batch_idx, word_idx, _ = ops.build_offsets(mask, seq_order=seq_order)
    vr = batch_idx[B:]
    packed = ops.compress(x, batch_idx, word_idx)
    # The layer reads each weight as stored ([k, n]) unless the measured tile table says its
    # product runs faster on a k-contiguous copy made in the prologue of the same call: time
    # every product the way the operator launches it at this row count.
    names = ("qkv_kernel", "attr_output_kernel", "inter_kernel", "output_kernel")
    import bytetransformer_amd as bt
    pays, fused_start, _ = bt.BertEncoderLayer(heads, cfg.head_size, w).plan(B, S, rows_hint=M)
    kn_qkv, kn_o, kn_1, kn_2 = [not p for p in pays]
    wt_qkv, wt_o, wt_1, wt_2 = [ops.transpose_weight(w[n]) if p else w[n]
                                for n, p in zip(names, pays)]
    qkv = ops.gemm_qkv_bias_split(packed, wt_qkv, w["qkv_bias"], heads, valid_rows=vr, w_kn=kn_qkv)
    scale = 1.0 / cfg.head_size ** 0.5
    att_fn = ops.attention_grouped     # the host library's default choice at every length
    att = att_fn(qkv, batch_idx, B, S, scale)
    proj = ops.gemm(att, wt_o, valid_rows=vr, w_kn=kn_o)
    inter = ops.gemm_bias_gelu(proj, wt_1, w["inter_bias"], valid_rows=vr, w_kn=kn_1)
    ffn2 = ops.gemm(inter, wt_2, valid_rows=vr, w_kn=kn_2)
    out_pad = torch.empty(B, S, H, dtype=torch.float16, device=dev)
    ln_buf = proj.clone()
    g1, b1 = w["attr_output_layernorm_gamma"], w["attr_output_layernorm_beta"]
    bo_bi, bo_wi = torch.empty_like(batch_idx), torch.empty_like(word_idx)
    x2d = x.view(T, H)
    # every launch after the attention is sized for batch * seq_len rows, as the operator sizes
    # it (the live row count is read on the device; `rows_hint` only steers the tile choice)
    att_m, proj_m, inter_m, ffn2_m, ln_m = att, proj, inter, ffn2, ln_buf

    # the layer's first launch: offsets + the k-contiguous copies of the weights that pay
    pro_out = (bo_bi, bo_wi, torch.empty_like(seq_order), None)
    pro_w = [w[n] for n, p in zip(names, pays) if p == 1]
    pro_wt = [t_ for t_, p in zip((wt_qkv, wt_o, wt_1, wt_2), pays) if p == 1]
    # ... and those that the first LayerNorm's launch makes
    ln_w = [w[n] for n, p in zip(names, pays) if p == 2]
    ln_wt = [t_ for t_, p in zip((wt_qkv, wt_o, wt_1, wt_2), pays) if p == 2]
    pro_warm = [w[n] for n, p in zip(names, pays) if not p]      # read as stored: first touch
    pro_bytes = sum(2 * x_.numel() * 2 for x_ in pro_w)

    all_wt = [torch.empty(w[n].shape[1], w[n].shape[0], dtype=torch.float16, device=dev)
              for n in names]
    rows = [
        # name, callable, bound, algorithmic work per launch (flops or bytes)
        ("build_offsets", lambda: ops.build_offsets(mask, out=(bo_bi, bo_wi)), "hbm",
         2 * B * S + 4 * (B + 1) + 4 * M),
        ("layer_prologue", lambda: ops.layer_prologue(mask, weights=pro_w, packed=pro_wt,
                                                      out=pro_out, warm=pro_warm), "hbm",
         2 * B * S + 4 * (B + 1) + 4 * M + pro_bytes),
        ("compress", lambda: ops.compress(x, batch_idx, word_idx, out=packed), "hbm",
         2 * M * H * 2 + 4 * M),
        ("gemm_qkv_bias_split", lambda: ops.gemm_qkv_bias_split(
            x2d, wt_qkv, w["qkv_bias"], heads, valid_rows=vr, out=qkv, a_row_index=word_idx,
            rows_hint=M, w_kn=kn_qkv),
         "mfma", 2 * M * H * 3 * H),
    ]
    if ops.gemm_qkv_mask_rows_supported(B, S, mask.dtype):
        # the same product with the live rows counted from the mask inside the launch (what a
        # layer starts with when no per-call weight copy pays; stand-alone entry otherwise)
        mr_out = (torch.empty_like(batch_idx), torch.empty_like(word_idx), torch.empty_like(seq_order))
        rows.append(("gemm_qkv_bias_split_mask_rows", lambda: ops.gemm_qkv_bias_split_mask_rows(
            x, mask, w["qkv_kernel"], w["qkv_bias"], heads, out=qkv, offsets_out=mr_out,
            rows_hint=M, w_kn=True), "mfma", 2 * M * H * 3 * H))
    rows += [
        ("attention", lambda: att_fn(qkv, batch_idx, B, S, scale, out=att, seq_order=seq_order),
         "mfma", 4 * H * sq),
        ("gemm_proj", lambda: ops.gemm(att_m, wt_o, valid_rows=vr, out=proj_m, rows_hint=M,
                                       w_kn=kn_o), "mfma",
         2 * M * H * H),
        ("layernorm", (lambda: ops.add_bias_residual_layernorm_copy(
            ln_m, x2d, w["attr_output_bias"], g1, b1, ln_w, ln_wt, valid_rows=vr,
            residual_row_index=word_idx)) if ln_w else (lambda: ops.add_bias_residual_layernorm(
                ln_m, x2d, w["attr_output_bias"], g1, b1, valid_rows=vr, residual_row_index=word_idx)),
         "hbm", 3 * M * H * 2 + sum(2 * t_.numel() * 2 for t_ in ln_w)),
        ("gemm_bias_gelu", lambda: ops.gemm_bias_gelu(proj_m, wt_1, w["inter_bias"], valid_rows=vr,
                                                      out=inter_m, rows_hint=M, w_kn=kn_1), "mfma",
         2 * M * H * F),
        ("gemm_ffn2", lambda: ops.gemm(inter_m, wt_2, valid_rows=vr, out=ffn2_m, rows_hint=M,
                                       w_kn=kn_2), "mfma",
         2 * M * F * H),
    ]
    if kn_1:
        # the same FFN1 launch on a k-contiguous copy of its weight: what the whole-encoder
        # entry, which owns pre-packed copies, runs - and what the as-stored layout costs
        wt_1_packed = ops.transpose_weight(w["inter_kernel"])
        rows.append(("gemm_bias_gelu_prepacked", lambda: ops.gemm_bias_gelu(
            proj_m, wt_1_packed, w["inter_bias"], valid_rows=vr, out=inter_m, rows_hint=M,
            w_kn=False), "mfma", 2 * M * H * F))
    rows += [
        ("layernorm_restore", lambda: ops.add_bias_residual_layernorm_restore(
            ffn2, proj, w["output_bias"], g1, b1, batch_idx, B, S, out_padded=out_pad,
            word_idx=word_idx),
         "hbm", 2 * M * H * 2 + T * H * 2),
        ("transpose_weights", lambda: ops.transpose_weights([w[n] for n in names], out=all_wt),
         "hbm", 2 * (4 * H * H + 2 * H * F) * 2),
    ]
    # plain device copy of known size: the reference dispatch that the rocprofv3
    # FETCH_SIZE / WRITE_SIZE counters are scaled by
    # (the row gather on an all-valid [64, 256, 2048] batch: a 64 MiB copy)
    cB, cS, cH = 64, 256, 2048
    calib_src = torch.empty(cB, cS, cH, dtype=torch.float16, device=dev).normal_()
    calib_dst = torch.empty(cB * cS, cH, dtype=torch.float16, device=dev)
    c_bi, c_wi, _ = ops.build_offsets(torch.ones(cB, cS, cS, dtype=torch.float16, device=dev))
    rows.append(("copy_calibration_64MiB",
                 lambda: ops.compress(calib_src, c_bi, c_wi, out=calib_dst), "hbm",
                 2 * calib_src.numel() * 2))
    # A plain copy moving as many bytes as each memory-bound kernel of the layer moves: what
    # a launch of that size can reach at all (the row gather over an identity index).
    def same_size_copy(name, total_bytes):
        r = max(1, int(total_bytes) // (2 * H * 2))          # rows: read + write of r*H halfs
        src = torch.empty(1, r, H, dtype=torch.float16, device=dev).normal_()
        dst = torch.empty(r, H, dtype=torch.float16, device=dev)
        bi = torch.tensor([0, r], dtype=torch.int32, device=dev)
        wi = torch.arange(r, dtype=torch.int32, device=dev)
        rows.append((name, lambda: ops.compress(src, bi, wi, out=dst), "hbm", 2 * r * H * 2))

    same_size_copy("copy_same_bytes_as_layernorm", 3 * M * H * 2 + sum(2 * t_.numel() * 2 for t_ in ln_w))
    same_size_copy("copy_same_bytes_as_layernorm_restore", 2 * M * H * 2 + T * H * 2)
    same_size_copy("copy_same_bytes_as_compress", 2 * M * H * 2)
    # The memory-bound kernels at a size where the launch cost (a few us, the same for
    # a plain copy) no longer dominates: 16x the rows of the workload.
    big = 16 * T
    big_out = torch.empty(big, H, dtype=torch.float16, device=dev).normal_()
    big_res = torch.empty(big, H, dtype=torch.float16, device=dev).normal_()
    rows.append(("layernorm_16x_rows", lambda: ops.add_bias_residual_layernorm(
        big_out, big_res, w["attr_output_bias"], g1, b1), "hbm", 3 * big * H * 2))
    table = {}
    for name, fn, bound, work in rows:
        ms = time_kernel(fn, iters)
        if bound == "mfma":
            ach, peak, unit = work / (ms * 1e-3) / 1e12, MFMA_F16_PEAK_TFLOPS, "TFLOP/s"
        else:
            ach, peak, unit = work / (ms * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s"
        table[name] = {"us": round(ms * 1e3, 2), "bound": bound, "achieved": round(ach, 2),
                       "peak": peak, "unit": unit, "frac": round(ach / peak, 4)}
    # each memory-bound kernel against the plain copy of the same byte count
    for kern, ref in (("layernorm", "copy_same_bytes_as_layernorm"),
                      ("layernorm_restore", "copy_same_bytes_as_layernorm_restore"),
                      ("compress", "copy_same_bytes_as_compress")):
        table[kern]["vs_same_size_copy"] = round(table[kern]["achieved"] / table[ref]["achieved"], 3)
    # which products ran on a per-call k-contiguous copy of their weight (the others read
    # the [k, n] weight as stored)
    for kern, p in zip(("gemm_qkv_bias_split", "gemm_proj", "gemm_bias_gelu", "gemm_ffn2"), pays):
        table[kern]["weight"] = ("[k,n] as stored", "[n,k] copy made in the prologue",
                                 "[n,k] copy made in the first LayerNorm's launch")[p]
    # the launches that one layer of the timed forward is made of (the others are stand-alone
    # entries, calibration copies and the variants the layer does not take at this shape)
    first = ["gemm_qkv_bias_split_mask_rows"] if fused_start else ["layer_prologue", "gemm_qkv_bias_split"]
    in_layer = first + ["attention", "gemm_proj", "layernorm", "gemm_bias_gelu", "gemm_ffn2",
                        "layernorm_restore"]
    for kern in table:
        table[kern]["in_layer"] = kern in in_layer
    return table


def hipblaslt_calibration(wl, dev, iters):
    """torch.matmul (hipBLASLt / rocBLAS behind PyTorch-ROCm) on the layer's four GEMM
    shapes at the workload's row count and on 8192^3: what the vendor library reaches on
    this box next to the in-tree kernels.  fp16 in and out, no epilogue."""
    import torch
    cfg = wl.cfg
    H, F, M = cfg.hidden, cfg.ffn_mult * cfg.hidden, wl.valid_tokens
    out = {}
    for name, (m, n, k) in (("qkv", (M, 3 * H, H)), ("proj", (M, H, H)), ("ffn1", (M, F, H)),
                            ("ffn2", (M, H, F)), ("square_8192", (8192, 8192, 8192))):
        a = torch.empty(m, k, dtype=torch.float16, device=dev).normal_()
        b = torch.empty(k, n, dtype=torch.float16, device=dev).normal_(std=0.02)
        c = torch.empty(m, n, dtype=torch.float16, device=dev)
        ms = time_kernel(lambda: torch.matmul(a, b, out=c), max(5, iters // 5 if m >= 8192 else iters))
        tf = 2.0 * m * n * k / (ms * 1e-3) / 1e12
        out[name] = {"m": m, "n": n, "k": k, "us": round(ms * 1e3, 2), "tflops": round(tf, 1),
                     "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        if name == "square_8192":
            # the in-tree product on the same large shape (plain epilogue, weight as stored and
            # pre-packed): what its k loop sustains once fill, stores and tile quantisation are
            # amortised, beside the vendor library's figure
            from bytetransformer_amd import ops
            bt_ = ops.transpose_weight(b)
            for key, w_, kn in (("in_tree_tflops_as_stored", b, True), ("in_tree_tflops_prepacked", bt_, False)):
                ms2 = time_kernel(lambda: ops.gemm(a, w_, out=c, w_kn=kn), max(5, iters // 5))
                out[name][key] = round(2.0 * m * n * k / (ms2 * 1e-3) / 1e12, 1)
                out[name][key.replace("tflops", "us")] = round(ms2 * 1e3, 2)
    return out


def in_tree_over_vendor(kernels, calib):
    """Run time of each in-tree product (with its epilogue, launched as the operator launches
    it) over the vendor library's plain product of the same shape, both timed in this run on
    this box: a figure that separates a change of the kernels from the spread between boxes.
    Below 1 the in-tree kernel is the faster one."""
    out = {}
    qkv = "gemm_qkv_bias_split"
    if not kernels[qkv]["in_layer"]:
        qkv += "_mask_rows"       # (the layer's first launch then also builds the offsets)
    for shape, kern in (("qkv", qkv), ("proj", "gemm_proj"), ("ffn1", "gemm_bias_gelu"),
                        ("ffn2", "gemm_ffn2")):
        out[shape] = round(kernels[kern]["us"] / calib[shape]["us"], 3)
    if "gemm_bias_gelu_prepacked" in kernels:
        out["ffn1_prepacked"] = round(kernels["gemm_bias_gelu_prepacked"]["us"] / calib["ffn1"]["us"], 3)
    sq = calib["square_8192"]
    out["square_8192_as_stored"] = round(sq["in_tree_us_as_stored"] / sq["us"], 3)
    out["square_8192_prepacked"] = round(sq["in_tree_us_prepacked"] / sq["us"], 3)
    return out


def vendor_compare(wl, dev, iters):
    """Counter mode (`--vendor-compare`): nothing but the FFN1 shape of the workload and
    8192^3, each through torch.matmul (the vendor library) and through the in-tree product
    (plain epilogue, weight pre-packed and as stored; FFN1 also with its bias + GELU
    epilogue), `iters` eager launches each, so that a rocprofv3 --pmc run of this command
    lists the two libraries' kernels side by side.  Prints the launch order as JSON."""
    import torch
    from bytetransformer_amd import ops
    cfg = wl.cfg
    H, F, M = cfg.hidden, cfg.ffn_mult * cfg.hidden, wl.valid_tokens
    order = []
    for name, (m, n, k) in (("ffn1", (M, F, H)), ("square_8192", (8192, 8192, 8192))):
        a = torch.empty(m, k, dtype=torch.float16, device=dev).normal_()
        b = torch.empty(k, n, dtype=torch.float16, device=dev).normal_(std=0.02)
        bias = torch.zeros(n, dtype=torch.float16, device=dev)
        c = torch.empty(m, n, dtype=torch.float16, device=dev)
        bt_ = ops.transpose_weight(b)
        runs = [("vendor torch.matmul", lambda: torch.matmul(a, b, out=c)),
                ("in-tree bt_gemm, weight [n,k]", lambda: ops.gemm(a, bt_, out=c, w_kn=False)),
                ("in-tree bt_gemm, weight [k,n]", lambda: ops.gemm(a, b, out=c, w_kn=True))]
        if name == "ffn1":
            runs.append(("in-tree bt_gemm_bias_gelu, weight [n,k]",
                         lambda: ops.gemm_bias_gelu(a, bt_, bias, out=c, w_kn=False)))
        for label, fn in runs:
            for _ in range(iters):
                fn()
            torch.cuda.synchronize()
            order.append({"shape": name, "m": m, "n": n, "k": k, "what": label, "launches": iters})
    print(json.dumps({"vendor_compare": order}))


def cpp_api_layer_ms(wl, iters=50):
    """Per-layer time of the C++ BertTransformer::infer loop without torch or Python: the
    stand-alone driver on synthetic tensors of the workload's shape and lengths (the
    reference's own timing loop, unit_test/bert_transformer_test.cc:190-202).  Runs as a
    child process; None when the driver is not built."""
    import re
    import subprocess
    import bytetransformer_amd as bt
    exe = os.path.join(bt.lib_dir(), "bert_transformer_test")
    if not os.path.exists(exe):
        return None
    cfg = wl.cfg
    cmd = [exe, str(cfg.batch), str(cfg.seq_len), str(cfg.head_num), str(cfg.head_size),
           "--synthetic", "--lens", ",".join(str(int(v)) for v in wl.lens), "--iters", str(iters)]
    try:
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                             timeout=120)
    except (OSError, subprocess.TimeoutExpired) as exc:
        print("bench: C++ driver failed (%s)" % exc, file=sys.stderr)
        return None
    m = re.search(r"layer time costs ([0-9.]+) ms", res.stdout)
    if res.returncode != 0 or not m:
        print("bench: C++ driver failed:\n%s" % res.stdout[-500:], file=sys.stderr)
        return None
    return float(m.group(1))


def oracle_forward(wl):
    """One complete forward of the CPU oracle (fp32 PyTorch restatement of the reference's
    encoder script) on the workload; returns (masked output, seconds per layer list)."""
    import numpy as np
    import torch
    from oracle import bert_oracle as O
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0")) or 10 ** 6)
    torch.set_num_threads(cores)
    x = torch.from_numpy(wl.x.astype(np.float32))
    mask = torch.from_numpy(wl.mask.astype(np.float32))
    layers32 = [{k: torch.from_numpy(np.asarray(v, np.float32)) for k, v in w.items()}
                for w in wl.layers]
    times = []
    with torch.no_grad():
        O.encoder_layer(x, mask, layers32[0], wl.cfg.head_num)       # warm-up
        h = x
        for w in layers32:
            t0 = time.perf_counter()
            h = O.encoder_layer(h, mask, w, wl.cfg.head_num)
            times.append(time.perf_counter() - t0)
    return O.masked_output(h.numpy(), wl.lens), times, cores


def measured_traffic(workload_name, kernel):
    """HBM bytes per launch of `kernel` from the committed rocprofv3 --pmc runs
    (profiles/traffic.json: FETCH_SIZE and WRITE_SIZE, each scaled by what the same
    counter reads for the 64 MiB calibration copy); None when not recorded."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f)[workload_name][kernel]["hbm_bytes_per_launch"]
    except (OSError, KeyError, ValueError):
        return None


def cpu_baseline(wl, first_pass_times, cores, target_s=10.0, budget_s=25.0):
    """The oracle's PyTorch fp32 encoder on the padded batch, all host cores.  The first
    complete forward (whose output the parity check uses) is already timed layer by layer;
    further whole layers are run until about target_s of CPU work is done (cut off at
    budget_s)."""
    import numpy as np
    import torch
    from oracle import bert_oracle as O
    torch.set_num_threads(cores)
    x = torch.from_numpy(wl.x.astype(np.float32))
    mask = torch.from_numpy(wl.mask.astype(np.float32))
    layers32 = [{k: torch.from_numpy(np.asarray(v, np.float32)) for k, v in w.items()}
                for w in wl.layers]
    done, el = len(first_pass_times), float(sum(first_pass_times))
    with torch.no_grad():
        while el < target_s:
            h = x
            for w in layers32:
                t0 = time.perf_counter()
                h = O.encoder_layer(h, mask, w, wl.cfg.head_num)
                el += time.perf_counter() - t0
                done += 1
                if el > budget_s:
                    break
            if el > budget_s:
                break
    ms_full = el / done * len(layers32) * 1e3
    return {"value": round(ms_full, 1), "unit": "ms", "cores": cores, "kind": "port",
            "sample": "%d layer passes (%.1f forwards of %d layers) of the same padded batch timed "
                      "in %.1f s, scaled to one forward; fp32 PyTorch CPU restatement of the "
                      "reference's encoder script"
                      % (done, done / len(layers32), len(layers32), el),
            "tokens_per_s": round(wl.valid_tokens / (ms_full * 1e-3), 1)}


def main():
    args = parse()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets one GPU per process; --gpus %d is not supported "
                 "(the path shards by batch with no collectives)" % args.gpus)
    import numpy as np
    import torch
    import bytetransformer_amd as bt
    from bytetransformer_amd import workload
    from oracle import bert_oracle as O

    wl = workload.make_workload(args.workload)
    cfg = wl.cfg
    # the torch-free C++ loop runs as a child process, before this process touches the GPU
    cpp_layer_ms = None if (args.no_cpp_driver or args.vendor_compare) else cpp_api_layer_ms(wl)
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    bt.load_th_op()
    if args.vendor_compare:
        vendor_compare(wl, dev, min(args.kernel_iters, 10))
        return
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    layers = [[t(w[n]) for n in workload.WEIGHT_NAMES] for w in wl.layers]
    x, mask = t(wl.x), t(wl.mask)
    op = torch.ops.ByteTransformer.BertTransformer

    def forward():
        h = x
        for w in layers:
            h = op(cfg.head_num, cfg.head_size, *w, h, mask, True, True)
        return h

    for _ in range(args.warmup):
        forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        last = forward()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # parity of what was just timed: the last timed forward's output against one complete
    # forward of the CPU oracle on the same inputs (budget of the fp16 configurations)
    expect, oracle_times, cores = oracle_forward(wl)
    got = last.cpu().numpy()
    if cfg.batch <= 2:                      # padded rows: rows past the lengths are not zeroed
        got = O.masked_output(got, wl.lens)
    mx, mean, pads_zero = O.parity_metrics(got, expect, wl.lens)
    parity = {"max_abs": float("%.4g" % mx), "mean_abs": float("%.4g" % mean),
              "pads_zero": bool(pads_zero), "tolerance": {"max_abs": 2e-2, "mean_abs": 2e-3},
              "against": "CPU oracle, one complete %d-layer forward on the same inputs" % cfg.layers}
    parity["ok"] = bool(mx <= 2e-2 and mean <= 2e-3 and pads_zero)

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return round((time.perf_counter() - t1) * 1e3 / args.steps, 4)

    # A serving loop sees a new mask tensor with every batch: the same forward with a mask
    # tensor the operator has not met before in each forward (fresh clones made outside the
    # timed region), so that whatever the operator does once per mask tensor is inside the figure.
    def fresh_mask_ms():
        n_fwd = args.warmup + args.steps
        masks = [mask.clone() for _ in range(n_fwd)]
        torch.cuda.synchronize()
        t1 = None
        for i, mk in enumerate(masks):
            if i == args.warmup:
                torch.cuda.synchronize()
                t1 = time.perf_counter()
            h = x
            for w in layers:
                h = op(cfg.head_num, cfg.head_size, *w, h, mk, True, True)
        torch.cuda.synchronize()
        return round((time.perf_counter() - t1) * 1e3 / args.steps, 4)

    fresh_ms = fresh_mask_ms()

    # the same forward through the other entry points (reported beside `value`, which
    # stays the reference's protocol: one operator call per layer)
    per_layer = [bt.BertEncoderLayer(cfg.head_num, cfg.head_size, w) for w in layers]
    whole = bt.BertEncoder(cfg.head_num, cfg.head_size, layers)
    graphed = whole.graph(cfg.batch, cfg.seq_len, valid_rows_hint=wl.valid_tokens)
    graphed.input.copy_(x)
    graphed.mask.copy_(mask)
    other = {
        "c_api_per_layer_ms": timed(lambda: bt.encoder_forward(per_layer, x, mask)),
        "whole_encoder_ms": timed(lambda: whole(x, mask, valid_rows_hint=wl.valid_tokens)),
        "whole_encoder_graph_ms": timed(graphed.replay),
    }

    # OperationType::FP32: the same batch and weights as float tensors (float kernels
    # throughout), a few steps only - reported beside the headline, never as `value`
    layers32 = [[w.float() for w in ws] for ws in layers]
    x32, mask32 = x.float(), mask.float()

    def forward32():
        h = x32
        for w in layers32:
            h = op(cfg.head_num, cfg.head_size, *w, h, mask32, True, True)
        return h

    forward32()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    n32 = max(1, min(args.steps, 10))
    for _ in range(n32):
        forward32()
    torch.cuda.synchronize()
    other["float_th_op_ms"] = round((time.perf_counter() - t1) * 1e3 / n32, 4)
    del layers32, x32, mask32

    gemm_f, attn_f = workload.layer_flops(cfg, wl.lens)
    kernels = kernel_table(wl, dev, args.kernel_iters)
    dominant = max((k for k in kernels if kernels[k]["bound"] == "mfma" and kernels[k]["in_layer"]),
                   key=lambda k: kernels[k]["us"])
    d = kernels[dominant]
    roofline = {"kernel": dominant, "bound": d["bound"], "achieved": d["achieved"],
                "peak": d["peak"], "unit": d["unit"], "frac": d["frac"],
                "traffic": measured_traffic(args.workload, dominant),
                "traffic_source": "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                  "runs of this command, not measured in this run)",
                "launch_us": d["us"]}
    pub = PUBLISHED_A100_MS.get(args.workload)
    calib = hipblaslt_calibration(wl, dev, args.kernel_iters)
    line = {
        "metric": "ms per %d-layer BERT fwd, bs%d, avg len 0.6*max (valid-token throughput alongside)"
                  % (cfg.layers, cfg.batch),
        "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": round(ms / pub, 4) if pub else None,
        "dtype": "fp16", "data": "synthetic",
        "config": {"workload": "%s: %d-layer encoder, hidden %d, heads %d, fp16, batch %d, max seq %d, "
                               "lens uniform [%d, %d], %d valid tokens, via torch.ops per layer"
                               % (cfg.name, cfg.layers, cfg.hidden, cfg.head_num, cfg.batch,
                                  cfg.seq_len, int(wl.lens.min()), int(wl.lens.max()),
                                  wl.valid_tokens),
                   "valid_tokens": wl.valid_tokens, "lens": wl.lens.tolist()},
        "tokens_per_s": round(wl.valid_tokens / (ms * 1e-3), 1),
        "model_tflops": round(cfg.layers * (gemm_f + attn_f) / (ms * 1e-3) / 1e12, 2),
        "roofline": roofline,
        "parity": parity,
        "fresh_mask_ms": fresh_ms,
        "other_entry_points": other,
        "cpp_api_layer_ms": cpp_layer_ms,
        "hipblaslt_calibration": calib,
        "in_tree_over_vendor": in_tree_over_vendor(kernels, calib),
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(wl, oracle_times, cores)
    print(json.dumps(line))
    if not parity["ok"]:
        sys.exit("bench.py: the timed operator's output is outside the parity budget: %s" % parity)


if __name__ == "__main__":
    main()
