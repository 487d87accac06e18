"""Latency sweep of the PyTorch operator over batch sizes and sequence lengths:
the measurement the reference makes with benchmark/bert_bench.sh:21-57 +
unit_test/python_scripts/bert_transformer_test.py:183-208 (12 layers, 12 heads x
64, fp16, average length 60 % of the maximum, 5 warm-up + N timed iterations,
one operator call per layer).

    python -m bytetransformer_amd.bert_bench [--batch-sizes 1 16] [--seqlens 64 512] [--iters 100]

Prints the reference's table (Batch Size, Seqlen, Precision, BT Latency) with the
published A100 ByteTransformer latency beside it where the reference's README
has one.
"""
import argparse
import time

import numpy as np
import torch

from . import load_th_op, workload

# ByteTransformer column of the reference's README tables (A100, ms): README.md:34-49,56-71
PUBLISHED_A100 = {
    1: {64: 0.90, 128: 0.97, 192: 1.36, 256: 1.43, 320: 1.69, 384: 1.72, 448: 1.86, 512: 2.00,
        576: 2.19, 640: 2.23, 704: 2.47, 768: 2.51, 832: 2.80, 896: 2.86, 960: 3.12, 1024: 3.16},
    16: {64: 2.09, 128: 3.18, 192: 5.08, 256: 6.85, 320: 7.49, 384: 8.44, 448: 8.89, 512: 9.22,
         576: 10.15, 640: 12.04, 704: 13.55, 768: 16.3, 832: 16.92, 896: 20.67, 960: 23.27,
         1024: 24.70},
}


def run_case(batch, seqlen, n_layers, head_num, head_size, avg_percent, iters, dev):
    avg = seqlen * avg_percent // 100
    low = max(2 * avg - seqlen, 0)
    rs = np.random.RandomState(seqlen * 131 + batch)
    lens = rs.randint(low, seqlen + 1, size=batch)           # the reference's length draw
    cfg = workload.EncoderConfig("sweep", batch, seqlen, head_num, head_size, layers=n_layers,
                                 lens=tuple(int(v) for v in lens))
    wl = workload.make_workload(cfg)

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    layers = [[t(w[n]) for n in workload.WEIGHT_NAMES] for w in wl.layers]
    x, mask = t(wl.x), t(wl.mask)
    op = torch.ops.ByteTransformer.BertTransformer
    for i in range(5 + iters):
        if i == 5:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        h = x
        for w in layers:
            h = op(head_num, head_size, *w, h, mask, True, True)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / iters, int(lens.sum())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch-sizes", type=int, nargs="+", default=[1, 2, 4, 8, 16])
    ap.add_argument("--seqlens", type=int, nargs="+",
                    default=[32, 64, 128, 192, 256, 320, 384, 448, 512, 576, 640, 704, 768, 832,
                             896, 960, 1024])
    ap.add_argument("--n-layers", type=int, default=12)
    ap.add_argument("--head-num", type=int, default=12)
    ap.add_argument("--head-size", type=int, default=64)
    ap.add_argument("--avg-seqlen-percent", type=int, default=60)
    ap.add_argument("--iters", type=int, default=100)
    args = ap.parse_args()
    load_th_op()
    dev = torch.device("cuda:0")
    print("%-12s%-10s%-11s%-18s%-14s%-16s" % ("Batch Size", "Seqlen", "Precision",
                                              "BT Latency (ms)", "valid tokens",
                                              "A100 published"), flush=True)
    for b in args.batch_sizes:
        for s in args.seqlens:
            ms, tokens = run_case(b, s, args.n_layers, args.head_num, args.head_size,
                                  args.avg_seqlen_percent, args.iters, dev)
            pub = PUBLISHED_A100.get(b, {}).get(s)
            print("%-12d%-10d%-11s%-18.3f%-14d%-16s" % (b, s, "fp16", ms, tokens,
                                                        "%.2f" % pub if pub else "-"), flush=True)


if __name__ == "__main__":
    main()
