"""Measures every fp16 GEMM tile shape of libbt_hip.so over a grid of row counts for
the four weight shapes of BERT-base and BERT-large, in both weight layouts ([k, n] as
stored and the [n, k] pre-pack) and both launch shapes (a padded batch of which 60 % of the
rows are live, and a launch whose rows are all live), and writes the table the launcher consults (csrc/kernels/gemm_tuned.inc; rebuild the kernels afterwards).

    python -m bytetransformer_amd.tune_gemm [--json timings.json] [--from-json run1.json run2.json ...]

Needs a GPU unless --from-json replays earlier measurements; several runs (ideally from
several machines) are merged by the upper quartile of each entry.  Shapes outside the table
keep using the launcher's analytic cost model."""
import argparse
import json
import os
import sys

M_STEP = 256                     # the tallest tile: run time steps with the count of row tiles
M_GRID = tuple(range(M_STEP, 16384 + 1, M_STEP))
HIDDEN = (768, 1024)
TILES = (0, 1, 2, 3, 4, 5, 6, 7, 8)
EPI_CODE = {"plain": 0, "gelu": 1, "qkv": 2}     # enum Epilogue of gemm.hip
SMALL_TILE_MAX_ROWS = 3000      # the 32x64 tile is not worth timing beyond this
INC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "kernels", "gemm_tuned.inc")


def _time_kernel(fn, iters):
    """GPU time per launch (us): the launches are captured into a HIP graph and one replay
    is bracketed by events, so host call overhead is excluded."""
    import torch
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(iters):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    beg.record()
    graph.replay()
    end.record()
    end.synchronize()
    return beg.elapsed_time(end) / iters * 1e3


def measure(iters=32):
    """Each weight shape as the layer launches it: with its epilogue (QKV: bias + head
    split, FFN1: bias + GELU, the two others plain), with a row capacity of m / 0.6 (the
    padded batch: launches are sized for batch x seq_len rows, of which m are live) and with
    a row capacity of m (every row live: the padded path, or a caller that sizes its launches
    for the live rows), the
    QKV product gathering its rows from the padded input through a word_idx of 16 runs, and
    with the weights cold: the launches of one timing loop walk through enough copies of
    the weight matrix to exceed the memory-side cache, as the layers of a model do.  Every
    shape is timed with the weight in both layouts."""
    import torch
    from . import ops
    dev = torch.device("cuda:0")
    cap_of = lambda m: (int(m / 0.6) + 255) // 256 * 256
    rows_cap = cap_of(max(M_GRID))
    out = []
    try:
        for h in HIDDEN:
            heads = h // 64
            for epi, n, k in (("qkv", 3 * h, h), ("plain", h, h), ("gelu", 4 * h, h),
                              ("plain", h, 4 * h)):
                a = torch.randn(rows_cap, k, device=dev).half()
                copies = min(iters, max(2, -(-300 * 2 ** 20 // (n * k * 2))))
                ws = [(torch.randn(k, n, device=dev) * 0.02).half() for _ in range(copies)]
                wts = [ops.transpose_weight(w) for w in ws]
                bias = torch.zeros(n, device=dev, dtype=torch.float16)
                c = torch.empty(rows_cap * n, device=dev, dtype=torch.float16)
                for m, full in [(m, f) for m in M_GRID for f in (0, 1)]:
                    vr = torch.tensor([m], dtype=torch.int32, device=dev)
                    turn = [0]
                    cap = m if full else cap_of(m)
                    # 16 sequences of cap / 16 padded rows each, m / 16 of them valid
                    runs = [torch.arange(b * (cap // 16), b * (cap // 16) + (m * (b + 1)) // 16
                                         - (m * b) // 16, dtype=torch.int32) for b in range(16)]
                    word_idx = torch.cat(runs + [torch.zeros(cap - m, dtype=torch.int32)]).to(dev)

                    kn = [False]

                    def call():
                        wt = (ws if kn[0] else wts)[turn[0] % copies]
                        turn[0] += 1
                        if epi == "qkv":
                            ops.gemm_qkv_bias_split(a[:cap], wt, bias, heads, valid_rows=vr,
                                                    rows_hint=m, a_row_index=word_idx, w_kn=kn[0],
                                                    out=c[:3 * cap * k].view(3, heads, cap, 64))
                        elif epi == "gelu":
                            ops.gemm_bias_gelu(a[:cap], wt, bias, valid_rows=vr, rows_hint=m,
                                               out=c[:cap * n].view(cap, n), w_kn=kn[0])
                        else:
                            ops.gemm(a[:cap], wt, valid_rows=vr, rows_hint=m,
                                     out=c[:cap * n].view(cap, n), w_kn=kn[0])

                    ops.set_option("gemm_tile", 1)
                    _time_kernel(call, 8)      # warm the clocks for this shape
                    for layout in (0, 1):
                        kn[0] = bool(layout)
                        us = {}
                        for tile in TILES:
                            if tile == 4 and m > SMALL_TILE_MAX_ROWS:
                                continue
                            ops.set_option("gemm_tile", tile)
                            us[str(tile)] = round(_time_kernel(call, iters), 2)
                        row = {"M": m, "N": n, "K": k, "epi": epi, "kn": layout, "full": full,
                               "us": us}
                        out.append(row)
                        print(json.dumps(row), flush=True)
    finally:
        ops.set_option("gemm_tile", -1)
    return out


def merge_runs(rows):
    """One row per (shape, layout, row count): every tile's time at the upper quartile of the
    runs that measured it (the second-largest of five).  Boxes differ - the tiles with
    dedicated loader waves by up to +-15 % from box to box where the 256 x 256 tile moves
    +-2 %, and one of five runs here had every loader-wave tile 20-30 % slower than the others
    - so a tile that is fast on most boxes and slow on some is priced at its slow side, and a
    table from one box alone would inherit that box's quirks."""
    import math
    seen = {}
    for r in rows:
        key = (r["M"], r["N"], r["K"], r.get("epi", "plain"), r.get("kn", 0), r.get("full", 0))
        for tile, us in r["us"].items():
            seen.setdefault(key, {}).setdefault(tile, []).append(us)
    pick = lambda v: sorted(v)[math.ceil(0.75 * (len(v) - 1))]
    return [{"M": m, "N": n, "K": k, "epi": epi, "kn": kn, "full": full,
             "us": {t: round(pick(v), 2) for t, v in by_tile.items()}}
            for (m, n, k, epi, kn, full), by_tile in seen.items()]


def write_inc(rows, path=INC):
    shapes = {}
    for r in merge_runs(rows):
        shapes.setdefault((r["N"], r["K"], EPI_CODE[r.get("epi", "plain")], r.get("kn", 0),
                           r.get("full", 0)), {})[r["M"]] = r["us"]
    lines = ["// Generated by `python -m bytetransformer_amd.tune_gemm` from timings on one MI355X:",
             "// microseconds per launch of each tile shape (index = tile id; 0 = not measured)",
             "// at kTunedRows live rows, per weight shape, weight layout and launch shape (full = 1:",
             "// every row of the launch live; 0: a padded batch with 60 % live rows).  Do not edit by hand.",
             "constexpr int kTunedPoints = %d;" % len(M_GRID),
             "constexpr int kTunedTiles = %d;" % len(TILES),
             "constexpr int kTunedStep = %d;" % M_STEP,
             "static const int kTunedRows[kTunedPoints] = {%s};" % ", ".join(map(str, M_GRID)),
             "struct TunedShape {",
             "  int n, k, epi, kn, full;   // epi: the Epilogue the shape was timed with; kn: 1 = [k, n] weight",
             "  float us[kTunedPoints][kTunedTiles];", "};",
             "static const TunedShape kTunedShapes[] = {"]
    for (n, k, epi, kn, full), by_m in sorted(shapes.items()):
        lines.append("    {%d, %d, %d, %d, %d, {" % (n, k, epi, kn, full))
        for m in M_GRID:
            us = by_m.get(m, {})
            lines.append("        {%s},   // %d rows" % (
                ", ".join("%.2ff" % us.get(str(t), 0.0) for t in TILES), m))
        lines.append("    }},")
    lines.append("};")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")
    return path


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--json", help="also save the raw timings here")
    ap.add_argument("--from-json", nargs="+", help="build the table from saved timings instead")
    args = ap.parse_args()
    if args.from_json:
        rows = []
        for p in args.from_json:
            rows += json.load(open(p))
    else:
        rows = measure()
    if args.json:
        json.dump(rows, open(args.json, "w"))
    print("wrote", write_inc(rows), file=sys.stderr)


if __name__ == "__main__":
    main()
