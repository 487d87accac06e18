"""Writes one layer's tensors in the reference's text-fixture format (one "%f"
per line, flattened row-major, fp32 text; file names of
unit_test/python_scripts/bert_transformer_test.py:170-181) for the C++ driver
bytetransformer_amd/lib/bert_transformer_test.  The expected output comes from
the CPU oracle on the fp16-rounded tensors and is multiplied by the row mask.

    python tests/export_text_fixtures.py OUT_DIR [batch seq heads] [--seed N]
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from bytetransformer_amd import workload  # noqa: E402
from oracle import bert_oracle as O  # noqa: E402

FILES = {n: n + ".in" for n in workload.WEIGHT_NAMES}


def export(out_dir, batch=4, seq=48, heads=2, seed=5, lens=None):
    os.makedirs(out_dir, exist_ok=True)
    cfg = workload.EncoderConfig("txt", batch, seq, heads, layers=1, seed=seed,
                                 lens=tuple(lens) if lens is not None else ())
    wl = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    w32 = {k: np.asarray(v, np.float32) for k, v in wl.layers[0].items()}
    exp = O.masked_output(
        O.encoder_layer(wl.x.astype(np.float32), wl.mask.astype(np.float32), w32, heads).numpy(),
        wl.lens)

    def save(name, arr):
        # "%f" keeps six decimals, like the reference's np.savetxt call
        np.savetxt(os.path.join(out_dir, name), np.asarray(arr, np.float32).ravel(),
                   delimiter="\n", fmt="%f")

    for n in workload.WEIGHT_NAMES:
        save(FILES[n], wl.layers[0][n])
    save("from_tensor.in", wl.x)
    save("atten_mask.in", wl.mask)
    save("transformer_out.out", exp)
    return wl


if __name__ == "__main__":
    args = [a for a in sys.argv[1:] if not a.startswith("--")]
    seed = int(sys.argv[sys.argv.index("--seed") + 1]) if "--seed" in sys.argv else 5
    out = args[0]
    b, s, h = (int(v) for v in args[1:4]) if len(args) >= 4 else (4, 48, 2)
    wl = export(out, b, s, h, seed)
    print("wrote fixtures for batch %d seq %d heads %d lens %s to %s" % (b, s, h, wl.lens.tolist(), out))
