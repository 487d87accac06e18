"""Writes the golden fixtures under tests/golden/ with the CPU oracle:

  cfg0_out.npy             masked output of the stated single-layer fp32
                           configuration (B2, S64, lens [64, 38], seed 0),
                           CUDA-kernel conventions (eps 1e-6, tanh GELU,
                           softmax +1e-6)
  workload_checksums.npz   sums / lengths that pin the seeded generator
  small_fp16_case.npz      a tiny fp16 layer (inputs, 12 weights, expected
                           output) for the GPU parity test

The reference ships no golden vectors of its own (its *.in / *.out files are
git-ignored), so these come from the restated oracle, which tests/test_oracle.py
pins independently.  Run from the repo root: python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from bytetransformer_amd import workload  # noqa: E402
from oracle import bert_oracle as O  # noqa: E402


def main():
    wl = workload.make_workload("cfg0")
    out = O.masked_output(O.encoder_layer(wl.x, wl.mask, wl.layers[0], 12).numpy(), wl.lens)
    np.save(os.path.join(HERE, "cfg0_out.npy"), out.astype(np.float32))
    np.savez(os.path.join(HERE, "workload_checksums.npz"),
             cfg0_x_sum=wl.x.astype(np.float64).sum(),
             cfg2_lens=workload.draw_lengths(workload.CONFIGS["cfg2"]),
             cfg3_lens=workload.draw_lengths(workload.CONFIGS["cfg3"]),
             cfg4_lens=workload.draw_lengths(workload.CONFIGS["cfg4"]))

    cfg = workload.EncoderConfig("small", 3, 48, 2, layers=1, dtype="fp16", lens=(48, 17, 30),
                                 seed=11)
    ws = workload.make_workload(cfg, bias_std=0.05, random_affine=True)
    w32 = {k: v.astype(np.float32) for k, v in ws.layers[0].items()}
    exp = O.masked_output(
        O.encoder_layer(ws.x.astype(np.float32), ws.mask.astype(np.float32), w32, 2).numpy(),
        ws.lens)
    np.savez_compressed(os.path.join(HERE, "small_fp16_case.npz"), x=ws.x, lens=ws.lens,
                        expected=exp.astype(np.float32), **ws.layers[0])
    print("wrote golden fixtures")


if __name__ == "__main__":
    main()
