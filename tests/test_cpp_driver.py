"""The stand-alone C++ driver and the reference's text-fixture format."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

import bytetransformer_amd as bt

sys.path.insert(0, os.path.dirname(__file__))
import export_text_fixtures as X  # noqa: E402

DRIVER = os.path.join(bt.lib_dir(), "bert_transformer_test")


def test_driver_is_built_and_prints_usage():
    assert os.path.exists(DRIVER), "run python -m bytetransformer_amd.build"
    out = subprocess.run([DRIVER], stdout=subprocess.PIPE, text=True, timeout=60)
    assert out.returncode == 0 and "<batch_size> <seq_len> <head_num> <size_per_head>" in out.stdout


def test_text_fixture_format(tmp_path):
    wl = X.export(str(tmp_path), batch=3, seq=8, heads=1, seed=2, lens=(8, 3, 5))
    names = sorted(os.listdir(tmp_path))
    assert len(names) == 15 and "transformer_out.out" in names and "atten_mask.in" in names
    x = np.loadtxt(tmp_path / "from_tensor.in", dtype=np.float32)
    assert x.shape == (3 * 8 * 64,)
    # six decimals of an fp16 value: within 5e-7 absolute
    assert np.abs(x - wl.x.astype(np.float32).ravel()).max() <= 5.1e-7
    first = open(tmp_path / "qkv_kernel.in").readline().strip()
    assert re.fullmatch(r"-?\d+\.\d{6}", first)
    mask = np.loadtxt(tmp_path / "atten_mask.in").reshape(3, 8, 8)
    assert mask[:, 0, :].sum(axis=1).tolist() == [8, 3, 5]
    out = np.loadtxt(tmp_path / "transformer_out.out").reshape(3, 8, 64)
    assert np.all(out[1, 3:] == 0) and np.any(out[1, :3] != 0)


@pytest.mark.gpu
@pytest.mark.parametrize("batch,seq,heads,extra", [(4, 48, 2, []), (2, 40, 2, []),
                                                   (5, 100, 4, ["--no-fused"]),
                                                   (4, 48, 2, ["--fp32"]), (2, 40, 2, ["--fp32"])])
def test_cpp_driver_matches_exported_expectation(device, tmp_path, batch, seq, heads, extra):
    print("cpp driver", batch, seq, heads, extra, flush=True)
    X.export(str(tmp_path), batch=batch, seq=seq, heads=heads, seed=batch)
    # float: the fixtures hold six decimals of each value, the float layer itself is good to 2e-4
    tol = "0.0005" if "--fp32" in extra else "0.02"
    cmd = [DRIVER, str(batch), str(seq), str(heads), "64", "--data", str(tmp_path), "--iters", "5",
           "--tol", tol] + extra
    out = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                         timeout=120)
    print(out.stdout[-600:], flush=True)
    assert out.returncode == 0, out.stdout[-2000:]
    m = re.search(r"max_diff ([0-9.]+)", out.stdout)
    assert m and float(m.group(1)) <= float(tol)
    assert "layer time costs" in out.stdout
