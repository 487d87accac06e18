"""The GEMM tuner's table writer (host logic; the timing itself needs a GPU)."""
import os
import re

from bytetransformer_amd import tune_gemm


def test_table_writer_lays_rows_out_by_row_count_and_tile(tmp_path):
    rows = [{"M": m, "N": 2304, "K": 768, "epi": "qkv", "kn": 1, "full": 0,
             "us": {str(t): float(m + t) for t in tune_gemm.TILES if t != 4}}
            for m in tune_gemm.M_GRID[:3]]
    path = tune_gemm.write_inc(rows, str(tmp_path / "t.inc"))
    text = open(path).read()
    assert "kTunedPoints = %d;" % len(tune_gemm.M_GRID) in text
    assert "kTunedTiles = %d;" % len(tune_gemm.TILES) in text
    assert "kTunedStep = %d;" % tune_gemm.M_STEP in text
    assert "{2304, 768, %d, 1, 0, {" % tune_gemm.EPI_CODE["qkv"] in text
    body = [l for l in text.splitlines() if l.strip().startswith("{") and "rows" in l]
    assert len(body) == len(tune_gemm.M_GRID)
    first = [float(v) for v in re.findall(r"([0-9.]+)f", body[0])]
    m0 = tune_gemm.M_GRID[0]
    assert first == [0.0 if t == 4 else float(m0 + t) for t in tune_gemm.TILES]
    # row counts that were not measured stay at 0 = "not measured"
    assert set(re.findall(r"([0-9.]+)f", body[-1])) == {"0.00"}


def test_committed_table_matches_the_tuner_grid():
    text = open(tune_gemm.INC).read()
    assert "kTunedPoints = %d;" % len(tune_gemm.M_GRID) in text
    assert "kTunedTiles = %d;" % len(tune_gemm.TILES) in text
    rows = re.search(r"kTunedRows\[kTunedPoints\] = \{([^}]*)\}", text).group(1)
    assert tuple(int(v) for v in rows.split(",")) == tune_gemm.M_GRID
    assert os.path.getsize(tune_gemm.INC) < 256 * 1024


def test_runs_are_merged_by_the_upper_quartile_of_each_entry():
    mk = lambda us: {"M": 256, "N": 768, "K": 768, "epi": "plain", "kn": 0, "us": us}
    five = [mk({"0": v, "1": 5.0}) for v in (10.0, 30.0, 11.0, 12.0, 9.0)] + [mk({"1": 7.0})]
    merged = tune_gemm.merge_runs(five)
    # tile 0: second-largest of five; tile 1: six values, index ceil(0.75 * 5) = 4
    assert len(merged) == 1 and merged[0]["us"] == {"0": 12.0, "1": 5.0}
    assert tune_gemm.merge_runs([mk({"0": 3.0})])[0]["us"] == {"0": 3.0}
