"""The benchmark sweeps (bench.py --sweep, kraken_amd/_logging/sweep.py) on one or two tiny shapes
each: the table the reference's benchmark/benchmark_*.py print (one column per backend, speed-up
over the first backend, best backend; benchmark/benchmark_all_reduce.py:140-193), the CSV, and the
cross-check of every backend against the first one, which runs inside run_sweep."""
import csv

import pytest
import torch

from kraken_amd._logging import sweep

pytestmark = pytest.mark.gpu

CASES = {
    "all_reduce": ([4096, 1 << 16], ["hip_1shot", "hip_2shot", "torch"]),
    "all_reduce_bias": ([(1, 5120), (16, 5120)], ["hip_1shot", "hip_2shot", "torch"]),
    "all_reduce_bias_rms_norm": ([(1, 5120), (16, 8192)], ["hip_fused", "hip_unfused", "torch"]),
    "matmul_reduce_scatter": ([(128, 256, 512), (256, 512, 256)], ["hip", "hip_ce", "torch"]),
    "all_gather_matmul": ([(32, 256, 512), (128, 384, 256)], ["hip", "hip_overlap", "torch"]),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_sweep_table_csv_and_cross_check(dev, tmp_path, capsys, monkeypatch, name):
    shapes, backends = CASES[name]
    assert set(sweep.SWEEPS) == set(CASES)
    checked = []
    real = torch.testing.assert_close

    def counting(got, want, **kw):
        checked.append(kw)
        return real(got, want, **kw)

    monkeypatch.setattr(torch.testing, "assert_close", counting)
    out = tmp_path / f"{name}.csv"
    rows = sweep.run_sweep(name, None, shapes, 8, str(out), iters=3, dev=dev)
    assert len(checked) == len(shapes) * len(backends)          # every backend against the first, every shape
    assert len(rows) == len(shapes)
    speedup = f"Speedup over {backends[0]}"
    for row in rows:
        assert list(row) == ["shape", "dtype", "world_size", *backends, speedup, "Best Backend"]
        assert row["Best Backend"] in backends and row["world_size"] == 8 and row["dtype"] == "bfloat16"
        assert all(0.5 < row[b] < 1e5 for b in backends)        # microseconds
        assert row[speedup] == pytest.approx(row[backends[0]] / min(row[b] for b in backends))
        assert row[speedup] >= 1.0
    printed = capsys.readouterr().out
    assert speedup in printed and "Best Backend" in printed and f"Results saved to {out}" in printed
    with open(out, newline="") as f:
        saved = list(csv.DictReader(f))
    assert [r["shape"] for r in saved] == [r["shape"] for r in rows]
    assert saved[0].keys() == rows[0].keys()
    # a backend subset in another order: the first one given is the baseline
    rows2 = sweep.run_sweep(name, [backends[2], backends[0]], shapes[:1], 8, None, iters=2, dev=dev)
    assert f"Speedup over {backends[2]}" in rows2[0] and backends[1] not in rows2[0]
    with pytest.raises(ValueError):
        sweep.run_sweep(name, ["no_such_backend"], shapes[:1], 8, None, iters=1, dev=dev)
