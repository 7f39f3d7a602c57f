"""The benchmark's JSON record: one line, small enough for the tail of standard
output a harness keeps, complete enough to recompute every roofline fraction."""

import io
import json

import bench


def _fake_results():
    """Results shaped like bench.run()'s, one per benchmark workload, with the
    longest texts a real run produces."""
    out = []
    for name, wl in bench.workloads().items():
        hbm = wl["kind"] == "rowwise"
        work = 268443648 if hbm else 1099511627776.0
        kernel_us = 43.31805706 if hbm else 833.97712
        peak = bench.HBM_PEAK_GBS if hbm else bench.MFMA_PEAK_TFLOPS
        achieved = work / (kernel_us * 1e-6) / (1e9 if hbm else 1e12)
        rf = {"bound": "hbm" if hbm else "mfma", "achieved": achieved, "peak": peak,
              "unit": "GB/s" if hbm else "TFLOP/s", "frac": achieved / peak, "traffic": 1755325842,
              "kernel_us": kernel_us}
        rf["algorithmic_bytes" if hbm else "algorithmic_flops"] = work
        if hbm:
            rf.update(kernel_us_same_buffers=42.3475646, buffer_sets=4)
        out.append({
            "workload": name, "metric": "FlashAttention fwd fp16 B4 H16 S4096 D128 causal TFLOPS",
            "value": achieved * 0.99, "unit": rf["unit"], "ms_per_step": kernel_us * 1.01e-3,
            "dtype": "f16 in/out, f32 accumulate", "config": str(wl["cfg"]), "roofline": rf,
            "cpu_baseline": {
                "value": 1.8545226833797817, "unit": rf["unit"], "cores": 16, "kind": "port",
                "sample": "torch a_cpu.float() @ b_cpu.float() on the first 2980 of 8192 rows "
                          "of A (all of B), 1 warm-up, median of 19",
                "seconds": 0.21567211500000383, "native_matmul_value": 0.001936248033676745,
                "native_matmul_sample": "a_cpu[:8] @ b_cpu[:, :512] in float16, single run",
                "host_cpus": 16}})
    return out


def test_record_is_one_short_line_with_every_workload():
    results = _fake_results()
    assert len(results) == 13
    rec = bench.build_record(results, 20, 5)
    line = json.dumps(rec, separators=(",", ":"))
    assert "\n" not in line
    assert len(line) < bench.MAX_RECORD_BYTES, len(line)
    back = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "roofline", "cpu_baseline"):
        assert key in back
    assert "results" not in back
    assert back["config"]["workload"] == bench.DEFAULT_WORKLOAD
    assert set(back["roofline"]["all"]) == set(bench.workloads())
    assert set(back["cpu_baseline"]["all"]) == set(bench.workloads())
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in back["cpu_baseline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in back["roofline"]
    # every fraction follows from the record alone
    for name, row in back["roofline"]["all"].items():
        scale = 1e9 if row["unit"] == "GB/s" else 1e12
        frac = row["work"] / (row["kernel_us"] * 1e-6) / scale / row["peak"]
        assert abs(frac - row["frac"]) < 2e-3 * row["frac"], name
    gated = set(back["config"]["targets_met"]) | set(back["config"]["targets_missed"])
    assert gated == set(bench.TARGET_FRAC)


def test_table_goes_out_before_the_record(monkeypatch, capsys):
    """main() prints the per-workload table on stderr and the JSON line last on
    stdout (nothing after it on either stream)."""
    results = _fake_results()
    order = []

    class Tap(io.StringIO):
        def __init__(self, name):
            super().__init__()
            self.name_ = name

        def write(self, s):
            if s.strip():
                order.append(self.name_)
            return super().write(s)

    err, out = Tap("err"), Tap("out")
    it = iter(results)
    monkeypatch.setattr(bench, "run", lambda *a, **k: next(it))
    monkeypatch.setattr("sys.stderr", err)
    monkeypatch.setattr("sys.stdout", out)
    monkeypatch.setattr("sys.argv", ["bench.py", "--full-out", ""])
    import torch

    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    bench.main()
    lines = [l for l in out.getvalue().splitlines() if l.strip()]
    assert len(lines) == 1
    assert json.loads(lines[0])["roofline"]["all"]
    assert order[-1] == "out" and "out" not in order[:-1]
    assert "rmsnorm_bf16_16384x4096" in err.getvalue()
