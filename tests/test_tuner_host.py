"""Host tests of the tuning driver pieces that need no GPU: parallel compile
with worker failure, record formats, GPU detection, argument parsing."""

import os
import re
import sys

import pytest

from deca_amd import Tuner as tuner_mod
from deca_amd.arch import MI355X
from deca_amd.kernels.rowwise_hip import RowConfig
from deca_amd.utils.helper import GPUDetector, byte_size

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- builders used by the worker pool (must be importable from a spawned process)
def _ok_builder(tag, path):
    with open(path, "w") as f:
        f.write(tag)
    return path


def _dying_builder(tag, path):
    import multiprocessing

    if tag == "dies" and multiprocessing.current_process().name != "MainProcess":
        os._exit(3)  # kills the pool worker: the pool breaks
    return _ok_builder(tag, path)


def _failing_builder(tag, path):
    if tag == "bad":
        raise RuntimeError("hipcc failed: synthetic error")
    return _ok_builder(tag, path)


def test_build_all_parallel_and_failed_config_is_dropped(capsys):
    args = {tag: (lambda t: lambda path: (t, path))(tag) for tag in ("a", "bad", "c")}
    paths = tuner_mod.build_all("test_tuner_host:_failing_builder", args, jobs=2)
    assert sorted(paths) == ["a", "c"]
    assert all(open(p).read() == t for t, p in paths.items())
    assert "bad failed to build" in capsys.readouterr().out


def test_build_all_survives_a_dead_worker():
    """A worker that dies breaks the pool; the affected configs are rebuilt
    serially in this process (where the builder does not die)."""
    args = {tag: (lambda t: lambda path: (t, path))(tag) for tag in ("x", "dies", "y")}
    paths = tuner_mod.build_all("test_tuner_host:_dying_builder", args, jobs=2)
    assert sorted(paths) == ["dies", "x", "y"]
    assert open(paths["dies"]).read() == "dies"


def test_build_all_serial_when_one_job():
    args = {"only": lambda path: ("only", path)}
    assert list(tuner_mod.build_all("test_tuner_host:_ok_builder", args, jobs=1)) == ["only"]


class _FakeRowOp:
    num_bytes = 268435456

    def describe(self):
        return "Softmax(M=16384, N=4096, float16)"


class _FakeGemmOp:
    num_flops = 2 * 8192**3

    def describe(self):
        return "GEMMTC(M=8192, N=8192, K=8192, float16)"


def test_rowwise_record_format():
    t = tuner_mod.Tuner("softmax", arch=MI355X(), arch_str="gfx950")
    msg, best, ref = t._report(_FakeRowOp(), RowConfig(256, 2, 8, hint=True), 3, 24, 42e-6, 84e-6,
                               1.2e-4, 7.5, 31.0)
    lines = msg.splitlines()
    assert re.fullmatch(r"\d{4}-\d\d-\d\d \d\d:\d\d:\d\d \[AMD Instinct MI355X\]", lines[0])
    assert lines[1] == (" DeCA Softmax(M=16384, N=4096, float16), config: "
                        "tpr=256,rpb=2,vec=8,mode=reg,hint=1 (cost-model rank 3/24)")
    assert re.fullmatch(r" throughput: 6391\.3 GB/s \(80% of DRAM peak\), runtime: 0\.0420 ms, "
                        r"max err: 1\.20e-04", lines[2])
    assert re.fullmatch(r" torch: 3195\.7 GB/s, runtime: 0\.0840 ms, ratio: 2\.000", lines[3])
    assert lines[4] == " compile time: 7.5 s, total tuning time: 31.0 s"
    assert best == pytest.approx(6391.3, abs=0.1) and ref == pytest.approx(3195.7, abs=0.1)


def test_gemm_record_format():
    t = tuner_mod.Tuner("GEMM", arch=MI355X(), arch_str="gfx950")
    msg, best, _ = t._report(_FakeGemmOp(), "256x256x64,warp=128x64,stages=2,raster=4,epi_smem=0",
                             1, 24, 0.9e-3, 1.0e-3, 2.4e-4, 20.0, 60.0)
    assert "throughput: 1221.7 TFLOPS (49% of fp32-acc MFMA peak)" in msg
    assert "torch: 1099.5 TFLOPS, runtime: 1.0000 ms, ratio: 1.111" in msg
    assert best == pytest.approx(1221.7, abs=0.1)


def test_tuner_rejects_unknown_operator():
    with pytest.raises(AssertionError):
        tuner_mod.Tuner("conv2d", arch=MI355X())


def test_gpu_lookup_and_detection_failure(capsys):
    assert GPUDetector.lookup("AMD Radeon Graphics", "gfx950:sramecc+:xnack-") is MI355X
    assert GPUDetector.lookup("AMD Instinct MI355X", "") is MI355X
    with pytest.raises(NotImplementedError):
        GPUDetector.lookup("NVIDIA H20", "sm_90")
    assert byte_size("float16") == 2 and byte_size("float32") == 4
    with pytest.raises(ValueError):
        byte_size("int8")

    class _NoDevice(GPUDetector):
        @classmethod
        def _device_info(cls, device_id=0):
            raise RuntimeError("no HIP device is visible")

    with pytest.raises(SystemExit) as e:
        _NoDevice.detect_gpu(verbose=True)
    assert e.value.code == -1
    assert "GPU detection failed" in capsys.readouterr().out


def test_arch_configure_device():
    class Info:
        name, gcn_arch = "", "gfx950:sramecc+:xnack-"
        cu_count, clock_khz, lds_per_block, total_mem = 128, 2000000, 65536, 64 * 2**30

    a = MI355X().configure_device(Info)
    assert a.name == "AMD Instinct MI355X" and a.gcn_arch == "gfx950"
    assert a.sm_nums == 128 and a.sm_clock_hz == 2.0e9 and a.max_dyn_smem_per_block == 65536
    assert a.peak_mma_sync_flops == pytest.approx(128 * 4096 * 2.0)  # GFLOPS
    base = MI355X()
    assert base.peak_mma_sync_flops == pytest.approx(2516582, rel=1e-6) and base.dram_bw == 8000


def test_driver_argument_parsing():
    sys.path.insert(0, ROOT)
    import test_flash_attn
    import test_gemm_tc
    import test_rowwise

    a = test_rowwise.parse_args(["--op", "rmsnorm", "--dtype", "bf16", "--shape", "8192", "8192"])
    assert (a.op, a.dtype, a.shape, a.top_n, a.finalists, a.rounds) == ("rmsnorm", "bf16",
                                                                      [8192, 8192], 24, 3, 5)
    g = test_gemm_tc.parse_args(["--sweep"])
    assert g.sweep and g.shape == [4096, 4096, 4096] and g.top_n == 24
    f = test_flash_attn.parse_args(["--causal"])
    assert f.causal and f.top_n == 16 and test_flash_attn.parse_shape(f.shape) == (4, 16, 4096, 4096, 128)
    assert test_flash_attn.parse_shape([1, 2, 128, 640, 64]) == (1, 2, 128, 640, 64)


def test_sweep_csv(tmp_path):
    import test_gemm_tc

    p = tmp_path / "s.csv"
    test_gemm_tc.write_sweep_csv([((2048, 2048, 2048), "cfg", 600.0, 500.0)], str(p))
    assert p.read_text().splitlines() == ["M,N,K,DeCA_TFLOPS,torch_TFLOPS,ratio",
                                          "2048,2048,2048,600.0000,500.0000,1.2000"]


def test_runtime_mod_error_metric_and_nan():
    """The verification metric on host tensors: max |d|, the reference's
    excess ratio, and NaN outputs counted as failures."""
    import torch

    from deca_amd.RuntimeMod import RuntimeMod

    rt = RuntimeMod(_FakeRowOp(), MI355X(), False, RowConfig())
    ref = torch.tensor([[1.0, -2.0, 0.0, 4.0]])
    out = ref + torch.tensor([[0.001, 0.0, 0.0, -0.004]])
    worst, excess = rt._errors(out, ref, 1e-2, 2e-3)
    assert worst == pytest.approx(0.004, rel=1e-3)
    assert excess == pytest.approx(0.004 / (1e-2 + 2e-3 * 4), rel=1e-3)
    bad = out.clone()
    bad[0, 1] = float("nan")
    assert rt._errors(bad, ref, 1e-2, 2e-3) == (float("inf"), float("inf"))
    # 4-D attention outputs are compared through the same row-block loop
    o4 = torch.zeros(2, 3, 5, 8)
    assert rt._errors(o4 + 0.5, o4, 1.0, 0.0) == (0.5, 0.5)
    with pytest.raises(RuntimeError, match="no kernel loaded"):
        rt.time_kernel_op()
    assert rt.is_flash_attn is False
    # the reference's method names (RuntimeMod.py:53-131): the tensor-core build is the build,
    # its schedule-based legacy path says what it is not
    assert RuntimeMod.build_with_tc is RuntimeMod.build and RuntimeMod.build_flash_attn is RuntimeMod.build
    assert RuntimeMod.load_flash_attn is RuntimeMod.load_kernel
    with pytest.raises(NotImplementedError, match="GEMMTC"):
        rt.build_without_tc()
    with pytest.raises(AssertionError, match="Schedule not built"):
        rt.get_sch()


def test_tuned_table_roundtrip(tmp_path):
    from deca_amd import tuned
    from deca_amd.kernels.flash_attn_hip import FAConfig
    from deca_amd.kernels.gemm_hip import GemmConfig

    path = str(tmp_path / "t.json")
    assert tuned.lookup("softmax|16384x4096|float16|gfx950", path) is None
    k1 = tuned.make_key("softmax", (16384, 4096), "float16")
    k2 = tuned.make_key("flash_attn", (4, 16, 4096, 4096, 128), "float16", "gfx950", causal=True)
    k3 = tuned.make_key("GEMM", (8192, 8192, 8192), "bfloat16")
    assert k1 == "softmax|16384x4096|float16|gfx950"
    assert k2 == "flash_attn|4x16x4096x4096x128|float16|causal|gfx950"
    tuned.store(k1, RowConfig(256, 2, 8, hint=True), 6391.3, "GB/s", path, runtime_ms=0.042)
    tuned.store(k2, FAConfig(256, 128, 8, 2), 800.0, "TFLOPS", path)
    tuned.store(k3, GemmConfig(256, 256, 64, 128, 64, 2, 4), 1200.0, "TFLOPS", path)
    assert tuned.lookup(k1, path) == RowConfig(256, 2, 8, hint=True)
    assert tuned.lookup(k2, path) == FAConfig(256, 128, 8, 2)
    assert tuned.lookup(k3, path) == GemmConfig(256, 256, 64, 128, 64, 2, 4)
    assert tuned.load(path)[k1]["runtime_ms"] == 0.042
    # the table shipped with the package covers every bench workload
    import bench

    assert len(bench.workloads()) == 13


def test_shipped_winners_come_from_the_tuner():
    """Every entry of the shipped table was written by `Tuner.tune` (the drivers'
    `--cache --retune`), timed back to back, after measuring a real share of the solver's
    list; the GEMM entries bench.py uses are the ones tuned on its U(-1,1) operands."""
    import bench
    from deca_amd import tuned

    table = tuned.load()
    for key, entry in table.items():
        assert entry.get("method") == "tuner", key
        assert entry.get("timing") == "back_to_back", key
        assert 1 <= entry["rank"] <= entry["candidates"] <= entry["solutions"], key
        assert entry["candidates"] >= min(16, entry["solutions"]), key
        assert entry["torch_throughput"] > 0 and entry["runtime_ms"] > 0, key
        if key.startswith("GEMM"):
            assert ("|U(-1,1)|" in key) == (entry.get("inputs") == "U(-1,1)"), key
    # bench.py finds all of its 13 workloads there (it raises on a missing key)
    assert len(bench.workloads()) == 13
    bf16 = table[tuned.make_key("GEMM", (8192, 8192, 8192), "bfloat16", "gfx950", False, "uniform")]
    # the bf16 winner was searched with the 16x16x32 and accumulation-register bodies on offer
    assert bf16["candidates"] >= 24


def test_tuner_timing_modes(monkeypatch):
    """`timing` reaches RuntimeMod, and the two procedures differ as documented: one event
    pair per call, or batches between one pair."""
    import pytest as _pytest

    from deca_amd.kernels import attn_bench as ab
    from deca_amd.operators import Softmax
    from deca_amd.RuntimeMod import RuntimeMod
    from deca_amd.Tuner import Tuner

    assert ab.TIMINGS == ("events", "back_to_back")
    assert Tuner("softmax", arch=object(), arch_str="gfx950").timing == "back_to_back"
    assert Tuner("softmax", arch=object(), arch_str="gfx950", timing="events").timing == "events"
    with _pytest.raises(AssertionError):
        Tuner("softmax", arch=object(), arch_str="gfx950", timing="wall")
    rt = RuntimeMod(Softmax(64, 128, "float16"), None, True, RowConfig(16, 4, 8), timing="back_to_back")
    assert rt.timing == "back_to_back" and RuntimeMod(rt.operator, None, True, None).timing == "events"
    # bench_back_to_back: warm-up by time, then `batches` batches sized from the settled time
    calls = []

    def timed(n):
        calls.append(n)
        return 1e-3

    monkeypatch.setattr(ab.time, "perf_counter", iter([0.0, 0.1, 0.2, 0.4, 0.5]).__next__)
    t = ab.bench_back_to_back(timed, warmup_s=0.3, measure_s=0.3, min_iters=20, batches=3)
    assert t == 1e-3 and calls[0] == 4 and calls[-3:] == [100, 100, 100]
    seen = ab.bench_interleaved_batches.__doc__
    assert "batch timers" in seen


def test_winners_are_kept_per_operand_distribution(tmp_path):
    from deca_amd import tuned
    from deca_amd.kernels.gemm_hip import GemmConfig

    n01 = tuned.make_key("GEMM", (4096, 4096, 4096), "float16")
    uni = tuned.make_key("GEMM", (4096, 4096, 4096), "float16", "gfx950", False, "uniform")
    assert n01 == "GEMM|4096x4096x4096|float16|gfx950" and uni == "GEMM|4096x4096x4096|float16|U(-1,1)|gfx950"
    path = str(tmp_path / "t.json")
    tuned.store(uni, GemmConfig(256, 256, 64, 128, 64, 2, 0), 1300.0, "TFLOPS", path, inputs="U(-1,1)")
    assert tuned.lookup(n01, path) is None and tuned.lookup(uni, path) is not None


def test_shipped_winners_are_solver_candidates():
    """Every entry of the shipped table is a configuration its solver still emits for
    that shape (a rule added to a solver must not leave a stale winner behind)."""
    from deca_amd import Solver, tuned
    from deca_amd.arch import MI355X

    arch = MI355X()
    table = tuned.load()
    assert table
    for key in table:
        op, dims = key.split("|")[0], tuple(int(d) for d in key.split("|")[1].split("x"))
        cfg = tuned.lookup(key)
        if op == "GEMM":
            candidates = Solver.solve_gemm_tc(arch, *dims)
        elif op == "flash_attn":
            candidates = Solver.solve_flash_attn(arch, *dims)
        else:
            candidates = Solver.solve_rowwise(arch, op, *dims)
        assert cfg in candidates, key


def test_rotating_sets_and_cycle():
    import torch

    from deca_amd.kernels.rowwise_bench import cycle, rotating_sets

    x, w, y = torch.ones(64, 32), torch.ones(32), torch.zeros(64, 32)
    per_set = (64 * 32 * 2 + 32) * 4
    sets = rotating_sets((x, w), y, cache_bytes=per_set, factor=4)
    assert len(sets) == 4 and sets[0][0] is x and sets[1][0] is not x
    assert all(torch.equal(s[0], x) and len(s) == 3 for s in sets)
    assert len(rotating_sets((x,), y, cache_bytes=0)) == 1
    seen = []
    call = cycle(lambda *a: seen.append(a[-1].data_ptr()), sets)
    for _ in range(6):
        call()
    assert seen[:4] == [s[-1].data_ptr() for s in sets] and seen[4:] == seen[:2]


def test_config_strings_parse_back():
    """Every config's printed form (what records, logs and bench.py --kernel-config use)
    parses back into the same object."""
    from deca_amd import tuned
    from deca_amd.kernels.flash_attn_hip import FAConfig
    from deca_amd.kernels.gemm_hip import GemmConfig
    from deca_amd.kernels.rowwise_hip import RowConfig

    cases = [
        ("GEMM", GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True)),
        ("GEMM", GemmConfig(128, 128, 32, 64, 32, 5, 4, False, False, True, True, 16, 2)),
        ("GEMM", GemmConfig(256, 256, 64, 128, 64, 2, 0, True, True, True, False, 16, 4, True)),
        ("GEMM", GemmConfig(256, 128, 64, 128, 64, 1, 1, True, False, False)),
        ("softmax", RowConfig(256, 2, 8, "reg", 1, True)),
        ("rmsnorm", RowConfig(1024, 1, 4, "twopass", 4)),
        ("flash_attn", FAConfig(256, 64, 8, 2, pipe=2)),
        ("flash_attn", FAConfig(128, 128, 4, 1)),
        ("flash_attn", FAConfig(256, 128, 8, 2, mfma=16, roll=True)),
        ("flash_attn", FAConfig(256, 64, 4, 3, trust=True)),
        ("flash_attn", FAConfig(256, 64, 4, 2, spread=4, trust=True)),
    ]
    for op, cfg in cases:
        assert tuned.parse_config(op, str(cfg)) == cfg
    with pytest.raises(ValueError):
        tuned.parse_config("GEMM", "256x256x64,warp=128x64,stages=2,raster=0,epi_smem=1,bogus=1")
