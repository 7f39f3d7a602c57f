"""The profile summariser: derived figures from synthetic rocprofv3 CSV files."""

import csv
import json
import os

import pytest

from deca_amd.arch import profile


def _write(path, header, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(header)
        w.writerows(rows)


def _passes(tmp, workload, dur_ns, steps=4, rowwise=False):
    out = str(tmp / f"prof_{workload}")
    n = steps * (3 if rowwise else 2)
    first = steps  # warm-up launches before, the pass over one buffer set after
    # the timed launches take dur_ns, everything else twice as long
    trace = []
    for i in range(n):
        d = dur_ns if first <= i < first + steps else 2 * dur_ns
        trace.append(["deca_main", 1000 * i * 10, 1000 * i * 10 + d])
    trace.append(["void at::native::fill", 5, 50])
    _write(os.path.join(out, "trace", "out_kernel_trace.csv"),
           ["Kernel_Name", "Start_Timestamp", "End_Timestamp"], trace)
    _write(os.path.join(out, "trace", "out_kernel_stats.csv"),
           ["Name", "Calls", "AverageNs", "MinNs", "MaxNs", "Percentage"],
           [["deca_main", n, 1.5 * dur_ns, dur_ns, 2 * dur_ns, 99.9], ["void at::native::fill", 1, 45, 45, 45, 0.1]])
    for name, counter, value in (("fetch", "FETCH_SIZE", 65536.0), ("write", "WRITE_SIZE", 131072.0)):
        _write(os.path.join(out, name, "out_counter_collection.csv"),
               ["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value", "Start_Timestamp", "End_Timestamp"],
               [[i, "deca_main", counter, value, 0, dur_ns] for i in range(3)]
               + [[9, "void at::native::fill", counter, 1.0, 0, 10]])
    if not rowwise:
        vals = {"SQ_VALU_MFMA_BUSY_CYCLES": 0.5 * profile.SIMDS * dur_ns * 2.0,  # 50 % busy at 2 GHz
                "SQ_INSTS_MFMA": 1000.0, "SQ_INSTS_VALU": 4000.0, "SQ_ACTIVE_INST_VALU": 1.0,
                "SQ_VALU_MFMA_COEXEC_CYCLES": 0.25 * 0.5 * profile.SIMDS * dur_ns * 2.0,
                "SQ_INSTS_LDS": 1500.0, "SQ_LDS_BANK_CONFLICT": 7.0,
                "GRBM_GUI_ACTIVE": profile.XCDS * dur_ns * 2.0}
        _write(os.path.join(out, "sq", "out_counter_collection.csv"),
               ["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value", "Start_Timestamp", "End_Timestamp"],
               [[d, "deca_main", c, v, 100, 100 + dur_ns] for d in range(2) for c, v in vals.items()])
    work = 268435456 if rowwise else 1099511627776
    rec = {"steps": steps, "config": {"workload": workload, "kernel_config": "Br=256,mfma=16"},
           "roofline": {"kernel_us": dur_ns / 1e3, "timed_launches": [first, steps],
                        "all": {workload: {"work": work}}}}
    with open(os.path.join(out, "trace.log"), "w") as f:
        f.write("[bench] noise\n" + json.dumps(rec) + "\n")
    return out


def test_passes_keep_counters_apart_from_traces():
    for wl in ("gemm_fp16_8192", "softmax_fp16_16384x4096", "fa_fp16_b4h16s4096d128_causal"):
        p = profile.passes(wl)
        assert ("sq" in p) == (profile.kernel_of(wl) != "rowwise")
        assert p["board"][0] is None and p["board"][1][-2:] == ["--power", "4"]
        assert profile.command(wl, "board", "/x")[0] == "python3"
        for name, (prof, bench) in p.items():
            if prof is None:
                continue
            assert ("--pmc" in prof) != ("--kernel-trace" in prof)
            assert bench[:2] == ["--workload", wl] and "--no-cpu" in bench
            cmd = profile.command(wl, name, "/x")
            # the program itself follows "--": no shell, env or launcher in between
            assert cmd[cmd.index("--") + 1] == "python3" and cmd[cmd.index("--") + 2].endswith("bench.py")
    sq = profile.passes("gemm_fp16_8192")["sq"][0][1:]
    assert sum(c.startswith("SQ_") for c in sq) <= 8 and sum(c.startswith("GRBM_") for c in sq) <= 2


def test_matrix_pipe_figures(tmp_path):
    out = _passes(tmp_path, "gemm_fp16_8192", 800_000)
    mp = profile.matrix_pipe(profile._rows(os.path.join(out, "sq", "out_counter_collection.csv")))
    assert abs(mp["clock_ghz"] - 2.0) < 1e-9 and abs(mp["busy"] - 0.5) < 1e-9
    assert abs(mp["peak_share"] - 0.5 * 2.0 / 2.4) < 1e-9
    assert abs(mp["coexec"] - 0.25) < 1e-9 and mp["valu_per_mfma"] == 4.0 and mp["lds_per_mfma"] == 1.5
    # a dispatch of 19 us: no clock, no busy share of the cycles -- only the share of the peak
    short = _passes(tmp_path, "gemm_fp16_2048", 19_000)
    mp = profile.matrix_pipe(profile._rows(os.path.join(short, "sq", "out_counter_collection.csv")))
    assert mp["clock_ghz"] is None and mp["busy"] is None and 0 < mp["peak_share"] <= 1.0


def test_summary_and_traffic_table(tmp_path):
    prof_dir = tmp_path / "profiles"
    prof_dir.mkdir()
    traffic = str(tmp_path / "traffic.json")
    out = _passes(tmp_path, "softmax_fp16_16384x4096", 42_000, rowwise=True)
    path = profile.summarise("softmax_fp16_16384x4096", out, str(prof_dir), traffic)
    text = open(path).read()
    assert os.path.basename(path) == "rowwise_softmax_fp16_16384x4096.md"
    assert "average 42000 ns (min 42000, max 42000)" in text  # the timed launches only
    trace = profile._rows(os.path.join(out, "trace", "out_kernel_trace.csv"))
    assert profile.event_timed_durations(trace, 0, 4) == [84000] * 4
    with pytest.raises(ValueError):
        profile.event_timed_durations(trace, 10, 4)
    assert "python -m deca_amd.arch.profile run softmax_fp16_16384x4096" in text
    assert "Matrix pipe" not in text
    entry = json.load(open(traffic))["workloads"]["softmax_fp16_16384x4096"]
    assert entry["traffic_bytes"] == (65536 * 2 + 131072) * 1024 == profile.traffic_bytes(65536.0, 131072.0)
    assert entry["config"] == "Br=256,mfma=16"
    out = _passes(tmp_path, "gemm_fp16_2048", 19_000)
    text = open(profile.summarise("gemm_fp16_2048", out, str(prof_dir), traffic)).read()
    assert "not derived" in text and "GHz (2.4 GHz nominal)" not in text
    out = _passes(tmp_path, "fa_fp16_b4h16s4096d128", 480_000)
    with open(os.path.join(out, "board.log"), "w") as f:
        f.write(json.dumps({"roofline": {"sclk_mhz": [2100.0, 2140.0], "socket_w": [1330.0, 1350.0],
                                         "achieved": 1140.2, "unit": "TFLOP/s"}}) + "\n")
    text = open(profile.summarise("fa_fp16_b4h16s4096d128", out, str(prof_dir), traffic)).read()
    assert "2.00 GHz" in text and "16x16x32" in text
    assert "Shader clock 2100-2140 MHz, socket power 1330-1350 W" in text
    # another configuration than the stored winner: its own file, nothing recorded
    path = profile.summarise("fa_fp16_b4h16s4096d128", out, str(prof_dir), traffic,
                             kernel_config="Br=256,Bc=64,q_smem=1", tag="q_smem")
    assert path.endswith("flash_attn_fa_fp16_b4h16s4096d128_q_smem.md")
    assert "--kernel-config 'Br=256,Bc=64,q_smem=1'" in open(path).read()
    assert set(json.load(open(traffic))["workloads"]) == {
        "softmax_fp16_16384x4096", "gemm_fp16_2048", "fa_fp16_b4h16s4096d128"}
