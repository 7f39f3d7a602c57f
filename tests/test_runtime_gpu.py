"""GPU tests of the public tuning surface: RuntimeMod (build / load_kernel /
time_evaluator / record), the bench helpers, GPU detection, and one short
Tuner run per operator family with its deca_performance.log record."""

import io
import os
import re

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arch():
    from deca_amd.utils.helper import GPUDetector

    return GPUDetector.create_gpu_instance(verbose=False)


def test_gpu_detection(arch):
    assert arch.gcn_arch == "gfx950" and arch.warp_size == 64
    assert arch.sm_nums > 0 and arch.max_dyn_smem_per_block >= 64 * 1024
    assert arch.peak_mma_sync_flops == pytest.approx(arch.sm_nums * 4096 * arch.sm_clock_hz / 1e9)


def test_device_and_function_info(hip):
    from deca_amd.kernels.rowwise_hip import RowConfig, build_rowwise, make_rowwise

    info = hip.device_info(0)
    assert info.gcn_arch.startswith("gfx950") and info.wave_size == 64 and info.cu_count > 0
    kern = build_rowwise(make_rowwise("softmax", 256, 4096, "float16", RowConfig(128, 1, 8)))
    fi = kern.info()
    assert 0 < fi["num_regs"] <= 128 and fi["scratch_bytes"] == 0
    kern.close()
    kern.close()  # idempotent


def test_loader_refuses_a_spilled_kernel_that_was_marked_spill_free():
    """Kernels that wait for part of their outstanding loads are marked `no_scratch`; a
    build of such a kernel that spills is refused at load time, not launched."""
    import kernel_cases
    from deca_amd.driver.driver import KernelRejected, load_kernel
    from deca_amd.kernels.attn_bench import make_qkv, math_attention
    from deca_amd.kernels.build import cached_build

    plain, marked = kernel_cases.spilling_specs()
    assert plain.key() == marked.key()  # one code object
    path = cached_build(plain)
    kern = load_kernel(plain, path)
    assert kern.info()["scratch_bytes"] > 0
    # unmarked it loads and is right (it only ever waits for all of its loads)
    q, k, v = make_qkv(1, 2, 256, 256, 320)
    o = torch.full_like(q, float("nan"))
    kern(q, k, v, o)
    torch.cuda.synchronize()
    assert (o.float() - math_attention(q, k, v, False)).abs().max().item() <= 2e-3
    kern.close()
    with pytest.raises(KernelRejected, match="spills"):
        load_kernel(marked, path)


def test_runtime_mod_rowwise_build_and_time(arch):
    from deca_amd.kernels.rowwise_hip import RowConfig
    from deca_amd.operators import RMSNorm, Softmax
    from deca_amd.RuntimeMod import RuntimeMod

    for op, cfg in ((Softmax(2048, 4096, "fp16"), RowConfig(256, 2, 8, hint=True)),
                    (RMSNorm(2048, 4096, "bf16", 1e-6), RowConfig(128, 1, 8))):
        rt = RuntimeMod(op, arch, False, cfg)
        assert rt.is_kernel_op and not rt.is_flash_attn
        with pytest.raises(RuntimeError, match="no kernel loaded"):
            rt.time_evaluator()
        rt.build()
        rt.time_evaluator()
        assert rt.execution_time > 0 and rt.throughput > 100 and rt.max_error < 5e-2
        assert re.fullmatch(
            rf"{re.escape(op.describe())} \n\t{re.escape(str(cfg))} \n\tcost time: \d+\.\d{{4}} ms, "
            r"throughput: \d+\.\d GB/s, max err: \d\.\d\de[-+]\d\d", rt.record)
        assert rt.get_mod().grid[0] == 2048 // cfg.rows_per_block


def test_runtime_mod_load_kernel_from_file(arch, tmp_path):
    from deca_amd.kernels.gemm_hip import GemmConfig, build_gemm_tc_to_file
    from deca_amd.operators import GEMMTC
    from deca_amd.RuntimeMod import RuntimeMod

    cfg = GemmConfig(128, 128, 64, 64, 64, 2, 4, False, True, True)
    shape = (1024, 1024, 512)
    path = build_gemm_tc_to_file(shape, cfg, arch.gcn_arch, str(tmp_path / "g.hsaco"))
    op = GEMMTC(*shape)
    rt = RuntimeMod(op, arch, True, cfg)
    rt.load_kernel(path)
    rt.time_evaluator()
    # outputs reach |c| ~ 100, where the fp16 grid spacing is 0.0625: the relative part of the tolerance covers it
    assert "TFLOPS" in rt.record and rt.throughput > 1 and rt.max_error <= 0.0625


def test_runtime_mod_rejects_wrong_results(arch, tmp_path):
    """A kernel built for another shape computes something else: the check
    against torch must raise, as the tuner relies on it to drop bad configs."""
    from deca_amd.kernels.rowwise_hip import RowConfig, build_rowwise_to_file
    from deca_amd.operators import Softmax
    from deca_amd.RuntimeMod import RuntimeMod

    cfg = RowConfig(128, 1, 8)
    # rows of 2048 instead of 4096: every output row is normalised over half a row
    path = build_rowwise_to_file("softmax", (2048, 2048), "float16", cfg, 1e-6, arch.gcn_arch,
                                 str(tmp_path / "wrong.hsaco"))
    rt = RuntimeMod(Softmax(1024, 4096), arch, False, cfg)
    rt.load_kernel(path)
    # the spec of the operator (1024 blocks of 128 lanes) launches the 2048-column kernel:
    # it stays inside the [1024, 4096] buffers (1024 rows x 2048 columns) and is wrong
    with pytest.raises(RuntimeError, match="exceeds"):
        rt.time_evaluator()


def test_runtime_mod_flash_attn(arch):
    from deca_amd.kernels.flash_attn_hip import FAConfig
    from deca_amd.operators import FlashAttention
    from deca_amd.RuntimeMod import RuntimeMod

    for causal in (False, True):
        op = FlashAttention(2, 4, 1024, 1024, 128, causal=causal)
        rt = RuntimeMod(op, arch, True, FAConfig(128, 64, 4, 2))
        assert rt.is_flash_attn
        rt.build()
        rt.time_evaluator()
        assert rt.max_error <= 2e-2 and rt.throughput > 1
        assert ("causal" in rt.record) == causal


def test_bench_helpers():
    from deca_amd.kernels.attn_bench import bench_cuda, bench_interleaved

    x = torch.randn(1 << 20, device="cuda")
    t = bench_cuda(lambda: x.mul_(1.0), warmup_s=0.02, measure_s=0.02, min_iters=5)
    assert 0 < t < 1e-2
    out = bench_interleaved({"a": lambda: x.add_(0.0), "b": lambda: x.mul_(1.0)}, rounds=1)
    assert set(out) == {"a", "b"} and all(v > 0 for v in out.values())


@pytest.mark.parametrize("operator,shape,kw", [
    ("softmax", (4096, 1024), {"dtype": "fp16"}),
    ("GEMM", (2048, 2048, 1024), {}),
    ("flash_attn", (2, 8, 1024, 1024, 64), {"causal": True}),
])
def test_tuner_end_to_end(arch, operator, shape, kw):
    """solve -> rank -> compile in worker processes -> verify + time -> finalists vs torch -> record"""
    from deca_amd.Tuner import Tuner

    log = io.StringIO()
    tuner = Tuner(operator, arch, arch.gcn_arch, top_n=3, jobs=3, finalists=2, rounds=1)
    cfg, best, ref = tuner.tune(*shape, log=log, **kw)
    assert best > 0 and ref > 0 and len(tuner.measurements) >= 1
    text = log.getvalue()
    assert re.search(r"^\d{4}-\d\d-\d\d \d\d:\d\d:\d\d \[", text, re.M)
    assert f"config: {cfg} (cost-model rank " in text
    assert re.search(r"compile time: \d+\.\d s, total tuning time: \d+\.\d s", text)
    unit = "GB/s" if operator == "softmax" else "TFLOPS"
    assert re.search(rf"throughput: \d+\.\d {unit} \(\d+% of ", text)
    assert os.environ.get("HIP_VISIBLE_DEVICES", "0") is not None
