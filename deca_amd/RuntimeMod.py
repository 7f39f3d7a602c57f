"""
Loads, verifies and times one tuned kernel.

Same constructor, methods and result attributes as the reference's
src/RuntimeMod.py (`build`, `build_with_tc`, `build_flash_attn`, `load_kernel`,
`load_flash_attn`, `time_evaluator`, `time_kernel_op`, `time_flash_attn`, `show`,
`get_mod`, `get_sch`; `execution_time`,
`throughput`, `max_error`, `record`).  Underneath, a kernel is a gfx950 code
object loaded through libdeca_hip.so instead of a TVM runtime module, and torch
tensors are handed over as raw device pointers instead of DLPack capsules.
There is no path that computes on the host: without the launcher library or a
GPU every method that would run a kernel raises.
"""

from __future__ import annotations

from deca_amd.operators.Op import Operator

# Rows of the reference compared per step: bounds the fp32 temporaries for
# vocab-sized inputs (reference: RuntimeMod.py:213-219).
_VERIFY_ELEMS = 1 << 24


class RuntimeMod:
    def __init__(self, operator: Operator, arch, use_tc: bool, compute_pattern,
                 timing: str = "events"):
        """
        Args:
            operator: the operator whose kernel is tuned
            arch: hardware model of the GPU
            use_tc: kept for signature compatibility (every GEMM here uses MFMA)
            compute_pattern: the config (`GemmConfig`, `RowConfig` or `FAConfig`)
            timing: "events" -- one event pair and one synchronisation per call, the
                reference's procedure (attn_bench.py:35-70); "back_to_back" -- batches of
                launches between one event pair (`deca_launch_timed`)
        """
        from deca_amd.kernels.attn_bench import TIMINGS

        assert timing in TIMINGS, timing
        self.timing = timing
        self.operator = operator
        self.arch = arch
        self.use_tc = use_tc
        self.compute_pattern = compute_pattern
        self.ir_mod = None  # KernelSpec of the config
        self.runtime_mod = None  # LoadedKernel
        self.execution_time: float = 0.0
        self.throughput: float = 0.0
        self.max_error: float = float("nan")
        self.record: str = ""

    # ---- building / loading ------------------------------------------------------------
    @property
    def is_flash_attn(self) -> bool:
        return bool(getattr(self.operator, "is_attention", False))

    @property
    def is_kernel_op(self) -> bool:
        """Operators that generate their kernel from a config (`build_mod`)."""
        return hasattr(self.operator, "build_mod")

    def _specialise(self):
        if not self.is_kernel_op:
            raise NotImplementedError(
                f"{type(self.operator).__name__} has no kernel template in this build"
            )
        self.ir_mod = self.operator.build_mod(self.compute_pattern)
        return self.ir_mod

    def build(self):
        """Specialise, compile (in-tree cache) and load the kernel."""
        self.runtime_mod = self.operator.compile(self._specialise())

    build_flash_attn = build
    build_with_tc = build  # every GEMM here is a config-generated MFMA kernel (RuntimeMod.py:79-87)

    def build_without_tc(self):
        """The reference's CUDA-core GEMM over a TVM schedule (RuntimeMod.py:67-77) has no
        counterpart here: the operators of this build all generate their kernel from a config."""
        raise NotImplementedError("no schedule-based GEMM in this build: use the GEMMTC operator")

    def load_kernel(self, path: str):
        """Load a code object written by one of the `build_*_to_file` functions."""
        from deca_amd.driver.driver import load_kernel

        self.runtime_mod = load_kernel(self._specialise(), path)

    load_flash_attn = load_kernel

    def get_mod(self):
        return self.ir_mod

    def get_sch(self):
        """The TVM schedule of the reference's legacy GEMM path (RuntimeMod.py:126-131); never
        built here, so this fails the way the reference does before its `build_*_tc`."""
        assert hasattr(self, "sch"), "Schedule not built"
        return self.sch

    def show(self):
        """Print the specialisation (template, macros, geometry) and, once
        loaded, the resources recorded in the code object."""
        print(self.get_mod().show())
        if self.runtime_mod is not None:
            print(self.runtime_mod.info())

    # ---- verification --------------------------------------------------------------------
    def _errors(self, out, ref, atol: float, rtol: float):
        """(max |out - ref|, max |out - ref| / (atol + rtol |ref|)) in row blocks.
        A NaN anywhere in the output makes both infinite (Python's max() would
        otherwise drop it and let a broken kernel pass)."""
        out2, ref2 = out.reshape(-1, out.shape[-1]), ref.reshape(-1, ref.shape[-1])
        step = max(1, _VERIFY_ELEMS // ref2.shape[-1])
        worst, excess = 0.0, 0.0
        for r0 in range(0, ref2.shape[0], step):
            r = ref2[r0 : r0 + step].float()
            d = (out2[r0 : r0 + step].float() - r).abs()
            block_worst = d.max().item()
            block_excess = (d / (atol + rtol * r.abs())).max().item()
            if block_worst != block_worst or block_excess != block_excess:  # NaN
                return float("inf"), float("inf")
            worst, excess = max(worst, block_worst), max(excess, block_excess)
        return worst, excess

    def _measure(self, verify: bool, abs_tol: float | None):
        """Runs the kernel once for verification (optional) and then times it.
        `abs_tol`: absolute tolerance (attention); None: the operator's (atol, rtol)."""
        import torch

        from deca_amd.kernels.attn_bench import bench_back_to_back, bench_cuda

        if self.runtime_mod is None:
            raise RuntimeError("no kernel loaded: call build() or load_kernel(path) first")
        op, kern = self.operator, self.runtime_mod
        inputs = op.make_inputs()
        args = op.kernel_args(inputs, op.make_output(inputs))
        if verify:
            kern(*args)
            torch.cuda.synchronize()
            ref = op.reference(inputs)
            if abs_tol is not None:
                self.max_error, _ = self._errors(args[-1], ref, abs_tol, 0.0)
                if not self.max_error <= abs_tol:
                    raise RuntimeError(
                        f"{self.compute_pattern}: max error {self.max_error} exceeds {abs_tol}")
            else:
                atol, rtol = op.tolerance
                self.max_error, excess = self._errors(args[-1], ref, atol, rtol)
                if not excess <= 1.0:
                    raise RuntimeError(
                        f"{self.compute_pattern}: max error {self.max_error:.3e} exceeds "
                        f"atol={atol} + rtol={rtol} * |ref| (x{excess:.2f})")
            del ref
        if getattr(op, "metric", "GB/s") == "GB/s":
            # memory-bound: cycle through buffer sets larger than the Infinity Cache
            from deca_amd.kernels.rowwise_bench import cycle, rotating_sets

            sets = rotating_sets(inputs, args[-1], getattr(self.arch, "mall_bytes", 0))
            if self.timing == "back_to_back":
                t = bench_back_to_back(lambda n: kern.time(sets, n))
            else:
                t = bench_cuda(cycle(kern, sets))
        elif self.timing == "back_to_back":
            t = bench_back_to_back(lambda n: kern.time([args], n))
        else:
            t = bench_cuda(lambda: kern(*args))
        self.execution_time = t
        return t

    # ---- timing ----------------------------------------------------------------------------
    def time_evaluator(self):
        """Time (and verify) the loaded kernel."""
        return self.time_flash_attn() if self.is_flash_attn else self.time_kernel_op()

    def time_flash_attn(self, verify: bool = True, atol: float = 2e-2):
        """Attention: verified against torch's fused attention on the device with an
        absolute tolerance (reference: RuntimeMod.py:156-190)."""
        op = self.operator
        t = self._measure(verify, atol)
        self.throughput = op.num_flops / t / 1e12
        self.record = (
            f"{op.describe()} \n\t{self.compute_pattern} \n\tcost time: {t * 1000:.4f} ms, "
            f"throughput: {self.throughput:.2f} TFLOPS, max err: {self.max_error:.2e}"
        )

    def time_kernel_op(self, verify: bool = True):
        """Row-wise operators and GEMM: verified against the operator's torch reference
        with |d| <= atol + rtol |ref|; GB/s for memory-bound operators, TFLOPS for
        operators with `metric == "TFLOPS"` (reference: RuntimeMod.py:192-238)."""
        op = self.operator
        t = self._measure(verify, None)
        if getattr(op, "metric", "GB/s") == "TFLOPS":
            self.throughput, unit = op.num_flops / t / 1e12, "TFLOPS"
        else:
            self.throughput, unit = op.num_bytes / t / 1e9, "GB/s"
        self.record = (
            f"{op.describe()} \n\t{self.compute_pattern} \n\tcost time: {t * 1000:.4f} ms, "
            f"throughput: {self.throughput:.1f} {unit}, max err: {self.max_error:.2e}"
        )
