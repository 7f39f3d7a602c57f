"""
Loads, verifies and times one tuned kernel.

Same constructor, methods and result attributes as the reference's
src/RuntimeMod.py; underneath, a kernel is a gfx950 code object loaded through
libdeca_hip.so (`deca_amd.driver`) instead of a TVM runtime module, and torch
tensors are handed over as raw device pointers instead of DLPack capsules.
There is no path that computes on the host: without the launcher library or a
GPU every method that would run a kernel raises.
"""

from __future__ import annotations

from deca_amd.operators.Op import Operator


class RuntimeMod:
    def __init__(self, operator: Operator, arch, use_tc: bool, compute_pattern):
        """
        Args:
            operator: Operator, kernel to be tuned
            arch: Arch, the architecture of the GPU
            use_tc: kept for signature compatibility (every GEMM here uses MFMA)
            compute_pattern: the config (`GemmConfig`, `RowConfig` or `FAConfig`)
        """
        self.operator = operator
        self.arch = arch
        self.use_tc = use_tc
        self.compute_pattern = compute_pattern

        self.ir_mod = None  # KernelSpec
        self.runtime_mod = None  # LoadedKernel
        self.execution_time: float = 0.0
        self.throughput: float = 0.0
        self.max_error: float = float("nan")
        self.record: str = ""

    @property
    def is_flash_attn(self) -> bool:
        return bool(getattr(self.operator, "is_attention", False))

    @property
    def is_kernel_op(self) -> bool:
        """Operators that generate their kernel from a config (`build_mod`)."""
        return hasattr(self.operator, "build_mod")

    def build(self):
        """Specialise, compile (in-tree cache) and load the kernel (reference: :53-65)."""
        if not self.is_kernel_op:
            raise NotImplementedError(
                f"{type(self.operator).__name__} has no kernel template in this build"
            )
        self.ir_mod = self.operator.build_mod(self.compute_pattern)
        if self.is_flash_attn:
            from deca_amd.kernels.flash_attn_hip import build_flash_attn

            self.runtime_mod = build_flash_attn(self.ir_mod)
        else:
            self.runtime_mod = self.operator.compile(self.ir_mod)

    def build_flash_attn(self):
        self.build()

    def load_flash_attn(self, path: str):
        """Load a FlashAttention kernel written by `build_flash_attn_to_file`."""
        self.load_kernel(path)

    def load_kernel(self, path: str):
        """Load a code object written by a `build_*_to_file` function (reference: :104-109)."""
        from deca_amd.driver.driver import load_kernel

        self.ir_mod = self.operator.build_mod(self.compute_pattern)
        self.runtime_mod = load_kernel(self.ir_mod, path)

    def show(self):
        """Print the specialisation (template, macros, geometry) and, once
        loaded, the resources recorded in the code object."""
        print(self.get_mod().show())
        if self.runtime_mod is not None:
            print(self.runtime_mod.info())

    def get_mod(self):
        return self.ir_mod

    def time_evaluator(self):
        """Time (and verify) the loaded kernel."""
        if self.runtime_mod is None:
            raise RuntimeError("no kernel loaded: call build() or load_kernel(path) first")
        if self.is_flash_attn:
            return self.time_flash_attn()
        return self.time_kernel_op()

    def time_flash_attn(self, verify: bool = True, atol: float = 2e-2):
        """
        Time (and optionally verify against torch SDPA on the device) the
        FlashAttention kernel (reference: :156-190).
        """
        import torch

        from deca_amd.kernels.attn_bench import bench_cuda, make_qkv, sdpa_flash

        op = self.operator
        B, H, S_q, S_kv, D = op.shape
        q, k, v = op.make_inputs() if hasattr(op, "make_inputs") else make_qkv(B, H, S_q, S_kv, D)
        o = torch.empty_like(q)
        func = self.runtime_mod

        if verify:
            func(q, k, v, o)
            torch.cuda.synchronize()
            ref = sdpa_flash(q, k, v, causal=op.causal, scale=op.softmax_scale)
            self.max_error = (o.float() - ref.float()).abs().max().item()
            if not self.max_error <= atol:
                raise RuntimeError(
                    f"{self.compute_pattern}: max error {self.max_error} exceeds {atol}"
                )

        t = bench_cuda(lambda: func(q, k, v, o))
        self.execution_time = t
        self.throughput = op.num_flops / t / 1e12
        self.record = (
            f"{op.name}(B={B}, H={H}, S_q={S_q}, S_kv={S_kv}, D={D}, {op.dtype}"
            f"{', causal' if op.causal else ''}) "
            f"\n\t{self.compute_pattern} \n\tcost time: {t * 1000:.4f} ms, "
            f"throughput: {self.throughput:.2f} TFLOPS, max err: {self.max_error:.2e}"
        )

    def time_kernel_op(self, verify: bool = True):
        """
        Time (and optionally verify against the operator's torch reference) a
        `build_mod` operator.  Throughput is reported in GB/s for memory-bound
        operators and in TFLOPS for operators with `metric == "TFLOPS"`
        (reference: :192-238).
        """
        import torch

        from deca_amd.kernels.attn_bench import bench_cuda

        op = self.operator
        inputs = op.make_inputs()
        out = op.make_output(inputs) if hasattr(op, "make_output") else torch.empty_like(inputs[0])
        args = op.kernel_args(inputs, out)
        func = self.runtime_mod

        if verify:
            func(*args)
            torch.cuda.synchronize()
            ref = op.reference(inputs)
            atol, rtol = op.tolerance
            self.max_error, excess = 0.0, 0.0
            # Row chunks keep the fp32 temporaries small for vocab-sized inputs.
            step = max(1, (1 << 24) // ref.shape[-1])
            for r0 in range(0, ref.shape[0], step):
                r = ref[r0 : r0 + step].float()
                diff = (out[r0 : r0 + step].float() - r).abs()
                self.max_error = max(self.max_error, diff.max().item())
                excess = max(excess, (diff / (atol + rtol * r.abs())).max().item())
            del ref
            if not excess <= 1.0:
                raise RuntimeError(
                    f"{self.compute_pattern}: max error {self.max_error:.3e} exceeds "
                    f"atol={atol} + rtol={rtol} * |ref| (x{excess:.2f})"
                )

        t = bench_cuda(lambda: func(*args))
        self.execution_time = t
        if getattr(op, "metric", "GB/s") == "TFLOPS":
            self.throughput = op.num_flops / t / 1e12
            unit = "TFLOPS"
        else:
            self.throughput = op.num_bytes / t / 1e9
            unit = "GB/s"
        self.record = (
            f"{op.describe()} \n\t{self.compute_pattern} \n\tcost time: {t * 1000:.4f} ms, "
            f"throughput: {self.throughput:.1f} {unit}, max err: {self.max_error:.2e}"
        )
