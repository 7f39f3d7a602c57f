"""
FP16 MFMA GEMM operator (C = A @ B, fp32 accumulation, fp16 output).

A tile configuration (`GemmConfig`) fully determines a specialisation of the
HIP template produced by `kernels.gemm_hip.make_gemm_tc`; the operator also
provides the inputs, the reference and the tolerance used by RuntimeMod.
(Reference: src/operators/GEMMTC.py.)
"""

import math

from deca_amd.kernels.gemm_hip import GemmConfig, check_config, make_gemm_tc
from deca_amd.operators.Op import Operator


class GEMMTC(Operator):
    # RuntimeMod reports compute-bound kernels in TFLOPS.
    metric = "TFLOPS"

    def __init__(self, M: int, N: int, K: int, dtype: str = "float16", acc: str = "fp32",
                 acc_splits: int = 1, name: str = "GEMMTC"):
        """
        Args:
            acc: accumulation precision; only "fp32" exists on the matrix cores
                 of CDNA4 (the reference's "fp16" mode, GEMMTC.py:29-43, is an
                 mma.sync feature)
        """
        assert dtype == "float16", "GEMMTC only supports float16 inputs"
        if acc != "fp32":
            raise NotImplementedError("MFMA accumulates in fp32 only")
        self.M, self.N, self.K = M, N, K
        self.dtype = dtype
        self.acc = acc
        self.acc_splits = 1
        self.num_flops = 2 * M * N * K
        super().__init__(name=name)

    @property
    def shape(self):
        return (self.M, self.N, self.K)

    @property
    def tolerance(self):
        """(atol, rtol) vs the fp32 reference: fp16 output rounding is ~5e-4
        relative, the accumulation error grows like sqrt(K) (reference:
        GEMMTC.py:51-63)."""
        return (1e-2 * math.sqrt(self.K / 1024), 2e-3)

    def is_valid(self, cfg: GemmConfig) -> bool:
        try:
            check_config(cfg, self.M, self.N, self.K)
            return True
        except AssertionError:
            return False

    def build_mod(self, cfg: GemmConfig):
        return make_gemm_tc(self.M, self.N, self.K, cfg)

    def compile(self, mod):
        from deca_amd.kernels.gemm_hip import build_gemm_tc

        return build_gemm_tc(mod)

    def make_inputs(self):
        from deca_amd.kernels.gemm_bench import make_inputs

        return make_inputs(self.M, self.N, self.K)

    def make_output(self, inputs):
        import torch

        return torch.empty(self.M, self.N, device=inputs[0].device, dtype=torch.float16)

    def reference(self, inputs):
        """fp32 GEMM of the fp16 inputs (torch's own fp16 GEMM may use
        reduced-precision reductions, so it is not used as the reference)."""
        import torch

        a, b = inputs
        tf32 = torch.backends.cuda.matmul.allow_tf32
        torch.backends.cuda.matmul.allow_tf32 = False
        try:
            return a.float() @ b.float()
        finally:
            torch.backends.cuda.matmul.allow_tf32 = tf32

    def kernel_args(self, inputs, out):
        """Tensors in the kernel's argument order: a, b, c."""
        return (*inputs, out)

    def describe(self) -> str:
        return f"{self.name}(M={self.M}, N={self.N}, K={self.K}, {self.dtype})"
