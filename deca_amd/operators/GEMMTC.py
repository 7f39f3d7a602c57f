"""
16-bit MFMA GEMM operator: C = A @ B with fp32 accumulation; fp16 (the
reference's type) or bf16 inputs and output.

A `GemmConfig` fully determines a specialisation of `csrc/gemm.hip`
(reference: src/operators/GEMMTC.py).
"""

import math

from deca_amd.kernels import gemm_hip
from deca_amd.operators.Op import Operator


class GEMMTC(Operator):
    metric = "TFLOPS"

    def __init__(self, M: int, N: int, K: int, dtype: str = "float16", acc: str = "fp32",
                 acc_splits: int = 1, name: str = "GEMMTC", inputs: str = "normal"):
        """`acc` must be "fp32": the matrix cores of CDNA4 have no fp16
        accumulation, so the reference's acc="fp16" / acc_splits modes
        (GEMMTC.py:29-43) do not exist here.  `inputs`: "normal" draws N(0, 1)
        operands as the reference does (gemm_bench.py:29-30), "uniform" U(-1, 1); on a
        power-limited board the operand statistics decide which tile body is fastest."""
        assert inputs in ("normal", "uniform")
        self.inputs = inputs
        from deca_amd.kernels.rowwise_bench import canonical_dtype

        dtype = canonical_dtype(dtype)  # "float16" (the reference's only type) or "bfloat16"
        if acc != "fp32" or acc_splits != 1:
            raise NotImplementedError("MFMA accumulates in fp32 only")
        super().__init__(name)
        self.M, self.N, self.K = M, N, K
        self.dtype, self.acc, self.acc_splits = dtype, acc, 1
        self.num_flops = 2 * M * N * K

    shape = property(lambda self: (self.M, self.N, self.K))

    @property
    def tolerance(self):
        """(atol, rtol) against the fp32 product: the fp16 output rounding is
        ~5e-4 relative and the accumulation error grows like sqrt(K)
        (reference: GEMMTC.py:51-63); bf16 has 3 fewer mantissa bits (x8)."""
        scale = 8.0 if self.dtype == "bfloat16" else 1.0
        return (1e-2 * math.sqrt(self.K / 1024) * scale, 2e-3 * scale)

    def _check(self, cfg):
        gemm_hip.check_config(cfg, self.M, self.N, self.K)

    def _specialise(self, cfg):
        return gemm_hip.make_gemm_tc(self.M, self.N, self.K, cfg, self.dtype)

    def _load(self, spec):
        return gemm_hip.build_gemm_tc(spec)

    def make_inputs(self):
        from deca_amd.kernels.gemm_bench import make_inputs

        from deca_amd.kernels.rowwise_bench import torch_dtype

        return make_inputs(self.M, self.N, self.K, dist=self.inputs, dtype=torch_dtype(self.dtype))

    def make_output(self, inputs):
        import torch

        return torch.empty(self.M, self.N, device=inputs[0].device, dtype=inputs[0].dtype)

    def reference(self, inputs):
        """fp32 product of the fp16 inputs, with TF32-style shortcuts off: torch's
        own fp16 GEMM may use reduced-precision reductions."""
        import torch

        a, b = inputs
        saved = torch.backends.cuda.matmul.allow_tf32
        torch.backends.cuda.matmul.allow_tf32 = False
        try:
            return a.float() @ b.float()
        finally:
            torch.backends.cuda.matmul.allow_tf32 = saved

    def describe(self) -> str:
        dist = ", U(-1,1) inputs" if self.inputs == "uniform" else ""
        return f"{self.name}(M={self.M}, N={self.N}, K={self.K}, {self.dtype}{dist})"
