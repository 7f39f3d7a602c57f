"""
Row-wise memory-bound operators over an [M, N] input (reduction over N):
Softmax over the last dimension, and RMSNorm with a weight,
y = x * rsqrt(mean(x^2) + eps) * w.  fp16 or bf16 I/O, fp32 math.

A `RowConfig` fully determines a specialisation of `csrc/rowwise.hip`
(reference: src/operators/Rowwise.py, Softmax.py, RMSNorm.py).
"""

from deca_amd.kernels import rowwise_hip
from deca_amd.operators.Op import Operator

# (atol, rtol) of the comparison with torch while tuning:
# |y - ref| <= atol + rtol * |ref|   (reference: Rowwise.py:15-20)
TOLERANCE = {
    ("softmax", "float16"): (1e-5, 1e-2),
    ("softmax", "bfloat16"): (1e-5, 3e-2),
    ("rmsnorm", "float16"): (1e-2, 1e-2),
    ("rmsnorm", "bfloat16"): (3e-2, 3e-2),
}


class RowwiseOperator(Operator):
    op_kind: str = ""

    def __init__(self, M: int, N: int, dtype: str = "float16", eps: float = 1e-6, name: str = ""):
        from deca_amd.kernels.rowwise_bench import canonical_dtype, rowwise_bytes

        super().__init__(name or type(self).__name__)
        self.M, self.N = M, N
        self.dtype = canonical_dtype(dtype)
        self.eps = eps
        self.num_bytes = rowwise_bytes(self.op_kind, M, N)

    shape = property(lambda self: (self.M, self.N))
    tolerance = property(lambda self: TOLERANCE[(self.op_kind, self.dtype)])

    def _check(self, cfg):
        rowwise_hip.check_config(cfg, self.op_kind, self.M, self.N, self.dtype)

    def _specialise(self, cfg):
        return rowwise_hip.make_rowwise(self.op_kind, self.M, self.N, self.dtype, cfg, self.eps)

    def _load(self, spec):
        return rowwise_hip.build_rowwise(spec)

    def make_inputs(self):
        from deca_amd.kernels.rowwise_bench import make_inputs

        return make_inputs(self.op_kind, self.M, self.N, self.dtype)

    def reference(self, inputs):
        from deca_amd.kernels.rowwise_bench import torch_ref

        return torch_ref(self.op_kind, inputs, self.eps)

    def describe(self) -> str:
        return f"{self.name}(M={self.M}, N={self.N}, {self.dtype})"


class Softmax(RowwiseOperator):
    """softmax(x, -1) for x [M, N] (M rows, e.g. tokens; N hidden / vocab size)."""

    op_kind = "softmax"

    def __init__(self, M: int, N: int, dtype: str = "float16", name: str = "Softmax"):
        super().__init__(M, N, dtype, name=name)


class RMSNorm(RowwiseOperator):
    """x * rsqrt(mean(x^2) + eps) * w for x [M, N], w [N]."""

    op_kind = "rmsnorm"

    def __init__(self, M: int, N: int, dtype: str = "float16", eps: float = 1e-6,
                 name: str = "RMSNorm"):
        super().__init__(M, N, dtype, eps, name=name)
