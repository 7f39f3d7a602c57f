"""
FlashAttention (forward) operator.

A tile configuration (`FAConfig`) fully determines a specialisation of the HIP
template produced by `kernels.flash_attn_hip.make_flash_attn_fwd`
(reference: src/operators/FlashAttention.py).
"""

import math

from deca_amd.kernels.flash_attn_hip import FAConfig, check_config, make_flash_attn_fwd
from deca_amd.operators.Op import Operator


class FlashAttention(Operator):
    metric = "TFLOPS"
    is_attention = True  # RuntimeMod times it against fused attention (absolute tolerance)

    def __init__(self, B: int, H: int, S_q: int, S_kv: int, D: int, dtype: str = "float16",
                 softmax_scale: float | None = None, causal: bool = False,
                 name: str = "FlashAttention"):
        """
        Args:
            B, H: batch size and number of heads
            S_q, S_kv: query / key-value sequence lengths
            D: head dimension
            dtype: only "float16" is supported (fp32 accumulation)
            softmax_scale: defaults to 1 / sqrt(D)
            causal: top-left aligned causal mask (requires S_q == S_kv)
        """
        assert dtype == "float16", "FlashAttention only supports float16 inputs"
        self.B, self.H, self.S_q, self.S_kv, self.D = B, H, S_q, S_kv, D
        self.dtype = dtype
        self.softmax_scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
        assert not causal or S_q == S_kv, "causal attention requires S_q == S_kv"
        self.causal = causal
        self.num_flops = 4 * B * H * S_q * S_kv * D // (2 if causal else 1)
        super().__init__(name=name)

    @property
    def shape(self):
        return (self.B, self.H, self.S_q, self.S_kv, self.D)

    def is_valid(self, cfg: FAConfig) -> bool:
        try:
            check_config(cfg, self.S_q, self.S_kv, self.D)
            return True
        except AssertionError:
            return False

    def build_mod(self, cfg: FAConfig):
        return make_flash_attn_fwd(
            self.B, self.H, self.S_q, self.S_kv, self.D, cfg, self.softmax_scale, self.causal
        )

    def compile(self, mod):
        from deca_amd.kernels.flash_attn_hip import build_flash_attn

        return build_flash_attn(mod)

    def make_inputs(self):
        from deca_amd.kernels.attn_bench import make_qkv

        return make_qkv(self.B, self.H, self.S_q, self.S_kv, self.D)

    def make_output(self, inputs):
        import torch

        return torch.empty_like(inputs[0])

    def kernel_args(self, inputs, out):
        """Tensors in the kernel's argument order: q, k, v, o."""
        return (*inputs, out)

    def describe(self) -> str:
        B, H, S_q, S_kv, D = self.shape
        return (f"{self.name}(B={B}, H={H}, S_q={S_q}, S_kv={S_kv}, D={D}, {self.dtype}"
                f"{', causal' if self.causal else ''})")
