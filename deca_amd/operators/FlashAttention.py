"""
FlashAttention (forward) operator: O = softmax(scale * Q K^T [+ causal]) V.

An `FAConfig` fully determines a specialisation of `csrc/flash_attn.hip`
(reference: src/operators/FlashAttention.py).
"""

import math

from deca_amd.kernels import flash_attn_hip
from deca_amd.operators.Op import Operator


class FlashAttention(Operator):
    metric = "TFLOPS"
    #: RuntimeMod verifies attention against torch's fused kernel with an
    #: absolute tolerance instead of the (atol, rtol) pair of the other operators
    is_attention = True

    def __init__(self, B: int, H: int, S_q: int, S_kv: int, D: int, dtype: str = "float16",
                 softmax_scale: float | None = None, causal: bool = False,
                 name: str = "FlashAttention"):
        """Q [B, H, S_q, D], K and V [B, H, S_kv, D], fp16 with fp32 accumulation;
        `softmax_scale` defaults to 1 / sqrt(D); `causal` is the top-left aligned
        mask and needs S_q == S_kv."""
        assert dtype == "float16", "FlashAttention only supports float16 inputs"
        assert not causal or S_q == S_kv, "causal attention requires S_q == S_kv"
        super().__init__(name)
        self.B, self.H, self.S_q, self.S_kv, self.D = B, H, S_q, S_kv, D
        self.dtype = dtype
        self.softmax_scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
        self.causal = causal
        self.num_flops = 4 * B * H * S_q * S_kv * D // (2 if causal else 1)

    shape = property(lambda self: (self.B, self.H, self.S_q, self.S_kv, self.D))

    def _check(self, cfg):
        flash_attn_hip.check_config(cfg, self.S_q, self.S_kv, self.D)

    def _specialise(self, cfg):
        return flash_attn_hip.make_flash_attn_fwd(*self.shape, cfg, self.softmax_scale, self.causal)

    def _load(self, spec):
        return flash_attn_hip.build_flash_attn(spec)

    def make_inputs(self):
        from deca_amd.kernels.attn_bench import make_qkv

        return make_qkv(*self.shape)

    def reference(self, inputs):
        from deca_amd.kernels.attn_bench import sdpa_flash

        q, k, v = inputs
        return sdpa_flash(q, k, v, causal=self.causal, scale=self.softmax_scale)

    def describe(self) -> str:
        B, H, S_q, S_kv, D = self.shape
        tail = ", causal" if self.causal else ""
        return f"{self.name}(B={B}, H={H}, S_q={S_q}, S_kv={S_kv}, D={D}, {self.dtype}{tail})"
