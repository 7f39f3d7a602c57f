"""Operator protocol shared by every tunable kernel family.

`RuntimeMod` and `Tuner` talk to an operator through a small duck-typed
protocol (reference: src/operators/Op.py is an empty base; the protocol lives
implicitly in GEMMTC.py:19-111 and Rowwise.py:23-73).  Here the base class
implements the protocol once as template methods; a kernel family supplies
three hooks:

    _check(cfg)      raise AssertionError if `cfg` is invalid for this shape
    _specialise(cfg) return the KernelSpec (template + macros + geometry)
    _load(spec)      compile (in-tree cache) and load the kernel on the device

plus its inputs (`make_inputs`), torch reference (`reference`), tolerance and
work count (`num_flops` or `num_bytes`).
"""

from __future__ import annotations


class Operator:
    #: unit RuntimeMod reports: "GB/s" (memory bound) or "TFLOPS" (compute bound)
    metric = "GB/s"

    def __init__(self, name: str):
        self.name = name

    def __call__(self, *args, **kwargs):
        raise NotImplementedError("operators are descriptors; launch kernels through RuntimeMod")

    # ---- hooks ---------------------------------------------------------------------
    def _check(self, cfg) -> None:
        raise NotImplementedError

    def _specialise(self, cfg):
        raise NotImplementedError

    def _load(self, spec):
        raise NotImplementedError

    # ---- protocol ------------------------------------------------------------------
    def is_valid(self, cfg) -> bool:
        try:
            self._check(cfg)
        except AssertionError:
            return False
        return True

    def build_mod(self, cfg):
        """The specialised kernel of `cfg` (the reference returns a TVM IRModule)."""
        return self._specialise(cfg)

    def compile(self, mod):
        """Compile and load what `build_mod` returned."""
        return self._load(mod)

    def make_output(self, inputs):
        import torch

        return torch.empty_like(inputs[0])

    def kernel_args(self, inputs, out):
        """Tensors in the kernel's argument order: the inputs, then the output."""
        return (*inputs, out)

    def describe(self) -> str:
        return self.name
