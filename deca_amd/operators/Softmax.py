"""Softmax over the last dimension of an [M, N] tensor (defined with the other
row-wise operators; kept as a module for `from operators.Softmax import Softmax`)."""

from deca_amd.operators.Rowwise import Softmax  # noqa: F401

__all__ = ["Softmax"]
