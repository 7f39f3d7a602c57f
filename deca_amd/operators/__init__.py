"""Operator descriptors: shape, work count, inputs, reference, tolerance and the
kernel specialisation of a config."""

from .FlashAttention import FlashAttention
from .GEMMTC import GEMMTC
from .Op import Operator
from .Rowwise import RMSNorm, RowwiseOperator, Softmax

__all__ = ["Operator", "RowwiseOperator", "Softmax", "RMSNorm", "GEMMTC", "FlashAttention"]
