"""RMSNorm over the last dimension of an [M, N] tensor (defined with the other
row-wise operators; kept as a module for `from operators.RMSNorm import RMSNorm`)."""

from deca_amd.operators.Rowwise import RMSNorm  # noqa: F401

__all__ = ["RMSNorm"]
