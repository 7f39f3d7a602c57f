"""
Row-wise reduction kernels (Softmax over the last dim, RMSNorm): config type,
resource estimates, validity rules and the specialisation of the HIP template
`csrc/rowwise.hip`.

Counterpart of the reference's src/kernels/rowwise_tir.py.  Every row of the
[M, N] input is handled by `threads_per_row` lanes; `rows_per_block` rows share
a workgroup.  Lane t owns the `vec`-element chunks `(c * threads_per_row + t)`
of its row, so a 64-lane wave touches contiguous 1 KiB (512 B) segments.

Modes (rowwise_tir.py:10-16):
- reg:     the whole row is cached in VGPRs (in the input dtype), read from
           HBM exactly once and written once.
- twopass: rows too long for registers are streamed twice: pass 1 computes an
           online (max, sum) / a sum of squares, pass 2 re-reads the row
           (mostly from L2 / Infinity Cache) and writes the output.

What changes on CDNA4: a wave has 64 lanes (so `threads` must be a multiple of
64, and a row may also be owned by a 16- or 32-lane slice of a wave), the
register budget is 512 VGPRs per lane and SIMD shared by the resident waves,
and reductions use DPP / ds_swizzle instead of `__shfl_xor_sync`.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass

from deca_amd.kernels.build import (
    DEFAULT_ARCH, FAST_MATH_OPTIONS, KernelSpec, build_kernel, cached_build, make_spec,
)

LOG2E = 1.4426950408889634
NEG_INF = -1e30
OPS = ("softmax", "rmsnorm")
DTYPES = ("float16", "bfloat16")
MODES = ("reg", "twopass")
WAVE = 64
MAX_VGPRS = 512  # unified VGPRs per lane available to a single wave
VGPRS_PER_SIMD = 512
MAX_ARCH_VGPRS = 256  # architectural VGPRs one wave can address
MAX_THREADS = 1024
TPR_CHOICES = (16, 32, 64, 128, 256, 512, 1024)
TEMPLATE = "rowwise.hip"


@dataclass(frozen=True)
class RowConfig:
    threads_per_row: int = 128
    rows_per_block: int = 1
    vec: int = 8  # elements per vector access (8 -> 16 B for 16-bit dtypes)
    mode: str = "reg"
    unroll: int = 1  # chunks loaded back to back per twopass iteration
    hint: bool = False  # non-temporal loads of read-once data and non-temporal stores

    @property
    def threads(self) -> int:
        return self.threads_per_row * self.rows_per_block

    def as_dict(self):
        return asdict(self)

    def __str__(self):
        s = f"tpr={self.threads_per_row},rpb={self.rows_per_block},vec={self.vec},mode={self.mode}"
        s += f",unroll={self.unroll}" if self.mode == "twopass" else ""
        return s + (",hint=1" if self.hint else "")


def num_chunks(cfg: RowConfig, N: int) -> int:
    return -(-N // (cfg.threads_per_row * cfg.vec))


def est_regs_per_thread(cfg: RowConfig, N: int, op: str) -> int:
    """VGPR estimate of the `E` cached elements per lane + bookkeeping.

    Fitted to the register counts hipcc (gfx950, -O3) records in the code
    object: the row stays packed in its 16-bit dtype (E / 2) and the compiler
    keeps fp32 values live between the reduction and the store -- the
    exponentials of softmax (76 VGPRs at E = 64, 49 at 32, 28 at 16), the
    converted inputs of RMSNorm (bf16: 101 at E = 64, 57 at 32, 38 at 16; fp16
    needs fewer).  (Reference: rowwise_tir.py:68-85, fitted to ptxas on sm_90.)
    """
    cached = num_chunks(cfg, N) if cfg.mode == "reg" else cfg.unroll
    elems = cached * cfg.vec
    if op == "softmax":
        return elems * 9 // 8 + 12
    return elems * 5 // 4 + 16 + cfg.vec // 2


def _fits(regs: int, threads: int) -> bool:
    """One workgroup of `threads` lanes with `regs` VGPRs each fits the CU's 4 SIMDs."""
    waves_per_simd = -(-(threads // WAVE) // 4)
    # (these kernels have no use for the accumulation half of the unified register file)
    return regs <= MAX_ARCH_VGPRS and (regs + 7) // 8 * 8 * waves_per_simd <= VGPRS_PER_SIMD


def lean_regs_per_thread(cfg: RowConfig, N: int) -> int:
    """Estimate for the lean form of the reg mode: only the packed row (E / 2) stays in
    registers between the passes, the fp32 values are computed again (78 VGPRs measured at
    E = 128 for softmax, 77-85 for RMSNorm)."""
    elems = num_chunks(cfg, N) * cfg.vec
    return elems * 5 // 8 + 16


def use_lean(cfg: RowConfig, N: int, op: str) -> bool:
    """The lean reg mode is compiled when the plain one would not fit its workgroup into
    the register files: that is what lets a 128256-element row be read from HBM once."""
    return (cfg.mode == "reg" and not _fits(est_regs_per_thread(cfg, N, op), cfg.threads)
            and _fits(lean_regs_per_thread(cfg, N), cfg.threads))


def regs_per_thread(cfg: RowConfig, N: int, op: str) -> int:
    """Estimate of the form that gets compiled (plain or lean)."""
    return lean_regs_per_thread(cfg, N) if use_lean(cfg, N, op) else est_regs_per_thread(cfg, N, op)


def check_config(cfg: RowConfig, op: str, M: int, N: int, dtype: str) -> None:
    assert op in OPS and dtype in DTYPES and cfg.mode in MODES
    assert cfg.vec in (2, 4, 8) and N % cfg.vec == 0
    assert not cfg.hint or cfg.vec in (4, 8), "cache hints need 8- or 16-byte accesses"
    assert cfg.threads_per_row in TPR_CHOICES
    assert cfg.threads % WAVE == 0 and cfg.threads <= MAX_THREADS
    assert M % cfg.rows_per_block == 0
    assert cfg.unroll >= 1
    if cfg.mode == "twopass":
        # at least one full loop iteration
        assert cfg.unroll <= N // (cfg.threads_per_row * cfg.vec)
    if cfg.mode == "reg":
        assert num_chunks(cfg, N) <= 32  # the row loop is fully unrolled
    # one workgroup must fit in the register files of the CU's 4 SIMDs
    assert _fits(regs_per_thread(cfg, N, op), cfg.threads)


def make_rowwise(
    op: str, M: int, N: int, dtype: str, cfg: RowConfig, eps: float = 1e-6
) -> KernelSpec:
    """Softmax: y = softmax(x, -1).  RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w.

    Returns the specialised kernel (template + macros + launch geometry):
    grid M / rows_per_block, block threads_per_row * rows_per_block
    (reference: rowwise_tir.py:99-128)."""
    check_config(cfg, op, M, N, dtype)
    defines = {
        "DECA_OP": OPS.index(op),
        "DECA_M": M,
        "DECA_N": N,
        "DECA_BF16": int(dtype == "bfloat16"),
        "DECA_TPR": cfg.threads_per_row,
        "DECA_RPB": cfg.rows_per_block,
        "DECA_VEC": cfg.vec,
        "DECA_MODE": MODES.index(cfg.mode),
        "DECA_UNROLL": cfg.unroll,
        "DECA_HINT": int(cfg.hint),
        "DECA_EPS": repr(float(eps)),
    }
    if use_lean(cfg, N, op):
        defines["DECA_LEAN"] = 1
    return make_spec(
        TEMPLATE, defines, grid=(M // cfg.rows_per_block, 1, 1), block=(cfg.threads, 1, 1),
        nargs=3 if op == "rmsnorm" else 2, options=FAST_MATH_OPTIONS,
        meta={"op": op, "dtype": dtype, "cfg": str(cfg)},
    )


def build_rowwise(spec: KernelSpec, target: str | None = None, dump_dir: str | None = None):
    """Compiles (or takes from the in-tree cache) and loads the kernel on the
    current device; `dump_dir` keeps the generated ISA for inspection."""
    from deca_amd.driver.driver import load_kernel

    arch = target or DEFAULT_ARCH
    if dump_dir:
        import os

        path = build_kernel(spec, arch, os.path.join(dump_dir, f"rowwise_{spec.key()}.hsaco"), dump_dir)
    else:
        path = cached_build(spec, arch)
    return load_kernel(spec, path)


def build_rowwise_to_file(
    op: str, shape, dtype: str, cfg: RowConfig, eps: float, arch: str, path: str
) -> str:
    """Builds in a worker process (no GPU context needed) and writes a code object."""
    M, N = shape
    spec = make_rowwise(op, M, N, dtype, cfg, eps)
    return build_kernel(spec, arch, path)
