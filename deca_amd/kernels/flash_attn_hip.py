"""
FlashAttention-2 style forward kernel: config type, resource estimates,
validity rules and the specialisation of the HIP template
`csrc/flash_attn.hip`.

Counterpart of the reference's src/kernels/flash_attn_tir.py.  Layout: Q, K, V,
O are contiguous [B, H, S, D] float16.

What changes on CDNA4: a wave is 64 lanes and owns a multiple of 32 query rows
(`Br % (32 * num_warps) == 0` instead of 16, flash_attn_tir.py:72); the two
products are computed transposed (S^T = K Q^T, O^T = V^T P^T) so that P stays in
registers between them -- the MFMA accumulator layout is not the operand layout,
unlike mma.sync m16n8k16 (:8-9); K/V tiles arrive by asynchronous global->LDS
loads (cp.async, :320-335).  Q is read from global memory straight into VGPRs and
stays there; with `q_in_smem` the Q tile is staged in LDS behind the K/V ring once
and each wave reads its fragments again in every KV step (:263-281, :345-348),
which trades `D/4` registers per query tile for LDS reads.  `swizzle=False` keeps
the LDS rows linear: the direct loads write whole 1 KiB runs, so rows cannot be
padded as the reference does (:105) and the unswizzled form is only the slow
baseline of the comparison.
"""

from __future__ import annotations

import math
from dataclasses import asdict, dataclass

from deca_amd.kernels.build import (
    DEFAULT_ARCH, FAST_MATH_OPTIONS, KernelSpec, build_kernel, cached_build, make_spec,
)

LOG2E = 1.4426950408889634
NEG_INF = -1e30
WAVE = 64
MAX_LDS = 160 * 1024
TEMPLATE = "flash_attn.hip"


@dataclass(frozen=True)
class FAConfig:
    Br: int = 128  # Q rows per workgroup
    Bc: int = 64  # KV rows per pipeline step
    num_warps: int = 4
    stages: int = 2  # K/V LDS ring depth (1..3; 3 requests tiles two steps ahead, plain loop)
    q_in_smem: bool = False  # re-read Q fragments from LDS every KV step (else VGPR resident)
    swizzle: bool = True  # XOR swizzle of the LDS rows (else linear rows, bank conflicts)
    # 0: S^T, softmax, O^T of one tile after the other.  1: S^T of tile j+1 is computed
    # before the softmax of tile j (two S^T accumulators).  2: as 1, and every matrix
    # instruction of an iteration carries a fixed share of its vector work.
    pipe: int = 0
    # MFMA tile: 32 -> v_mfma_f32_32x32x16, 16 -> v_mfma_f32_16x16x32 (plain and slot loop).
    # The plain loops on 16x16x32 tiles take the row sums on the matrix pipe (one more product
    # per k-step with a ones operand) instead of by one add per score: +3.9 % / +1.2 % for the
    # trusted winners of D = 64 / 128, +1 % for the rolled causal loop at D = 128.
    mfma: int = 32
    # Plain loop over two LDS stages: False unrolls it by two (each copy of the step knows its
    # ring slot and the scheduler overlaps the end of one step with the start of the next),
    # True keeps one copy with the slot as a run-time value (about 50 registers fewer: for
    # the tiles whose unrolled loop does not fit the register file of two waves per SIMD).
    roll: bool = False
    # Plain ring loops (two or three stages) and slot loop: the K/V loads of the next tile are dealt over the
    # first `spread` groups of matrix instructions of a step instead of issued in one burst
    # behind the step's barrier, where all waves queue up at the CU's one load path
    # (measured: +1 % for the D = 128 slot loop with 8, +3 % for the D = 64 plain loop with 2-4,
    # -1...-2 % for the rolled 16x16x32 loop).
    spread: int = 0
    # Plain ring loops: a tile's exponentials are taken against the running max as it stands,
    # without the tile's own max (half a vector instruction per score, the exchange between the
    # lanes of a query and the update arithmetic).  A lane's p are bounded by their own sum,
    # which is checked before the second product: a tile that outgrew the running max (the
    # first one always takes its max) is computed again with it.  Same quotient O / l.
    # Measured: +3.6 % at D = 64 and D = 128 (S = 4096, full); nothing with the causal mask.
    trust: bool = False

    @property
    def threads(self) -> int:
        return self.num_warps * WAVE

    def as_dict(self):
        return asdict(self)

    def __str__(self):
        return (
            f"Br={self.Br},Bc={self.Bc},warps={self.num_warps},stages={self.stages},"
            f"q_smem={int(self.q_in_smem)},swz={int(self.swizzle)}"
            + (f",pipe={int(self.pipe)}" if self.pipe else "")
            + (f",mfma={self.mfma}" if self.mfma != 32 else "")
            + (",roll=1" if self.roll else "")
            + (f",spread={self.spread}" if self.spread else "")
            + (",trust=1" if self.trust else "")
        )


def default_spread(cfg: FAConfig) -> int:
    """The window the solver offers: 8 slots in the slot loop, 4 groups in the unrolled
    two-stage plain loop, none elsewhere (the kernel has it for the three-stage ring as well,
    where it measured -1.5 ... +1.4 %: the third stage already takes the burst out of the
    step that waits for it)."""
    if cfg.stages != 2 or cfg.roll:
        return 0
    return 8 if int(cfg.pipe) == 2 else (4 if int(cfg.pipe) == 0 else 0)


def smem_bytes(cfg: FAConfig, D: int) -> int:
    """`stages` K tiles and `stages` V tiles of Bc x D halves, and the Q tile when it is
    staged (flash_attn_tir.py:54-56; rows are never padded here)."""
    return (2 * cfg.stages * cfg.Bc + (cfg.Br if cfg.q_in_smem else 0)) * D * 2


def est_regs_per_thread(cfg: FAConfig, D: int) -> int:
    """Unified VGPR estimate per lane of the live fragments."""
    mq = cfg.Br // cfg.num_warps // 32
    o_acc = (D // 32) * mq * 16
    s_acc = (cfg.Bc // 32) * mq * 16
    p_h = s_acc // 2
    if int(cfg.pipe) == 1:
        s_acc *= 2
    elif int(cfg.pipe) == 2:
        # tile j's scores turn into packed halves while tile j+1's chains come to life
        s_acc, p_h = s_acc * 7 // 4, p_h // 2
    # Q fragments: all of them, or two k-steps' worth in flight (flash_attn_tir.py:65)
    q_frag = 2 * mq * 4 if cfg.q_in_smem else mq * (D // 16) * 4
    kv_frag = 2 * 4 * 2  # a few K / V fragments in flight
    return o_acc + s_acc + p_h + q_frag + kv_frag + 4 * mq + 40


# Largest register estimate that hipcc was seen to allocate without spilling, by
# (pipe, stages).  A wave that is alone on its SIMD may use all 512 registers, and the
# compiler then spends them on scheduling freedom: measured allocations are 1.35-1.4x the
# estimate for the plain loop with one LDS stage, 1.5x and more with two (the two unrolled
# steps overlap), 1.0-1.3x for the loops whose order is fixed by hand.  Beyond these the
# kernels spill to scratch memory inside the loop and run 2-15x slower.
SPILL_FREE_EST_REGS = {(0, 1): 365, (0, 2): 330, (0, 3): 330, (1, 2): 480, (2, 2): 480}


def expect_spill_free(cfg: FAConfig, D: int) -> bool:
    """Whether the compiler is expected to fit the kernel's registers (see above)."""
    limit = SPILL_FREE_EST_REGS.get((int(cfg.pipe), cfg.stages))
    return limit is not None and est_regs_per_thread(cfg, D) <= limit


def register_fill(cfg: FAConfig, D: int) -> float:
    """Estimated registers as a share of what a wave gets at the occupancy the kernel is
    compiled for.  From about 0.95 the unrolled two-stage plain loop spills (measured:
    D = 128, Br=256, Bc=128, 8 waves: 0.98, 3 to 67 spilled registers; rolled: none)."""
    return est_regs_per_thread(cfg, D) / (512 / target_waves_per_simd(cfg, D))


def target_waves_per_simd(cfg: FAConfig, D: int) -> int:
    """Waves per SIMD the kernel is compiled for: what the estimated registers and the LDS
    footprint let co-reside.  Without it the compiler spends the whole 512-register file on
    a workgroup of 4 waves or fewer (the only bound it knows is the block size), and a second
    workgroup that the LDS has room for cannot share the SIMDs."""
    regs8 = (est_regs_per_thread(cfg, D) + 7) // 8 * 8
    by_regs = 512 // regs8
    by_lds = (MAX_LDS // smem_bytes(cfg, D)) * cfg.num_warps // 4
    return max(1, min(by_regs, by_lds, 8))


def slot_schedule_ok(Bc: int, D: int, mfma: int = 32) -> bool:
    """Whether the slot-interleaved loop (`pipe == 2`) can be scheduled: the S^T chains are
    issued in pairs, and the exponentials, spread over the matrix instructions at a fixed
    rate, must be packed before the O^T instruction that consumes them (the same check as
    `Sched::ok()` in the kernel)."""
    if mfma == 16:
        kt, dk, kk, dt, acc = Bc // 16, D // 32, Bc // 32, D // 16, 4
    else:
        kt, dk, kk, dt, acc = Bc // 32, D // 16, Bc // 16, D // 32, 16
    if Bc % 64 or kt % 2:
        return False
    s_slots, pv_slots = kt * dk, kk * dt
    ns, ne = s_slots + pv_slots, kt * acc
    ne_s, pve = ne * 5 // 8, pv_slots - dt - 2
    if pve < 1:
        return False

    def e_end(t: int) -> int:
        if t < 0:
            return 0
        if t < s_slots:
            return (t + 1) * ne_s // s_slots
        return min(ne, ne_s + ((t - s_slots + 1) * (ne - ne_s) + pve - 1) // pve)

    return all(e_end(s_slots + k * dt - 2) >= 8 * (k + 1) for k in range(kk)) and e_end(ns - 3) == ne


def check_config(cfg: FAConfig, S_q: int, S_kv: int, D: int) -> None:
    # as the reference (flash_attn_tir.py:70-72); the LDS swizzles only touch the low chunk
    # bits of a row, so any row of a multiple of 8 chunks works
    assert D % 64 == 0 and D >= 64, "head dim must be a multiple of 64"
    assert cfg.Br % (32 * cfg.num_warps) == 0
    assert cfg.Bc % 32 == 0
    assert S_q % cfg.Br == 0 and S_kv % cfg.Bc == 0
    cpr = D // 8
    assert (cfg.Bc * cpr) % cfg.threads == 0
    assert 2 * (cfg.Bc * cpr) // cfg.threads <= 63
    assert cfg.threads <= 1024
    assert cfg.stages in (1, 2, 3)
    assert cfg.stages < 3 or int(cfg.pipe) == 0, "three stages: plain loop only"
    assert cfg.stages < 3 or 4 * (cfg.Bc * cpr) // cfg.threads <= 63
    assert int(cfg.pipe) in (0, 1, 2)
    assert cfg.mfma in (32, 16)
    assert cfg.mfma == 32 or int(cfg.pipe) != 1, "the 16x16x32 form exists for the plain and the slot loop"
    assert not cfg.pipe or cfg.stages == 2
    assert not cfg.roll or (int(cfg.pipe) == 0 and cfg.stages >= 2), "roll is a form of the plain ring loop"
    assert cfg.spread >= 0
    assert not cfg.spread or (cfg.stages >= 2 and int(cfg.pipe) in (0, 2)), \
        "the load window exists in the plain ring loops and the slot loop"
    assert not cfg.trust or (int(cfg.pipe) == 0 and cfg.stages >= 2), "trust is a form of the plain ring loops"
    assert int(cfg.pipe) != 2 or slot_schedule_ok(cfg.Bc, D, cfg.mfma)
    # a wave's Q rows go to LDS as whole 1 KiB runs
    assert not cfg.q_in_smem or (cfg.Br // cfg.num_warps * cpr) % WAVE == 0
    assert smem_bytes(cfg, D) <= MAX_LDS
    assert est_regs_per_thread(cfg, D) <= 512


# The kernel's running max follows a tile's max only when that lies more than this
# many powers of two above it: p stays below 2^tau (fp16 P and fp32 sums hold that as
# well as p <= 1), the quotient O / l is unchanged, and the O^T rescale is skipped for
# almost every tile.
LAZY_MAX_TAU = 8


def make_flash_attn_fwd(
    B: int, H: int, S_q: int, S_kv: int, D: int, cfg: FAConfig,
    softmax_scale: float | None = None, causal: bool = False,
) -> KernelSpec:
    """`causal` applies the top-left aligned mask (key j visible to query i iff j <= i).
    1-D grid of (S_q / Br) * B * H workgroups (reference: 2-D, flash_attn_tir.py:147; the
    kernel remaps ids so that each XCD owns whole (batch, head) slices), block `threads`."""
    check_config(cfg, S_q, S_kv, D)
    assert not causal or S_q == S_kv, "causal attention requires S_q == S_kv"
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    assert scale > 0, "the running max is taken of the unscaled scores: the scale must be positive"
    defines = {
        "DECA_B": B, "DECA_H": H, "DECA_SQ": S_q, "DECA_SKV": S_kv, "DECA_D": D,
        "DECA_BR": cfg.Br, "DECA_BC": cfg.Bc, "DECA_NW": cfg.num_warps,
        "DECA_STAGES": cfg.stages, "DECA_CAUSAL": int(causal),
        "DECA_SCALE": repr(float(scale)), "DECA_PIPE": int(cfg.pipe),
        "DECA_MIN_WAVES": target_waves_per_simd(cfg, D), "DECA_LAZY_TAU": LAZY_MAX_TAU,
    }
    if cfg.mfma == 16:
        defines["DECA_MFMA16"] = 1
    if cfg.roll:
        defines["DECA_ROLL"] = 1
    if cfg.q_in_smem:
        defines["DECA_QSMEM"] = 1
    if not cfg.swizzle:
        defines["DECA_SWIZZLE"] = 0
    if cfg.spread:
        defines["DECA_SPREAD"] = cfg.spread
    if cfg.trust:
        defines["DECA_TRUST"] = 1
    # The three-stage ring waits for part of its outstanding loads, which is only right
    # while the tile loads are the loop's only vector-memory traffic: a build that spills
    # (scratch stores share the counter and retire out of order) is refused at load time.
    return make_spec(
        TEMPLATE, defines, grid=((S_q // cfg.Br) * B * H, 1, 1), block=(cfg.threads, 1, 1), nargs=4,
        options=FAST_MATH_OPTIONS,
        meta={"cfg": str(cfg), "causal": causal, "no_scratch": cfg.stages > 2},
    )


FA_HIPCC_OPTIONS = FAST_MATH_OPTIONS


def build_flash_attn_to_file(
    shape, cfg: FAConfig, softmax_scale, arch: str, path: str, causal: bool = False
) -> str:
    """Builds in a worker process (no GPU context needed) and writes a code object."""
    B, H, S_q, S_kv, D = shape
    return build_kernel(make_flash_attn_fwd(B, H, S_q, S_kv, D, cfg, softmax_scale, causal), arch, path)


def build_flash_attn(spec: KernelSpec, target: str | None = None, dump_dir: str | None = None):
    """Compiles (or takes from the in-tree cache) and loads the kernel;
    `dump_dir` keeps the generated ISA for inspection."""
    import os

    from deca_amd.driver.driver import load_kernel

    arch = target or DEFAULT_ARCH
    if dump_dir:
        path = build_kernel(spec, arch, os.path.join(dump_dir, f"fa_{spec.key()}.hsaco"), dump_dir)
    else:
        path = cached_build(spec, arch)
    return load_kernel(spec, path)
