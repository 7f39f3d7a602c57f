"""
Enumerates the valid kernel configurations of one operator at one shape.

Same entry points as the reference's src/Solver.py (`solve_rowwise` :389,
`solve_gemm_tc` :473, `solve_flash_attn` :304), with the constraint sets
re-derived for CDNA4: 64-lane waves, a 512-entry unified VGPR file per lane and
SIMD shared by the resident waves, 160 KiB of LDS per CU with no L1 carve-out.

Each constraint set is written once against a tiny expression interface
(`_IntOps` on Python ints, `_Z3Ops` on Z3 bit-vectors).  When z3 is importable
the all-SAT loop with blocking clauses of the reference is used; otherwise the
(small, finite) domain product is enumerated exhaustively.  Both return the
same set; results are sorted so that the order does not depend on the solver.
Importing this module touches no GPU.
"""

from __future__ import annotations

import itertools

try:  # pragma: no cover - z3 is optional
    import z3 as _z3
except Exception:  # noqa: BLE001
    _z3 = None


# ---------------------------------------------------------------------------
# expression interface
# ---------------------------------------------------------------------------
class _IntOps:
    @staticmethod
    def const(v):
        return int(v)

    # Division by zero follows the bit-vector theory (all ones / the dividend),
    # so that both back ends agree on partially defined expressions.
    @staticmethod
    def udiv(a, b):
        return a // b if b else (1 << 32) - 1

    @staticmethod
    def urem(a, b):
        return a % b if b else a

    @staticmethod
    def ule(a, b):
        return a <= b

    @staticmethod
    def uge(a, b):
        return a >= b

    @staticmethod
    def eq(a, b):
        return a == b

    @staticmethod
    def ite(c, a, b):
        return a if c else b

    @staticmethod
    def implies(a, b):
        return (not a) or b

    @staticmethod
    def all_of(*xs):
        return all(xs)

    @staticmethod
    def any_of(*xs):
        return any(xs)


class _Z3Ops:  # pragma: no cover - exercised only when z3 is installed
    BITS = 32

    @classmethod
    def const(cls, v):
        return _z3.BitVecVal(int(v), cls.BITS)

    @staticmethod
    def udiv(a, b):
        return _z3.UDiv(a, b)

    @staticmethod
    def urem(a, b):
        return _z3.URem(a, b)

    @staticmethod
    def ule(a, b):
        return _z3.ULE(a, b)

    @staticmethod
    def uge(a, b):
        return _z3.UGE(a, b)

    @staticmethod
    def eq(a, b):
        return a == b

    @staticmethod
    def ite(c, a, b):
        return _z3.If(c, a, b)

    @staticmethod
    def implies(a, b):
        return _z3.Implies(a, b)

    @staticmethod
    def all_of(*xs):
        return _z3.And(*xs)

    @staticmethod
    def any_of(*xs):
        return _z3.Or(*xs)


def _enumerate(domains: dict, constraints, count: int, backend: str = "auto"):
    """All assignments of `domains` (name -> tuple of ints) that satisfy
    `constraints(ops, vars) -> list of boolean expressions`, as sorted tuples in
    the key order of `domains`, at most `count` of them.

    `backend`: "enum" (and "auto") walk the finite domains exhaustively; "z3"
    runs the same constraints through a Z3 all-SAT loop with blocking clauses,
    as the reference does (Solver.py:543-558).  The Z3 path is only taken when
    it is asked for by name: no environment this package was developed in has
    z3, so that path has never been executed."""
    names = list(domains)
    use_z3 = backend == "z3"
    if use_z3:
        if _z3 is None:
            raise RuntimeError("z3 backend requested but z3 is not importable")
        ops = _Z3Ops
        vs = {n: _z3.BitVec(n, _Z3Ops.BITS) for n in names}
        s = _z3.Solver()
        for n in names:
            s.add(_z3.Or([vs[n] == v for v in domains[n]]))
        s.add(*constraints(ops, vs))
        found = []
        while len(found) < count and s.check() == _z3.sat:
            m = s.model()
            vals = tuple(m[vs[n]].as_long() for n in names)
            found.append(vals)
            s.add(_z3.Or([vs[n] != v for n, v in zip(names, vals)]))
        return sorted(found)
    found = []
    for vals in itertools.product(*(domains[n] for n in names)):
        if all(constraints(_IntOps, dict(zip(names, vals)))):
            found.append(vals)
    return sorted(found)[:count]


def _satisfiable(domains: dict, constraints, backend: str = "auto") -> bool:
    return len(_enumerate(domains, constraints, 1, backend)) > 0


# ---------------------------------------------------------------------------
# row-wise (Softmax / RMSNorm)
# ---------------------------------------------------------------------------
ROWWISE_DOMAINS = {
    "tpr": (16, 32, 64, 128, 256, 512, 1024),
    "rpb": (1, 2, 4, 8, 16),
    "vec": (4, 8),
    "mode": (0, 1),
    "unroll": (1, 2, 4),
    "hint": (0, 1),
}


def _rowwise_constraints(arch, op: str, M: int, N: int, type_size: int, force_reg: bool):
    wave = arch.warp_size
    simds = arch.simds_per_cu

    def build(o, v):
        tpr, rpb, vec, mode, unroll, hint = (v[k] for k in ROWWISE_DOMAINS)
        c = o.const
        n, m = c(N), c(M)
        threads = tpr * rpb
        span = tpr * vec
        chunks = o.udiv(n + span - 1, span)
        out = [
            # whole waves, at most one workgroup's worth of lanes
            o.uge(threads, c(wave)), o.ule(threads, c(arch.max_threads_per_block)),
            o.eq(o.urem(threads, c(wave)), c(0)),
            o.eq(o.urem(n, vec), c(0)),
            o.eq(o.urem(m, rpb), c(0)),
            # a row keeps every vector lane of its lanes busy at least once
            o.ule(span, n),
            # enough workgroups to give every CU at least one
            o.uge(o.udiv(m, rpb), c(arch.sm_nums)),
            # cache-hinted accesses are 8 or 16 bytes
            o.implies(o.eq(hint, c(1)), o.uge(vec * type_size, c(8))),
        ]
        # VGPRs of the cached elements + bookkeeping, as in
        # rowwise_hip.est_regs_per_thread
        elems = o.ite(o.eq(mode, c(0)), chunks, unroll) * vec
        if op == "softmax":
            regs = o.udiv(elems * 9, c(8)) + 12
        else:
            regs = o.udiv(elems * 5, c(4)) + 16 + o.udiv(vec, c(2))
        waves_per_simd = o.udiv(o.udiv(threads, c(wave)) + (simds - 1), c(simds))

        def fits(r):
            return o.all_of(o.ule(r, c(arch.max_arch_vgprs)),
                            o.ule(o.udiv(r + 7, c(8)) * 8 * waves_per_simd, c(arch.vgprs_per_simd)))

        # reg mode falls back to its lean form (only the packed row stays in registers
        # between the passes), as in rowwise_hip.use_lean
        lean = o.udiv(chunks * vec * 5, c(8)) + 16
        out += [
            o.any_of(fits(regs), o.all_of(o.eq(mode, c(0)), fits(lean))),
            # reg mode is fully unrolled; twopass needs one full loop iteration
            o.implies(o.eq(mode, c(0)), o.all_of(o.eq(unroll, c(1)), o.ule(chunks, c(32)))),
            o.implies(o.eq(mode, c(1)), o.ule(unroll, o.udiv(n, span))),
        ]
        if force_reg:
            out.append(o.eq(mode, c(0)))
        return out

    return build


def solve_rowwise(
    arch,
    op: str,
    M: int,
    N: int,
    type_size: int = 2,
    twopass_min_n: int = 16384,
    count: int = 1024,
    backend: str = "auto",
):
    """
    Enumerate row-wise (Softmax / RMSNorm) kernel configurations.
    Args:
        arch: Arch, the target GPU
        op: "softmax" or "rmsnorm"
        M, N: rows and reduced dimension
        type_size: bytes per element (2 for fp16 / bf16)
        twopass_min_n: rows at least this long may also be streamed twice
            (always allowed when no register-cached config fits)
        count: the maximum number of solutions to find
    Returns:
        list of RowConfig
    """
    from deca_amd.kernels.rowwise_hip import RowConfig

    reg_only = _rowwise_constraints(arch, op, M, N, type_size, force_reg=True)
    force_reg = N < twopass_min_n and _satisfiable(ROWWISE_DOMAINS, reg_only, backend)
    cons = reg_only if force_reg else _rowwise_constraints(arch, op, M, N, type_size, False)
    return [
        RowConfig(
            threads_per_row=tpr, rows_per_block=rpb, vec=vec,
            mode="twopass" if mode else "reg", unroll=unroll, hint=bool(hint),
        )
        for tpr, rpb, vec, mode, unroll, hint in _enumerate(ROWWISE_DOMAINS, cons, count, backend)
    ]


# ---------------------------------------------------------------------------
# FP16 MFMA GEMM
# ---------------------------------------------------------------------------
GEMM_DOMAINS = {
    "bm": (64, 128, 256),
    "bn": (64, 128, 256),
    "bk": (32, 64),
    "wm": (32, 64, 128),
    "wn": (32, 64, 128),
    "st": (1, 2, 3, 4, 5),
    "epi": (0, 1),
    "direct": (0, 1),
    "mfma": (32, 16),  # 32: v_mfma_f32_32x32x16, 16: v_mfma_f32_16x16x32
}
GEMM_RASTERS = (0, 1, 2, 4, 8, 16)  # 0: 8 x 4 sub-blocks of tiles per XCD, neighbours in flight


def _gemm_constraints(arch, M: int, N: int, K: int, type_size: int):
    from deca_amd.kernels.gemm_hip import EPI_PAD, SPILL_FREE_EST_REGS

    wave = arch.warp_size
    simds = arch.simds_per_cu

    def build(o, v):
        bm, bn, bk, wm, wn, st, epi, direct, mfma = (v[k] for k in GEMM_DOMAINS)
        c = o.const
        m_, n_, k_ = c(M), c(N), c(K)
        waves = o.udiv(bm, wm) * o.udiv(bn, wn)
        threads = waves * wave
        out = [
            # wave tiles divide the workgroup tile, workgroup tiles divide the problem
            o.eq(o.urem(bm, wm), c(0)), o.eq(o.urem(bn, wn), c(0)),
            o.eq(o.urem(m_, bm), c(0)), o.eq(o.urem(n_, bn), c(0)), o.eq(o.urem(k_, bk), c(0)),
            # ring depth: asynchronous direct loads use 2..4 slots, staged loads 1..2,
            # never more than there are K tiles
            o.implies(o.eq(direct, c(1)), o.uge(st, c(2))),
            o.implies(o.eq(direct, c(0)), o.ule(st, c(2))),
            o.ule(st, o.udiv(k_, bk)),
            # the 16x16x32 body is written for the direct ring; its k-steps are 32 deep, and
            # with one k-step per K-tile it takes two tiles per loop iteration
            o.implies(o.eq(mfma, c(16)), o.eq(direct, c(1))),
            o.implies(o.all_of(o.eq(mfma, c(16)), o.eq(bk, c(32))),
                      o.eq(o.urem(o.udiv(k_, bk), c(2)), c(0))),
            # at most 32 accumulator tiles of 16 x 16 per wave: 128 x 128 wave tiles spill
            o.implies(o.eq(mfma, c(16)), o.ule(o.udiv(wm, c(16)) * o.udiv(wn, c(16)), c(32))),
            # 1 to 16 waves per workgroup
            o.uge(threads, c(wave)), o.ule(threads, c(arch.max_threads_per_block)),
            # cooperative 16-byte loads (and epilogue stores) evenly cover the tiles
            o.eq(o.urem(bm * o.udiv(bk, c(8)), threads), c(0)),
            o.eq(o.urem(bk * o.udiv(bn, c(8)), threads), c(0)),
            o.implies(o.eq(epi, c(1)), o.eq(o.urem(bm * o.udiv(bn, c(8)), threads), c(0))),
        ]
        # LDS: `st` A and B tiles; the staged epilogue reuses them
        pipe = st * (bm * bk + bk * bn) * type_size
        epi_bytes = o.ite(o.eq(epi, c(1)), bm * (bn + EPI_PAD) * type_size, c(0))
        out += [o.ule(pipe, c(arch.max_dyn_smem_per_block)),
                o.ule(epi_bytes, c(arch.max_dyn_smem_per_block))]
        # unified VGPRs: fp32 accumulators + two fragment sets + staging + bookkeeping,
        # as in gemm_hip.est_regs_per_thread
        acc = o.udiv(wm * wn, c(wave))
        frags = 4 * (o.udiv(wm, c(32)) + o.udiv(wn, c(32)))
        frags16 = 4 * (o.udiv(wm, c(16)) + 2 * o.udiv(wn, c(16)))  # A once, B twice
        chunks = o.udiv(o.udiv(bm * bk + bk * bn, c(8)), threads)
        staging = o.ite(o.eq(direct, c(1)), chunks, chunks * 4)
        regs = acc + o.ite(o.eq(mfma, c(16)), frags16, 2 * frags) + staging + 40
        regs8 = o.udiv(regs + 7, c(8)) * 8
        waves_per_simd = o.udiv(waves + (simds - 1), c(simds))
        out += [o.ule(regs, c(min(arch.vgprs_per_simd, SPILL_FREE_EST_REGS))),
                o.ule(regs8 * waves_per_simd, c(arch.vgprs_per_simd))]
        # the loads of the (st - 2) youngest tiles stay in flight across a wait: the
        # vector-memory counter holds 6 bits
        out.append(o.implies(o.all_of(o.eq(direct, c(1)), o.uge(st, c(3))),
                             o.ule((st - 2) * chunks, c(63))))
        # enough workgroups to give every CU at least one
        out.append(o.uge(o.udiv(m_, bm) * o.udiv(n_, bn), c(arch.sm_nums)))
        return out

    return build


def solve_gemm_tc(arch, M: int, N: int, K: int, type_size: int = 2, count: int = 65536,
                  backend: str = "auto"):
    """
    Enumerate FP16 MFMA GEMM tile configurations (see `GemmConfig`).
    Args:
        arch: Arch, the target GPU
        M, N, K: the GEMM shape (C[M, N] = A[M, K] @ B[K, N])
        type_size: bytes per input element (2 for fp16)
        count: the maximum number of solutions to find
    Returns:
        list of GemmConfig
    """
    from dataclasses import replace

    from deca_amd.kernels.gemm_hip import GemmConfig, agpr_split_fits, check_config, default_spread

    tiles = _enumerate(GEMM_DOMAINS, _gemm_constraints(arch, M, N, K, type_size), count, backend)
    results = []
    for bm, bn, bk, wm, wn, st, epi, direct, mfma in tiles:
        # The rasterisation group only needs to divide the workgroup rows and the
        # XCD remap needs a multiple of 8 workgroups; neither interacts with the
        # other constraints, so both are expanded here (reference: Solver.py:550-558).
        xcd = ((M // bm) * (N // bn)) % arch.num_xcd == 0
        for ras in GEMM_RASTERS:
            if ras != 0 and (M // bm) % ras != 0:
                continue
            cfg = GemmConfig(BM=bm, BN=bn, BK=bk, warp_m=wm, warp_n=wn, stages=st,
                             raster=ras, epi_smem=bool(epi), xcd=xcd or ras == 0,
                             direct=bool(direct), mfma=mfma)
            # a grid that leaves a partial last wave may split its tiles in four; the
            # block order (raster 0) needs whole rounds of 8 sub-blocks of 8 x 4 tiles
            cands = [cfg, replace(cfg, tail=True, xcd=True)]
            if mfma == 16 and wm >= 64:
                # the barrier of a K-tile after half of the row blocks of its last k-step
                cands += [replace(c, early=wm // 32) for c in cands]
            if mfma == 16:
                # the accumulators in accumulation registers, where both halves of the
                # register file have room for their share
                cands += [replace(c, agpr=True) for c in cands if agpr_split_fits(c)]
                # the tile loads dealt over the MFMA groups instead of issued in a burst
                if default_spread(cfg):
                    cands += [replace(c, spread=default_spread(cfg)) for c in cands]
            for cand in cands:
                if ras == 0 or cand.tail or cand.spread:
                    try:
                        check_config(cand, M, N, K)
                    except AssertionError:
                        continue
                results.append(cand)
    return results[:count]


# ---------------------------------------------------------------------------
# FlashAttention forward
# ---------------------------------------------------------------------------
FA_DOMAINS = {
    "br": (32, 64, 128, 256),
    "bc": (32, 64, 128),
    "nw": (1, 2, 4, 8),
    "st": (1, 2, 3),  # as the reference (Solver.py:334); 3 in the plain loop only
    "pipe": (0, 1, 2),
    "mfma": (32, 16),  # 16: v_mfma_f32_16x16x32 tiles (plain and slot loop)
    "qs": (0, 1),  # Q tile staged in LDS and re-read every KV step (Solver.py:335)
}
# `swizzle` stays out of the search (the reference enumerates it, Solver.py:336): linear LDS
# rows are never faster here, `FAConfig(swizzle=False)` exists for the comparison only.


def _fa_constraints(arch, B: int, H: int, S_q: int, S_kv: int, D: int, type_size: int,
                    max_est_regs: int):
    from deca_amd.kernels.flash_attn_hip import SPILL_FREE_EST_REGS, slot_schedule_ok

    wave = arch.warp_size
    simds = arch.simds_per_cu

    def build(o, v):
        br, bc, nw, st, pipe, mfma, qs = (v[k] for k in FA_DOMAINS)
        c = o.const
        slot_bcs = {m: [b for b in FA_DOMAINS["bc"] if slot_schedule_ok(b, D, m)] or [0]
                    for m in FA_DOMAINS["mfma"]}
        threads = nw * wave
        cpr = D // 8
        out = [
            # each wave owns a multiple of 32 Q rows; the tiles divide the sequences
            o.eq(o.urem(br, nw * 32), c(0)),
            o.eq(o.urem(c(S_q), br), c(0)), o.eq(o.urem(c(S_kv), bc), c(0)),
            # do not pipeline deeper than the number of KV tiles
            o.ule(st, o.udiv(c(S_kv), bc)),
            # cooperative 16-byte loads evenly cover a K/V tile; the outstanding
            # loads of one tile pair fit the 6-bit vector-memory counter
            o.eq(o.urem(bc * cpr, threads), c(0)),
            o.ule(o.udiv(bc * cpr, threads) * 2, c(63)),
            # (two tile pairs with the three-deep ring, which only the plain loop has)
            o.implies(o.eq(st, c(3)), o.all_of(o.eq(pipe, c(0)), o.ule(o.udiv(bc * cpr, threads) * 4, c(63)))),
            o.ule(threads, c(arch.max_threads_per_block)),
            # LDS: `st` K tiles and `st` V tiles, and the Q tile when it is staged
            # (a wave's Q rows are then loaded as whole 1 KiB runs)
            o.ule((st * bc * 2 + qs * br) * (D * type_size), c(arch.max_dyn_smem_per_block)),
            o.implies(o.eq(qs, c(1)), o.eq(o.urem(o.udiv(br, nw) * cpr, c(wave)), c(0))),
            # the software-pipelined loop runs one K tile ahead: two slots, two tiles
            o.implies(o.uge(pipe, c(1)), o.all_of(o.eq(st, c(2)), o.uge(o.udiv(c(S_kv), bc), c(2)))),
            # the slot-interleaved loop issues the S^T chains in pairs of 32-key blocks
            *[o.implies(o.all_of(o.eq(pipe, c(2)), o.eq(mfma, c(m))),
                        o.any_of(*[o.eq(bc, c(b)) for b in slot_bcs[m]])) for m in slot_bcs],
            # the 16x16x32 form exists for the plain and the slot loop
            o.implies(o.eq(mfma, c(16)), o.any_of(o.eq(pipe, c(0)), o.eq(pipe, c(2)))),
        ]
        # registers: O^T accumulator + S^T accumulator + P + Q fragments + K/V fragments
        mq = o.udiv(br, nw * 32)
        o_acc = mq * (D // 32 * 16)
        # two S^T tiles in the pipelined loop; in the slot-interleaved one, tile j's scores
        # turn into packed halves while tile j+1's chains come to life
        s_one = mq * o.udiv(bc, c(2))
        s_acc = o.ite(o.eq(pipe, c(1)), s_one * 2, o.ite(o.eq(pipe, c(2)), o.udiv(s_one * 7, c(4)), s_one))
        p_h = o.ite(o.eq(pipe, c(2)), o.udiv(mq * o.udiv(bc, c(4)), c(2)), mq * o.udiv(bc, c(4)))
        q_frag = o.ite(o.eq(qs, c(1)), mq * 8, mq * (D // 16 * 4))
        regs = o_acc + s_acc + p_h + q_frag + 16 + mq * 4 + 40
        regs8 = o.udiv(regs + 7, c(8)) * 8
        waves_per_simd = o.udiv(nw + (simds - 1), c(simds))
        out += [o.ule(regs, c(max_est_regs)), o.ule(regs8 * waves_per_simd, c(arch.vgprs_per_simd))]
        # what the compiler was seen to allocate without spilling, per loop shape
        for (p_, st_), limit in SPILL_FREE_EST_REGS.items():
            out.append(o.implies(o.all_of(o.eq(pipe, c(p_)), o.eq(st, c(st_))), o.ule(regs, c(limit))))
        # enough workgroups to give every CU at least one
        out.append(o.uge(o.udiv(c(S_q), br) * (B * H), c(arch.sm_nums)))
        return out

    return build


def solve_flash_attn(arch, B: int, H: int, S_q: int, S_kv: int, D: int, type_size: int = 2,
                     max_est_regs: int = 512, count: int = 1024, backend: str = "auto"):
    """
    Enumerate FlashAttention forward tile configurations.
    Args:
        arch: Arch, the target GPU
        B, H, S_q, S_kv, D: the attention shape
        type_size: bytes per input element (2 for fp16)
        max_est_regs: upper bound of the estimated unified VGPRs per lane
        count: the maximum number of solutions to find
    Returns:
        list of FAConfig
    """
    from deca_amd.kernels.flash_attn_hip import FAConfig

    if D % 64 != 0 or D < 64:  # flash_attn_tir.py:70-72
        return []
    from dataclasses import replace

    from deca_amd.kernels.flash_attn_hip import default_spread, register_fill

    cons = _fa_constraints(arch, B, H, S_q, S_kv, D, type_size, max_est_regs)
    results = []
    for br, bc, nw, st, pipe, mfma, qs in _enumerate(FA_DOMAINS, cons, count, backend):
        cfg = FAConfig(Br=br, Bc=bc, num_warps=nw, stages=st, pipe=int(pipe), mfma=mfma,
                       q_in_smem=bool(qs))
        forms = [cfg]
        # the plain ring loop in its one-copy form, where the unrolled one is expected to
        # run out of registers (it interacts with no other constraint: expanded here)
        if int(pipe) == 0 and st >= 2 and register_fill(cfg, D) >= 0.95:
            forms.append(replace(cfg, roll=True))
        # the next tile's loads dealt over the first matrix-instruction groups of a step
        if default_spread(cfg):
            forms.append(replace(cfg, spread=default_spread(cfg)))
        # the plain ring loops with the tile's exponentials taken against the running max as
        # it stands (no max of the tile first; a tile that outgrew it is done again)
        if int(pipe) == 0 and st >= 2:
            forms += [replace(f, trust=True) for f in forms]
        results += forms
    return results
