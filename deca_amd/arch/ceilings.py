"""
Measures what one MI355X sustains on nothing but roofline-limited work: the
ceilings behind the constants of `arch/MI355X.py` and behind every "fraction of
peak" this package reports.  The reference pastes such measurements into its
arch files as comments (arch/H20.py:35-60); here they can be taken again:

    python -m deca_amd.arch.ceilings             # HBM streams and matrix-pipe loops
    python -m deca_amd.arch.ceilings --sclk      # + shader clock while the tuned 8192^3 GEMM runs

- HBM: a 16-byte-per-lane copy, a read-only and a write-only stream of 128 MiB
  buffers, rotating over 8 buffer pairs (2 GiB, several times the 256 MiB Infinity
  Cache) so that every launch streams from memory.
- LDS and the L2 -> LDS path: per workgroup of 8 waves (one workgroup per CU), some waves
  stream conflict-free ds_read_b128, others direct global->LDS loads from an L2-resident
  region; alone and together, which shows what the two share.
- Vector ALU: register-only loops of the instructions the softmax of FlashAttention is made
  of, and of an MFMA followed by such work in the same wave (what one wave overlaps by itself).
- Matrix pipe: register-only loops of v_mfma_f32_32x32x16_f16 and
  v_mfma_f32_16x16x32_f16 (no memory traffic) on N(0,1) and on all-zero operands:
  with real data the board's power limit, not its 2.4 GHz clock, sets the rate.
"""

from __future__ import annotations

import argparse
import itertools
import subprocess
import sys
import threading
import time

from deca_amd.kernels.build import cached_build, make_spec

TEMPLATE = "ceilings.hip"
STREAM_BYTES = 128 * 1024 * 1024
ROTATE = 8
MFMA_ITERS = 4096
MFMA_FLOPS = {3: 2 * 32 * 32 * 16, 4: 2 * 16 * 16 * 32}


def stream_spec(mode: int, threads: int, unroll: int, nt: int, wgs: int):
    chunks = STREAM_BYTES // 16
    grid = wgs if wgs else -(-chunks // (threads * unroll))
    return make_spec(TEMPLATE, {"DECA_CEILING": mode, "DECA_THREADS": threads, "DECA_CHUNKS": chunks,
                                "DECA_UNROLL": unroll, "DECA_NT": nt},
                     (grid, 1, 1), (threads, 1, 1), 2, options=[])


def mfma_spec(mode: int, nacc: int, blocks: int):
    return make_spec(TEMPLATE, {"DECA_CEILING": mode, "DECA_THREADS": 256, "DECA_ITERS": MFMA_ITERS,
                                "DECA_NACC": nacc}, (blocks, 1, 1), (256, 1, 1), 2, options=[])


LDS_ITERS = 4000
LDS_MIXES = [(8, 0), (4, 0), (0, 4), (0, 2), (4, 4), (6, 2)]  # (reading waves, loading waves)


def lds_spec(readers: int, loaders: int):
    return make_spec(TEMPLATE, {"DECA_CEILING": 5, "DECA_READERS": readers, "DECA_LOADERS": loaders,
                                "DECA_ITERS": LDS_ITERS}, (256, 1, 1), (512, 1, 1), 2, options=[])


VALU_ITERS = 4096
VALU_OPS = {0: "16 v_fma_f32", 1: "16 v_exp_f32", 2: "16 v_cvt_pk_f16_f32", 3: "16 v_max3_f32",
            4: "4 x (MFMA 32x32x16 + 2 v_exp_f32)", 5: "4 x (MFMA 32x32x16 + 8 v_fma_f32)",
            6: "4 x MFMA 32x32x16",
            7: "4 x (MFMA 32x32x16 + 2 v_fma_f32 + v_exp_f32 + v_cvt_pk_f16_f32 + v_max3_f32)",
            8: "4 x (MFMA 32x32x16 + 2 x (2 v_fma_f32 + v_exp_f32 + v_cvt_pk_f16_f32 + v_max3_f32))",
            9: "4 x (MFMA 32x32x16 + 2 x (2 v_fma_f32 + v_exp_f32 + v_cvt_pk_f16_f32 + v_max3_f32) "
               "+ 2 v_accvgpr_read_b32)",
            10: "16 dependent v_fma_f32", 11: "16 dependent v_exp_f32", 12: "16 dependent v_max3_f32",
            13: "16 x (v_exp_f32, dependent v_add_f32)"}
VALU_CHAIN_OPS = (0, 1, 10, 11, 12, 13)  # these also run with one and two waves per SIMD


VALU_RUNS = [(op, 0) for op in VALU_OPS if op != 9 and op < 10] + [(4, 1), (5, 1), (6, 1), (7, 1), (8, 1), (9, 1)]


def valu_spec(op: int, agpr: int = 0, waves_per_simd: int = 8):
    blocks = 256 * waves_per_simd
    return make_spec(TEMPLATE, {"DECA_CEILING": 6, "DECA_OP": op, "DECA_ITERS": VALU_ITERS,
                                "DECA_ACC_AGPR": agpr},
                     (blocks, 1, 1), (256, 1, 1), 2, options=[])


STREAM_VARIANTS = [(t, u, nt, w) for t, u, nt, w in itertools.product(
    (256, 512, 1024), (1, 2, 4), (0, 1), (0, 2048))]
MFMA_VARIANTS = [(3, 8, 1024), (3, 8, 2048), (4, 16, 1024), (4, 16, 2048)]


def all_specs():
    specs = [stream_spec(m, *v) for m in (0, 1, 2) for v in STREAM_VARIANTS]
    return (specs + [mfma_spec(*v) for v in MFMA_VARIANTS] + [lds_spec(*m) for m in LDS_MIXES]
            + [valu_spec(op, agpr) for op, agpr in VALU_RUNS]
            + [valu_spec(op, 0, w) for op in VALU_CHAIN_OPS for w in (1, 2)])


def build():
    from concurrent.futures import ThreadPoolExecutor

    unique = {spec.key(): spec for spec in all_specs()}  # grids differ, code objects do not
    with ThreadPoolExecutor(8) as pool:
        list(pool.map(cached_build, unique.values()))


def measure_streams(out=sys.stdout):
    import torch

    from deca_amd.driver.driver import load_kernel

    n = STREAM_BYTES // 4
    bufs = [(torch.randn(n, device="cuda"), torch.empty(n, device="cuda")) for _ in range(ROTATE)]
    names = {0: "copy", 1: "read only", 2: "write only"}
    moved = {0: 2 * STREAM_BYTES, 1: STREAM_BYTES, 2: STREAM_BYTES}
    for mode in (0, 1, 2):
        best = (0.0, None)
        for v in STREAM_VARIANTS:
            spec = stream_spec(mode, *v)
            kern = load_kernel(spec, cached_build(spec))
            kern.time(bufs, ROTATE)
            t = min(kern.time(bufs, 4 * ROTATE) for _ in range(3))
            rate = moved[mode] / t / 1e9
            if rate > best[0]:
                best = (rate, v, t)
        rate, (threads, unroll, nt, wgs), t = best
        print(f"HBM {names[mode]:10s}: {rate:7.0f} GB/s ({t * 1e6:.1f} us per {STREAM_BYTES >> 20} MiB"
              f"{' in + out' if mode == 0 else ''}; best of {len(STREAM_VARIANTS)} variants: "
              f"{threads} lanes, {unroll} in flight, {'non-temporal' if nt else 'plain'}, "
              f"{'grid-stride over ' + str(wgs) + ' workgroups' if wgs else 'one pass per lane'})",
              file=out, flush=True)


def run_copy(launches: int = 16, out=sys.stdout):
    """Only the plain copy (512 lanes, non-temporal, one 16-byte access per lane), `launches`
    times over rotating 128 MiB buffers: the kernel of known traffic that the L2 <-> fabric
    counters of rocprofv3 (FETCH_SIZE, WRITE_SIZE) are scaled against."""
    import torch

    from deca_amd.driver.driver import load_kernel

    n = STREAM_BYTES // 4
    bufs = [(torch.randn(n, device="cuda"), torch.empty(n, device="cuda")) for _ in range(ROTATE)]
    spec = stream_spec(0, 512, 1, 1, 0)
    kern = load_kernel(spec, cached_build(spec))
    for i in range(launches):
        kern(*bufs[i % ROTATE])
    torch.cuda.synchronize()
    assert torch.equal(bufs[0][0], bufs[0][1])
    print(f"copy: {launches} launches of {STREAM_BYTES} bytes in, {STREAM_BYTES} bytes out", file=out, flush=True)


def measure_lds(out=sys.stdout):
    """Bytes per nominal 2.4 GHz clock and CU (these loops draw little power: the shader
    clock stays at its maximum)."""
    import torch

    from deca_amd.driver.driver import load_kernel

    src = torch.zeros(65 * 65536, dtype=torch.uint8, device="cuda")
    res = torch.empty(256 * 512, device="cuda")
    for readers, loaders in LDS_MIXES:
        spec = lds_spec(readers, loaders)
        kern = load_kernel(spec, cached_build(spec))
        kern.time([(src, res)], 1)
        t = min(kern.time([(src, res)], 3) for _ in range(3))
        clocks = t * 2.4e9
        per_wave = LDS_ITERS * 8 * 1024
        print(f"LDS: {readers} waves ds_read_b128 + {loaders} waves global->LDS per CU: {t * 1e3:.3f} ms; "
              f"had each stream run all of it: reads {readers * per_wave / clocks:5.1f} B/clk/CU, "
              f"loads {loaders * per_wave / clocks:5.1f} B/clk/CU", file=out, flush=True)


def measure_valu(out=sys.stdout):
    """Clocks per trip and SIMD at the nominal 2.4 GHz: 2048 workgroups of 4 waves are 8 waves
    per SIMD over the 256 CUs, all resident at once."""
    import torch

    from deca_amd.driver.driver import load_kernel

    x = torch.rand(8192, device="cuda")
    x[4096:] = 0  # the MFMA operands: zeros draw no power, the clock stays at its maximum
    res = torch.empty(2048 * 256, device="cuda")
    runs = [(op, agpr, 8) for op, agpr in VALU_RUNS] + [(op, 0, w) for op in VALU_CHAIN_OPS for w in (1, 2)]
    for op, agpr, waves in runs:
        what = VALU_OPS[op] + (", accumulators in AGPRs" if agpr else "")
        spec = valu_spec(op, agpr, waves)
        kern = load_kernel(spec, cached_build(spec))
        kern.time([(x, res)], 1)
        t = min(kern.time([(x, res)], 3) for _ in range(3))
        clocks = t * 2.4e9 / VALU_ITERS / waves
        print(f"VALU: {what} per trip, {waves} waves per SIMD: {t * 1e3:.3f} ms, {clocks:6.1f} clocks per trip "
              f"and wave", file=out, flush=True)


def measure_mfma(out=sys.stdout):
    import torch

    from deca_amd.driver.driver import load_kernel

    operands = {"N(0,1)": torch.randn(4096 * 8, device="cuda").half(),
                "zeros": torch.zeros(4096 * 8, device="cuda").half()}
    for mode, nacc, blocks in MFMA_VARIANTS:
        spec = mfma_spec(mode, nacc, blocks)
        kern = load_kernel(spec, cached_build(spec))
        res = torch.empty(blocks * 256, device="cuda")
        flops = blocks * 4 * MFMA_ITERS * nacc * MFMA_FLOPS[mode]
        form = "32x32x16" if mode == 3 else "16x16x32"
        for name, x in operands.items():
            kern.time([(x, res)], 2)
            t = min(kern.time([(x, res)], 5) for _ in range(3))
            print(f"MFMA {form} f16, {blocks} workgroups x 4 waves x {nacc} tiles, {name:6s}: "
                  f"{flops / t / 1e12:6.0f} TFLOP/s ({t * 1e3:.3f} ms)", file=out, flush=True)


def board_state():
    """Shader clock, socket power and power cap as rocm-smi reports them, on one line."""
    try:
        text = subprocess.run(["rocm-smi", "--showclocks", "--showpower", "--showmaxpower"],
                              capture_output=True, text=True, timeout=20).stdout
    except (OSError, subprocess.SubprocessError) as err:
        return f"rocm-smi failed: {err}"
    keep = [line.split(":", 1)[1].strip() for line in text.splitlines()
            if "sclk" in line or "Power (W)" in line]
    try:  # the socket power comes from amd-smi where rocm-smi does not print it
        text = subprocess.run(["amd-smi", "metric", "-p"], capture_output=True, text=True, timeout=20).stdout
        keep += [line.strip() for line in text.splitlines() if "SOCKET_POWER" in line]
    except (OSError, subprocess.SubprocessError):
        pass
    return " | ".join(keep)


def sample_while(launch, label, out, seconds=3):
    """Prints the board state once a second while `launch()` (a batch of asynchronous
    launches) repeats on a worker thread."""
    import torch

    stop = threading.Event()

    def work():
        while not stop.is_set():
            launch()
            torch.cuda.synchronize()

    worker = threading.Thread(target=work)
    worker.start()
    for _ in range(seconds):
        time.sleep(1.0)
        print(f"{label}: {board_state()}", file=out, flush=True)
    stop.set()
    worker.join()


def measure_sclk(out=sys.stdout):
    """Shader clock and socket power reported by rocm-smi while the tuned 8192^3 GEMM, the
    tuned FlashAttention kernels and the register-only MFMA loop repeat."""
    import torch

    from deca_amd import tuned
    from deca_amd.driver.driver import load_kernel
    from deca_amd.kernels.attn_bench import attn_flops, make_qkv
    from deca_amd.kernels.flash_attn_hip import build_flash_attn, make_flash_attn_fwd
    from deca_amd.kernels.gemm_hip import build_gemm_tc, make_gemm_tc

    n = 8192
    cfg = tuned.lookup(tuned.make_key("GEMM", (n, n, n), "float16", "gfx950", False, "uniform"))
    kern = build_gemm_tc(make_gemm_tc(n, n, n, cfg))
    print(f"idle: {board_state()}", file=out, flush=True)
    makers = {"U(-1,1)": lambda: (2 * torch.rand(n, n, device="cuda") - 1).half(),
              "zeros": lambda: torch.zeros(n, n, device="cuda", dtype=torch.float16)}
    for name, make in makers.items():
        a, b = make(), make()
        c = torch.empty(n, n, device="cuda", dtype=torch.float16)
        sample_while(lambda: [kern(a, b, c) for _ in range(50)], f"GEMM {n}^3 [{cfg}] on {name}", out)
        t = kern.time([(a, b, c)], 20)
        print(f"  -> {2 * n**3 / t / 1e12:.0f} TFLOP/s", file=out, flush=True)
    for d in (128, 64):
        shape = (4, 16, 4096, 4096, d)
        fcfg = tuned.lookup(tuned.make_key("flash_attn", shape, "float16", "gfx950", False))
        fa = build_flash_attn(make_flash_attn_fwd(*shape, fcfg, None, False))
        q, k, v = make_qkv(*shape)
        o = torch.empty_like(q)
        sample_while(lambda: [fa(q, k, v, o) for _ in range(50)], f"FlashAttention D{d} [{fcfg}] on N(0,1)", out)
        t = fa.time([(q, k, v, o)], 20)
        print(f"  -> {attn_flops(*shape, False) / t / 1e12:.0f} TFLOP/s", file=out, flush=True)
    spec = mfma_spec(3, 8, 2048)
    loop = load_kernel(spec, cached_build(spec))
    x = torch.randn(4096 * 8, device="cuda").half()
    res = torch.empty(2048 * 256, device="cuda")
    sample_while(lambda: [loop(x, res) for _ in range(10)], "MFMA 32x32x16 register-only loop on N(0,1)", out)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--build", action="store_true", help="compile the probe kernels and exit")
    ap.add_argument("--sclk", action="store_true", help="also sample the shader clock under the GEMM")
    ap.add_argument("--copy-only", action="store_true",
                    help="run only the plain copy kernel (the calibration target of the traffic counters)")
    args = ap.parse_args(argv)
    build()
    if args.build:
        return
    if args.copy_only:
        run_copy()
        return
    measure_streams()
    measure_lds()
    measure_valu()
    measure_mfma()
    if args.sclk:
        measure_sclk()


if __name__ == "__main__":
    main()
