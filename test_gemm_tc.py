"""
Auto-tune the FP16 MFMA GEMM (C = A @ B, fp32 accumulation) on an MI355X and
compare it with torch.matmul (hipBLASLt / rocBLAS).

Usage:
    python test_gemm_tc.py --shape 4096 4096 4096
    python test_gemm_tc.py --sweep

Same flags, messages, `deca_performance.log` records and sweep CSV as the
reference's test_gemm_tc.py; this file is a tuning driver, not a pytest module.
"""

# Compile workers are spawned processes that re-import the builder module, so
# nothing heavy (torch, the HIP driver) is imported at module level here.
import argparse
import csv
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

__test__ = False  # keep pytest from collecting the driver


def parse_args(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--shape", nargs=3, type=int, default=[4096, 4096, 4096],
                        metavar=("M", "N", "K"))
    parser.add_argument("--sweep", action="store_true", default=False,
                        help="tune the square 2K-16K benchmark grid")
    parser.add_argument("--dtype", choices=["fp16", "bf16"], default="fp16",
                        help="type of A, B and C (accumulation is always fp32)")
    parser.add_argument("--inputs", choices=["uniform", "normal"], default="uniform",
                        help="operand distribution: U(-1,1), the benchmark's, or N(0,1) as the "
                             "reference draws them (gemm_bench.py:26-31); winners are stored "
                             "per distribution")
    parser.add_argument("--top_n", type=int, default=24,
                        help="number of ranked configs to compile and measure (0 = all)")
    parser.add_argument("--jobs", type=int, default=min(16, os.cpu_count() or 1),
                        help="parallel compile workers")
    parser.add_argument("--finalists", type=int, default=3,
                        help="best configs re-timed against torch in the final round")
    parser.add_argument("--cache", nargs="?", const="", default=None, metavar="JSON",
                        help="store the winner in (and reuse it from) a JSON file; without a "
                             "path, the table shipped with the package")
    parser.add_argument("--retune", action="store_true", default=False,
                        help="with --cache: search again and replace the stored winner")
    parser.add_argument("--rounds", type=int, default=5,
                        help="interleaved timing rounds of the final comparison")
    parser.add_argument("--timing", choices=["back_to_back", "events"], default="back_to_back",
                        help="back_to_back: batches of launches between one event pair (what "
                             "bench.py times); events: one event pair and one synchronisation "
                             "per call, as the reference times")
    return parser.parse_args(argv)


def _cache_path(args):
    if args.cache is None:
        return None
    from deca_amd import tuned

    return args.cache or tuned.DEFAULT_PATH


def tune(args, shape, arch, arch_str, log):
    from deca_amd.Tuner import Tuner

    tuner = Tuner("GEMM", arch, arch_str, args.top_n, args.jobs, args.finalists, args.rounds,
                  cache_path=_cache_path(args), retune=args.retune, timing=args.timing)
    return tuner.tune(*shape, log=log, dtype=args.dtype, inputs=args.inputs)


def write_sweep_csv(summary, path):
    """Writes DeCA and torch TFLOPS for the 2K-16K sweep."""
    with open(path, "w", newline="") as f:
        writer = csv.writer(f)
        writer.writerow(["M", "N", "K", "DeCA_TFLOPS", "torch_TFLOPS", "ratio"])
        for (M, N, K), _, tflops, torch_tflops in summary:
            ratio = tflops / torch_tflops if torch_tflops else float("nan")
            writer.writerow([M, N, K, f"{tflops:.4f}", f"{torch_tflops:.4f}", f"{ratio:.4f}"])


def main(argv=None):
    from deca_amd.kernels.gemm_bench import standard_shapes
    from deca_amd.utils.helper import GPUDetector

    args = parse_args(argv)
    arch = GPUDetector.create_gpu_instance()
    arch_str = arch.gcn_arch

    shapes = standard_shapes() if args.sweep else [tuple(args.shape)]
    log_path = os.path.join(ROOT, "deca_performance.log")
    summary = []
    with open(log_path, "a") as log:
        for shape in shapes:
            try:
                cfg, tflops, torch_tflops = tune(args, shape, arch, arch_str, log)
            except RuntimeError as e:
                # e.g. out of memory; keep sweeping the other shapes
                if not args.sweep:
                    raise
                print(f"skipping {shape}: {e}", flush=True)
                continue
            summary.append((shape, cfg, tflops, torch_tflops))

    if len(summary) > 1:
        print(f"\nSummary of FP16 MFMA GEMM on {arch.name}:")
        print(f"{'M':>6} {'N':>6} {'K':>6} | {'DeCA':>6} {'torch':>6} {'ratio':>6} | config")
        for (M, N, K), cfg, tflops, torch_tflops in summary:
            print(f"{M:>6} {N:>6} {K:>6} | {tflops:>6.1f} {torch_tflops:>6.1f} "
                  f"{tflops / torch_tflops:>6.3f} | {cfg}")

    if args.sweep:
        csv_path = os.path.join(ROOT, "gemm_tc_2K_to_16K.csv")
        write_sweep_csv(summary, csv_path)
        print(f"wrote {len(summary)} shapes to {csv_path}", flush=True)
    return summary


if __name__ == "__main__":
    main()
