"""
Auto-tune the row-wise Softmax / RMSNorm forward kernels on an MI355X and
compare them with eager torch (`torch.softmax`, `F.rms_norm`).

Usage:
    python test_rowwise.py --op softmax --shape 16384 4096
    python test_rowwise.py --op rmsnorm --dtype bf16 --sweep

Same flags, messages and `deca_performance.log` records as the reference's
test_rowwise.py; this file is a tuning driver, not a pytest module.
"""

# Compile workers are spawned processes that re-import the builder module, so
# nothing heavy (torch, the HIP driver) is imported at module level here.
import argparse
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

__test__ = False  # keep pytest from collecting the driver


def parse_args(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--op", choices=["softmax", "rmsnorm"], default="softmax")
    parser.add_argument("--dtype", choices=["fp16", "bf16"], default="fp16")
    parser.add_argument("--shape", nargs=2, type=int, default=[16384, 4096], metavar=("M", "N"))
    parser.add_argument("--sweep", action="store_true", default=False,
                        help="tune the standard row-wise benchmark grid")
    parser.add_argument("--eps", type=float, default=1e-6, help="RMSNorm epsilon")
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

    tuner = Tuner(args.op, arch, arch_str, args.top_n, args.jobs, args.finalists, args.rounds,
                  cache_path=_cache_path(args), retune=args.retune, timing=args.timing)
    return tuner.tune(*shape, log=log, dtype=args.dtype, eps=args.eps)


def main(argv=None):
    from deca_amd.kernels.rowwise_bench import standard_shapes
    from deca_amd.utils.helper import GPUDetector

    args = parse_args(argv)
    arch = GPUDetector.create_gpu_instance()
    arch_str = arch.gcn_arch

    shapes = standard_shapes(args.op) if args.sweep else [tuple(args.shape)]
    log_path = os.path.join(ROOT, "deca_performance.log")
    summary = []
    with open(log_path, "a") as log:
        for shape in shapes:
            try:
                cfg, gbps, torch_gbps = tune(args, shape, arch, arch_str, log)
            except RuntimeError as e:
                # e.g. out of memory; keep sweeping the other shapes
                if not args.sweep:
                    raise
                print(f"skipping {shape}: {e}", flush=True)
                continue
            summary.append((shape, cfg, gbps, torch_gbps))

    if len(summary) > 1:
        print(f"\nSummary of {args.op} ({args.dtype}) on {arch.name}:")
        print(f"{'M':>6} {'N':>7} | {'DeCA':>7} {'torch':>7} {'%peak':>5} {'ratio':>6} | config")
        for (M, N), cfg, gbps, torch_gbps in summary:
            print(
                f"{M:>6} {N:>7} | {gbps:>7.0f} {torch_gbps:>7.0f} "
                f"{100 * gbps / arch.dram_bw:>5.0f} {gbps / torch_gbps:>6.3f} | {cfg}"
            )
    return summary


if __name__ == "__main__":
    main()
