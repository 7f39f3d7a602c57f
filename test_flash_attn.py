"""
Auto-tune the FlashAttention forward kernel on an MI355X and compare it with
torch's fused scaled_dot_product_attention.

Usage:
    python test_flash_attn.py --shape 4 16 4096 128            # B H S D
    python test_flash_attn.py --shape 4 16 4096 128 --causal
    python test_flash_attn.py --sweep

Same flags, messages and `deca_performance.log` records as the reference's
test_flash_attn.py; this file is a tuning driver, not a pytest module.
"""

import argparse
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

__test__ = False  # keep pytest from collecting the driver


def parse_args(argv=None):
    parser = argparse.ArgumentParser()
    parser.add_argument("--shape", nargs="*", type=int, default=[4, 16, 4096, 128],
                        help="B H S D (S_q = S_kv) or B H S_q S_kv D")
    parser.add_argument("--sweep", action="store_true", default=False,
                        help="tune the standard FlashAttention-2 benchmark grid")
    parser.add_argument("--causal", action="store_true", default=False,
                        help="top-left aligned causal mask (S_q == S_kv)")
    parser.add_argument("--top_n", type=int, default=16,
                        help="number of ranked configs to compile and measure (0 = all)")
    parser.add_argument("--jobs", type=int, default=min(16, os.cpu_count() or 1),
                        help="parallel compile workers")
    parser.add_argument("--finalists", type=int, default=3,
                        help="best configs re-timed against SDPA in the final round")
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


def parse_shape(s):
    if len(s) == 4:
        B, H, S, D = s
        return (B, H, S, S, D)
    assert len(s) == 5, "--shape expects B H S D or B H S_q S_kv D"
    return tuple(s)


def _cache_path(args):
    if args.cache is None:
        return None
    from deca_amd import tuned

    return args.cache or tuned.DEFAULT_PATH


def tune(args, shape, arch, arch_str, log):
    from deca_amd.Tuner import Tuner

    tuner = Tuner("flash_attn", arch, arch_str, args.top_n, args.jobs, args.finalists, args.rounds,
                  cache_path=_cache_path(args), retune=args.retune, timing=args.timing)
    return tuner.tune(*shape, log=log, causal=args.causal)


def main(argv=None):
    from deca_amd.kernels.attn_bench import standard_shapes
    from deca_amd.utils.helper import GPUDetector

    args = parse_args(argv)
    arch = GPUDetector.create_gpu_instance()
    arch_str = arch.gcn_arch

    if args.sweep:
        shapes = [(B, H, S, S, D) for B, H, S, D in standard_shapes()]
    else:
        shapes = [parse_shape(args.shape)]
    log_path = os.path.join(ROOT, "deca_performance.log")
    summary = []
    with open(log_path, "a") as log:
        for shape in shapes:
            cfg, tflops, sdpa_tflops = tune(args, shape, arch, arch_str, log)
            summary.append((shape, cfg, tflops, sdpa_tflops))

    if len(summary) > 1:
        print(f"\nSummary of FlashAttention forward ({'causal' if args.causal else 'full'}) "
              f"on {arch.name}:")
        print(f"{'B':>3} {'H':>3} {'S':>6} {'D':>4} | {'DeCA':>7} {'SDPA':>7} {'ratio':>6} | config")
        for (B, H, S_q, _, D), cfg, tflops, sdpa_tflops in summary:
            print(f"{B:>3} {H:>3} {S_q:>6} {D:>4} | {tflops:>7.1f} {sdpa_tflops:>7.1f} "
                  f"{tflops / sdpa_tflops:>6.3f} | {cfg}")
        from deca_amd.kernels import attn_bench

        print(f"SDPA column: torch.nn.functional.scaled_dot_product_attention, back end: "
              f"{attn_bench.SDPA_BACKEND}")
    return summary


if __name__ == "__main__":
    main()
