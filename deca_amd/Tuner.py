"""
The tuning loop shared by the three drivers: solve -> rank -> compile the
top-N in parallel worker processes -> load, verify and time each on the GPU ->
re-time the finalists interleaved with torch -> append a record to
deca_performance.log.

The reference's `Tuner` is an empty shell (src/Tuner.py:3-26) and each of its
drivers carries its own copy of this loop (test_gemm_tc.py:70-171,
test_rowwise.py:45-147, test_flash_attn.py:52-157); here the drivers are thin
front-ends over one implementation with the same stages, messages and log
format.
"""

from __future__ import annotations

import multiprocessing as mp
import os
import tempfile
import time
from concurrent.futures import ProcessPoolExecutor, as_completed
from concurrent.futures.process import BrokenProcessPool
from datetime import datetime

DEFAULT_ARCH_STR = "gfx950"


def _run_build(fn_path: str, args: tuple):
    """Worker entry: imports `module:function` and calls it (no GPU context)."""
    import importlib

    mod, name = fn_path.split(":")
    return getattr(importlib.import_module(mod), name)(*args)


def build_all(fn_path: str, args_of: dict, jobs: int, prefix: str = "deca_tune_"):
    """Compiles configs in parallel; returns {cfg: path of the code object}.

    `args_of[cfg]` is a function path -> argument tuple for `fn_path`
    ("package.module:function").  A dead worker breaks the whole pool; the
    affected configs are rebuilt serially (reference: test_gemm_tc.py:70-98).
    """
    tmpdir = tempfile.mkdtemp(prefix=prefix)
    path_of = {cfg: os.path.join(tmpdir, f"cfg{i}.hsaco") for i, cfg in enumerate(args_of)}
    paths, crashed = {}, []
    if jobs <= 1:
        crashed = list(args_of)
    else:
        with ProcessPoolExecutor(max_workers=jobs, mp_context=mp.get_context("spawn")) as pool:
            futures = {
                pool.submit(_run_build, fn_path, args_of[cfg](path_of[cfg])): cfg for cfg in args_of
            }
            for fut in as_completed(futures):
                cfg = futures[fut]
                try:
                    paths[cfg] = fut.result()
                except BrokenProcessPool:
                    crashed.append(cfg)
                except Exception as e:  # noqa: BLE001
                    print(f"{cfg} failed to build: {str(e)[-200:]}", flush=True)
    for cfg in crashed:
        try:
            paths[cfg] = _run_build(fn_path, args_of[cfg](path_of[cfg]))
        except Exception as e:  # noqa: BLE001
            print(f"{cfg} failed to build: {str(e)[-200:]}", flush=True)
    return paths


class Tuner:
    """Tunes one operator at one shape.

    Args:
        operator: "GEMM" (fp16 MFMA GEMM), "softmax", "rmsnorm" or "flash_attn"
        arch: hardware model (detected from the visible device when omitted)
    """

    OPERATORS = ("GEMM", "softmax", "rmsnorm", "flash_attn")

    def __init__(self, operator: str = "GEMM", arch=None, arch_str: str | None = None,
                 top_n: int | None = None, jobs: int | None = None, finalists: int = 3,
                 rounds: int = 5, cache_path: str | None = None, retune: bool = False,
                 timing: str = "back_to_back"):
        from deca_amd.kernels.attn_bench import TIMINGS

        assert operator in self.OPERATORS
        assert timing in TIMINGS, timing
        # "back_to_back": candidates and finalists are timed in batches of launches between
        # one event pair, as bench.py times them; "events": one event pair and one
        # synchronisation per call, the reference's procedure (attn_bench.py:35-70)
        self.timing = timing
        self.operator = operator
        if arch is None:
            from deca_amd.utils.helper import GPUDetector

            arch = GPUDetector.create_gpu_instance()
        self.arch = arch
        self.arch_str = arch_str or getattr(arch, "gcn_arch", DEFAULT_ARCH_STR)
        self.top_n = top_n
        self.jobs = jobs if jobs is not None else min(16, os.cpu_count() or 1)
        self.finalists = finalists
        self.rounds = rounds
        # JSON file of stored winners (see deca_amd/tuned.py); None: always search
        self.cache_path = cache_path
        self.retune = retune  # search even when a winner is stored (and replace it)

    # -- the three compute levels of the reference's stub map onto the stages ----
    def tune_cpt_0(self, *shape, **kw):
        """Register level: enumerate the configs whose fragments fit the VGPR file."""
        return self._solve(self._make_op(shape, **kw), shape, **kw)

    def tune_cpt_1(self, configs, *shape, **kw):
        """LDS level: rank by the analytical model (occupancy, LDS and L2 traffic)."""
        return self._rank(configs, shape, **kw)

    def tune_cpt_2(self, *shape, log=None, **kw):
        """Global level: measure on the device and report."""
        return self.tune(*shape, log=log, **kw)

    # -- operator specifics -------------------------------------------------------
    def _make_op(self, shape, dtype="float16", eps=1e-6, causal=False, inputs="normal", **_):
        from deca_amd import operators as ops

        if self.operator == "GEMM":
            return ops.GEMMTC(*shape, dtype=dtype, inputs=inputs)
        if self.operator == "softmax":
            return ops.Softmax(*shape, dtype)
        if self.operator == "rmsnorm":
            return ops.RMSNorm(*shape, dtype, eps)
        return ops.FlashAttention(*shape, causal=causal)

    def _solve(self, op, shape, **kw):
        from deca_amd import Solver

        if self.operator == "GEMM":
            return Solver.solve_gemm_tc(self.arch, *shape)
        if self.operator in ("softmax", "rmsnorm"):
            return Solver.solve_rowwise(self.arch, self.operator, *shape)
        return Solver.solve_flash_attn(self.arch, *shape)

    def _rank(self, configs, shape, causal=False, **_):
        from deca_amd.cost_model import CostModel as cm

        top = self.top_n or None
        if self.operator == "GEMM":
            # at most 3 tile orders per tile set among the measured candidates
            return cm.rank_gemm_configs(configs, self.arch, *shape, top_n=top,
                                        per_tile=3 if top else None)
        if self.operator in ("softmax", "rmsnorm"):
            return cm.rank_rowwise_configs(configs, self.arch, self.operator, *shape, top_n=top)
        return cm.rank_fa_configs(configs, self.arch, shape, causal, top_n=top)

    def _builder(self, op, shape):
        """(function path, cfg -> (path -> args))."""
        if self.operator == "GEMM":
            return ("deca_amd.kernels.gemm_hip:build_gemm_tc_to_file",
                    lambda cfg: lambda path: (tuple(shape), cfg, self.arch_str, path, op.dtype))
        if self.operator in ("softmax", "rmsnorm"):
            return ("deca_amd.kernels.rowwise_hip:build_rowwise_to_file",
                    lambda cfg: lambda path: (self.operator, tuple(shape), op.dtype, cfg, op.eps,
                                              self.arch_str, path))
        return ("deca_amd.kernels.flash_attn_hip:build_flash_attn_to_file",
                lambda cfg: lambda path: (tuple(op.shape), cfg, op.softmax_scale, self.arch_str,
                                          path, op.causal))

    def _torch_fn(self, op, inputs):
        if self.operator == "GEMM":
            from deca_amd.kernels.gemm_bench import torch_ref

            return lambda: torch_ref(inputs)
        if self.operator in ("softmax", "rmsnorm"):
            return lambda: op.reference(inputs)
        from deca_amd.kernels.attn_bench import sdpa_flash

        q, k, v = inputs
        return lambda: sdpa_flash(q, k, v, causal=op.causal, scale=op.softmax_scale)

    def _report(self, op, best_cfg, rank, n_ranked, best_t, torch_t, err, compile_time, total):
        ratio = torch_t / best_t
        head = (
            f"{datetime.now().strftime('%Y-%m-%d %H:%M:%S')} [{self.arch.name}]\n"
            f" DeCA {op.describe()}, config: {best_cfg} (cost-model rank {rank}/{n_ranked})\n"
        )
        if self.operator in ("softmax", "rmsnorm"):
            best = op.num_bytes / best_t / 1e9
            ref = op.num_bytes / torch_t / 1e9
            peak = 100 * best / self.arch.dram_bw
            body = (
                f" throughput: {best:.1f} GB/s ({peak:.0f}% of DRAM peak), "
                f"runtime: {best_t * 1e3:.4f} ms, max err: {err:.2e}\n"
                f" torch: {ref:.1f} GB/s, runtime: {torch_t * 1e3:.4f} ms, ratio: {ratio:.3f}\n"
            )
        else:
            best = op.num_flops / best_t / 1e12
            ref = op.num_flops / torch_t / 1e12
            peak = 100 * best * 1e3 / self.arch.peak_mma_sync_flops
            what = "fp32-acc MFMA peak" if self.operator == "GEMM" else "MFMA peak"
            base = "torch" if self.operator == "GEMM" else "SDPA"
            body = (
                f" throughput: {best:.1f} TFLOPS ({peak:.0f}% of {what}), "
                f"runtime: {best_t * 1e3:.4f} ms, max err: {err:.2e}\n"
                f" {base}: {ref:.1f} TFLOPS, runtime: {torch_t * 1e3:.4f} ms, ratio: {ratio:.3f}\n"
            )
        tail = f" compile time: {compile_time:.1f} s, total tuning time: {total:.1f} s\n"
        return head + body + tail, best, ref

    # -- the loop -----------------------------------------------------------------
    def tune(self, *shape, log=None, **kw):
        """Returns (best config, its throughput, torch's throughput)."""
        import torch

        from deca_amd.kernels.attn_bench import (
            batch_timer, bench_interleaved, bench_interleaved_batches,
        )
        from deca_amd.RuntimeMod import RuntimeMod

        from deca_amd import tuned

        start = time.time()
        op = self._make_op(shape, **kw)
        key = tuned.make_key(self.operator, getattr(op, "shape", shape), op.dtype, self.arch_str,
                             bool(getattr(op, "causal", False)), getattr(op, "inputs", "normal"))
        cached = tuned.lookup(key, self.cache_path) if self.cache_path and not self.retune else None
        if cached is not None and op.is_valid(cached):
            # a stored winner: verify and time it alone instead of searching
            configs = ranked = [cached]
            print(f"Using the stored {op.name} config of {key}", flush=True)
        else:
            configs = self._solve(op, shape, **kw)
            ranked = self._rank(configs, shape, **kw)
            print(f"Find {len(configs)} {op.name} configs, measuring {len(ranked)}", flush=True)

        fn_path, args_for = self._builder(op, shape)
        paths = build_all(fn_path, {cfg: args_for(cfg) for cfg in ranked}, self.jobs)
        compile_time = time.time() - start

        res = []
        for cfg in ranked:
            if cfg not in paths:
                continue
            rt = RuntimeMod(op, self.arch, True, cfg, timing=self.timing)
            try:
                rt.load_kernel(paths[cfg])
                rt.time_evaluator()
                print(rt.record, flush=True)
                res.append((rt.throughput, cfg, rt.execution_time, rt.max_error))
            except Exception as e:  # noqa: BLE001
                text = str(e) if os.environ.get("DECA_VERBOSE") else str(e)[-200:]
                print(f"{cfg} is not a valid config: {text}", flush=True)
            finally:
                if rt.runtime_mod is not None:
                    rt.runtime_mod.close()
            torch.cuda.empty_cache()
        end = time.time()
        if not res:
            raise RuntimeError(f"no valid {op.name} config for {shape}")
        self.measurements = [(str(cfg), thr, t, err) for thr, cfg, t, err in res]

        res.sort(key=lambda x: x[0], reverse=True)
        finalists = res[: self.finalists]
        err_of = {cfg: err for _, cfg, _, err in res}

        # Final numbers: the finalists and torch timed alternately on the same
        # tensors, so that clock drift hits all of them alike.
        from deca_amd.driver.driver import load_kernel

        inputs = op.make_inputs()
        out = op.make_output(inputs) if hasattr(op, "make_output") else torch.empty_like(inputs[0])
        args = op.kernel_args(inputs, out)
        keep = []
        b2b = self.timing == "back_to_back"
        if self.operator in ("softmax", "rmsnorm"):
            # memory-bound: DeCA and torch both cycle through buffer sets larger
            # than the Infinity Cache, so that both stream from HBM
            from deca_amd.kernels.rowwise_bench import cycle, rotating_sets

            sets = rotating_sets(inputs, out, getattr(self.arch, "mall_bytes", 0))
            fns = {"torch": cycle(lambda *a: op.reference(a[:-1]), sets)}
            for _, cfg, _, _ in finalists:
                kern = load_kernel(op.build_mod(cfg), paths[cfg])
                keep.append(kern)
                fns[cfg] = (lambda n, kern=kern: kern.time(sets, n)) if b2b else cycle(kern, sets)
        else:
            fns = {"torch": self._torch_fn(op, inputs)}
            for _, cfg, _, _ in finalists:
                kern = load_kernel(op.build_mod(cfg), paths[cfg])
                keep.append(kern)
                fns[cfg] = ((lambda n, kern=kern: kern.time([args], n)) if b2b
                            else (lambda kern=kern: kern(*args)))
        if b2b:
            fns["torch"] = batch_timer(fns["torch"])
            times = bench_interleaved_batches(fns, rounds=self.rounds)
        else:
            times = bench_interleaved(fns, rounds=self.rounds)
        torch_t = times.pop("torch")
        best_cfg, best_t = min(times.items(), key=lambda x: x[1])
        msg, best, ref = self._report(
            op, best_cfg, ranked.index(best_cfg) + 1, len(ranked), best_t, torch_t,
            err_of[best_cfg], compile_time, end - start,
        )
        print("✅✅✅ " + msg, flush=True)
        if log is not None:
            log.write(msg + "\n")
            log.flush()
        if self.cache_path:
            unit = "GB/s" if self.operator in ("softmax", "rmsnorm") else "TFLOPS"
            tuned.store(key, best_cfg, best, unit, self.cache_path, runtime_ms=round(best_t * 1e3, 4),
                        max_err=float(f"{err_of[best_cfg]:.3e}"), measured_on=self.arch.name,
                        # provenance: this search measured `candidates` configs of the
                        # solver's `solutions`, and the winner was the cost model's `rank`-th
                        method="tuner", timing=self.timing, candidates=len(ranked),
                        solutions=len(configs), rank=ranked.index(best_cfg) + 1,
                        torch_throughput=round(float(ref), 2),
                        **({"inputs": "U(-1,1)"} if getattr(op, "inputs", "normal") == "uniform" else {}))
        for kern in keep:
            kern.close()
        return best_cfg, best, ref
