"""Rank quality of the cost models, from the tuning drivers' own output.

    python -m deca_amd.cost_model.rank_report LOG [LOG ...] > profiles/rank_quality.md
    python -m deca_amd.cost_model.rank_report --pairs q_smem=0:q_smem=1 stages=2:stages=3 -- LOG ...

A driver (`test_gemm_tc.py`, `test_rowwise.py`, `test_flash_attn.py`) prints one
record per measured configuration, in the order the cost model ranked them, and
a final report with the winner.  From that text: how many of the solver's
configurations were measured, at which rank the measured best stood, and what
measuring only the first few would have cost.  The reference ranks with the same
kind of model (src/cost_model/CostModel.py:274-283) and publishes no such figure.
"""

from __future__ import annotations

import re
import sys

_FIND = re.compile(r"^Find (\d+) (\S+) configs, measuring (\d+)")
_RECORD = re.compile(r"^(\S.*?) \n\t(\S+) \n\tcost time: ([\d.]+) ms, throughput: ([\d.]+) (\S+?),", re.M)


def parse_runs(text: str) -> list:
    """One dict per tuning run in `text`: operator description, solver solutions,
    measured candidates as (config, throughput) in cost-model order."""
    runs, starts = [], [m for m in re.finditer(_FIND.pattern, text, re.M)]
    for i, m in enumerate(starts):
        body = text[m.end(): starts[i + 1].start() if i + 1 < len(starts) else len(text)]
        records = _RECORD.findall(body)
        if not records:
            continue
        runs.append({
            "what": records[0][0].strip(), "solutions": int(m.group(1)), "asked": int(m.group(3)),
            "unit": records[0][4], "measured": [(cfg, float(thr)) for _, cfg, _, thr, _ in records],
        })
    return runs


def spearman(values: list) -> float:
    """Rank correlation between the model's order (the list order) and the measured
    throughputs (1.0: the model sorts them perfectly)."""
    n = len(values)
    if n < 2:
        return 1.0
    order = sorted(range(n), key=lambda i: -values[i])
    measured_rank = [0] * n
    for r, i in enumerate(order):
        measured_rank[i] = r
    d2 = sum((i - measured_rank[i]) ** 2 for i in range(n))
    return 1.0 - 6.0 * d2 / (n * (n * n - 1))


def quality(run: dict) -> dict:
    thr = [t for _, t in run["measured"]]
    best = max(thr)
    rank = thr.index(best) + 1

    def best_of_first(k):
        return max(thr[:k]) / best

    return {"what": run["what"], "solutions": run["solutions"], "measured": len(thr),
            "best_rank": rank, "best": best, "unit": run["unit"], "first": thr[0] / best,
            "top3": best_of_first(3), "top8": best_of_first(8), "spearman": spearman(thr),
            "best_cfg": run["measured"][rank - 1][0]}


def table(runs: list) -> str:
    rows = ["| tuned shape | solver solutions | measured | rank of the measured best | "
            "rank 1 / best | best of first 3 / best | best of first 8 / best | rank correlation | "
            "measured best |", "|---|---|---|---|---|---|---|---|---|"]
    for run in runs:
        q = quality(run)
        rows.append(f"| {q['what']} | {q['solutions']} | {q['measured']} | {q['best_rank']} | "
                    f"{q['first']:.3f} | {q['top3']:.3f} | {q['top8']:.3f} | {q['spearman']:.2f} | "
                    f"`{q['best_cfg']}` {q['best']:.1f} {q['unit']} |")
    return "\n".join(rows)


def pair_effects(run: dict, old: str, new: str) -> dict:
    """What one field of the configuration does, everything else equal: over all measured
    pairs of configurations whose text differs only in `old` -> `new` (e.g. "stages=2",
    "stages=3"), the ratios new / old, the pair with the fastest `new` member, and the
    same ratios among pairs whose better member is within 10 % of the run's best.  An empty
    `old` pairs the configurations that carry `new` with their twins without it (fields that
    are only printed when set, e.g. "" -> "trust=1")."""
    thr = dict(run["measured"])
    best = max(thr.values())
    if old:
        pairs = [(c, c.replace(old, new)) for c in thr if old in c.split(",") and c.replace(old, new) in thr]
    else:
        pairs = [(",".join(f for f in c.split(",") if f != new), c) for c in thr if new in c.split(",")]
        pairs = [(a, b) for a, b in pairs if a in thr]
    ratios = sorted(thr[b] / thr[a] for a, b in pairs)
    near = sorted(thr[b] / thr[a] for a, b in pairs if max(thr[a], thr[b]) >= 0.9 * best)
    top = max(pairs, key=lambda ab: thr[ab[1]], default=None)

    def mid(v):
        return v[len(v) // 2] if v else float("nan")

    return {"pairs": len(pairs), "median": mid(ratios), "min": ratios[0] if ratios else float("nan"),
            "max": ratios[-1] if ratios else float("nan"), "near_pairs": len(near), "near_median": mid(near),
            "near_min": near[0] if near else float("nan"), "near_max": near[-1] if near else float("nan"),
            "top": None if top is None else (top[1], thr[top[1]], thr[top[0]]), "best": best}


def pairs_table(runs: list, fields: list) -> str:
    rows = ["| tuned shape | field | pairs | new / old: median (min ... max) | ... among pairs within "
            "10 % of the best | fastest config with the new value | its twin with the old | "
            "best of the run |", "|---|---|---|---|---|---|---|---|"]
    for run in runs:
        for field in fields:
            old, new = field.split(":")
            e = pair_effects(run, old, new)
            top = "-" if e["top"] is None else f"`{e['top'][0]}` {e['top'][1]:.1f}"
            twin = "-" if e["top"] is None else f"{e['top'][2]:.1f}"
            rows.append(f"| {run['what']} | {old} -> {new} | {e['pairs']} | {e['median']:.3f} "
                        f"({e['min']:.3f} ... {e['max']:.3f}) | {e['near_pairs']} pairs: {e['near_median']:.3f} "
                        f"({e['near_min']:.3f} ... {e['near_max']:.3f}) | {top} | {twin} | {e['best']:.1f} |")
    return "\n".join(rows)


def main(argv=None):
    args = list(argv if argv is not None else sys.argv[1:])
    fields = []
    if args and args[0] == "--pairs":
        cut = args.index("--")
        fields, args = args[1:cut], args[cut + 1:]
    if not args:
        raise SystemExit(__doc__)
    runs = []
    for p in args:
        with open(p) as f:
            runs += parse_runs(f.read())
    print(pairs_table(runs, fields) if fields else table(runs))


if __name__ == "__main__":
    main()
