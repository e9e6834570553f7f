#!/usr/bin/env python3
"""Tuner driver for the MI355X SGEMM config table.

Same job and command line as the reference's tune.py (reference rocm_sgemm/config/tune.py:531-711):
for every (size, A/B/C layout) pick the fastest config by timing trials through the `tuner` binary,
merge with an existing JSON, write `{configurations: [{range, layout, config}]}`.

What differs, because the kernels do:
  * the search space is the MFMA parameterisation of space.py (macro tile, K-tile, wave grid, MFMA
    shape, split_k, group_m), not the nine VALU thread-tile parameters (reference tune.py:55-65);
  * every tile shape is precompiled, so one `tuner --sweep` process times the whole family for a
    problem instead of one hipRTC compile + process per trial (reference tune.py:163-190);
  * the space is small enough (tens of shapes x a few launch parameters) to be searched
    exhaustively in two phases, so no Optuna/TPE sampler is needed (Optuna is also not part of
    this environment): phase 1 sweeps all shapes at group_m = 4 with the split_k values that bring
    the grid to at least one workgroup per CU, phase 2 re-times the best shapes over every group_m,
    phases 3 and 4 try the best configs without the stream-K tail and with the partial tiles summed
    inside the launch / by a second kernel.
    `--budget` caps the number of trials per (size, layout) as in the reference.
  * `--explore` leaves the precompiled family, which is what the reference's tuner does for every
    trial (it compiles any valid point of its space through hipRTC, reference tuner.cpp:183-216,
    234-383, tune.py:163-232): tile shapes from outside the family - given on the command line, or
    the neighbours in the search space of the family's three fastest shapes for each problem - are
    compiled into a side library (build.build(out_dir=...), a minute for a dozen shapes), timed by a
    trial binary linked against it, and compared with the family's best.  A shape that wins is
    reported; it joins the library by being added to space._BASE_SHAPES.

usage examples
  python tune.py                                   # 1024..8192 cubes, all 8 layouts
  python tune.py --sizes 4096,4096,4096 --layouts r,r,r c,c,c
  python tune.py --input gemm_config.json --sizes 128,4096,4096 --output gemm_config_tuned.json
  python tune.py --explore --sizes 2048,2048,2048 --layouts r,r,r          # neighbours of the best shapes
  python tune.py --explore 256,128,16,2,2,32,2,1 128,128,16,2,2,32,4,1 --sizes 8192,8192,8192 --layouts r,r,r
"""

import argparse
import json
import os
import re
import subprocess
import sys
from pathlib import Path

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import space  # noqa: E402

LAYOUT_ALIASES = {"r": 0, "row_major": 0, "c": 1, "col_major": 1}
SWEEP_LINE = re.compile(
    r"cfg (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) avg_ms ([\d.]+) min_ms ([\d.]+) "
    r"tflops ([\d.]+) ok ([01])")


def parse_sizes(items):
    out = []
    for it in items:
        m, n, k = (int(x) for x in it.split(","))
        out.append((m, n, k))
    return out


def parse_layouts(items):
    out = []
    for it in items:
        a, b, c = (LAYOUT_ALIASES[x.strip()] for x in it.split(","))
        out.append((a, b, c))
    return out


def parse_baselines(items):
    out = []
    for it in items:
        vals = [int(x) for x in it.split(",")]
        if len(vals) != len(space.CONFIG_KEYS):
            raise ValueError(f"baseline needs {len(space.CONFIG_KEYS)} ints "
                             f"({','.join(space.CONFIG_KEYS)}), got {it!r}")
        out.append(dict(zip(space.CONFIG_KEYS, vals)))
    return out


def split_candidates(shape, M, N, K):
    """split_k values worth trying: none, plus those that lift the grid towards >= 1 workgroup
    per CU when the output alone gives fewer."""
    bm, bn, bk = shape[0], shape[1], shape[2]
    tiles = -(-M // bm) * -(-N // bn)
    out = [1]
    if tiles < 2 * space.NUM_CU:
        for s in space.PARAM_SPACE["split_k"]:
            if s > 1 and tiles * s <= 8 * space.NUM_CU and K >= s * bk * 2:
                out.append(s)
    return out


class Tuner:
    def __init__(self, tuner_bin, budget=150, iters=20, max_memory=space.LDS_BYTES_PER_CU, seed=42,
                 runner=subprocess.run, verbose=True, shapes=None):
        self.tuner_bin = tuner_bin
        self.budget = budget
        self.iters = iters
        self.max_memory = max_memory
        self.seed = seed  # the search is exhaustive and deterministic; kept for CLI compatibility
        self.runner = runner
        self.verbose = verbose
        # the tile shapes the trial binary's library holds (its sweep times all of them)
        self.shapes = [s for s in (space.family() if shapes is None else shapes)
                       if space.max_lds_bytes(s[0], s[1], s[2]) <= max_memory]

    def log(self, *a):
        if self.verbose:
            print(*a, flush=True)

    # -- one tuner process -----------------------------------------------------------------------
    def sweep(self, M, N, K, layout, splits, groups):
        a, b, c = layout
        cmd = [self.tuner_bin, "--sweep", str(M), str(N), str(K), str(a), str(b), str(c),
               "--iters", str(self.iters), "--splits", ",".join(map(str, splits)),
               "--groups", ",".join(map(str, groups))]
        try:
            proc = self.runner(cmd, capture_output=True, text=True, timeout=1200)
        except subprocess.TimeoutExpired:
            return []
        if proc.returncode != 0:
            self.log(f"  tuner failed ({proc.returncode}): {proc.stderr[-300:]}")
            return []
        return self.parse_sweep(proc.stdout)

    @staticmethod
    def parse_sweep(text):
        out = []
        for m in SWEEP_LINE.finditer(text):
            n = len(space.CONFIG_KEYS)
            vals = [int(m.group(i)) for i in range(1, n + 1)]
            cfg = dict(zip(space.CONFIG_KEYS, vals))
            out.append({"config": cfg, "avg_ms": float(m.group(n + 1)), "min_ms": float(m.group(n + 2)),
                        "tflops": float(m.group(n + 3)), "ok": m.group(n + 4) == "1"})
        return out

    def single(self, M, N, K, layout, cfg):
        a, b, c = layout
        cmd = [self.tuner_bin, str(M), str(N), str(K)] + [str(cfg[k]) for k in space.CONFIG_KEYS] \
            + [str(a), str(b), str(c), str(self.iters)]
        try:
            proc = self.runner(cmd, capture_output=True, text=True, timeout=300)
        except subprocess.TimeoutExpired:
            return None
        if proc.returncode != 0:
            return None
        m = re.search(r"time:\s*([\d.]+)\s+ms", proc.stdout)
        return float(m.group(1)) if m else None

    # -- search ------------------------------------------------------------------------------------
    def tune_problem(self, M, N, K, layout, baselines=()):
        """Returns the result record of the best config for one (size, layout)."""
        trials = []
        splits = sorted({s for shape in self.shapes for s in split_candidates(shape, M, N, K)})
        # phase 1: every shape x useful split at the default band height
        phase1 = self.sweep(M, N, K, layout, splits, [space.DEFAULT_CONFIG["group_m"]])
        trials += [t for t in phase1 if t["ok"]]
        for cfg in baselines:
            if space.config_ok(cfg, M, N, K) and not any(t["config"] == cfg for t in trials):
                ms = self.single(M, N, K, layout, cfg)
                if ms is not None:
                    trials.append({"config": dict(cfg), "avg_ms": ms, "min_ms": ms, "tflops": 0.0,
                                   "ok": True})
        if not trials:
            return None
        # one sweep process times the whole family, so phase 1 is never cut short; the budget
        # bounds the total by limiting phase 2
        trials.sort(key=lambda t: t["avg_ms"])
        # phase 2: the best few (shape, split) over every band height, within the budget
        left = max(0, self.budget - len(trials))
        groups = [g for g in space.PARAM_SPACE["group_m"] if g != space.DEFAULT_CONFIG["group_m"]]
        seen = {tuple(t["config"].values()) for t in trials}
        for t in list(trials[:3]):
            for g in groups:
                if left <= 0:
                    break
                cfg = dict(t["config"], group_m=g)
                if tuple(cfg.values()) in seen:
                    continue
                seen.add(tuple(cfg.values()))
                ms = self.single(M, N, K, layout, cfg)
                left -= 1
                if ms is not None:
                    trials.append({"config": cfg, "avg_ms": ms, "min_ms": ms, "tflops": 0.0,
                                   "ok": True})
        # phase 3: the best config so far with the stream-K tail switched off
        best = min(trials, key=lambda t: t["avg_ms"])
        if left > 0 and best["config"]["split_k"] == 1 and best["config"]["wave_slots"] == 0:
            cfg = dict(best["config"], wave_slots=1)
            if tuple(cfg.values()) not in seen:
                ms = self.single(M, N, K, layout, cfg)
                if ms is not None:
                    trials.append({"config": cfg, "avg_ms": ms, "min_ms": ms, "tflops": 0.0,
                                   "ok": True})
        # phase 4: the best few configs that leave partial tiles (K split or stream-K tail) with the
        # summation forced into the GEMM launch and forced into a second kernel
        trials.sort(key=lambda t: t["avg_ms"])
        for t in list(trials[:3]):
            if t["config"]["split_k"] == 1 and t["config"]["wave_slots"] == 1:
                continue
            if not space.sums_in_launch(tuple(t["config"][k] for k in space.SHAPE_KEYS)):
                continue
            for sums in (1, 2):
                if left <= 0:
                    break
                cfg = dict(t["config"], partial_sums=sums)
                if tuple(cfg.values()) in seen:
                    continue
                seen.add(tuple(cfg.values()))
                ms = self.single(M, N, K, layout, cfg)
                left -= 1
                if ms is not None:
                    trials.append({"config": cfg, "avg_ms": ms, "min_ms": ms, "tflops": 0.0,
                                   "ok": True})
        best = min(trials, key=lambda t: t["avg_ms"])
        shape = tuple(best["config"][k] for k in space.SHAPE_KEYS)
        self.log(f"  best {best['config']}  {best['avg_ms']:.4f} ms "
                 f"({2.0 * M * N * K / best['avg_ms'] * 1e-9:.1f} TFLOP/s, {len(trials)} trials)")
        by_shape = {}
        for t in trials:  # fastest trial of every tile shape, fastest shape first
            key = tuple(t["config"][k] for k in space.SHAPE_KEYS)
            if key not in by_shape or t["avg_ms"] < by_shape[key]:
                by_shape[key] = t["avg_ms"]
        return {"M": M, "N": N, "K": K, "layout": layout, "config": best["config"],
                "shape_ranking": sorted(by_shape.items(), key=lambda kv: kv[1]),
                "avg_time_ms": best["avg_ms"], "evaluations": len(trials),
                "memory_used_bytes": space.max_lds_bytes(*shape[:3], shape[6], shape[7]),
                "space_coverage_percent": round(100.0 * len({tuple(t['config'][k] for k in space.SHAPE_KEYS) for t in trials}) / max(1, len(self.shapes)), 1)}

    def tune_all(self, sizes, layouts, baselines_for=None):
        results = {}
        for (M, N, K) in sizes:
            for layout in layouts:
                self.log(f"tuning {M}x{N}x{K} A,B,C={layout}")
                base = baselines_for(M, N, K, layout) if baselines_for else ()
                rec = self.tune_problem(M, N, K, layout, base)
                if rec is not None:
                    results[(M, N, K) + tuple(layout)] = rec
        return results


# -- exploration: tile shapes from outside the compiled family --------------------------------------

def parse_shapes(items):
    out = []
    for it in items:
        vals = tuple(int(x) for x in it.split(","))
        if len(vals) != len(space.SHAPE_KEYS):
            raise ValueError(f"a tile shape is {len(space.SHAPE_KEYS)} ints ({','.join(space.SHAPE_KEYS)}), got {it!r}")
        if not space.shape_ok(vals):
            raise ValueError(f"tile shape {vals} violates the kernel's constraints")
        out.append(vals)
    return out


def default_side_build(out_dir, shapes):
    """Compiles `shapes` (and the default config's shape) into <out_dir>/librocm_sgemm.so and links
    <out_dir>/config/tuner against it.  Returns the path of that trial binary."""
    sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
    from rocm_sgemm_amd import build as lib_build  # noqa: E402
    lib_build.build(out_dir=out_dir, shapes=shapes, tuner=True, verbose=False)
    return os.path.join(out_dir, "config", "tuner")


def explore(sizes, layouts, shapes, family_tuner, out_dir, max_shapes=12, side_build=default_side_build,
            make_tuner=None, log=print):
    """Times tile shapes from outside the family against the family's best for every (size, layout).

    `shapes`: the shapes to try; empty = for every problem the neighbours (space.neighbours) of the
    family's three fastest shapes, at most `max_shapes` in all.  `family_tuner` is a Tuner on the
    shipped trial binary; `side_build(out_dir, shapes)` builds the side library and returns its
    trial binary; `make_tuner(path, shapes)` makes the Tuner for it (tests replace both).
    Returns [{M, N, K, layout, family: {config, avg_ms}, explored: {config, avg_ms} | None,
    winner: bool, shape_ranking: [...]}]."""
    shipped = space.shipped_family()
    family_recs = {}
    for (M, N, K) in sizes:
        for layout in layouts:
            log(f"family sweep {M}x{N}x{K} A,B,C={layout}")
            family_recs[(M, N, K) + tuple(layout)] = family_tuner.tune_problem(M, N, K, layout)
    candidates = [s for s in shapes if s not in shipped]
    if not candidates:
        pool = []
        for rec in family_recs.values():
            if rec is None:
                continue
            for shape, _ in rec["shape_ranking"][:3]:
                for n in space.neighbours(shape):
                    if n not in shipped and n not in pool:
                        pool.append(n)
        # round-robin over the problems' neighbourhoods would be fairer; sorted keeps it reproducible
        candidates = sorted(pool)[:max_shapes]
    if not candidates:
        log("nothing to explore: every candidate is in the family already")
        return []
    added = space.explore(candidates)
    log(f"compiling {len(added)} tile shapes outside the family: {added}")
    side_bin = side_build(out_dir, added)
    side = make_tuner(side_bin, added) if make_tuner else Tuner(
        side_bin, budget=family_tuner.budget, iters=family_tuner.iters, max_memory=family_tuner.max_memory,
        runner=family_tuner.runner, verbose=family_tuner.verbose, shapes=added)
    out = []
    for key, fam in family_recs.items():
        M, N, K = key[:3]
        layout = key[3:]
        log(f"exploring {M}x{N}x{K} A,B,C={layout}")
        rec = side.tune_problem(M, N, K, layout)
        # the side library also holds the default config's shape: only shapes outside the family count
        ranking = [(s, ms) for s, ms in (rec["shape_ranking"] if rec else []) if s not in shipped]
        best = None
        if rec is not None and tuple(rec["config"][k] for k in space.SHAPE_KEYS) not in shipped:
            best = {"config": rec["config"], "avg_ms": rec["avg_time_ms"]}
        elif ranking:
            best = {"config": dict(zip(space.SHAPE_KEYS, ranking[0][0])), "avg_ms": ranking[0][1]}
        fam_best = {"config": fam["config"], "avg_ms": fam["avg_time_ms"]} if fam else None
        winner = bool(best and fam_best and best["avg_ms"] < fam_best["avg_ms"])
        if best and fam_best:
            log(f"  family {fam_best['avg_ms']:.4f} ms, best outside {best['avg_ms']:.4f} ms "
                f"({(fam_best['avg_ms'] / best['avg_ms'] - 1.0) * 100.0:+.1f} %): "
                + ("the explored shape wins" if winner else "the family holds"))
        out.append({"M": M, "N": N, "K": K, "layout": list(layout), "family": fam_best, "explored": best,
                    "winner": winner, "shape_ranking": [[list(s), ms] for s, ms in ranking]})
    return out


# -- JSON in / out (schema of reference config/gemm_config.json:1-30 with the new config keys) -----

def load_existing_json(path):
    if not path or not Path(path).exists():
        return {}
    with open(path) as f:
        data = json.load(f)
    out = {}
    for e in data.get("configurations", []):
        key = (e["range"]["M"], e["range"]["N"], e["range"]["K"],
               LAYOUT_ALIASES[e["layout"]["A"]], LAYOUT_ALIASES[e["layout"]["B"]],
               LAYOUT_ALIASES[e["layout"]["C"]])
        cfg = {k: int(e["config"].get(k, space.DEFAULT_CONFIG[k])) for k in space.CONFIG_KEYS}
        out[key] = {"M": key[0], "N": key[1], "K": key[2], "layout": key[3:], "config": cfg,
                    "avg_time_ms": e.get("avg_time_ms")}
    return out


def merge_results(existing, new):
    """New results win; untouched entries are preserved (reference tune.py:426-474)."""
    merged = dict(existing)
    merged.update(new)
    return merged


def to_json(results):
    entries = []
    for key in sorted(results):
        r = results[key]
        a, b, c = r["layout"]
        e = {"range": {"M": r["M"], "N": r["N"], "K": r["K"]},
             "layout": {"A": space.LAYOUTS[a], "B": space.LAYOUTS[b], "C": space.LAYOUTS[c]},
             "config": {k: int(r["config"][k]) for k in space.CONFIG_KEYS}}
        if r.get("avg_time_ms") is not None:
            e["avg_time_ms"] = round(float(r["avg_time_ms"]), 5)
        entries.append(e)
    return {"configurations": entries}


def main(argv=None):
    ap = argparse.ArgumentParser(description="MI355X SGEMM tuner (exhaustive two-phase search)",
                                 formatter_class=argparse.RawDescriptionHelpFormatter,
                                 epilog=__doc__)
    ap.add_argument("--input", "-i", help="existing JSON; its entries are kept and used as baselines")
    ap.add_argument("--sizes", nargs="*", help="M,N,K ...")
    ap.add_argument("--layouts", nargs="*", help="A,B,C as row_major/col_major or r/c ...")
    ap.add_argument("--baselines", nargs="*",
                    help="configs as " + ",".join(space.CONFIG_KEYS) + " always included in the trials")
    ap.add_argument("--budget", type=int, default=150, help="max trials per (size, layout)")
    ap.add_argument("--seed", type=int, default=42, help="unused: the search is deterministic")
    ap.add_argument("--gpu-arch", default="gfx950", help="only gfx950 is supported")
    ap.add_argument("--max-memory", type=int, default=space.LDS_BYTES_PER_CU,
                    help="LDS bytes a config may use (default: 160 KB)")
    ap.add_argument("--iters", type=int, default=20, help="timed launches per trial")
    ap.add_argument("--tuner", default=os.path.join(HERE, "tuner"), help="trial binary")
    ap.add_argument("--output", default="gemm_config_tuned.json")
    ap.add_argument("--explore", nargs="*", metavar="SHAPE", default=None,
                    help="time tile shapes from outside the compiled family (" + ",".join(space.SHAPE_KEYS)
                         + " each); without shapes: the neighbours of the family's fastest shapes")
    ap.add_argument("--explore-dir", default=os.path.join(os.path.dirname(HERE), "_build", "explore"),
                    help="where the side library and its trial binary are built")
    ap.add_argument("--explore-max", type=int, default=12, help="most shapes compiled when none are named")
    ap.add_argument("--explore-prebuilt", action="store_true",
                    help="the side library in --explore-dir already holds the named shapes: do not compile "
                         "(build it beforehand with `python -m rocm_sgemm_amd.build --explore SHAPE ...`)")
    args = ap.parse_args(argv)

    if args.gpu_arch != "gfx950":
        ap.error("this library is built for gfx950 only")
    sizes = parse_sizes(args.sizes) if args.sizes else [(s, s, s) for s in (1024, 2048, 4096, 8192)]
    layouts = parse_layouts(args.layouts) if args.layouts else \
        [(a, b, c) for a in (0, 1) for b in (0, 1) for c in (0, 1)]
    existing = load_existing_json(args.input)
    cli_baselines = parse_baselines(args.baselines) if args.baselines else []

    def baselines_for(M, N, K, layout):
        out = list(cli_baselines)
        e = existing.get((M, N, K) + tuple(layout))
        if e is not None:
            out.append(e["config"])
        return out

    tuner = Tuner(args.tuner, budget=args.budget, iters=args.iters, max_memory=args.max_memory,
                  seed=args.seed)
    if args.explore is not None:
        prebuilt = (lambda out_dir, shapes: os.path.join(out_dir, "config", "tuner")) if args.explore_prebuilt \
            else default_side_build
        found = explore(sizes, layouts, parse_shapes(args.explore), tuner, args.explore_dir, args.explore_max,
                        side_build=prebuilt)
        with open(args.output, "w") as f:
            json.dump({"explored": found}, f, indent=4)
        wins = [r for r in found if r["winner"]]
        print(f"explored {len(found)} problems, {len(wins)} won by a shape outside the family; wrote {args.output}")
        return 0
    new = tuner.tune_all(sizes, layouts, baselines_for)
    merged = merge_results(existing, new)
    with open(args.output, "w") as f:
        json.dump(to_json(merged), f, indent=4)
    print(f"wrote {len(merged)} configurations ({len(new)} tuned now) to {args.output}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
