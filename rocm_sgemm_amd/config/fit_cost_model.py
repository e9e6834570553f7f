#!/usr/bin/env python3
"""Fits the constants of the library's cost model (rocm_sgemm_predict_us) to tuner sweeps.

The planner behind rocm_sgemm_find_config chooses configs for problems that are not table entries
by a small analytic model of a launch's duration.  Its structure is fixed (see `predict`, which
restates the C++ `predict_us` of csrc/planner.cpp term by term); its constants are fitted here.

Input: logs of `tuner --sweep M N K a b c --splits 1,2,4,8 --groups 4` (one line per timed config:
`cfg <12 ints> avg_ms .. min_ms .. tflops .. ok 1`), one file per problem, named
`sweep_<M>_<N>_<K>*.log`.  `--collect DIR` writes them: it runs the tuner binary (on a GPU) on
every problem of fit_problems.txt, the list the compiled constants were fitted on.  The fit minimises the squared error of log(time), weighting each config
by exp(-(t / t_best - 1) / 0.25) so that the ordering among a problem's fast configs matters most.

usage: fit_cost_model.py --collect DIR [--iters n] [--first i] [--count n]
                                                        sweeps the problems (all, or n from the i-th) of fit_problems.txt into DIR
       fit_cost_model.py 'DIR/sweep_*.log' [...]       prints the fitted constants, the quality of
                                                        picking configs by the model (chosen / best
                                                        time per problem) and a 3-fold check
"""

import glob
import math
import re
import sys

import numpy as np

# (sweeps written before the waves_k field existed have ten integers per line)
LINE = re.compile(r"cfg (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+) (\d+)(?: (\d+))?(?: \d+)? avg_ms ([\d.]+) "
                  r"min_ms ([\d.]+) tflops ([\d.]+) ok ([01])")
KEYS = ["macro_m", "macro_n", "k_tile", "waves_m", "waves_n", "mfma", "stages", "split_k", "group_m",
        "wave_slots", "waves_k"]
CUS = 256

# name: (value compiled into csrc/planner.cpp, lower bound, upper bound)
CONSTANTS = {
    "eff_128x64": (0.989, 0.5, 1.0),   # sustained matrix-pipe efficiency by wave-tile area >= 8192
    "eff_64x64": (0.984, 0.5, 1.0),    # >= 4096
    "eff_64x32": (1.0, 0.4, 1.0),    # >= 2048
    "eff_32x32": (0.971, 0.3, 1.0),    # smaller
    "k_tile_64": (0.982, 0.9, 1.3),
    "mfma_16": (0.933, 0.8, 1.1),
    "register_staged": (1.032, 0.7, 1.1),
    "stages_3_4": (0.985, 0.9, 1.1),
    "masked_4_byte": (0.861, 0.6, 1.1),   # problem not all multiples of 4
    "masked_16_byte": (0.93, 0.8, 1.05),  # ragged multiples of 4
    "l2_tbs": (40.0, 3.0, 40.0),           # L2 -> LDS panel bandwidth over the chip
    "l2_tbs_4_byte": (11.75, 2.0, 40.0),
    "launch_us": (4.44, 2.0, 15.0),
    "split_us": (2.57, 0.0, 15.0),
    "split_tbs": (4.15, 1.0, 10.0),
    "tail_us": (6.15, 0.0, 20.0),
    "tail_tbs": (5.1, 1.0, 12.0),
    "fill_us_per_kb": (0.0281, 0.0, 0.2),  # exposed per round of tiles: the (stages - 1) K-tiles loaded before the first MFMA
}
NAMES = list(CONSTANTS)


def compiled_constants():
    return {k: v[0] for k, v in CONSTANTS.items()}


def tail_applies(c, tiles, k_tiles, k):
    """csrc/planner.cpp tail_applies(): (applies, slots, tiles of the last wave)."""
    waves = c["waves_m"] * c["waves_n"] * max(c.get("waves_k", 1), 1)
    per_cu = 1 if waves >= 4 else 4 // max(waves, 1)
    slots = c["wave_slots"] if c["wave_slots"] > 1 else CUS * per_cu
    r = tiles % slots
    tile_us = 2.0 * c["macro_m"] * c["macro_n"] * k / 553.0e3 * per_cu
    saved = tile_us * (1 - r / slots)
    ok = (c["split_k"] == 1 and c["wave_slots"] != 1 and k_tiles >= 8 and r > 0 and 100 * r <= 85 * slots
          and (c["wave_slots"] > 1 or saved >= 12.0))
    return ok, slots, r


def predict(p, c, M, N, K, batch=1):
    """Restatement of csrc/planner.cpp predict_us() with the constants in `p`."""
    waves = c["waves_m"] * c["waves_n"] * max(c.get("waves_k", 1), 1)
    per_cu = 1 if waves >= 4 else 4 // max(waves, 1)
    area = (c["macro_m"] // c["waves_m"]) * (c["macro_n"] // c["waves_n"])
    eff = (p["eff_128x64"] if area >= 8192 else p["eff_64x64"] if area >= 4096
           else p["eff_64x32"] if area >= 2048 else p["eff_32x32"])
    if c["k_tile"] >= 64:
        eff *= p["k_tile_64"]
    if c["mfma"] == 16:
        eff *= p["mfma_16"]
    if c["stages"] == 0:
        eff *= p["register_staged"]
    if c["stages"] >= 3:
        eff *= p["stages_3_4"]
    aligned = M % 4 == 0 and N % 4 == 0 and K % 4 == 0
    full = M % c["macro_m"] == 0 and N % c["macro_n"] == 0 and K % c["k_tile"] == 0
    if not aligned:
        eff *= p["masked_4_byte"]
    elif not full:
        eff *= p["masked_16_byte"]
    tiles = -(-M // c["macro_m"]) * -(-N // c["macro_n"]) * batch
    k_tiles = -(-K // c["k_tile"])
    compute = 2.0 * c["macro_m"] * c["macro_n"] * K / (614.5e3 * eff)
    l2 = p["l2_tbs_4_byte"] if (not aligned and c["stages"] != 0) else p["l2_tbs"]
    panels = (c["macro_m"] + c["macro_n"]) * K * 4.0 / (l2 * 1e6 / CUS)
    tile_us = (compute ** 4 + panels ** 4) ** 0.25 * per_cu
    out_mb = M * N * 4.0 / 1e6 * batch
    # what a workgroup loads before its first MFMA: nothing overlaps it at the start of a round
    fill_kb = (max(c["stages"], 2) - 1) * c["k_tile"] * (c["macro_m"] + c["macro_n"]) * 4.0 / 1024.0
    t = p["launch_us"]
    if c["split_k"] > 1:
        split = min(c["split_k"], k_tiles)
        groups, slots = tiles * split, CUS * per_cu
        t += -(-groups // slots) * (tile_us / split + p["fill_us_per_kb"] * fill_kb)
        return t + p["split_us"] + (split + 1) * out_mb / p["split_tbs"]
    tail, slots, r = tail_applies(c, tiles, k_tiles, K)
    tail = tail and batch == 1
    t += (tiles // slots) * tile_us + -(-tiles // slots) * p["fill_us_per_kb"] * fill_kb
    if r > 0:
        if tail:
            tile_mb = c["macro_m"] * c["macro_n"] * 4.0 / 1e6
            t += tile_us * r / slots + p["tail_us"] + (2.0 * slots + r) * tile_mb / p["tail_tbs"]
        else:
            t += tile_us
    return t


def load(patterns):
    """[((M, N, K), [(microseconds, config dict), ...]), ...] from sweep logs."""
    import os
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import space
    family = set(space.family())
    data = []
    for pattern in patterns:
        for path in sorted(glob.glob(pattern)):
            m = re.search(r"sweep_(\d+)_(\d+)_(\d+)", path)
            if not m:
                continue
            rows = []
            with open(path) as f:
                for line in f:
                    g = LINE.search(line)
                    if g and g.group(15) == "1":
                        ints = [int(v) if v is not None else 1 for v in g.groups()[:11]]
                        cfg = dict(zip(KEYS, ints))
                        if tuple(cfg[k] for k in space.SHAPE_KEYS) in family:  # shapes since dropped
                            rows.append((float(g.group(12)) * 1e3, cfg))
            if rows:
                data.append((tuple(map(int, m.groups())), rows))
    return data


def planner_candidate(c):
    """The shapes the planner lets the model choose from (csrc/planner.cpp plan_config)."""
    return (c["stages"] >= 2 and c["mfma"] == 32
            and ((c["macro_m"] >= 64 and c["macro_n"] >= 64) or c.get("waves_k", 1) > 1))


def pick_quality(p, data):
    """Per problem: time of the config the model would pick / time of the fastest config."""
    out = []
    for (M, N, K), rows in data:
        best = min(t for t, _ in rows)
        cand = [r for r in rows if planner_candidate(r[1])] or rows
        out.append(min(cand, key=lambda r: predict(p, r[1], M, N, K))[0] / best)
    return np.array(out)


def fit(data):
    from scipy.optimize import least_squares

    def residuals(x):
        p = dict(zip(NAMES, x))
        out = []
        for (M, N, K), rows in data:
            best = min(t for t, _ in rows)
            for t, c in rows:
                out.append(math.exp(-(t / best - 1) / 0.25) * (math.log(predict(p, c, M, N, K)) - math.log(t)))
        return np.array(out)

    x0 = np.array([CONSTANTS[k][0] for k in NAMES])
    lo = np.array([CONSTANTS[k][1] for k in NAMES])
    hi = np.array([CONSTANTS[k][2] for k in NAMES])
    return dict(zip(NAMES, least_squares(residuals, x0, bounds=(lo, hi)).x))


def collect(out_dir, iters=20, first=0, count=None):
    """Sweeps the problems [first, first + count) of fit_problems.txt with the tuner binary (needs a GPU)."""
    import os
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(here, "fit_problems.txt")) as f:
        problems = [tuple(map(int, line.split())) for line in f if line.strip() and not line.startswith("#")]
    problems = problems[first:first + count if count is not None else None]
    for i, (M, N, K) in enumerate(problems):
        log = os.path.join(out_dir, f"sweep_{M}_{N}_{K}.log")
        cmd = [os.path.join(here, "tuner"), "--sweep", str(M), str(N), str(K), "0", "0", "0", "--iters",
               str(iters), "--splits", "1,2,4,8", "--groups", "4"]
        with open(log, "w") as out:
            rc = subprocess.run(cmd, stdout=out, stderr=subprocess.STDOUT, timeout=600).returncode
        print(f"[{i + 1}/{len(problems)}] {M} x {N} x {K}: rc {rc}", flush=True)
        if rc != 0:
            return rc
    return 0


def main(argv):
    if len(argv) < 2:
        print(__doc__)
        return 2
    if argv[1] == "--collect":
        opt = lambda name, default: int(argv[argv.index(name) + 1]) if name in argv else default  # noqa: E731
        return collect(argv[2], opt("--iters", 20), opt("--first", 0), opt("--count", None))
    data = load(argv[1:])
    if not data:
        print("no sweep logs matched", file=sys.stderr)
        return 1
    print(f"{len(data)} problems, {sum(len(r) for _, r in data)} timed configs")
    q = pick_quality(compiled_constants(), data)
    print(f"compiled constants: chosen / best time, mean {q.mean():.3f}, worst {q.max():.3f}")
    p = fit(data)
    for k in NAMES:
        print(f"  {k:18s} {p[k]:8.3f}   (compiled {CONSTANTS[k][0]})")
    q = pick_quality(p, data)
    print(f"fitted constants:   chosen / best time, mean {q.mean():.3f}, worst {q.max():.3f}")
    for fold in range(3):
        train = [d for i, d in enumerate(data) if i % 3 != fold]
        test = [d for i, d in enumerate(data) if i % 3 == fold]
        if train and test:
            q = pick_quality(fit(train), test)
            print(f"fold {fold}: held-out mean {q.mean():.3f}, worst {q.max():.3f}")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
