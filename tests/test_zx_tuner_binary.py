"""The tuner's trial binary on the GPU, and the Python driver on top of the real binary.

Counterpart of the reference's argv contract (reference rocm_sgemm/config/tuner.cpp:440-512) and
of its driver running one process per trial and parsing the time (reference
rocm_sgemm/config/tune.py:146-190).  A trial binary whose correctness gate said `ok 0` everywhere,
or whose line format drifted from the driver's regular expression, fails here.
"""

import os
import re
import subprocess
import sys

import pytest

import rocm_sgemm_amd as rs

pytestmark = pytest.mark.gpu

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CONFIG_DIR = os.path.join(REPO, "rocm_sgemm_amd", "config")
TUNER = os.path.join(CONFIG_DIR, "tuner")
sys.path.insert(0, CONFIG_DIR)
import space  # noqa: E402
import tune  # noqa: E402

M, N, K = 384, 256, 512
LAYOUT = (0, 1, 0)  # A row-major, B column-major, C row-major


def test_single_config_mode_times_and_verifies_one_trial():
    print("CASE tuner single", M, N, K, flush=True)
    cfg = rs.find_config(M, N, K, *LAYOUT).as_dict()
    cmd = [TUNER, str(M), str(N), str(K)] + [str(cfg[k]) for k in space.CONFIG_KEYS] \
        + [str(x) for x in LAYOUT] + ["3"]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr  # 5 = wrong result, 3 = unsupported config
    m = re.search(r"time:\s*([\d.]+)\s+ms\s+min:\s*([\d.]+)\s+ms\s+avg_tflops:\s*([\d.]+)", out.stdout)
    assert m is not None, out.stdout
    avg_ms, min_ms, tflops = map(float, m.groups())
    assert 0.0 < min_ms <= avg_ms * 1.5 and avg_ms < 5.0 and tflops > 0.5
    # a tile shape that is not compiled is refused, as the reference's launcher refuses a null slot
    bad = [TUNER, str(M), str(N), str(K), "96", "96", "32", "2", "2", "32", "2", "1", "4", "0", "1", "0", "0", "0", "0"]
    refused = subprocess.run(bad, capture_output=True, text=True, timeout=120)
    assert refused.returncode == 3 and "No kernel available" in refused.stderr


def test_sweep_mode_lines_parse_and_every_family_shape_is_correct():
    print("CASE tuner sweep", M, N, K, flush=True)
    cmd = [TUNER, "--sweep", str(M), str(N), str(K)] + [str(x) for x in LAYOUT] \
        + ["--iters", "3", "--splits", "1,2", "--groups", "4"]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.startswith("cfg ")]
    assert lines and all(tune.SWEEP_LINE.fullmatch(l) for l in lines), \
        [l for l in lines if not tune.SWEEP_LINE.fullmatch(l)][:3]
    trials = tune.Tuner.parse_sweep(out.stdout)
    assert len(trials) == len(lines)
    assert all(t["ok"] for t in trials), [t["config"] for t in trials if not t["ok"]]
    assert all(t["min_ms"] > 0 and t["tflops"] > 0 for t in trials)
    # every compiled tile shape was tried, unsplit and split in two
    shapes = {tuple(t["config"][k] for k in space.SHAPE_KEYS) for t in trials}
    family = {tuple(getattr(f, k) for k in space.SHAPE_KEYS) for f in rs.family()}
    assert shapes == family
    assert {t["config"]["split_k"] for t in trials} == {1, 2}


def test_driver_with_the_real_trial_binary_returns_a_runnable_config():
    print("CASE tuner driver", M, N, K, flush=True)
    tuner = tune.Tuner(TUNER, budget=100, iters=3, verbose=False)
    rec = tuner.tune_problem(M, N, K, LAYOUT)
    assert rec is not None and rec["evaluations"] >= len(rs.family())
    cfg = rec["config"]
    assert rs.config_supported(cfg, LAYOUT[2], LAYOUT[0], LAYOUT[1])
    assert 0.0 < rec["avg_time_ms"] < 1.0
    # the record goes into the JSON schema the generator reads
    entry = tune.to_json({(M, N, K) + LAYOUT: rec})["configurations"][0]
    assert entry["range"] == {"M": M, "N": N, "K": K}
    assert entry["layout"] == {"A": "row_major", "B": "col_major", "C": "row_major"}
    assert set(entry["config"]) == set(space.CONFIG_KEYS)


def test_exploration_times_a_tile_shape_from_outside_the_family():
    """tune.py --explore end to end on the GPU: the family sweep on the shipped trial binary, then
    a tile shape the library does not ship (128 x 128 x 32 with a three-stage ring), compiled by
    the build into a side library with a trial binary of its own, timed and verified there
    (a trial whose result is wrong says `ok 0` and is dropped, so a record means `ok 1`)."""
    from rocm_sgemm_amd import build as lib_build
    shape = lib_build.EXPLORE_CHECK_SHAPE
    side_tuner = os.path.join(lib_build.EXPLORE_CHECK_DIR, "config", "tuner")
    assert os.path.exists(side_tuner), "the build makes the side library (build_explore_check)"
    assert shape not in space.shipped_family() and not rs.config_supported(dict(zip(space.SHAPE_KEYS, shape)))
    print("CASE tuner explore", shape, flush=True)
    fam = tune.Tuner(TUNER, budget=5, iters=3, verbose=False)
    try:
        found = tune.explore([(1024, 768, 2048)], [(0, 0, 0)], [shape], fam, lib_build.EXPLORE_CHECK_DIR,
                             side_build=lambda out_dir, shapes: side_tuner, log=lambda *a: None)
    finally:
        space.explore([])  # leave the family as shipped for the other tests
    assert len(found) == 1
    rec = found[0]
    assert rec["family"] is not None and rec["family"]["avg_ms"] > 0
    assert tuple(rec["family"]["config"][k] for k in space.SHAPE_KEYS) in space.shipped_family()
    assert rec["explored"] is not None, "the explored shape produced no verified trial"
    got = tuple(rec["explored"]["config"][k] for k in space.SHAPE_KEYS)
    assert got in (shape, space.swapped(shape)) and rec["explored"]["avg_ms"] > 0
    # both were timed on the same problem: the two figures are of one order
    assert 0.2 < rec["explored"]["avg_ms"] / rec["family"]["avg_ms"] < 5.0
    # the shipped library refuses the shape, the side library's trial binary runs it
    cfg = dict(zip(space.SHAPE_KEYS, shape), split_k=1, group_m=4, wave_slots=0, partial_sums=0)
    argv = ["1024", "768", "2048"] + [str(cfg[k]) for k in space.CONFIG_KEYS] + ["0", "0", "0", "3"]
    assert subprocess.run([TUNER] + argv, capture_output=True, text=True, timeout=120).returncode == 3
    assert subprocess.run([side_tuner] + argv, capture_output=True, text=True, timeout=120).returncode == 0
