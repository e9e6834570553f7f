"""bench_float --counters: the benchmark program collects rocprofv3 hardware counters row by row
(matrix-pipe busy %, LDS bank conflicts, HBM bytes).  Collected last: it starts rocprofv3 child
processes, which is slow and the only test that depends on the profiler being installed."""

import os
import re
import shutil
import subprocess

import pytest

pytestmark = pytest.mark.gpu

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(REPO, "rocm_sgemm_amd", "benchmark", "bench_float")


def test_bench_float_counter_rows():
    if shutil.which("rocprofv3") is None:
        pytest.skip("rocprofv3 is not installed")
    print("CASE bench_float --counters", flush=True)
    env = dict(os.environ, TMPDIR="/tmp")
    out = subprocess.run([BENCH, "--shapes", "1024", "--layouts", "rrr", "--warmup", "2", "--iters", "5",
                          "--counters"], capture_output=True, text=True, timeout=600, env=env, cwd="/tmp")
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    rows = [l for l in out.stdout.splitlines() if "}/counters" in l]
    assert len(rows) == 1, out.stdout
    m = re.search(r"\}/counters\s+(-?[\d.]+)\s+(-?[\d.]+)\s+(-?[\d.]+)\s+(-?[\d.]+)\s+(-?[\d.]+)", rows[0])
    assert m is not None, rows[0]
    busy, busy_of_cu, conflicts, hbm_mb, hbm_gbps = map(float, m.groups())
    assert 1.0 < busy <= 100.0
    # over the cycles in which the CUs hold waves the figure leaves out the dispatch overhead the
    # profiler adds around a launch, so it is the higher of the two
    assert busy < busy_of_cu <= 100.0
    assert 0.0 <= conflicts < 5.0
    # at least the algorithmic traffic of a 1024^3 product (12.6 MB), at most a few times that
    assert 12.0 < hbm_mb < 80.0
    assert hbm_gbps > 0.0
