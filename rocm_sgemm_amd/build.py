#!/usr/bin/env python3
"""Builds librocm_sgemm.so (gfx950), the tuner trial binary, bench_float, kernel_phases and issue_cost with hipcc, in-tree.

Plays the role of the reference's CMake targets `rocm_sgemm` and `tuner`
(reference rocm_sgemm/CMakeLists.txt:11-89): run the config generator, compile one translation
unit per kernel instantiation in parallel, link.  Flags differ on purpose: gfx950 only, no
-ffast-math and no -mcumode (plain IEEE fp32 on the matrix cores), packed-fp32 VALU ops disabled.

usage: python -m rocm_sgemm_amd.build [--jobs N] [--force] [--no-tuner]
"""

import argparse
import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
GEN_DIR = os.path.join(PKG_DIR, "_build", "gen")
OBJ_DIR = os.path.join(PKG_DIR, "_build", "obj")
CONFIG_JSON = os.path.join(PKG_DIR, "config", "gemm_config.json")
LIB_PATH = os.path.join(PKG_DIR, "librocm_sgemm.so")
TUNER_PATH = os.path.join(PKG_DIR, "config", "tuner")
BENCH_SRC = os.path.join(PKG_DIR, "benchmark", "bench_float.cpp")
BENCH_PATH = os.path.join(PKG_DIR, "benchmark", "bench_float")
PHASES_SRC = os.path.join(PKG_DIR, "benchmark", "kernel_phases.hip")
PHASES_PATH = os.path.join(PKG_DIR, "benchmark", "kernel_phases")
ISSUE_SRC = os.path.join(PKG_DIR, "benchmark", "issue_cost.hip")
ISSUE_PATH = os.path.join(PKG_DIR, "benchmark", "issue_cost")
CALLER_SRC = os.path.join(REPO_DIR, "tests", "cxx", "reference_style_caller.cpp")
CALLER_PATH = os.path.join(REPO_DIR, "tests", "cxx", "reference_style_caller")
# a caller that includes the reference's own host headers by path: built only where that tree is
HEADER_CALLER_SRC = os.path.join(REPO_DIR, "tests", "cxx", "reference_header_caller.cpp")
HEADER_CALLER_PATH = os.path.join(REPO_DIR, "tests", "cxx", "reference_header_caller")
REFERENCE_DIR = "/root/reference"

ARCH = "gfx950"
COMMON_FLAGS = [
    "-std=c++17", "-O3", "-fPIC", f"--offload-arch={ARCH}",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    "-I", os.path.join(REPO_DIR, "include"), "-I", CSRC, "-I", GEN_DIR,
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build the library")
    return exe


def _digest(paths, extra=""):
    h = hashlib.sha256(extra.encode())
    for p in sorted(paths):
        with open(p, "rb") as f:
            h.update(p.encode())
            h.update(f.read())
    return h.hexdigest()


def _compile(job):
    src, obj, stamp_text, force = job
    stamp = obj + ".stamp"
    if not force and os.path.exists(obj) and os.path.exists(stamp):
        with open(stamp) as f:
            if f.read() == stamp_text:
                return src, 0, "", True
    lang = ["-x", "hip"] if src.endswith((".hip", ".cpp")) else []
    cmd = [hipcc()] + COMMON_FLAGS + lang + ["-c", src, "-o", obj,
                                             "-Rpass-analysis=kernel-resource-usage"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode == 0:
        with open(stamp, "w") as f:
            f.write(stamp_text)
    return src, proc.returncode, proc.stdout + proc.stderr, False


def _check_no_spills(log, src):
    """A kernel that spills registers to scratch memory is a bug in the tile-shape constraints.
    Returns one line per spilling kernel."""
    bad = []
    name = None
    for line in log.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            n = int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            if n != 0:
                bad.append((name, n))
    return [f"{os.path.basename(src)}: {name} spills {n} bytes per lane" for name, n in bad]


def build(jobs=None, force=False, tuner=True, verbose=True, defines=(), lib_path=None,
          obj_dir=None, out_dir=None, shapes=None):
    """Generates, compiles and links.  `defines` (extra -D macros), `lib_path` and `obj_dir` exist
    so that an experimental variant can be built beside the shipped library.  `out_dir` builds a
    whole side tree instead - generated sources, objects, `librocm_sgemm.so` and `config/tuner`
    under that directory - for the tuner's exploration mode, which compiles tile shapes from
    outside the shipped family (config/space.py: explore()) without touching the shipped library;
    only the library and the trial binary are built there, and `shapes` limits the side library
    to those tile shapes (plus the default config's)."""
    sys.path.insert(0, os.path.join(PKG_DIR, "config"))
    import generate_config  # noqa: E402

    global COMMON_FLAGS, GEN_DIR, TUNER_PATH
    base = (COMMON_FLAGS, GEN_DIR, TUNER_PATH)
    if out_dir is not None:
        out_dir = os.path.abspath(out_dir)
        GEN_DIR = os.path.join(out_dir, "gen")
        TUNER_PATH = os.path.join(out_dir, "config", "tuner")
        os.makedirs(os.path.dirname(TUNER_PATH), exist_ok=True)
        lib_path = os.path.join(out_dir, "librocm_sgemm.so")
        obj_dir = os.path.join(out_dir, "obj")
        COMMON_FLAGS = [GEN_DIR if f == base[1] else f for f in COMMON_FLAGS]
    COMMON_FLAGS = COMMON_FLAGS + [f"-D{d}" for d in defines]
    try:
        return _build(generate_config, jobs, force, tuner, verbose, lib_path or LIB_PATH,
                      obj_dir or OBJ_DIR, side_tree=out_dir is not None, shapes=shapes)
    finally:
        COMMON_FLAGS, GEN_DIR, TUNER_PATH = base


def _build(generate_config, jobs, force, tuner, verbose, LIB_PATH, OBJ_DIR, side_tree=False, shapes=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    kernel_sources = generate_config.generate(CONFIG_JSON, GEN_DIR, shapes)
    host_sources = [os.path.join(CSRC, "dispatch.cpp"), os.path.join(CSRC, "planner.cpp"),
                    os.path.join(CSRC, "api.cpp")]
    headers = [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".hpp")]
    headers += [os.path.join(REPO_DIR, "include", "rocm_sgemm.h"),
                os.path.join(REPO_DIR, "include", "rocm_sgemm", "gemm.hpp"),
                os.path.join(REPO_DIR, "include", "rocm_sgemm", "layout.hpp")]
    header_digest = _digest(headers, " ".join(COMMON_FLAGS))
    table_digest = _digest([os.path.join(GEN_DIR, "config_table.inc"),
                            os.path.join(GEN_DIR, "kernel_table.inc")])

    work = []
    for src in kernel_sources + host_sources:
        obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
        extra = table_digest if src in host_sources else ""
        work.append((src, obj, _digest([src], header_digest + extra), force))

    jobs = jobs or min(16, os.cpu_count() or 4)
    failed = []
    spilling = []
    done = 0
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, rc, log, cached in pool.map(_compile, work):
            done += 1
            if rc != 0:
                failed.append((src, log))
                continue
            if not cached:
                spilling += _check_no_spills(log, src)
            if verbose and not cached:
                print(f"[{done}/{len(work)}] compiled {os.path.basename(src)}", flush=True)
    if failed:
        for src, log in failed:
            sys.stderr.write(f"--- {src}\n{log}\n")
        raise RuntimeError(f"{len(failed)} translation units failed to compile")
    if spilling and not os.environ.get("RSG_ALLOW_SPILLS"):
        for obj in (w[1] for w in work):  # nothing that spills stays cached as good
            if any(os.path.basename(obj)[:-2] in line for line in spilling) and os.path.exists(obj + ".stamp"):
                os.remove(obj + ".stamp")
        raise RuntimeError("kernels use scratch memory (register spills):\n  " + "\n  ".join(spilling))

    objs = [w[1] for w in work]
    link = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB_PATH] + objs
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + (proc.stdout + proc.stderr)[-4000:])
    if verbose:
        print(f"linked {LIB_PATH}")

    if tuner:
        cmd = [hipcc()] + COMMON_FLAGS + ["-x", "hip", os.path.join(PKG_DIR, "config", "tuner.cpp"),
                                          "-o", TUNER_PATH, "-L", os.path.dirname(LIB_PATH), "-lrocm_sgemm",
                                          "-Wl,-rpath,$ORIGIN/.."]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("tuner build failed:\n" + (proc.stdout + proc.stderr)[-4000:])
        if verbose:
            print(f"linked {TUNER_PATH}")
        if side_tree:
            return LIB_PATH
        # a program written against the reference's public header, linked against this library
        cmd = [hipcc(), "-std=c++17", "-O2", f"--offload-arch={ARCH}", "-Wno-unused-command-line-argument",
               "-I", os.path.join(REPO_DIR, "include"), "-x", "hip", CALLER_SRC, "-o", CALLER_PATH,
               "-L", PKG_DIR, "-lrocm_sgemm", "-Wl,-rpath,$ORIGIN/../../rocm_sgemm_amd"]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("reference-style caller failed to build:\n"
                               + (proc.stdout + proc.stderr)[-4000:])
        if verbose:
            print(f"linked {CALLER_PATH}")
        # the same with the reference's real common/matrix.hpp and common/hip_utils.hpp beside this
        # repository's <rocm_sgemm/gemm.hpp> (nothing of the reference is copied; the binary
        # travels with the tree to machines that do not have the reference)
        if os.path.exists(os.path.join(REFERENCE_DIR, "common", "matrix.hpp")):
            cmd = [hipcc(), "-std=c++17", "-O2", f"--offload-arch={ARCH}", "-Wno-unused-command-line-argument",
                   "-I", os.path.join(REPO_DIR, "include"), "-I", REFERENCE_DIR,
                   "-x", "hip", HEADER_CALLER_SRC, "-o", HEADER_CALLER_PATH,
                   "-L", PKG_DIR, "-lrocm_sgemm", "-Wl,-rpath,$ORIGIN/../../rocm_sgemm_amd"]
            proc = subprocess.run(cmd, capture_output=True, text=True)
            if proc.returncode != 0:
                raise RuntimeError("reference-header caller failed to build:\n"
                                   + (proc.stdout + proc.stderr)[-4000:])
            if verbose:
                print(f"linked {HEADER_CALLER_PATH}")
        # the benchmark program (counterpart of the reference's bench_float), rocBLAS / hipBLASLt rows optional
        rocblas = os.path.exists("/opt/rocm/include/rocblas/rocblas.h")
        cmd = [hipcc(), "-std=c++17", "-O2", f"--offload-arch={ARCH}", "-Wno-unused-command-line-argument",
               "-I", os.path.join(REPO_DIR, "include"), "-x", "hip", BENCH_SRC, "-o", BENCH_PATH,
               "-L", PKG_DIR, "-lrocm_sgemm", "-Wl,-rpath,$ORIGIN/..", "-lpthread"]
        if rocblas:
            cmd += ["-DBENCH_WITH_ROCBLAS", "-L", "/opt/rocm/lib", "-lrocblas", "-Wl,-rpath,/opt/rocm/lib"]
        if os.path.exists("/opt/rocm/include/hipblaslt/hipblaslt.h"):
            cmd += ["-DBENCH_WITH_HIPBLASLT", "-L", "/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,/opt/rocm/lib"]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("bench_float failed to build:\n" + (proc.stdout + proc.stderr)[-4000:])
        if verbose:
            print(f"linked {BENCH_PATH}")
        # per-workgroup time stamps of a launch: its own instantiations of the kernels, compiled with
        # the stamps switched on (the library is built without them); links nothing of the library
        cmd = [hipcc()] + COMMON_FLAGS + ["-DROCM_SGEMM_PHASE_STAMPS", "-I", os.path.join(PKG_DIR, "csrc"),
                                          "-x", "hip", PHASES_SRC, "-o", PHASES_PATH]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("kernel_phases failed to build:\n" + (proc.stdout + proc.stderr)[-4000:])
        if verbose:
            print(f"linked {PHASES_PATH}")
        # what an instruction costs next to back-to-back MFMAs: a microbenchmark, links nothing of the library
        cmd = [hipcc()] + COMMON_FLAGS + ["-x", "hip", ISSUE_SRC, "-o", ISSUE_PATH]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError("issue_cost failed to build:\n" + (proc.stdout + proc.stderr)[-4000:])
        if verbose:
            print(f"linked {ISSUE_PATH}")
    return LIB_PATH


# A tile shape from outside the shipped family whose side library the build always makes, so that
# the exploration path (generator -> side library -> its own trial binary) is exercised end to end
# by a GPU test without compiling anything on the GPU box: 128 x 128 x 32 with a three-stage ring.
EXPLORE_CHECK_SHAPE = (128, 128, 32, 2, 2, 32, 3, 1)
EXPLORE_CHECK_DIR = os.path.join(PKG_DIR, "_build", "explore_check")


def build_explore_check(jobs=None, force=False, verbose=False):
    """Side library + trial binary of EXPLORE_CHECK_SHAPE under EXPLORE_CHECK_DIR."""
    sys.path.insert(0, os.path.join(PKG_DIR, "config"))
    import space  # noqa: E402
    if EXPLORE_CHECK_SHAPE in space.shipped_family():
        raise RuntimeError("the exploration check's tile shape has joined the family: choose another")
    try:
        shapes = space.explore([EXPLORE_CHECK_SHAPE])
        build(jobs=jobs, force=force, out_dir=EXPLORE_CHECK_DIR, shapes=shapes, verbose=verbose)
    finally:
        space.explore([])  # leave the family as shipped
    return os.path.join(EXPLORE_CHECK_DIR, "config", "tuner")


def main():
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--jobs", type=int, default=None)
    ap.add_argument("--force", action="store_true", help="recompile everything")
    ap.add_argument("--no-tuner", action="store_true")
    ap.add_argument("--define", action="append", default=[], help="extra -D macro (experiments)")
    ap.add_argument("--lib-path", default=None, help="where to link the library (experiments)")
    ap.add_argument("--obj-dir", default=None, help="object directory (experiments)")
    ap.add_argument("--explore", nargs="+", metavar="SHAPE", default=None,
                    help="build a side library of these tile shapes (macro_m,macro_n,k_tile,waves_m,waves_n,"
                         "mfma,stages,waves_k each) and its trial binary under --explore-dir, for "
                         "`config/tune.py --explore ... --explore-prebuilt`; the shipped library is not touched")
    ap.add_argument("--explore-dir", default=os.path.join(PKG_DIR, "_build", "explore"))
    a = ap.parse_args()
    if a.explore:
        sys.path.insert(0, os.path.join(PKG_DIR, "config"))
        import space  # noqa: E402
        shapes = space.explore([tuple(int(x) for x in s.split(",")) for s in a.explore])
        build(jobs=a.jobs, force=a.force, out_dir=a.explore_dir, shapes=shapes)
        print(f"side library of {len(shapes)} tile shapes in {a.explore_dir}")
        return
    build(jobs=a.jobs, force=a.force, tuner=not a.no_tuner, defines=a.define, lib_path=a.lib_path,
          obj_dir=a.obj_dir)


if __name__ == "__main__":
    main()
