"""Search space of the MI355X SGEMM kernels: parameters, resource model and constraints.

Shared by the config generator (which compiles every tile shape listed here into the library) and
the tuner (which times them).  Takes the place of the reference tuner's nine categorical
parameters and its constraint check (reference rocm_sgemm/config/tune.py:55-65, 100-144), which
describe a wave32 VALU kernel (thread tiles, threads_n); an MFMA kernel is described by

    macro_m x macro_n   output tile of a workgroup
    k_tile              depth staged through LDS per pipeline step
    waves_m x waves_n   wave64 grid of the workgroup
    mfma                32 -> v_mfma_f32_32x32x2_f32, 16 -> v_mfma_f32_16x16x4_f32
    stages              0 -> operands staged through registers into two LDS stages;
                        n >= 2 -> loaded straight into a ring of n LDS stages (ragged problems
                        run the edge-masked variants of the same kernel: 16-byte loads when the
                        operand lines are 16-byte aligned, 4-byte loads otherwise)
    waves_k             replicas of the wave grid along K: replica w multiplies the w-th part of
                        every K-tile over the whole wave tile and the partial tiles are summed
                        through LDS (1 = none); block size = 64 * waves_m * waves_n * waves_k
    split_k, group_m    launch-time only: K slices and tile-order band height
    partial_sums        launch-time only: who adds up the partial tiles of a K split or a stream-K
                        tail: 0 = the library decides (a second kernel), 1 = a second kernel, 2 = the GEMM launch
    wave_slots          launch-time only: 0 = deal the K range of a short last wave of tiles out
                        to all CUs (stream-K tail; slots asked from the runtime), 1 = never

and is bounded by CDNA4's 160 KB LDS per CU, 512 unified registers per lane and 256 CUs.
"""

from itertools import product

LDS_BYTES_PER_CU = 160 * 1024
REGS_PER_LANE = 512  # unified VGPR + AGPR budget of one wave at occupancy 1
NUM_CU = 256
NUM_XCD = 8

PARAM_SPACE = {
    "macro_m": [16, 32, 64, 128, 256],
    "macro_n": [16, 32, 64, 128, 256],
    "k_tile": [16, 32, 64, 128],
    "waves_m": [1, 2, 4],
    "waves_n": [1, 2, 4],
    "mfma": [32, 16],
    "stages": [0, 2, 3, 4],
    "split_k": [1, 2, 4, 8, 16],
    "group_m": [1, 2, 4, 8, 16],
    "wave_slots": [0, 1],
    "waves_k": [1, 2, 4],
    "partial_sums": [0, 1, 2],
}

# A tile shape (what is compiled) is the tuple of SHAPE_KEYS; a config adds the launch-time
# parameters.  CONFIG_KEYS is the field order of struct rocm_sgemm_config, of the tuner binary's
# command line and of its `cfg` lines: fields are appended as they are added, so waves_k sits
# behind the first three launch-time parameters and partial_sums behind it.
SHAPE_KEYS = ("macro_m", "macro_n", "k_tile", "waves_m", "waves_n", "mfma", "stages", "waves_k")
CONFIG_KEYS = SHAPE_KEYS[:7] + ("split_k", "group_m", "wave_slots", "waves_k", "partial_sums")
LAYOUTS = ("row_major", "col_major")


def lds_bytes(macro_m, macro_n, k_tile, x_kc, y_kc, stages=0, waves_k=1):
    """LDS footprint; mirrors tile_config::LDS_BYTES in csrc/sgemm_mfma_kernel.hpp: padded images
    in two stages when register-staged, unpadded images in `stages` stages when direct-to-LDS;
    with waves along K, at least the waves_k partial-tile images."""
    if stages >= 2:
        exchange = waves_k * macro_m * macro_n * 4 if waves_k > 1 else 0
        return max(stages * (macro_m + macro_n) * k_tile * 4, exchange)
    x = macro_m * (k_tile + 4) if x_kc else k_tile * (macro_m + 4)
    y = macro_n * (k_tile + 4) if y_kc else k_tile * (macro_n + 4)
    return 2 * (x + y) * 4


def max_lds_bytes(macro_m, macro_n, k_tile, stages=0, waves_k=1):
    return max(lds_bytes(macro_m, macro_n, k_tile, a, b, stages, waves_k) for a in (0, 1) for b in (0, 1))


def registers_per_lane(shape):
    """Estimate of registers per lane: accumulators + two fragment sets + staging + addressing.
    A pre-filter only: the build rejects any kernel the compiler has to spill."""
    macro_m, macro_n, k_tile, waves_m, waves_n, mfma = shape[:6]
    threads = 64 * waves_m * waves_n * shape[7]
    acc = (macro_m // waves_m) * (macro_n // waves_n) // 64
    tiles = (macro_m // waves_m + macro_n // waves_n) // mfma
    frags = 2 * 4 * tiles
    staging = (macro_m + macro_n) * k_tile // threads
    return acc + frags + staging + staging // 2 + 16


def register_budget(shape):
    """Registers per lane available to one wave: the SIMD's 512 shared by its resident waves."""
    waves = shape[3] * shape[4] * shape[7]
    return REGS_PER_LANE // max(1, -(-waves // 4))


def shape_ok(shape):
    """Constraints a tile shape must satisfy to be compiled (static_asserts of tile_config)."""
    macro_m, macro_n, k_tile, waves_m, waves_n, mfma, stages, waves_k = shape
    if mfma not in (32, 16):
        return False
    if waves_k < 1 or (waves_k > 1 and stages < 2):  # waves along K: direct-to-LDS kernels only
        return False
    if stages != 0 and not 2 <= stages <= 8:
        return False
    if macro_m % (mfma * waves_m) or macro_n % (mfma * waves_n):
        return False
    tm = macro_m // waves_m // mfma
    tn = macro_n // waves_n // mfma
    if tm not in (1, 2, 4, 8) or tn not in (1, 2, 4, 8):
        return False
    # every wave multiplies an even number of k-blocks (of 4 * (64 / mfma) depth) of a K-tile
    if k_tile % (8 * (64 // mfma) * waves_k):
        return False
    threads = 64 * waves_m * waves_n * waves_k
    if threads > 1024:
        return False
    if (macro_m * k_tile // 4) % threads or (macro_n * k_tile // 4) % threads:
        return False
    if waves_k > 1 and (macro_m * macro_n // 4) % threads:  # the summed tile is stored by all threads
        return False
    if max_lds_bytes(macro_m, macro_n, k_tile, stages, waves_k) > LDS_BYTES_PER_CU:
        return False
    if registers_per_lane(shape) > register_budget(shape):
        return False
    if stages >= 2:
        chunks = (macro_m + macro_n) * k_tile // 4 // threads
        if (stages - 2) * chunks >= 64:  # loads in flight are counted by a 6-bit counter
            return False
        if (mfma // max(1, 64 // k_tile)) % (k_tile // 4):  # swizzle independent of the MFMA tile
            return False
    return True


def sums_in_launch(shape):
    """Whether the kernels of a tile shape can add up partial tiles themselves (the kernel's
    tile_config::SUMS_IN_LAUNCH): at most four waves, each owning at most 64 x 64 of the macro
    tile.  For the other shapes partial_sums makes no difference."""
    macro_m, macro_n, _, waves_m, waves_n, _, _, waves_k = shape
    waves = waves_m * waves_n * max(waves_k, 1)
    return waves <= 4 and macro_m * macro_n // waves <= 64 * 64


def swapped(shape):
    """Shape of the kernel that serves a column-major C (operands and tile swapped)."""
    macro_m, macro_n, k_tile, waves_m, waves_n, mfma, stages, waves_k = shape
    return (macro_n, macro_m, k_tile, waves_n, waves_m, mfma, stages, waves_k)


# Tile shapes compiled into the library (closed under `swapped`).  A deliberately small subset of
# the valid points of PARAM_SPACE: big tiles for the compute-bound squares, small ones so that
# skinny or small problems still produce >= 256 workgroups.
_BASE_SHAPES = [
    # direct-to-LDS (stages >= 2); four waves, one per SIMD, each with the whole register file
    (256, 256, 32, 2, 2, 32, 2, 1),
    (256, 128, 32, 2, 2, 32, 2, 1),
    (128, 128, 32, 2, 2, 32, 2, 1),
    (128, 64, 32, 2, 2, 32, 3, 1),
    (64, 64, 32, 2, 2, 32, 2, 1),
    # the same tile with a three-stage ring, for problems whose operand lines are not 16-byte
    # aligned: their 4-byte loads take longer to land, and a K-tile more in flight covers that
    # (1000 x 3000 x 777: 2 - 3 % in the six layouts with such loads on the deep side, 3001 x 1001 x
    # 1501 2.7 %; aligned problems and 1023^3 are 0.5 - 2 % better off with two stages)
    (64, 64, 32, 2, 2, 32, 3, 1),
    # eight waves: two per SIMD cover each other's stalls in prologue and epilogue
    (256, 128, 32, 4, 2, 32, 2, 1),
    (128, 128, 64, 4, 2, 32, 2, 1),
    # K-tile of 16 in a direct-to-LDS ring: 48 KB of LDS and 128 accumulators, so two workgroups
    # share a CU and one's prologue and epilogue hide behind the other's main loop.  Found by the
    # tuner's exploration mode (8192 x 8192 x 1024: 1.5 % over the best shape of the family then)
    (256, 128, 16, 2, 2, 32, 2, 1),
    # K-tiles of 64: half as many pipeline steps (barriers, waits) per unit of depth (the 128 x 128
    # form with four waves came within 1 % of the fastest shape in none of 79 sweeps and in none of
    # 492 tuned entries; the eight-wave form above does)
    (64, 64, 64, 2, 2, 32, 2, 1),
    # waves along K: small macro tiles whose waves still own a 64 x 64 (or 64 x 32) wave tile, for
    # problems that need many tiles to fill the GPU
    (64, 64, 64, 1, 1, 32, 3, 4),
    (64, 32, 64, 1, 1, 32, 3, 4),
    (128, 64, 32, 2, 1, 32, 3, 2),
    (64, 64, 128, 1, 1, 32, 2, 4),
    # 16-row tiles on v_mfma_f32_16x16x4_f32 for problems with M or N <= 16: half the wasted rows of
    # a 32-row tile, and stages small enough for two or three workgroups per CU, i.e. more loads in
    # flight for what is a stream over the other operand (found by the tuner's exploration mode:
    # 4096 x 16 x 4096 14.8 against 16.9 us, 16 x 16384 x 1024 13.2 against 13.9)
    (16, 32, 64, 1, 1, 16, 4, 2),
    (16, 64, 64, 1, 1, 16, 3, 2),
    # register-staged (stages = 0): K-tiles of 16 for very shallow problems
    (256, 128, 16, 2, 2, 32, 0, 1),
]


_FAMILY = None
_EXTRA_SHAPES = []


def _closed(shapes):
    out = []
    for s in shapes:
        for t in (tuple(s), swapped(tuple(s))):
            if not shape_ok(t):
                raise ValueError(f"tile shape {t} violates the kernel's constraints")
            if t not in out:
                out.append(t)
    return out


def family():
    """Tile shapes compiled into the library, plus (exploration only) those of explore()."""
    global _FAMILY
    if _FAMILY is None:
        _FAMILY = _closed(_BASE_SHAPES)
    return list(_FAMILY) + [s for s in _EXTRA_SHAPES if s not in _FAMILY]


def shipped_family():
    """The family without exploration shapes."""
    family()
    return list(_FAMILY)


def explore(shapes):
    """Adds tile shapes from outside the shipped family for this process: the generator then emits
    kernels for them (into a side library, see build.build(out_dir=...)) and the tuner times them.
    Returns the shapes added (closed under `swapped`)."""
    global _EXTRA_SHAPES
    _EXTRA_SHAPES = [s for s in _closed(shapes) if s not in shipped_family()]
    return list(_EXTRA_SHAPES)


def neighbours(shape):
    """Valid tile shapes one step away from `shape` in the search space (another K-tile, ring depth,
    wave grid or waves along K on the same macro tile; the macro tile halved or doubled along one
    side), for the tuner's exploration mode."""
    bm, bn, bk, wm, wn, mfma, stages, wk = shape
    out = set()
    for k in PARAM_SPACE["k_tile"]:
        for st in PARAM_SPACE["stages"]:
            out.add((bm, bn, k, wm, wn, mfma, st, wk))
    for a in PARAM_SPACE["waves_m"]:
        for b in PARAM_SPACE["waves_n"]:
            for w in PARAM_SPACE["waves_k"]:
                out.add((bm, bn, bk, a, b, mfma, stages, w))
    for m2, n2 in ((bm * 2, bn), (bm, bn * 2), (bm // 2, bn), (bm, bn // 2)):
        if m2 in PARAM_SPACE["macro_m"] and n2 in PARAM_SPACE["macro_n"]:
            out.add((m2, n2, bk, wm, wn, mfma, stages, wk))
    out.discard(tuple(shape))
    return sorted(s for s in out if shape_ok(s))


def all_valid_shapes():
    """Every point of PARAM_SPACE that satisfies the constraints (superset of family())."""
    keys = SHAPE_KEYS
    return [s for s in product(*(PARAM_SPACE[k] for k in keys)) if shape_ok(s)]


def config_ok(cfg, M, N, K):
    """Constraints on a full config for a given problem: shape in the family, split_k sane."""
    shape = tuple(cfg[k] for k in SHAPE_KEYS)
    if shape not in family():
        return False
    if cfg["split_k"] < 1 or cfg["group_m"] < 1:
        return False
    # every slice must hold at least one K-tile
    if cfg["split_k"] > 1 and K < cfg["split_k"] * cfg["k_tile"]:
        return False
    return True


def workgroups(cfg, M, N):
    gm = -(-M // cfg["macro_m"])
    gn = -(-N // cfg["macro_n"])
    return gm * gn * cfg["split_k"]


DEFAULT_CONFIG = {
    "macro_m": 128,
    "macro_n": 128,
    "k_tile": 32,
    "waves_m": 2,
    "waves_n": 2,
    "mfma": 32,
    "stages": 2,
    "split_k": 1,
    "group_m": 4,
    "wave_slots": 0,
    "waves_k": 1,
    "partial_sums": 0,
}
