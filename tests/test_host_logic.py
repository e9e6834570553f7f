"""Host-side logic of the library, no GPU needed: exported symbols, config lookup, tile order,
argument validation (all of which run before any HIP call), search-space model and generator."""

import ctypes
import itertools
import json
import math
import os
import re
import subprocess
import sys

import pytest

import rocm_sgemm_amd as rs

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(REPO, "rocm_sgemm_amd", "config"))
import generate_config  # noqa: E402
import space  # noqa: E402


# ---- the C ABI library loads and exports what the headers declare -------------------------------

def test_library_exports_every_declared_c_symbol():
    header = open(os.path.join(REPO, "include", "rocm_sgemm.h")).read()
    declared = set(re.findall(r"\b(rocm_sgemm_[a-z0-9_]+)\s*\(", header))
    assert declared == set(rs.C_SYMBOLS)
    L = rs.lib()
    for name in declared:
        assert getattr(L, name) is not None


def test_library_exports_the_eight_reference_cxx_symbols():
    # what `nm -u` shows for a caller compiled against the reference header
    # (void rocm_sgemm::gemm<(m_layout)c,(m_layout)a,(m_layout)b,float>(float*, float*, float*,
    #  unsigned long, unsigned long, unsigned long, ihipStream_t*&))
    out = subprocess.run(["nm", "-D", "--defined-only", rs.lib_path()], check=True,
                         capture_output=True, text=True).stdout
    for sym in rs.CXX_SYMBOLS:
        assert sym in out
    assert len(set(rs.CXX_SYMBOLS)) == 8
    dem = subprocess.run(["c++filt", rs.cxx_symbol(1, 0, 1)], check=True, capture_output=True,
                         text=True).stdout
    assert "rocm_sgemm::gemm<(rocm_sgemm::m_layout)1, (rocm_sgemm::m_layout)0, (rocm_sgemm::m_layout)1, float>" in dem
    assert "ihipStream_t*&" in dem


def test_version_string():
    assert "gfx950" in rs.version()


# ---- config lookup (reference generate_config.py:174-267 semantics) ----------------------------

def _mirror(key, cfg):
    """(M, N, K, a, b, c) under a config launches exactly what (N, M, K, !b, !a, !c) launches under
    the config with macro_m / macro_n and waves_m / waves_n exchanged: a column-major C is computed
    as C^T = B^T A^T with operands, problem and tile shape exchanged."""
    M, N, K, a, b, c = key
    d = cfg.as_dict()
    d.update(macro_m=cfg.macro_n, macro_n=cfg.macro_m, waves_m=cfg.waves_n, waves_n=cfg.waves_m)
    return (N, M, K, 1 - b, 1 - a, 1 - c), rs.Config.from_dict(d)


def _with_mirrors(table):
    """What the library searches: the tuned entries plus the mirror image of every entry whose
    mirror is not a tuned entry itself, in key order."""
    keys = {k for k, _ in table}
    extra = [_mirror(k, cfg) for k, cfg in table]
    return sorted(list(table) + [(k, cfg) for k, cfg in extra if k not in keys], key=lambda e: e[0])


def _py_select(table, M, N, K, a, b, c):
    """Independent restatement of the lookup rule for cross-checking the C++ one."""
    for key, cfg in table:
        if key == (M, N, K, a, b, c):
            return cfg

    def dist(key):
        return sum((math.log2(x) - math.log2(y)) ** 2 for x, y in zip((M, N, K), key[:3]))

    def whole(dims):
        return dims[0] % 4 == 0 and dims[1] % 4 == 0 and dims[2] % 4 == 0

    same = [(dist(k), i) for i, (k, _) in enumerate(table) if k[3:] == (a, b, c)]
    kind = [(d, i) for d, i in same if whole(table[i][0][:3]) == whole((M, N, K))]
    pool = kind or same or [(dist(k), i) for i, (k, _) in enumerate(table)]
    best = min(pool, key=lambda t: (t[0], t[1]))
    return table[best[1]][1]


def _fit_split(cfg, M, N, K):
    cfg = dict(cfg)
    if cfg["split_k"] > 1:
        tiles = -(-M // cfg["macro_m"]) * -(-N // cfg["macro_n"])
        k_tiles = -(-K // cfg["k_tile"])
        if tiles * cfg["split_k"] * 4 <= 256 * 3 and k_tiles >= 8:
            cfg["split_k"], cfg["wave_slots"] = 1, 0
        elif tiles * cfg["split_k"] > 4 * 256:
            cfg["split_k"] = max(1, min(cfg["split_k"], -(-2 * 256 // tiles)))
    return cfg


def _py_plan(table, M, N, K, a, b, c):
    """Restatement of the planning rule around the library's own cost model: table entries are
    returned as they are; otherwise the nearest entry's config, unless one of the four nearest
    entries of the same layouts and kind (split_k fitted first) or one of the larger direct-to-LDS
    tile shapes (or smaller ones with waves along K) at split_k 1, 2, 3, 4, 6 or 8 is predicted at least
    5 % faster."""
    nearest = _py_select(table, M, N, K, a, b, c).as_dict()
    if any(key == (M, N, K, a, b, c) for key, _ in table):
        return nearest

    def dist(key):
        return sum((math.log2(x) - math.log2(y)) ** 2 for x, y in zip((M, N, K), key[:3]))

    def kind(dims):
        return dims[0] % 4 == 0 and dims[1] % 4 == 0 and dims[2] % 4 == 0

    pool = [(dist(k), i) for i, (k, _) in enumerate(table) if k[3:] == (a, b, c) and kind(k[:3]) == kind((M, N, K))]
    pool.sort(key=lambda t: (t[0], t[1]))
    best = _fit_split(nearest, M, N, K)
    nearest_us = best_us = rs.predict_us(best, M, N, K)
    candidates = [_fit_split(table[i][1].as_dict(), M, N, K) for _, i in pool[:4]]
    for fam in rs.family():
        if fam.stages < 2 or ((fam.macro_m < 64 or fam.macro_n < 64) and fam.waves_k <= 1):
            continue
        if fam.mfma != 32 and not ((fam.macro_m == 16 and M <= 16) or (fam.macro_n == 16 and N <= 16)):
            continue  # 16-row (16-column) tiles only where the problem has no more rows (columns)
        k_tiles = -(-K // fam.k_tile)
        for split in (1, 2, 3, 4, 6, 8):
            if split > 1 and k_tiles < 2 * split:
                break
            candidates.append(dict(fam.as_dict(), split_k=split, group_m=4, wave_slots=0))
    for cand in candidates:
        us = rs.predict_us(cand, M, N, K)
        if us < best_us and us <= 0.95 * nearest_us:
            best, best_us = cand, us
    return best


def test_cost_model_orders_the_obvious_cases():
    big = dict(macro_m=256, macro_n=256, k_tile=32, waves_m=4, waves_n=2, mfma=32, stages=2, split_k=1,
               group_m=4, wave_slots=0)
    small = dict(big, macro_m=64, macro_n=64, waves_m=2, waves_n=2)
    # more depth costs more; a big problem prefers big tiles, a small one small tiles
    assert rs.predict_us(big, 4096, 4096, 8192) > rs.predict_us(big, 4096, 4096, 4096)
    assert rs.predict_us(big, 8192, 8192, 8192) < rs.predict_us(small, 8192, 8192, 8192)
    assert rs.predict_us(small, 512, 512, 512) < rs.predict_us(big, 512, 512, 512)
    # 400 tiles on 256 CUs: the stream-K tail is worth a whole wave of tiles
    assert rs.predict_us(big, 5120, 5120, 5120) < 0.85 * rs.predict_us(dict(big, wave_slots=1), 5120, 5120, 5120)
    # 16 tiles of 128 x 128 with K = 16384: unsplit and without a tail 240 CUs idle
    mid = dict(big, macro_m=128, macro_n=128, waves_m=2, waves_n=2)
    assert rs.predict_us(mid, 512, 512, 16384) < 0.3 * rs.predict_us(dict(mid, wave_slots=1), 512, 512, 16384)
    assert rs.lib().rocm_sgemm_predict_us(None, 1, 1, 1, 1) < 0
    # sixteen 1024^3 products fill the GPU like one large problem: no K split, and a config the model
    # rates at least as fast for the batch as the one a single product gets (since the main loop
    # lost its stalls, small tiles cost next to nothing, so it may well be the same config);
    # one of them alone is planned as before
    one, many = rs.find_config(1024, 1024, 1024), rs.find_config(1024, 1024, 1024, batch_count=16)
    assert one.as_dict() == dict(rs.table())[(1024, 1024, 1024, 0, 0, 0)].as_dict()
    assert many.split_k == 1
    assert rs.predict_us(many, 1024, 1024, 1024, 16) <= rs.predict_us(one, 1024, 1024, 1024, 16)
    assert rs.find_config(512, 512, 2048, batch_count=32).split_k == 1


def test_cost_model_matches_the_fitting_scripts_restatement():
    """config/fit_cost_model.py restates the C++ cost model term by term (that is what its fit
    runs on) and carries the compiled constants; the two must agree on random configs and sizes,
    on every branch: K split, stream-K tail, plain partial wave, all three problem kinds."""
    import random
    import fit_cost_model as fcm
    p = fcm.compiled_constants()
    rnd = random.Random(3)
    family = [f.as_dict() for f in rs.family()]
    seen = set()
    for _ in range(3000):
        c = dict(rnd.choice(family), split_k=rnd.choice([1, 1, 2, 4, 8]), group_m=4,
                 wave_slots=rnd.choice([0, 0, 0, 1, 48]))
        step = rnd.choice([1, 4, 64])
        M, N, K = [max(step, rnd.randint(32, 6000) // step * step) for _ in range(3)]
        batch = rnd.choice([1, 1, 1, 3, 40])
        got, want = rs.predict_us(c, M, N, K, batch), fcm.predict(p, c, M, N, K, batch)
        assert abs(got - want) <= 1e-9 * want, (c, M, N, K, batch, got, want)
        if batch > 1:
            continue
        tiles = -(-M // c["macro_m"]) * -(-N // c["macro_n"])
        seen.add(("split" if c["split_k"] > 1 else
                  "tail" if fcm.tail_applies(c, tiles, -(-K // c["k_tile"]), K)[0] else "plain", step))
    assert len(seen) == 9


def test_table_is_sorted_by_reference_key_order():
    keys = [k for k, _ in rs.table()]
    assert keys == sorted(keys) and len(set(keys)) == len(keys)


def test_exact_hits_return_their_entry():
    for key, cfg in rs.table():
        M, N, K, a, b, c = key
        assert rs.find_config(M, N, K, a, b, c).as_dict() == cfg.as_dict()


@pytest.mark.parametrize("shape", [(1000, 3000, 777), (4095, 4097, 4093), (128, 4096, 4096),
                                   (16384, 16384, 16384), (1, 1, 1), (3000, 3000, 3000),
                                   (1024, 1024, 16384), (8192, 8192, 1024), (1448, 1448, 1448),
                                   (3840, 3840, 3840), (4010, 4010, 4010), (2000, 2000, 2048), (256, 256, 16384),
                                   (512, 512, 8192), (2048, 2048, 16384), (96, 4096, 4096),
                                   (1000, 1000, 4096), (5000, 5000, 5024), (640, 640, 640)])
def test_nearest_neighbour_fallback_matches_restatement(shape):
    table = _with_mirrors(rs.table())
    for a, b, c in itertools.product((0, 1), repeat=3):
        got = rs.find_config(*shape, a, b, c)
        assert got.as_dict() == _py_plan(table, *shape, a, b, c)
        assert rs.nearest_config(*shape, a, b, c).as_dict() == _py_select(table, *shape, a, b, c).as_dict()


def test_mirror_image_of_a_tuned_entry_is_an_entry():
    """A rectangular entry tuned in one layout serves its mirror image (transposed problem, layouts
    of A and B exchanged and flipped, C flipped) with the tile shape exchanged - unless the mirror
    was tuned itself, in which case its own entry wins."""
    tuned = dict(rs.table())
    checked = 0
    for key, cfg in rs.table():
        mkey, mcfg = _mirror(key, cfg)
        assert _mirror(mkey, mcfg)[0] == key and _mirror(mkey, mcfg)[1].as_dict() == cfg.as_dict()
        want = tuned[mkey] if mkey in tuned else mcfg
        assert rs.find_config(*mkey).as_dict() == want.as_dict(), (key, mkey)
        assert rs.nearest_config(*mkey).as_dict() == want.as_dict()
        assert rs.config_supported(want, mkey[5], mkey[3], mkey[4])
        checked += mkey not in tuned
    assert checked > 0  # the shipped table does hold rectangular entries without a tuned mirror


def test_whole_tile_and_ragged_problems_look_up_entries_of_their_own_kind():
    """3840^3 (aligned operand lines) lies as close to the 4095 x 4097 x 4093 entry (odd leading
    dimensions) as to 4096^3, and 4010^3 the other way round; each must get an entry of its own
    kind.  2000 x 2000 x 2040 is ragged in all three dimensions but every one is a multiple of 4,
    so it counts as aligned."""
    table = {k: c.as_dict() for k, c in rs.table()}
    if (4095, 4097, 4093, 0, 0, 0) not in table or (4096, 4096, 4096, 0, 0, 0) not in table:
        pytest.skip("the shipped table holds neither of the two entries")
    def aligned(k):
        return k[0] % 4 == 0 and k[1] % 4 == 0 and k[2] % 4 == 0
    whole_entries = [c for k, c in table.items() if k[3:] == (0, 0, 0) and aligned(k)]
    ragged_entries = [c for k, c in table.items() if k[3:] == (0, 0, 0) and not aligned(k)]
    assert rs.nearest_config(2000, 2000, 2040).as_dict() in whole_entries
    assert rs.nearest_config(3840, 3840, 3840).as_dict() in whole_entries
    assert rs.nearest_config(4010, 4010, 4010).as_dict() in ragged_entries
    assert rs.nearest_config(4010, 4010, 4010).as_dict() == table[(4095, 4097, 4093, 0, 0, 0)]


def test_inherited_split_k_is_fitted_to_the_problem():
    """A problem a quarter as wide and as tall as a table entry that splits K (an eighth as wide, for
    a skinny entry) inherits that entry's config from the nearest-entry rule, split_k included -
    which would put a fraction of the entry's workgroups on 256 CUs.  The plan must fill the GPU instead: either unsplit with the
    stream-K tail dealing the K range out to every CU, or with tiles x split_k covering at least
    half the CUs.  A table entry itself is never altered."""
    table = {k: c.as_dict() for k, c in rs.table()}
    tried = 0
    for (M, N, K, a, b, c), entry in table.items():
        if (a, b, c) != (0, 0, 0) or entry["split_k"] <= 1 or max(M, N) < 1024:
            continue
        assert rs.find_config(M, N, K).as_dict() == entry  # the entry itself is served as it is
        m, n = (M // 4, N // 4) if min(M, N) >= 256 else ((M // 8, N) if M > N else (M, N // 8))
        nearest = rs.nearest_config(m, n, K).as_dict()
        if (m, n, K, 0, 0, 0) in table or nearest["split_k"] <= 1:
            continue
        tried += 1
        small = rs.find_config(m, n, K).as_dict()
        groups = -(-m // small["macro_m"]) * -(-n // small["macro_n"]) * small["split_k"]
        inherited = -(-m // nearest["macro_m"]) * -(-n // nearest["macro_n"]) * nearest["split_k"]
        assert (small["split_k"] == 1 and small["wave_slots"] == 0) or groups >= min(128, inherited), (m, n, K, small)
        # the plan is the nearest entry's config (its split fitted to this problem) or one the
        # model rates faster than that
        fitted = _fit_split(nearest, m, n, K)
        assert small in (nearest, fitted) or rs.predict_us(small, m, n, K) < rs.predict_us(fitted, m, n, K)
    if tried == 0:
        pytest.skip("no row-major table entry splits K at present")


def test_every_table_config_has_a_kernel_for_its_layout():
    # the reference can leave a null slot (kernel_launcher.hpp:89-94); this table must not
    for (M, N, K, a, b, c), cfg in rs.table():
        assert rs.config_supported(cfg, c, a, b), (M, N, K, a, b, c, cfg)


def test_family_is_closed_under_operand_swap():
    shapes = {tuple(f.as_dict()[k] for k in space.SHAPE_KEYS) for f in rs.family()}
    assert shapes == set(space.family())
    for s in shapes:
        assert space.swapped(s) in shapes


# ---- argument validation: all of it happens before the first HIP call ---------------------------

FAKE = 0x1000  # never dereferenced: validation fails first


def test_rejects_null_pointers_and_zero_dims():
    for args in [(None, FAKE, FAKE, 4, 4, 4), (FAKE, None, FAKE, 4, 4, 4), (FAKE, FAKE, None, 4, 4, 4),
                 (FAKE, FAKE, FAKE, 0, 4, 4), (FAKE, FAKE, FAKE, 4, 0, 4), (FAKE, FAKE, FAKE, 4, 4, 0)]:
        with pytest.raises(rs.SgemmError) as e:
            rs.gemm(*args)
        assert e.value.status == rs.STATUS_INVALID_ARG


def test_general_form_rejects_bad_leading_dimensions_strides_and_batches():
    def call(**kw):
        args = dict(M=8, N=8, K=8, batch_count=1)
        args.update(kw)
        rs.gemm_strided_batched(FAKE, FAKE, FAKE, **args)
    for kw, text in [(dict(lda=7), "leading dimension"), (dict(ldb=4), "leading dimension"),
                     (dict(ldc=1), "leading dimension"), (dict(stride_a=-1), "negative"),
                     (dict(batch_count=0), "batch count"), (dict(batch_count=70000), "batch count"),
                     (dict(batch_count=2, stride_c=63), "overlap"),
                     (dict(batch_count=2, stride_c=64, ldc=9), "overlap")]:
        with pytest.raises(rs.SgemmError) as e:
            call(**kw)
        assert e.value.status == rs.STATUS_INVALID_ARG and text in str(e.value), (kw, str(e.value))


def test_rejects_bad_layout_and_oversized_dim():
    L = rs.lib()
    assert L.rocm_sgemm_f32(2, 0, 0, FAKE, FAKE, FAKE, 4, 4, 4, None) == rs.STATUS_INVALID_ARG
    assert b"layout" in L.rocm_sgemm_last_error()
    assert L.rocm_sgemm_f32(0, 0, 0, FAKE, FAKE, FAKE, 2**31, 4, 4, None) == rs.STATUS_INVALID_ARG
    with pytest.raises(ValueError):
        rs.gemm(FAKE, FAKE, FAKE, 4, 4, 4, layout_a="diagonal")


def test_unknown_tile_shape_raises_no_kernel():
    # the condition under which the reference throws std::runtime_error("No kernel available ...")
    cfg = rs.family()[0].as_dict()
    cfg["macro_m"] = 96
    assert not rs.config_supported(cfg)
    with pytest.raises(rs.NoKernelError) as e:
        rs.gemm_with_config(cfg, FAKE, FAKE, FAKE, 128, 128, 128)
    assert "No kernel available" in str(e.value)


def test_bad_split_is_a_bad_config():
    cfg = rs.family()[0].as_dict()
    cfg["split_k"] = 0
    with pytest.raises(rs.SgemmError) as e:
        rs.gemm_with_config(cfg, FAKE, FAKE, FAKE, 128, 128, 128)
    assert e.value.status == rs.STATUS_BAD_CONFIG


# ---- XCD-aware tile order ----------------------------------------------------------------------

@pytest.mark.parametrize("grid_m,grid_n,group_m", [(1, 1, 4), (16, 16, 4), (32, 32, 8), (7, 13, 4),
                                                   (13, 7, 16), (1, 40, 4), (40, 1, 4), (3, 3, 1),
                                                   (17, 16, 4), (64, 2, 8)])
def test_tile_order_is_a_bijection(grid_m, grid_n, group_m):
    seen = set()
    for wg in range(grid_m * grid_n):
        tm, tn = rs.map_workgroup(wg, grid_m, grid_n, group_m)
        assert 0 <= tm < grid_m and 0 <= tn < grid_n
        seen.add((tm, tn))
    assert len(seen) == grid_m * grid_n


def test_tile_order_keeps_an_xcd_compact():
    """At 4096^2 with 256x256 tiles (16 x 16 grid, one wave of 256 workgroups) the 32 workgroups
    of one XCD (ids congruent mod 8) must cover a 4 x 8 patch: 4 A panels + 8 B panels per L2."""
    for xcd in range(8):
        tiles = [rs.map_workgroup(wg, 16, 16, 4) for wg in range(xcd, 256, 8)]
        assert len({t[0] for t in tiles}) == 4
        assert len({t[1] for t in tiles}) == 8


def test_tile_order_rejects_out_of_range():
    with pytest.raises(rs.SgemmError):
        rs.map_workgroup(256, 16, 16, 4)


# ---- search space model and generator ----------------------------------------------------------

def test_space_constraints():
    assert space.shape_ok((256, 256, 16, 2, 2, 32, 0, 1))
    assert not space.shape_ok((256, 256, 64, 2, 2, 32, 0, 1))  # 2 stages of 256x(64+4)x2 floats > 160 KB
    assert not space.shape_ok((96, 128, 16, 2, 2, 32, 0, 1))  # wave tile not a multiple of 32
    assert not space.shape_ok((128, 128, 24, 2, 2, 32, 0, 1))  # odd number of k-blocks
    assert not space.shape_ok((128, 128, 32, 1, 1, 32, 0, 1))  # register budget
    assert space.lds_bytes(256, 256, 16, 1, 0) == 2 * (256 * 20 + 16 * 260) * 4
    # direct-to-LDS: unpadded images, `stages` of them
    assert space.lds_bytes(256, 256, 32, 1, 0, 2) == 2 * 512 * 32 * 4
    assert space.shape_ok((256, 256, 32, 2, 4, 32, 2, 1))
    assert not space.shape_ok((256, 256, 32, 2, 4, 32, 3, 1))  # 3 x 64 KB > 160 KB
    assert not space.shape_ok((128, 128, 32, 2, 2, 32, 1, 1))  # a ring has at least two stages
    assert all(space.max_lds_bytes(*s[:3], s[6], s[7]) <= space.LDS_BYTES_PER_CU for s in space.family())
    assert set(space.family()) <= set(space.all_valid_shapes())
    # waves along K: direct-to-LDS only, an even number of k-blocks per wave, <= 1024 threads,
    # and LDS for the partial-tile images
    assert space.shape_ok((64, 64, 64, 1, 1, 32, 2, 4))
    assert not space.shape_ok((64, 64, 64, 1, 1, 32, 0, 4))
    assert not space.shape_ok((64, 64, 32, 1, 1, 32, 2, 4))  # one k-block per wave
    assert not space.shape_ok((256, 256, 32, 2, 4, 32, 2, 2))  # 2 x 256 x 256 floats > 160 KB
    assert space.lds_bytes(64, 64, 32, 1, 0, 2, 4) == 4 * 64 * 64 * 4  # the images, more than the stages
    # which shapes can add up partial tiles inside the launch (at most four waves of at most 64 x 64 each)
    assert space.sums_in_launch((128, 128, 32, 2, 2, 32, 2, 1)) and space.sums_in_launch((64, 64, 64, 1, 1, 32, 3, 4))
    assert space.sums_in_launch((128, 64, 32, 2, 1, 32, 3, 2))
    assert not space.sums_in_launch((256, 256, 32, 2, 2, 32, 2, 1))  # 128 x 128 per wave
    assert not space.sums_in_launch((256, 128, 32, 4, 2, 32, 2, 1))  # eight waves


def test_generator_outputs(tmp_path):
    cfg = dict(space.DEFAULT_CONFIG)
    doc = {"configurations": [
        {"range": {"M": 512, "N": 256, "K": 128},
         "layout": {"A": "col_major", "B": "row_major", "C": "col_major"}, "config": cfg},
        {"range": {"M": 64, "N": 256, "K": 128},
         "layout": {"A": "row_major", "B": "row_major", "C": "row_major"}, "config": cfg},
    ]}
    j = tmp_path / "t.json"
    j.write_text(json.dumps(doc))
    srcs = generate_config.generate(str(j), str(tmp_path / "gen"))
    assert len(srcs) == 4 * len(space.family())
    # a direct-to-LDS shape compiles a full-tile kernel and two masked kernels (16-byte and 4-byte
    # loads), a register-staged shape a full-tile and one masked kernel
    dtl = [p for p in srcs if "_s2_" in os.path.basename(p)]
    assert dtl and all(open(p).read().count("launch_kernel<") == 3 for p in dtl)
    staged = [p for p in srcs if "_s" not in os.path.basename(p).split("_m")[1]]
    assert staged and all(open(p).read().count("launch_kernel<") == 2 for p in staged)

    table = (tmp_path / "gen" / "config_table.inc").read_text()
    assert table.index("{64u, 256u, 128u, 0, 0, 0") < table.index("{512u, 256u, 128u, 1, 0, 1")
    ktab = (tmp_path / "gen" / "kernel_table.inc").read_text()
    assert f"kernel_family_size = {len(space.family())}" in ktab
    # null slots: the two masked direct-to-LDS variants of a register-staged shape, the
    # register-staged variant of a direct-to-LDS shape; four orientations each
    assert ktab.count("nullptr") == 4 * sum(2 if f[6] == 0 else 1 for f in space.family())
    bad = dict(cfg, macro_m=96)
    doc["configurations"][0]["config"] = bad
    j.write_text(json.dumps(doc))
    with pytest.raises(ValueError):
        generate_config.generate(str(j), str(tmp_path / "gen2"))


def test_shipped_json_matches_compiled_table():
    entries = generate_config.load_table(os.path.join(REPO, "rocm_sgemm_amd", "config",
                                                      "gemm_config.json"))
    compiled = rs.table()
    assert len(entries) == len(compiled)
    for e, (key, cfg) in zip(entries, compiled):
        assert tuple(e[:6]) == key and e[6] == cfg.as_dict()


# ---- tuner driver (fake trial binary) ------------------------------------------------------------

import tune  # noqa: E402


class _FakeProc:
    def __init__(self, out):
        self.returncode, self.stdout, self.stderr = 0, out, ""


def _fake_runner(best_shape, best_group):
    """Pretends to be the trial binary: every config takes 2 ms except the planted optimum."""
    calls = []

    def run(cmd, capture_output=True, text=True, timeout=None):
        calls.append(cmd)
        if cmd[1] == "--sweep":
            splits = [int(x) for x in cmd[cmd.index("--splits") + 1].split(",")]
            groups = [int(x) for x in cmd[cmd.index("--groups") + 1].split(",")]
            lines = []
            for s in space.family():
                for sp in splits:
                    for g in groups:
                        ms = 1.0 if (s == best_shape and sp == 1) else 2.0
                        lines.append("cfg " + " ".join(map(str, s[:7] + (sp, g, 0, s[7], 0)))
                                     + f" avg_ms {ms:.4f} min_ms {ms:.4f} tflops 1.00 ok 1")
            lines.append("cfg 32 32 32 1 1 32 0 1 4 0 1 0 avg_ms 0.0100 min_ms 0.0100 tflops 9.00 ok 0")
            return _FakeProc("\n".join(lines))
        cfg = dict(zip(space.CONFIG_KEYS, map(int, cmd[4:4 + len(space.CONFIG_KEYS)])))
        shape = tuple(cfg[k] for k in space.SHAPE_KEYS)
        ms = 0.5 if (shape == best_shape and cfg["group_m"] == best_group) else 1.5
        return _FakeProc(f"time: {ms:.4f} ms  min: {ms:.4f} ms  avg_tflops: 1  max_tflops: 1\n")
    return run, calls


def test_tuner_driver_finds_planted_optimum_and_merges(tmp_path):
    best_shape = (256, 128, 32, 4, 2, 32, 2, 1)
    run, calls = _fake_runner(best_shape, 8)
    t = tune.Tuner("tuner", budget=400, runner=run, verbose=False)
    rec = t.tune_problem(4096, 4096, 4096, (0, 1, 0))
    assert tuple(rec["config"][k] for k in space.SHAPE_KEYS) == best_shape
    assert rec["config"]["group_m"] == 8 and rec["config"]["split_k"] == 1
    assert rec["avg_time_ms"] == 0.5  # the wrong-result line (ok 0) must never win
    # merge keeps untouched entries and the schema round-trips through the generator
    existing = tune.load_existing_json(os.path.join(REPO, "rocm_sgemm_amd", "config", "gemm_config.json"))
    merged = tune.merge_results(existing, {(4096, 4096, 4096, 0, 1, 0): rec})
    assert len(merged) == len(existing)
    out = tmp_path / "tuned.json"
    out.write_text(json.dumps(tune.to_json(merged)))
    entries = generate_config.load_table(str(out))
    hit = [e for e in entries if tuple(e[:6]) == (4096, 4096, 4096, 0, 1, 0)][0]
    assert hit[6]["macro_m"] == 256 and hit[6]["macro_n"] == 128 and hit[6]["group_m"] == 8


def test_tuner_budget_and_split_candidates():
    run, calls = _fake_runner((128, 128, 64, 4, 2, 32, 2, 1), 4)
    t = tune.Tuner("tuner", budget=5, runner=run, verbose=False)
    rec = t.tune_problem(1024, 1024, 16384, (0, 0, 0))
    # the family sweep is one process and always complete; the budget only stops phase 2
    assert not any(c[1] != "--sweep" for c in calls)
    assert tuple(rec["config"][k] for k in space.SHAPE_KEYS) == (128, 128, 64, 4, 2, 32, 2, 1)
    assert tune.split_candidates((256, 256, 16, 2, 2, 32, 0, 1), 8192, 8192, 8192) == [1]
    assert 4 in tune.split_candidates((256, 256, 16, 2, 2, 32, 0, 1), 1024, 1024, 16384)
    assert tune.parse_layouts(["r,c,r", "col_major,row_major,col_major"]) == [(0, 1, 0), (1, 0, 1)]
    assert tune.parse_sizes(["128,4096,4096"]) == [(128, 4096, 4096)]


def test_tuner_exploration_finds_a_planted_optimum_outside_the_family(tmp_path):
    """--explore: the planted optimum is a tile shape the library does not ship.  The family sweep
    cannot see it; the exploration compiles it (here: a stand-in for the side build records what it
    was asked to compile), times it through the side trial binary and reports it as the winner."""
    planted = (256, 128, 16, 2, 2, 32, 4, 1)
    assert space.shape_ok(planted) and planted not in space.shipped_family()
    assert planted in space.neighbours((256, 128, 32, 2, 2, 32, 2, 1))
    built = []

    def runner_for(which):
        def run(cmd, capture_output=True, text=True, timeout=None):
            # the shipped binary knows the family only, the side binary what was compiled into it
            shapes = space.shipped_family() if which == "family" else built[-1][1]
            if cmd[1] == "--sweep":
                splits = [int(x) for x in cmd[cmd.index("--splits") + 1].split(",")]
                lines = []
                for sh in shapes:
                    for sp in splits:
                        ms = 0.5 if sh == planted and sp == 1 else (1.0 if sh == (256, 128, 32, 2, 2, 32, 2, 1) and sp == 1 else 2.0)
                        lines.append("cfg " + " ".join(map(str, sh[:7] + (sp, 4, 0, sh[7], 0)))
                                     + f" avg_ms {ms:.4f} min_ms {ms:.4f} tflops 1.00 ok 1")
                return _FakeProc("\n".join(lines))
            return _FakeProc("time: 3.0000 ms  min: 3.0000 ms  avg_tflops: 1  max_tflops: 1\n")
        return run

    def side_build(out_dir, shapes):
        built.append((out_dir, list(shapes)))
        return os.path.join(out_dir, "config", "tuner")

    fam = tune.Tuner("tuner", budget=30, runner=runner_for("family"), verbose=False)
    try:
        found = tune.explore([(4096, 4096, 4096)], [(0, 0, 0)], [], fam, str(tmp_path), max_shapes=64,
                             side_build=side_build,
                             make_tuner=lambda path, shapes: tune.Tuner(path, budget=30, runner=runner_for("side"),
                                                                        verbose=False, shapes=shapes),
                             log=lambda *a: None)
        assert len(built) == 1 and planted in built[0][1]
        assert all(sh not in space.shipped_family() for sh in built[0][1])
        assert len(found) == 1 and found[0]["winner"]
        assert tuple(found[0]["explored"]["config"][k] for k in space.SHAPE_KEYS) == planted
        assert found[0]["explored"]["avg_ms"] == 0.5 and found[0]["family"]["avg_ms"] == 1.0
        # named shapes are taken as they are; one that is in the family already is not compiled again
        built.clear()
        found = tune.explore([(4096, 4096, 4096)], [(0, 0, 0)], [planted, (256, 256, 32, 2, 2, 32, 2, 1)], fam,
                             str(tmp_path), side_build=side_build,
                             make_tuner=lambda path, shapes: tune.Tuner(path, budget=30, runner=runner_for("side"),
                                                                        verbose=False, shapes=shapes),
                             log=lambda *a: None)
        assert [sorted(b[1]) for b in built] == [sorted({planted, space.swapped(planted)})]
        assert found[0]["winner"]
    finally:
        space.explore([])  # leave the family as shipped for the other tests
    assert space.family() == space.shipped_family()
    assert tune.parse_shapes(["256,128,16,2,2,32,4,1"]) == [planted]
    with pytest.raises(ValueError):
        tune.parse_shapes(["256,256,32,2,4,32,3,1"])  # three stages of 64 KB exceed the LDS


def test_workspace_query_is_host_only_and_consistent_with_the_plan():
    """rocm_sgemm_workspace_bytes: what the planned config of a problem keeps as partial products.
    No GPU is touched; a plan that neither splits K nor deals out a tail keeps nothing, a K split
    keeps split_k packed M x N partials."""
    assert rs.workspace_bytes(4096, 4096, 4096) == 0  # 256 tiles of 256 x 256: one full wave
    seen_split = False
    for (M, N, K) in [(1024, 1024, 16384), (512, 512, 8192), (300, 260, 4096), (32, 4096, 4096), (8, 4096, 4096),
                      (256, 256, 16384), (192, 192, 8192)]:
        for lay in (("row_major",) * 3, ("col_major",) * 3):
            cfg = rs.find_config(M, N, K, *lay)
            got = rs.workspace_bytes(M, N, K, *lay)
            if cfg.split_k > 1:
                k_tiles = -(-K // cfg.k_tile)
                slice_tiles = -(-k_tiles // min(cfg.split_k, k_tiles))
                assert got == 4 * M * N * -(-k_tiles // slice_tiles), (M, N, K, lay, cfg.as_dict())
                seen_split = True
            else:
                assert got % (4 * cfg.macro_m * cfg.macro_n) == 0, (M, N, K, lay)  # whole partial tiles, or none
    assert seen_split
    with pytest.raises(rs.SgemmError):
        rs.workspace_bytes(0, 16, 16)


def test_cmake_imported_target_builds_a_reference_style_caller(tmp_path):
    """The CMake change a maintainer of the reference makes: `add_subdirectory(rocm_sgemm)` becomes
    an imported target of the same name that points at this library.  A ten-line project with that
    target must configure and link a caller written against the reference's header (the one that
    includes the reference's own common/ headers where that tree exists)."""
    import shutil
    cmake = shutil.which("cmake")
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if cmake is None or not os.path.exists(hipcc):
        pytest.skip("needs cmake and hipcc")
    with_reference = os.path.exists("/root/reference/common/matrix.hpp")
    source = os.path.join(REPO, "tests", "cxx",
                          "reference_header_caller.cpp" if with_reference else "reference_style_caller.cpp")
    (tmp_path / "CMakeLists.txt").write_text(f"""cmake_minimum_required(VERSION 3.21)
project(caller_of_rocm_sgemm LANGUAGES CXX)
set(MI355X_SGEMM "{REPO}")
# --- the snippet of the integration guide ---
add_library(rocm_sgemm SHARED IMPORTED)
set_target_properties(rocm_sgemm PROPERTIES
    IMPORTED_LOCATION ${{MI355X_SGEMM}}/rocm_sgemm_amd/librocm_sgemm.so
    INTERFACE_INCLUDE_DIRECTORIES ${{MI355X_SGEMM}}/include)
# --- a caller, as the reference's test/CMakeLists.txt:8 links its own ---
add_executable(caller "{source}")
target_compile_options(caller PRIVATE -x hip --offload-arch=gfx950 -Wno-unused-command-line-argument)
{"target_include_directories(caller PRIVATE /root/reference)" if with_reference else ""}
target_link_libraries(caller PRIVATE rocm_sgemm)
""")
    build = tmp_path / "build"
    conf = subprocess.run([cmake, "-S", str(tmp_path), "-B", str(build), f"-DCMAKE_CXX_COMPILER={hipcc}",
                           "-DCMAKE_BUILD_TYPE=Release"], capture_output=True, text=True, timeout=300)
    assert conf.returncode == 0, conf.stdout + conf.stderr
    made = subprocess.run([cmake, "--build", str(build), "-j", "4"], capture_output=True, text=True, timeout=600)
    assert made.returncode == 0, made.stdout + made.stderr
    exe = build / "caller"
    assert exe.exists()
    # it is linked against this library and leaves none of the eight gemm<> symbols undefined
    needed = subprocess.run(["readelf", "-d", str(exe)], capture_output=True, text=True).stdout
    assert "librocm_sgemm.so" in needed
    undefined = subprocess.run(["nm", "-D", "--undefined-only", str(exe)], capture_output=True, text=True).stdout
    assert "rocm_sgemm4gemm" in undefined  # resolved at load time from the imported library


def test_side_library_of_the_exploration_check_holds_the_shape_the_shipped_one_lacks():
    """The build makes a side library with one tile shape from outside the family (a GPU test
    times it through the side library's own trial binary).  Host part: that library's family is
    the explored shape, its transpose and the default config's shape, and only it supports the
    shape."""
    from rocm_sgemm_amd import build as lib_build
    side = os.path.join(lib_build.EXPLORE_CHECK_DIR, "librocm_sgemm.so")
    if not os.path.exists(side):  # a tree whose build step has not run yet
        lib_build.build_explore_check()
    assert os.path.exists(side) and os.path.exists(os.path.join(lib_build.EXPLORE_CHECK_DIR, "config", "tuner"))
    shape = lib_build.EXPLORE_CHECK_SHAPE
    cfg = rs.Config.from_dict(dict(zip(space.SHAPE_KEYS, shape)))
    assert shape not in space.shipped_family() and space.shape_ok(shape)
    assert not rs.config_supported(cfg)
    # in a process of its own: the loader would hand back the shipped library for the same soname
    probe = ("import ctypes, sys; L = ctypes.CDLL(sys.argv[1]); c = (ctypes.c_int * 12)(*map(int, sys.argv[2:14])); "
             "print(L.rocm_sgemm_config_supported(c, 0, 0, 0), L.rocm_sgemm_family_size())")
    out = subprocess.run([sys.executable, "-c", probe, side] + [str(v) for v in cfg.as_dict().values()],
                         capture_output=True, text=True, check=True).stdout.split()
    default_shape = tuple(space.DEFAULT_CONFIG[k] for k in space.SHAPE_KEYS)
    assert out == ["1", str(len({shape, space.swapped(shape), default_shape}))]


def test_bench_held_out_shapes_are_not_table_entries():
    """bench.py's held-out rows measure the planner, so none of them may be a tuned entry."""
    sys.path.insert(0, REPO)
    import bench
    keys = {tuple(e[:6]) for e in generate_config.load_table(
        os.path.join(REPO, "rocm_sgemm_amd", "config", "gemm_config.json"))}
    assert len(bench.HELD_OUT) >= 4
    for (m, n, k, la, lb, lc) in bench.HELD_OUT:
        assert (m, n, k, la, lb, lc) not in keys
        assert (n, m, k, 1 - lb, 1 - la, 1 - lc) not in keys  # nor its mirror image, which is the same launch
    assert len({(la, lb, lc) for (_, _, _, la, lb, lc) in bench.HELD_OUT}) >= 4  # mixed layouts


# ---- a caller written against the reference's public header ---------------------------------------

CALLER = os.path.join(REPO, "tests", "cxx", "reference_style_caller")


def test_reference_style_caller_leaves_exactly_the_eight_symbols_undefined():
    """tests/cxx/reference_style_caller.cpp uses the API the way the reference's test and bench do;
    what it leaves for the library to define must be exactly the eight gemm instantiations."""
    assert os.path.exists(CALLER), "run `python -m rocm_sgemm_amd.build` first"
    out = subprocess.run(["nm", "-u", CALLER], check=True, capture_output=True, text=True).stdout
    undefined = {line.split()[-1] for line in out.splitlines() if "rocm_sgemm" in line}
    assert undefined == set(rs.CXX_SYMBOLS)


def test_leading_dimension_limit_is_reported_not_wrapped():
    # 32-bit tile offsets: tile extent x leading dimension must stay below 2^29 elements
    with pytest.raises(rs.SgemmError) as e:
        rs.gemm_with_config(rs.family()[0], FAKE, FAKE, FAKE, 256, 256, 2**22)
    assert e.value.status == rs.STATUS_INVALID_ARG and "leading dimension" in str(e.value)


# ---- bench_float (counterpart of the reference's benchmark/gemm) -----------------------------------

BENCH = os.path.join(REPO, "rocm_sgemm_amd", "benchmark", "bench_float")


def test_bench_float_command_line():
    """Same flags as the reference bench (benchmark/gemm/bench.cpp:175-228): --shapes,
    --batch_count, --help; Google Benchmark pass-through flags are accepted."""
    assert os.path.exists(BENCH), "run `python -m rocm_sgemm_amd.build` first"
    out = subprocess.run([BENCH, "--help"], capture_output=True, text=True)
    assert out.returncode == 0
    for flag in ("--shapes", "--batch_count", "--identity_b", "--warmup", "--iters", "--vendor"):
        assert flag in out.stdout
    bad = subprocess.run([BENCH, "--no-such-flag"], capture_output=True, text=True)
    assert bad.returncode == 2 and "unknown argument" in bad.stderr
    bad = subprocess.run([BENCH, "--layouts", "rx"], capture_output=True, text=True)
    assert bad.returncode == 2


def test_report_parses_bench_rows_and_builds_the_table(tmp_path):
    """report.py reads rows of the reference bench's console format (the sample row is the one
    quoted in reference docs/generate_report.py:33) plus bench_float's rocBLAS and hipBLASLt rows."""
    sys.path.insert(0, os.path.join(REPO, "rocm_sgemm_amd", "benchmark"))
    import report
    text = "\n".join([
        "{A:m_layout::col_major,B:m_layout::col_major,C:m_layout::col_major,m:1024,n:1024,k:1024}/manual_time"
        "      0.207 ms        0.278 ms         3713    11.5848      56.6933Gi/s     24.7665     0.16149",
        "  rocBLAS {A:m_layout::col_major,B:m_layout::col_major,C:m_layout::col_major,m:1024,n:1024,k:1024}/manual_time"
        "      0.300 ms        0.310 ms          100     7.0000      40.0000Gi/s     0.4     0.29   4.5",
        "  hipBLASLt {A:m_layout::col_major,B:m_layout::col_major,C:m_layout::row_major,m:1024,n:1024,k:1024}/manual_time"
        "      0.300 ms        0.310 ms          100    10.0000      40.0000Gi/s     0.4     0.29   4.5",
        "\x1b[32m{A:m_layout::col_major,B:m_layout::col_major,C:m_layout::row_major,m:1024,n:1024,k:1024}/manual_time"
        "      0.200 ms        0.270 ms         100    12.5000      58.0000Gi/s     0.3     0.19\x1b[0m",
        "noise line",
    ])
    rows = report.parse(text)
    assert [r[0] for r in rows] == ["rocm_sgemm", "rocblas", "hipblaslt", "rocm_sgemm"]
    assert rows[0][-1] == 11.5848 and rows[1][-1] == 7.0 and rows[3][3] == "row_major"
    md = report.table(rows)
    line = [l for l in md.splitlines() if l.startswith("| 1024x1024x1024")][0]
    assert "11.58" in line and "12.50" in line and "7.00" in line and "10.00" in line
    assert "125.0%" in line  # best of this library / best vendor figure
    log = tmp_path / "bench.log"
    log.write_text(text)
    out = tmp_path / "r.md"
    assert report.main(["--log", str(log), "--output", str(out)]) == 0
    assert "rocBLAS (best C)" in out.read_text() and "hipBLASLt (best C)" in out.read_text()


# ---- sampled correctness gate of the tuner trial binary and bench_float --------------------------

SAMPLED_CHECK_PROBE = r"""
#include <cstdio>
#include <limits>
#include <vector>
#include "sampled_check.hpp"
int main()
{
    using namespace rocm_sgemm::check;
    const size_t M = 37, N = 29, K = 53;
    std::vector<float> A(M * K), B(K * N), C(M * N);
    for(size_t i = 0; i < A.size(); ++i) A[i] = static_cast<float>((i * 7 + 3) % 11) - 5.0f;
    for(size_t i = 0; i < B.size(); ++i) B[i] = static_cast<float>((i * 5 + 1) % 9) - 4.0f;
    for(size_t i = 0; i < M; ++i)
        for(size_t j = 0; j < N; ++j)
        {
            float acc = 0.0f;
            for(size_t k = 0; k < K; ++k) acc += A[i * K + k] * B[k * N + j];
            C[i * N + j] = acc;
        }
    const double good = sampled_scaled_error(C.data(), A.data(), B.data(), M, N, K, false, false, false);
    // every entry sampled (samples >> M * N), one NaN anywhere must be seen
    std::vector<float> one_nan = C;
    one_nan[5 * N + 7]         = std::numeric_limits<float>::quiet_NaN();
    const double nan_err = sampled_scaled_error(one_nan.data(), A.data(), B.data(), M, N, K, false, false, false, 20000);
    std::vector<float> unwritten(M * N, std::numeric_limits<float>::quiet_NaN());
    const double all_nan = sampled_scaled_error(unwritten.data(), A.data(), B.data(), M, N, K, false, false, false);
    std::vector<float> off = C;
    off[0] += 1.0f; // corner (0, 0) is always sampled
    const double wrong = sampled_scaled_error(off.data(), A.data(), B.data(), M, N, K, false, false, false);
    std::printf("%d %d %d %d\n", within_tolerance(good), within_tolerance(nan_err), within_tolerance(all_nan),
                within_tolerance(wrong));
    return 0;
}
"""


def test_sampled_check_fails_on_nan_and_unwritten_outputs(tmp_path):
    """The gate behind `ok 0|1` of a tuner trial and behind bench_float --verify: an exact product
    passes; a NaN sample, an output left at its NaN pre-fill and a wrong value all fail
    (std::max(worst, NaN) would have returned `worst` and passed them)."""
    src = tmp_path / "probe.cpp"
    src.write_text(SAMPLED_CHECK_PROBE)
    exe = tmp_path / "probe"
    subprocess.run(["g++", "-std=c++17", "-O1", "-I", os.path.join(REPO, "rocm_sgemm_amd", "benchmark"),
                    str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert out == ["1", "0", "0", "0"], out


def test_no_kernel_spills_and_registers_leave_the_occupancy_that_lds_allows(tmp_path):
    """Reads the register, LDS and scratch sizes of every compiled GEMM kernel from the library's
    code-object metadata.  A kernel that spills, or whose register count halves the number of
    workgroups its LDS footprint lets a CU hold, still computes the right product, only slower;
    no parity test sees that."""
    bundler, readelf = "/opt/rocm/llvm/bin/clang-offload-bundler", "/opt/rocm/llvm/bin/llvm-readelf"
    if not (os.path.exists(bundler) and os.path.exists(readelf)):
        pytest.skip("needs the ROCm LLVM tools")
    fat = tmp_path / "fat.bin"
    subprocess.run(["objcopy", "-O", "binary", "--only-section=.hip_fatbin", rs.lib_path(), str(fat)], check=True)
    data = fat.read_bytes()
    starts = [m.start() for m in re.finditer(b"__CLANG_OFFLOAD_BUNDLE__", data)] + [len(data)]
    kernels = []
    for a, b in zip(starts, starts[1:]):
        (tmp_path / "bundle").write_bytes(data[a:b])
        subprocess.run([bundler, "--unbundle", "--type=o", f"--input={tmp_path / 'bundle'}",
                        "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--output={tmp_path / 'co'}"], check=True)
        notes = subprocess.run([readelf, "--notes", str(tmp_path / "co")], capture_output=True, text=True).stdout
        for block in notes.split("- .agpr_count:")[1:]:
            field = lambda key: re.search(rf"\.{key}:\s*(\S+)", block).group(1)  # noqa: E731
            kernels.append((field("name"), int(field("vgpr_count")), int(field("group_segment_fixed_size")),
                            int(field("private_segment_fixed_size")), int(field("max_flat_workgroup_size"))))
    gemm = [k for k in kernels if "sgemm_mfma_kernel" in k[0]]
    assert len(gemm) >= 4 * sum(3 if s[6] else 2 for s in space.family())
    for name, registers, lds, scratch, threads in gemm:
        assert scratch == 0, (name, scratch)
        waves = threads // 64
        groups_by_lds = min(160 * 1024 // lds, 8)
        waves_per_simd = 512 // ((registers + 7) // 8 * 8)  # VGPRs and AGPRs share 512 per lane
        groups_by_registers = waves_per_simd * 4 // waves if waves <= 4 else waves_per_simd // (waves // 4)
        # register-staged kernels keep their staging registers; two workgroups per CU is their design point
        assert groups_by_registers >= min(groups_by_lds, 2), (name, registers, lds)
