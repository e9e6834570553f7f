"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle.

Bars (written here, as the tolerance is part of the test):
  * identity-B and integer-valued inputs: bit-exact;
  * the reference's own rule: |C - sgemm_cpu(A, B)| <= 1e-4 on its 13 shapes x 8 layouts with
    mt19937(1) / uniform(-1, 1) inputs (reference test/gemm/test.cpp:82-176);
  * everything else: max|C - C_ref| / (K * max|A| * max|B|) <= 1e-6 against fp64 accumulation.
"""

import ctypes

import numpy as np
import pytest

import oracle
import rocm_sgemm_amd as rs
from helpers import (ALL_LAYOUTS, check_exact_int, check_strided_batched_exact, int_matrices, lay_id,
                     run_gemm, to_device)

pytestmark = pytest.mark.gpu

LAYOUT_IDS = [lay_id(*l) for l in ALL_LAYOUTS]
REL_TOL = 1e-6
REF_ABS_TOL = 1e-4

# reference test/gemm/test.cpp:113-176
REFERENCE_SHAPES = [(128, 128, 128), (128, 256, 128), (128, 128, 256), (256, 128, 128),
                    (256, 256, 256), (320, 320, 320), (320, 512, 512), (512, 320, 320),
                    (512, 512, 320), (512, 320, 512), (512, 512, 512), (1024, 256, 256),
                    (256, 1024, 256)]


def _announce(*what):
    print("CASE", *what, flush=True)


# ---- the reference's own test suite -------------------------------------------------------------

@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_reference_suite(la, lb, lc):
    for (M, N, K) in REFERENCE_SHAPES:
        _announce("reference_suite", M, N, K, la, lb, lc)
        a = oracle.fill_uniform(M, K, la, 1)  # same seed for A and B, as in the reference
        b = oracle.fill_uniform(K, N, lb, 1)
        got = run_gemm(a, b, M, N, K, la, lb, lc)
        want = oracle.sgemm_f32(a, b, M, N, K, lc, la, lb, threads=8)
        assert np.max(np.abs(got - want)) <= REF_ABS_TOL, (M, N, K)
        ref64 = oracle.sgemm_f64acc(a, b, M, N, K, lc, la, lb)
        assert oracle.scaled_error(got, ref64, a, b, K) <= REL_TOL, (M, N, K)


# ---- bit-exact closed forms ----------------------------------------------------------------------

@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_identity_b_is_bit_exact(la, lb, lc):
    for (M, K) in [(256, 256), (300, 77), (1024, 512)]:
        _announce("identity_b", M, K, la, lb, lc)
        a = oracle.fill_uniform(M, K, la, 7)
        eye = oracle.to_storage(np.eye(K, dtype=np.float32), lb)
        got = run_gemm(a, eye, M, K, K, la, lb, lc)
        want = oracle.to_storage(oracle.as_matrix(a, M, K, la), lc)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_identity_a_is_bit_exact(la, lb, lc):
    K, N = 200, 333
    _announce("identity_a", K, N, la, lb, lc)
    b = oracle.fill_uniform(K, N, lb, 3)
    eye = oracle.to_storage(np.eye(K, dtype=np.float32), la)
    got = run_gemm(eye, b, K, N, K, la, lb, lc)
    want = oracle.to_storage(oracle.as_matrix(b, K, N, lb), lc)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_all_ones_gives_k():
    for K in (1, 15, 16, 17, 4093):
        _announce("all_ones", K)
        M, N = 130, 70
        got = run_gemm(np.ones(M * K, np.float32), np.ones(K * N, np.float32), M, N, K, 0, 0, 0)
        assert np.array_equal(got, np.full(M * N, float(K), np.float32))


# Integer-valued inputs make every summation order exact, so this pins the index paths, the MFMA
# lane maps, the M/N/K edge masks and split-K of EVERY compiled kernel without any tolerance.
# (512, 256, 96) and (256, 512, 352) are whole tiles for every shape, so they run the full-tile
# (direct-to-LDS where the shape has one) kernels; 352 = 11 K-tiles of 32 wraps every LDS ring.
# (300, 260, 128), (36, 68, 192) and (300, 260, 100) have leading dimensions that are multiples of
# 4 in every layout: they run the masked direct-to-LDS kernels, the last with a ragged last K-tile.
# (300, 257, 100) and (257, 300, 100) have one odd dimension: depending on the layout one operand's
# lines are 16-byte aligned and the other's are not (16-byte loads for one, 4-byte for the other).
EDGE_SHAPES = [(1, 1, 1), (33, 65, 17), (255, 257, 129), (300, 260, 100), (64, 64, 64),
               (512, 256, 96), (256, 512, 352), (257, 511, 263), (300, 260, 128), (36, 68, 192),
               (300, 257, 100), (257, 300, 100)]


@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_every_kernel_exact_on_integers(la, lb, lc):
    rng = np.random.default_rng(100 + la * 4 + lb * 2 + lc)
    # (split_k, wave_slots, partial_sums): plain, uniform split-K, and a tail split forced by
    # pretending the GPU runs only 3 workgroups at once - the last two with the partial tiles
    # summed by a second kernel (1) and by the GEMM launch itself where the kernel can (2)
    for fam in rs.family():
        for split, slots, sums in ((1, 1, 0), (3, 1, 1), (3, 1, 2), (1, 3, 1), (1, 3, 2)):
            cfg = dict(fam.as_dict(), split_k=split, group_m=3, wave_slots=slots, partial_sums=sums)
            for (M, N, K) in EDGE_SHAPES:
                _announce("int_exact", cfg, M, N, K, la, lb, lc)
                check_exact_int(M, N, K, la, lb, lc, rng, cfg)


@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_default_dispatch_exact_on_integers(la, lb, lc):
    rng = np.random.default_rng(5)
    for (M, N, K) in [(1000, 3000, 777), (128, 4096, 512), (4096, 128, 512), (1024, 1024, 2048),
                      (777, 1, 1000), (1, 555, 1000), (2048, 2048, 64)]:
        _announce("dispatch_int_exact", M, N, K, la, lb, lc)
        check_exact_int(M, N, K, la, lb, lc, rng)


def test_full_and_edge_kernels_agree_bitwise():
    """A misaligned base pointer forces the edge-masked kernel on a tile-aligned problem; both
    kernels sum in the same order, so the results must be identical."""
    import torch
    M = N = K = 512
    _announce("full_vs_edge", M)
    a, b = oracle.fill_uniform_pair(M, N, K, 0, 0, seed=4)
    dA = to_device(np.concatenate([np.zeros(1, np.float32), a]))
    dB = to_device(b)
    dC1 = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
    dC2 = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
    rs.gemm(dC1, dA.data_ptr() + 4, dB, M, N, K, stream=torch.cuda.current_stream())
    rs.gemm(dC2, to_device(a), dB, M, N, K, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert torch.equal(dC1, dC2)


# ---- benchmark configurations ----------------------------------------------------------------------

def test_config1_1024_cube_row_major_seed0():
    M = N = K = 1024
    _announce("config1", M)
    a, b = oracle.fill_uniform_pair(M, N, K, 0, 0, seed=0)
    got = run_gemm(a, b, M, N, K, 0, 0, 0)
    want32 = oracle.sgemm_f32(a, b, M, N, K, 0, 0, 0, threads=8)
    assert np.max(np.abs(got - want32)) <= 2e-4  # K = 1024: twice the reference's K <= 512 bound
    ref64 = oracle.sgemm_f64acc(a, b, M, N, K, 0, 0, 0)
    assert oracle.scaled_error(got, ref64, a, b, K) <= REL_TOL


def _device_uniform(rows, cols, seed):
    import torch
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    return torch.rand(rows * cols, generator=g, device="cuda:0", dtype=torch.float32) * 2.0 - 1.0


def _sampled_check(dA, dB, dC, M, N, K, la, lb, lc, samples=4096, seed=0):
    """fp64 dot products of sampled entries (all four borders included) against the HIP result.
    Only the sampled rows of A and columns of B leave the GPU."""
    import torch
    rng = np.random.default_rng(seed)
    rows = rng.integers(0, M, samples)
    cols = rng.integers(0, N, samples)
    nb = samples // 8
    rows[:nb], rows[nb:2 * nb] = 0, M - 1
    cols[2 * nb:3 * nb], cols[3 * nb:4 * nb] = 0, N - 1
    urows, rinv = np.unique(rows, return_inverse=True)
    ucols, cinv = np.unique(cols, return_inverse=True)
    A = dA.view(M, K) if la == 0 else dA.view(K, M).t()
    B = dB.view(K, N) if lb == 0 else dB.view(N, K).t()
    C = dC.view(M, N) if lc == 0 else dC.view(N, M).t()
    Ar = A[torch.from_numpy(urows).cuda()].double()  # u x K
    Bc = B[:, torch.from_numpy(ucols).cuda()].double()  # K x v
    ref = (Ar[torch.from_numpy(rinv).cuda()] * Bc.t()[torch.from_numpy(cinv).cuda()]).sum(dim=1)
    got = C[torch.from_numpy(rows).cuda(), torch.from_numpy(cols).cuda()].double()
    scale = K * float(dA.abs().max()) * float(dB.abs().max())
    err = float((got - ref).abs().max()) / scale
    assert np.isfinite(err) and err <= REL_TOL, err
    return err


def _run_device(dA, dB, M, N, K, la, lb, lc):
    import torch
    dC = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
    rs.gemm(dC, dA, dB, M, N, K, lc, la, lb, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    return dC


def test_sampled_checker_agrees_with_oracle():
    """The torch-side sampled reference used at full sizes is itself checked against the oracle's
    sampled fp64 dots on a size the oracle handles."""
    import torch
    M, N, K = 257, 300, 129
    a, b = oracle.fill_uniform_pair(M, N, K, 1, 0, seed=9)
    rows = np.array([0, 256, 13, 200]); cols = np.array([0, 299, 7, 150])
    want = oracle.dot_f64_samples(a, b, M, N, K, 1, 0, rows, cols)
    A = to_device(a).view(K, M).t().double()
    B = to_device(b).view(K, N).double()
    got = (A[torch.from_numpy(rows).cuda()] * B[:, torch.from_numpy(cols).cuda()].t()).sum(1)
    assert np.max(np.abs(got.cpu().numpy() - want)) < 1e-12


def test_config2_4096_identity_b_bit_exact():
    import torch
    M = N = K = 4096
    _announce("config2", M)
    dA = _device_uniform(M, K, 1)
    dB = torch.eye(K, dtype=torch.float32, device="cuda:0").reshape(-1)
    dC = _run_device(dA, dB, M, N, K, 0, 0, 0)
    assert torch.equal(dC.view(torch.int32), dA.view(torch.int32))


@pytest.mark.parametrize("size", [4096, 8192])
@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_config3_square_all_layouts(size, la, lb, lc):
    M = N = K = size
    _announce("config3", size, la, lb, lc)
    dA, dB = _device_uniform(M, K, 2), _device_uniform(K, N, 3)
    dC = _run_device(dA, dB, M, N, K, la, lb, lc)
    _sampled_check(dA, dB, dC, M, N, K, la, lb, lc)


@pytest.mark.parametrize("shape", [(8192, 8192, 1024), (1024, 1024, 16384), (128, 4096, 4096),
                                   (4096, 128, 4096)])
def test_config4_rectangular(shape):
    M, N, K = shape
    _announce("config4", M, N, K)
    dA, dB = _device_uniform(M, K, 4), _device_uniform(K, N, 5)
    dC = _run_device(dA, dB, M, N, K, 0, 0, 0)
    _sampled_check(dA, dB, dC, M, N, K, 0, 0, 0)


@pytest.mark.parametrize("shape", [(4095, 4097, 4093), (1000, 3000, 777)])
@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_config5_unaligned_all_layouts(shape, la, lb, lc):
    M, N, K = shape
    _announce("config5", M, N, K, la, lb, lc)
    dA, dB = _device_uniform(M, K, 6), _device_uniform(K, N, 7)
    dC = _run_device(dA, dB, M, N, K, la, lb, lc)
    _sampled_check(dA, dB, dC, M, N, K, la, lb, lc)


def test_config5_16384_cube():
    M = N = K = 16384
    _announce("config5", M)
    dA, dB = _device_uniform(M, K, 8), _device_uniform(K, N, 9)
    dC = _run_device(dA, dB, M, N, K, 0, 0, 0)
    _sampled_check(dA, dB, dC, M, N, K, 0, 0, 0, samples=2048)


# ---- size-independent properties at full size -------------------------------------------------------

def test_linearity_in_power_of_two_scale_is_exact():
    """(2A)B = 2(AB) and A(B/4) = (AB)/4 bit for bit (scaling by a power of two commutes with
    every rounding as long as nothing under- or overflows)."""
    import torch
    M = N = K = 2048
    _announce("linearity", M)
    dA, dB = _device_uniform(M, K, 10), _device_uniform(K, N, 11)
    base = _run_device(dA, dB, M, N, K, 0, 1, 0)
    assert torch.equal(_run_device(dA * 2.0, dB, M, N, K, 0, 1, 0), base * 2.0)
    assert torch.equal(_run_device(dA, dB * 0.25, M, N, K, 0, 1, 0), base * 0.25)


def test_subnormal_inputs_and_results_are_not_flushed():
    """The reference multiplies with ordinary fp32 FMAs, which on its targets keep subnormal values
    (gradual underflow), and its CPU check does the same.  The matrix-core path must not flush
    them: products and sums in the subnormal range (around 4e-39, below the smallest normal
    1.18e-38) and subnormal inputs (around 1e-40) come out as the fp64 product says, to the
    precision subnormal numbers have (their spacing is 1.4e-45, i.e. about 4e-7 of these sums per
    rounding), in a full-tile, a ragged and a column-major case and through a K split."""
    rng = np.random.default_rng(3)
    for (M, N, K, la, lb, lc, split) in [(64, 64, 64, 0, 0, 0, 1), (300, 260, 100, 0, 1, 0, 1),
                                         (512, 256, 96, 1, 0, 1, 1), (128, 128, 512, 0, 0, 0, 4)]:
        _announce("subnormal", M, N, K, la, lb, lc, split)
        cfg = dict(rs.find_config(M, N, K, la, lb, lc).as_dict(), split_k=split)
        for scale_a, scale_b in ((1e-25, 1e-15), (1e-40, 1e10)):
            A = (rng.uniform(0.5, 1.0, (M, K)) * scale_a).astype(np.float32)
            B = (rng.uniform(0.5, 1.0, (K, N)) * scale_b).astype(np.float32)
            assert scale_a > 1e-30 or float(A.max()) < 1.2e-38  # the second case feeds subnormal inputs
            want = A.astype(np.float64) @ B.astype(np.float64)
            got = run_gemm(oracle.to_storage(A, la), oracle.to_storage(B, lb), M, N, K, la, lb, lc, config=cfg)
            got = got.reshape(M, N) if lc == 0 else got.reshape(N, M).T
            assert not (got == 0).any(), (M, N, K, scale_a)
            assert float(np.max(np.abs(got - want) / want)) < 4e-7 * K, (M, N, K, scale_a)


def test_nan_and_infinity_propagate_as_ieee_says_and_nowhere_else():
    """A NaN in row i of A makes row i of C NaN, an infinity (with positive B) makes its row
    infinite, and every other row equals, bit for bit, what it is without them - in a ragged problem
    (masked kernels), a full-tile one and through a K split, for both storage orders of C."""
    rng = np.random.default_rng(8)
    for (M, N, K, la, lb, lc, split) in [(300, 260, 100, 0, 0, 0, 1), (256, 256, 128, 1, 1, 1, 1),
                                         (255, 257, 1029, 0, 1, 0, 3)]:
        _announce("nan_inf", M, N, K, la, lb, lc, split)
        cfg = dict(rs.find_config(M, N, K, la, lb, lc).as_dict(), split_k=split)
        A = rng.uniform(-1.0, 1.0, (M, K)).astype(np.float32)
        B = rng.uniform(0.5, 1.0, (K, N)).astype(np.float32)
        def product(a):
            flat = run_gemm(oracle.to_storage(a, la), oracle.to_storage(B, lb), M, N, K, la, lb, lc, config=cfg)
            return flat.reshape(M, N) if lc == 0 else flat.reshape(N, M).T
        clean = product(A)
        special = A.copy()
        special[5, 7], special[9, K - 1], special[M - 1, 0] = np.nan, np.inf, -np.inf
        got = product(special)
        assert np.isnan(got[5]).all() and (got[9] == np.inf).all() and (got[M - 1] == -np.inf).all()
        others = [i for i in range(M) if i not in (5, 9, M - 1)]
        assert np.array_equal(got[others].view(np.uint32), clean[others].view(np.uint32))


def test_run_to_run_determinism_including_split_k():
    import torch
    M, N, K = 512, 384, 4096
    _announce("determinism", M, N, K)
    dA, dB = _device_uniform(M, K, 12), _device_uniform(K, N, 13)
    cfg = dict(rs.family()[0].as_dict(), split_k=4)
    outs = []
    for _ in range(3):
        dC = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
        rs.gemm_with_config(cfg, dC, dA, dB, M, N, K, stream=torch.cuda.current_stream())
        torch.cuda.synchronize()
        outs.append(dC)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])


# ---- the C++ entry points, as a program compiled against the reference header would call them ----

@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_cxx_template_symbols_match_c_abi(la, lb, lc):
    import torch
    M, N, K = 320, 512, 512
    _announce("cxx_symbol", la, lb, lc)
    a, b = oracle.fill_uniform(M, K, la, 1), oracle.fill_uniform(K, N, lb, 1)
    want = run_gemm(a, b, M, N, K, la, lb, lc)
    fn = getattr(rs.lib(), rs.cxx_symbol(lc, la, lb))
    fn.restype = None
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_size_t] * 3 + [ctypes.POINTER(ctypes.c_void_p)]
    dA, dB = to_device(a), to_device(b)
    dC = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    fn(dC.data_ptr(), dA.data_ptr(), dB.data_ptr(), M, N, K, ctypes.byref(stream))
    torch.cuda.synchronize()
    assert np.array_equal(dC.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_refused_cxx_call_leaves_a_hip_error_and_c_untouched():
    """A zero dimension or a null pointer: the C++ entry point throws nothing and enqueues nothing,
    but the check the reference's callers make after every call (hipPeekAtLastError,
    reference test/gemm/test.cpp:69) must see a failure, as it does after the reference's launch of
    an empty grid."""
    import torch
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipPeekAtLastError.restype = ctypes.c_int
    hip.hipGetLastError.restype = ctypes.c_int
    fn = getattr(rs.lib(), rs.cxx_symbol(0, 0, 0))
    fn.restype = None
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_size_t] * 3 + [ctypes.POINTER(ctypes.c_void_p)]
    dA = torch.ones(64 * 64, dtype=torch.float32, device="cuda:0")
    dC = torch.full((64 * 64,), 7.0, dtype=torch.float32, device="cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    hip.hipGetLastError()  # start clean
    for args in ((dC.data_ptr(), dA.data_ptr(), dA.data_ptr(), 0, 64, 64),
                 (dC.data_ptr(), None, dA.data_ptr(), 64, 64, 64)):
        _announce("refused_cxx_call", args[3:])
        fn(*args, ctypes.byref(stream))
        assert hip.hipPeekAtLastError() != 0
        assert hip.hipGetLastError() != 0 and hip.hipPeekAtLastError() == 0  # reading it clears it
        assert "must be" in rs.lib().rocm_sgemm_last_error().decode()
    torch.cuda.synchronize()
    assert bool((dC == 7.0).all())
    # and a good call after it works and leaves no error
    fn(dC.data_ptr(), dA.data_ptr(), dA.data_ptr(), 64, 64, 64, ctypes.byref(stream))
    torch.cuda.synchronize()
    assert hip.hipPeekAtLastError() == 0 and bool((dC == 64.0).all())


def test_runs_on_a_side_stream_without_blocking_semantics():
    import torch
    M, N, K = 256, 256, 256
    _announce("side_stream")
    a, b = oracle.fill_uniform_pair(M, N, K, 0, 0, seed=2)
    want = run_gemm(a, b, M, N, K, 0, 0, 0)
    side = torch.cuda.Stream()
    dA, dB = to_device(a), to_device(b)
    dC = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
    torch.cuda.synchronize()
    rs.gemm(dC, dA, dB, M, N, K, stream=side)
    side.synchronize()
    assert np.array_equal(dC.cpu().numpy(), want)


def test_reference_style_cxx_caller_runs():
    """The program in tests/cxx (compiled against include/rocm_sgemm/gemm.hpp only, calling the
    eight template instantiations like the reference's own test does) passes on the GPU."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cxx", "reference_style_caller")
    _announce("cxx_caller")
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.count("PASS") == 9


def test_caller_with_the_reference_headers_runs():
    """tests/cxx/reference_header_caller.cpp includes the reference's real common/matrix.hpp
    (global ::m_layout, matrix<T, Layout>) and common/hip_utils.hpp next to this repository's
    <rocm_sgemm/gemm.hpp> and calls the eight instantiations the way the reference test does
    (reference test/gemm/test.cpp:36-96).  It can only be compiled where the reference tree is;
    the binary travels with this tree."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tests", "cxx",
                       "reference_header_caller")
    if not os.path.exists(exe):
        pytest.skip("reference_header_caller was not built (the reference tree was absent at build time)")
    _announce("reference_header_caller")
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count("PASS") == 17 and "FAIL" not in out.stdout  # 16 cases + the summary


def test_bench_float_rows_parse_like_the_reference_bench():
    """bench_float prints rows in the reference bench's console format; the two regular
    expressions are the ones the reference's report script applies to them
    (docs/generate_report.py:36 and :52).  Also checks the identity-B and fp64 verification."""
    import os
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rocm_sgemm_amd",
                       "benchmark", "bench_float")
    _announce("bench_float", exe)
    out = subprocess.run([exe, "--shapes", "256:384,256,256", "--warmup", "2", "--iters", "5",
                          "--identity_b", "--verify", "--batch_count", "2"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    name_re = re.compile(r"\{A:m_layout::(\w+),B:m_layout::(\w+),C:m_layout::(\w+),m:(\d+),n:(\d+),k:(\d+)\}")
    tflops_re = re.compile(r"\s+(\d+(?:\.\d+)?)\s+[\d.]+Gi/s")
    rows = []
    for line in out.stdout.splitlines():
        m = name_re.match(line)
        if m:
            t = tflops_re.search(line)
            assert t is not None, line
            assert float(t.group(1)) > 0.0
            assert "identity:bit-exact" in line and "(FAIL)" not in line, line
            rows.append(m.groups())
    # two shapes x eight layout combinations, C column-major first as in the reference
    assert len(rows) == 16
    assert rows[0][:3] == ("col_major", "col_major", "col_major") and rows[0][3:] == ("256", "256", "256")
    assert rows[7][:3] == ("row_major", "row_major", "row_major")
    assert rows[8][3:] == ("384", "256", "256")


def test_bench_float_mfma_ceiling_is_a_ceiling():
    """--mfma_ceiling times a kernel of MFMAs only: its rate bounds every SGEMM kernel from above
    and cannot exceed the published peak (256 CUs x 256 flop per cycle x 2.4 GHz); the per-XCD
    lines account for all 1024 waves, each of which finds the matrix pipe busy for the whole loop."""
    import os
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rocm_sgemm_amd",
                       "benchmark", "bench_float")
    _announce("bench_float --mfma_ceiling", exe)
    out = subprocess.run([exe, "--mfma_ceiling"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    whole = re.search(r"= ([\d.]+) TFLOP/s = ([\d.]+) % of ([\d.]+)", out.stdout)
    assert whole is not None, out.stdout
    tflops, peak = float(whole.group(1)), float(whole.group(3))
    assert 0.8 * peak < tflops <= 1.005 * peak, out.stdout
    xcds = re.findall(r"XCD (\d):\s+(\d+) waves, shader clock (\d+) MHz, loop [\d.]+ us = ([\d.]+) %", out.stdout)
    assert sum(int(x[1]) for x in xcds) == 1024 and len(xcds) == 8, out.stdout
    for _, _, mhz, busy in xcds:
        assert 1500 <= int(mhz) <= 2450 and 99.0 <= float(busy) <= 100.5, out.stdout


def test_kernel_phases_accounts_for_a_launch():
    """kernel_phases instantiates the GEMM kernels with time stamps switched on (the library is
    built without them) and prints where a launch's time goes.  The phases of a workgroup must add
    up to its life, every workgroup must appear under one of the eight XCDs, and the main loop can
    be no shorter than its MFMAs."""
    import os
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rocm_sgemm_amd",
                       "benchmark", "kernel_phases")
    _announce("kernel_phases 2048 1024", exe)
    out = subprocess.run([exe, "2048", "1024"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    blocks = out.stdout.strip().split("\n\n")
    assert len(blocks) == 2, out.stdout
    for block, groups in zip(blocks, (256, 256)):
        rows = re.findall(r"^\s+(\d)\s+(\d+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s+(\d+) MHz",
                          block, re.M)
        assert len(rows) == 8 and sum(int(r[1]) for r in rows) == groups, block
        for _, _, start, prologue, loop, epilogue, end, end_max, mhz in rows:
            total = float(start) + float(prologue) + float(loop) + float(epilogue)
            assert abs(total - float(end)) <= 0.05 and float(end_max) >= float(end) - 0.01, block
            assert 1500 <= int(mhz) <= 2450, block
        busy = re.search(r"pipe busy ([\d.]+) % of the loop", block)
        assert busy is not None and 50.0 <= float(busy.group(1)) <= 100.5, block
        each = re.search(r"back to back: ([\d.]+) us each = ([\d.]+) TFLOP/s", block)
        assert each is not None and 40.0 < float(each.group(2)) < 157.3, block


def test_issue_cost_of_instructions_next_to_mfmas():
    """issue_cost measures what one instruction of each kind adds to a stream of back-to-back
    MFMAs.  The design of the main loop rests on two of its findings: a vector-ALU instruction
    costs several cycles of matrix-pipe time (about 13 measured), scalar instructions, LDS reads,
    direct-to-LDS loads and barriers next to nothing."""
    import os
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rocm_sgemm_amd",
                       "benchmark", "issue_cost")
    _announce("issue_cost", exe)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    alone = float(re.search(r"MFMAs alone: ([\d.]+) cycles each", out.stdout).group(1))
    assert 63.9 <= alone <= 64.6, out.stdout  # a v_mfma_f32_32x32x2_f32 holds the pipe for 64 cycles
    cost = {(m.group(1).strip(), int(m.group(2))): float(m.group(3))
            for m in re.finditer(r"^cost (.+?)\s+every\s+(\d+) MFMAs:\s+(-?[\d.]+) cycles", out.stdout, re.M)}
    assert len(cost) == 9, out.stdout
    assert 6.0 <= cost[("vector-ALU add", 8)] <= 25.0 and 6.0 <= cost[("vector-ALU add", 1)] <= 25.0, out.stdout
    assert cost[("two vector-ALU adds", 8)] >= cost[("vector-ALU add", 8)], out.stdout
    for free in (("four scalar-ALU adds", 1), ("ds_read_b128", 8), ("ds_read_b128", 2),
                 ("direct-to-LDS load, 16 bytes per lane", 4), ("s_barrier", 16)):
        assert cost[free] <= 2.0, (free, out.stdout)
    assert cost[("direct-to-LDS load, 4 bytes per lane", 1)] <= 3.0, out.stdout


def test_bench_float_l2_to_lds_probe():
    """--l2_to_lds streams direct-to-LDS loads from windows that fit the L2s and from windows that
    do not: a CU cannot take more than 64 bytes per cycle, and what comes from beyond the L2 is
    slower than what comes from it."""
    import os
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rocm_sgemm_amd",
                       "benchmark", "bench_float")
    _announce("bench_float --l2_to_lds", exe)
    out = subprocess.run([exe, "--l2_to_lds"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    rows = re.findall(r"window\s+(\d+) KB per workgroup,\s+(\d+) workgroups .*?:\s+([\d.]+) bytes per cycle and CU", out.stdout)
    assert len(rows) == 8, out.stdout
    rate = {(int(w), int(g)): float(r) for w, g, r in rows}
    assert all(1.0 < r <= 64.5 for r in rate.values()), out.stdout
    groups = max(g for _, g in rate)
    assert rate[(1024, groups)] < rate[(64, groups)], out.stdout


def test_bench_float_vendor_rows_compute_the_same_product():
    """--vendor adds a rocBLAS and a hipBLASLt row under each of this library's rows; with
    --verify each vendor row carries the same sampled fp64 error figure, which pins the operand
    mapping used for them (row-major C served as the column-major C^T = B^T A^T) on a
    non-square problem for all eight layout combinations."""
    import os
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "rocm_sgemm_amd",
                       "benchmark", "bench_float")
    _announce("bench_float --vendor", exe)
    out = subprocess.run([exe, "--shapes", "384,256,512", "--warmup", "1", "--iters", "3", "--uniform",
                          "--verify", "--vendor"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    err_re = re.compile(r"err:([0-9.e+-]+)")
    seen = {"rocBLAS": 0, "hipBLASLt": 0}
    for line in out.stdout.splitlines():
        who = line.split()[0] if line.strip() else ""
        if who in seen and "{A:m_layout::" in line:
            m = err_re.search(line)
            assert m is not None, line
            assert float(m.group(1)) <= 1e-6, line
            seen[who] += 1
    assert seen == {"rocBLAS": 8, "hipBLASLt": 8}, out.stdout


@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_edge_masks_do_not_leak_neighbouring_data(la, lb, lc):
    """Ragged shapes make the 128-bit loads of an edge tile overrun into the neighbouring row /
    column / depth line.  Zero-valued padding would hide a missing mask (0 * finite = 0), so the
    neighbours are poisoned with Inf: any leak turns an exact integer result into NaN.
    Poison: A rows 0-2 entirely and A[odd rows][0:3]; B columns 0-2 entirely and B[0:3][odd
    columns].  Outputs C[i][j] with i, j even and >= 4 touch no poisoned element and must be exact."""
    rng = np.random.default_rng(17)
    family = rs.family()
    # every register-staged shape, and every direct-to-LDS shape, whose masked kernels
    # move 16 bytes per lane on problems with ragged dimensions that are multiples of 4 and 4 bytes
    # per lane on all others (the last K-tile of a depth-contiguous operand runs on into the next
    # row, which is poisoned)
    staged = [(f, [(70, 90, 19), (258, 262, 35), (131, 67, 70), (300, 300, 200)])
              for f in family if f.stages == 0]
    direct = [(f, [(300, 300, 200), (132, 68, 100), (260, 264, 36), (70, 90, 19), (258, 262, 35),
                   (131, 67, 70)]) for f in family if f.stages > 0]
    assert direct, "the family holds no direct-to-LDS shape"
    for fam, shapes in staged + direct:
        cfg = dict(fam.as_dict(), split_k=1, group_m=2, wave_slots=3)
        for (M, N, K) in shapes:
            _announce("edge_poison", cfg, M, N, K, la, lb, lc)
            A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
            B = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
            want = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
            A[0:3, :] = np.inf
            A[1::2, 0:3] = np.inf
            B[:, 0:3] = np.inf
            B[0:3, 1::2] = np.inf
            got = oracle.as_matrix(
                run_gemm(oracle.to_storage(A, la), oracle.to_storage(B, lb), M, N, K, la, lb, lc, cfg),
                M, N, lc)
            clean_got, clean_want = got[4::2, 4::2], want[4::2, 4::2]
            assert np.array_equal(clean_got, clean_want), (
                cfg, M, N, K, np.argwhere(clean_got != clean_want)[:4])


@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_nothing_outside_an_operand_reaches_the_result(la, lb, lc):
    """A and B sit in the middle of arenas filled with Inf, so whatever lies before or after an
    operand in memory is poison.  A ragged last K-tile makes the loads of a row-contiguous
    operand run past its last depth line, i.e. past its end; those must come back as zeros from
    the range check of the load itself (for every piece a lane moves, also the ones addressed
    through the scalar offset), or Inf * 0 = NaN lands in every output.  Offsets that are
    multiples of 4 floats keep the operands 16-byte aligned (16-byte loads), odd ones do not
    (4-byte loads); shapes without an LDS ring take their register-staged kernel."""
    import torch
    rng = np.random.default_rng(23)
    family = rs.family()
    picks = family
    for fam in picks:
        cfg = dict(fam.as_dict(), split_k=1, group_m=2, wave_slots=1)
        for (M, N, K, off) in [(132, 68, 100, 1024), (260, 264, 36, 512), (131, 67, 70, 1021),
                               (132, 67, 100, 1024), (131, 68, 36, 512)]:
            _announce("inf_arena", cfg, M, N, K, off, la, lb, lc)
            A, B, C = int_matrices(rng, M, N, K)
            a, b = oracle.to_storage(A, la), oracle.to_storage(B, lb)
            arena_a = torch.full((a.size + 2 * off,), float("inf"), dtype=torch.float32, device="cuda:0")
            arena_b = torch.full((b.size + 2 * off,), float("inf"), dtype=torch.float32, device="cuda:0")
            arena_a[off:off + a.size] = torch.from_numpy(a).to("cuda:0")
            arena_b[off:off + b.size] = torch.from_numpy(b).to("cuda:0")
            dC = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
            rs.gemm_with_config(cfg, dC, arena_a.data_ptr() + 4 * off, arena_b.data_ptr() + 4 * off,
                                M, N, K, lc, la, lb, stream=torch.cuda.current_stream())
            torch.cuda.synchronize()
            got, want = dC.cpu().numpy(), oracle.to_storage(C, lc)
            bad = np.flatnonzero(got.view(np.uint32) != want.view(np.uint32))
            assert bad.size == 0, (cfg, M, N, K, off, bad[:5], got[bad[:5]], want[bad[:5]])


def test_sixteen_byte_loads_that_straddle_the_end_of_a_padded_operand():
    """16-byte direct-to-LDS loads are chosen when pointers and leading dimensions are 16-byte
    aligned and K is a multiple of 4 - also when a row-contiguous operand's own width is not a
    multiple of 4 under a padded leading dimension (column-major A with M = 130, lda = 132).  The
    last 16-byte piece of the final depth line then straddles the operand's end: its first two
    floats are data, the other two lie beyond the allocation.  The range check must drop the
    out-of-range dwords only, not the whole piece.  Padding holds NaN, the buffers end exactly at
    the operands' extents, integer-valued data: bit-exact or wrong."""
    rng = np.random.default_rng(61)
    for fam in [f for f in rs.family() if f.stages > 0]:
        cfg = dict(fam.as_dict(), split_k=1, group_m=2, wave_slots=1)
        for (M, N, K, la, lb, lc, pads) in [(130, 64, 72, 1, 0, 0, (2, 0, 0)),   # X row-contiguous, ragged
                                            (64, 134, 72, 0, 0, 0, (0, 2, 0)),   # Y column-contiguous, ragged
                                            (130, 134, 40, 1, 0, 0, (2, 2, 0)),  # both
                                            (130, 134, 40, 1, 0, 1, (2, 2, 2))]:  # swapped for a column-major C
            _announce("straddling_piece", cfg, M, N, K, la, lb, lc, pads)
            check_strided_batched_exact(rng, M, N, K, la, lb, lc, 1, 1, 0, pads, config=cfg)


def test_partial_tiles_summed_in_the_launch_equal_the_second_kernel_bit_for_bit():
    """The parts of a tile are added in the same order whoever adds them - the wave that draws the
    last ticket inside the GEMM launch, or the reduction kernel - so uniform inputs must give the
    same bits, call after call (the counters of a launch are left at zero for the next one, and the
    workspace is reused with other contents in between)."""
    import torch
    fams = {(f.macro_m, f.macro_n, f.k_tile, f.waves_k): f for f in rs.family() if f.stages >= 2 and f.mfma == 32}
    cases = [((64, 64, 64, 4), (768, 384, 2304), dict(split_k=3, wave_slots=1)),
             ((64, 32, 64, 4), (300, 777, 4100), dict(split_k=5, wave_slots=1)),
             ((128, 128, 32, 1), (1000, 1100, 2048), dict(split_k=1, wave_slots=7)),
             ((64, 64, 32, 1), (1030, 2050, 777), dict(split_k=2, wave_slots=1)),
             ((128, 64, 32, 2), (382, 1059, 3350), dict(split_k=1, wave_slots=0)),
             ((64, 64, 128, 4), (1024, 1024, 4096), dict(split_k=2, wave_slots=1))]
    for key, (M, N, K), launch in cases:
        dA, dB = _device_uniform(M, K, M + 1), _device_uniform(K, N, N + 2)
        outs = []
        for sums in (1, 2, 2, 1, 2):
            cfg = dict(fams[key].as_dict(), group_m=4, partial_sums=sums, **launch)
            _announce("partial_sums", cfg, M, N, K)
            dC = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
            rs.gemm_with_config(cfg, dC, dA, dB, M, N, K, stream=torch.cuda.current_stream())
            torch.cuda.synchronize()
            outs.append(dC)
        for other in outs[1:]:
            assert torch.equal(outs[0].view(torch.int32), other.view(torch.int32)), (key, M, N, K)
        _sampled_check(dA, dB, outs[1], M, N, K, 0, 0, 0)


def test_stream_k_tail_matches_plain_run_and_is_deterministic():
    """The stream-K tail (K range of a short last wave of tiles dealt out to all slots) changes
    only the summation order of the affected tiles: results stay within the fp64 tolerance, repeat
    bit for bit, and untouched tiles are bit-identical to a run without it."""
    import torch
    M, N, K = 1280, 1024, 2048
    _announce("stream_k_tail", M, N, K)
    dA, dB = _device_uniform(M, K, 21), _device_uniform(K, N, 22)
    base = dict(rs.family()[0].as_dict(), group_m=4)  # 256 x 256 tiles: 5 x 4 = 20 tiles
    outs = {}
    for slots in (1, 16, 16):  # 16 slots: one full wave + a tail of 4 tiles dealt to 16 workgroups
        dC = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
        rs.gemm_with_config(dict(base, wave_slots=slots), dC, dA, dB, M, N, K,
                            stream=torch.cuda.current_stream())
        torch.cuda.synchronize()
        outs.setdefault(slots, []).append(dC)
    plain, split_a, split_b = outs[1][0], outs[16][0], outs[16][1]
    assert torch.equal(split_a, split_b)
    _sampled_check(dA, dB, split_a, M, N, K, 0, 0, 0)
    same = (plain.view(M, N) == split_a.view(M, N))
    tiles_same = same.view(5, 256, 4, 256).all(dim=3).all(dim=1)
    assert int(tiles_same.sum()) == 16  # the 16 tiles of the full wave are untouched
    assert float((plain - split_a).abs().max()) < 1e-3


@pytest.mark.parametrize("slots", [3, 5, 7, 13])
def test_stream_k_tail_runs_that_straddle_two_tiles_are_exact(slots):
    """A problem that is a single short wave (4 tiles of 256 x 256) dealt out to a number of slots
    that does not divide the K range: most workgroups own the end of one tile and the beginning
    of the next.  Integer-valued inputs, so the sum of the segments must be exact."""
    rng = np.random.default_rng(40 + slots)
    base = dict(rs.family()[0].as_dict(), group_m=2, wave_slots=slots)
    for (M, N, K) in ((512, 512, 1024), (500, 300, 1111)):
        for (la, lb, lc) in ((0, 0, 0), (1, 1, 1), (0, 1, 0)):
            _announce("stream_k_straddle", slots, M, N, K, la, lb, lc)
            check_exact_int(M, N, K, la, lb, lc, rng, base)


def test_concurrent_calls_from_threads_on_separate_streams():
    """The library keeps no state between calls: four host threads, each with its own stream and
    problem (one of them split-K, one with a stream-K tail, so workspaces are in play), must all be exact."""
    import threading
    import torch
    rng = np.random.default_rng(3)
    jobs = []
    base = rs.family()[0].as_dict()
    small = [f for f in rs.family() if f.macro_m == 64 and f.macro_n == 64][0].as_dict()
    for idx, (shape, cfg) in enumerate([((512, 384, 640), dict(base)),
                                         ((300, 260, 1000), dict(base, split_k=4)),
                                         ((260, 300, 520), dict(small, wave_slots=7, partial_sums=2)),
                                         ((129, 1000, 77), dict(small))]):
        M, N, K = shape
        A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
        B = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
        want = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float32)
        jobs.append(dict(shape=shape, cfg=cfg, dA=to_device(A.reshape(-1)), dB=to_device(B.reshape(-1)),
                         dC=torch.empty(M * N, dtype=torch.float32, device="cuda:0"), want=want,
                         stream=torch.cuda.Stream(), error=None))
    torch.cuda.synchronize()

    def work(job):
        try:
            M, N, K = job["shape"]
            for _ in range(20):
                rs.gemm_with_config(job["cfg"], job["dC"], job["dA"], job["dB"], M, N, K,
                                    stream=job["stream"])
            job["stream"].synchronize()
        except Exception as e:  # surfaced in the main thread below
            job["error"] = e

    _announce("threads")
    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    torch.cuda.synchronize()
    for job in jobs:
        assert job["error"] is None, job["error"]
        M, N, K = job["shape"]
        assert np.array_equal(job["dC"].cpu().numpy().reshape(M, N), job["want"]), job["shape"]


def test_call_can_be_captured_in_a_hip_graph_and_replayed():
    """A call that needs no workspace enqueues exactly one kernel and allocates nothing, so it can
    be recorded into a HIP graph.  Each replay (with fresh inputs, and eager work plus
    synchronisation in between) must equal the eager result bit for bit."""
    import torch
    M = N = K = 1024
    _announce("graph_capture", M)
    cfg = rs.find_config(M, N, K).as_dict()
    cfg.update(split_k=1, wave_slots=1)  # one launch, no workspace
    dA, dB = _device_uniform(M, K, 31), _device_uniform(K, N, 32)
    dC = torch.zeros(M * N, dtype=torch.float32, device="cuda:0")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        rs.gemm_with_config(cfg, dC, dA, dB, M, N, K, stream=torch.cuda.current_stream())  # warm-up
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rs.gemm_with_config(cfg, dC, dA, dB, M, N, K, stream=torch.cuda.current_stream())
    for seed in (41, 42, 43):
        dA.copy_(_device_uniform(M, K, seed))
        dB.copy_(_device_uniform(K, N, seed + 100))
        dC.zero_()
        graph.replay()
        torch.cuda.synchronize()
        replayed = dC.clone()
        eager = torch.empty_like(dC)
        rs.gemm_with_config(cfg, eager, dA, dB, M, N, K, stream=torch.cuda.current_stream())
        torch.cuda.synchronize()
        assert torch.equal(replayed, eager), seed


@pytest.mark.parametrize("what", ["split_k", "stream_k_tail"])
def test_captured_call_with_partials_owns_its_workspace(what):
    """A call that needs a workspace (split-K, stream-K tail) recorded into a HIP graph must not
    bake the library's per-stream buffer into the graph: that buffer is freed when a later eager
    call on the stream outgrows it and by release_workspaces().  The order below is the usual one
    (eager warm-up creates the buffer, capture follows, a bigger product comes later); every
    replay, with fresh integer-valued inputs, must equal the int64 product bit for bit."""
    import torch
    rng = np.random.default_rng(77)
    M, N, K = 300, 260, 1000
    base = rs.family()[0].as_dict()
    cfg = dict(base, split_k=4, wave_slots=1) if what == "split_k" else dict(base, split_k=1, wave_slots=3)
    _announce("graph_capture_workspace", what, cfg, M, N, K)
    A, B, C = int_matrices(rng, M, N, K)
    dA, dB = to_device(A.reshape(-1)), to_device(B.reshape(-1))
    dC = torch.zeros(M * N, dtype=torch.float32, device="cuda:0")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        rs.gemm_with_config(cfg, dC, dA, dB, M, N, K, stream=stream)  # the stream now has a buffer
    stream.synchronize()
    assert np.array_equal(dC.cpu().numpy().reshape(M, N), C)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        rs.gemm_with_config(cfg, dC, dA, dB, M, N, K, stream=torch.cuda.current_stream())
    # a larger eager product on the same stream outgrows the stream's buffer; then everything the
    # library holds is given back
    M2, N2, K2 = 700, 650, 1200
    A2, B2, C2 = int_matrices(rng, M2, N2, K2)
    dC2 = torch.zeros(M2 * N2, dtype=torch.float32, device="cuda:0")
    rs.gemm_with_config(dict(base, split_k=6, wave_slots=1), dC2, to_device(A2.reshape(-1)),
                        to_device(B2.reshape(-1)), M2, N2, K2, stream=stream)
    stream.synchronize()
    assert np.array_equal(dC2.cpu().numpy().reshape(M2, N2), C2)
    rs.release_workspaces()
    filler = torch.full((64 << 20,), float("nan"), device="cuda:0")  # reuse whatever was freed
    for _ in range(3):
        A, B, C = int_matrices(rng, M, N, K)
        dA.copy_(to_device(A.reshape(-1)))
        dB.copy_(to_device(B.reshape(-1)))
        dC.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dC.cpu().numpy().reshape(M, N), C)
    del filler


# ---- general form: leading dimensions, strided batches, alpha / beta ---------------------------------

@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_strided_batched_general_form_exact_on_integers(la, lb, lc):
    """C_b <- alpha A_b B_b + beta C_b with padded leading dimensions and batch strides, against
    the int64 computation.  NaN in the padding of A / B must not reach C, the padding of C must not
    be written, and beta = 0 must not read C (it holds NaN)."""
    rng = np.random.default_rng(700 + la * 4 + lb * 2 + lc)
    cases = [  # M, N, K, batch, alpha, beta, pads (A, B, C)
        (70, 50, 33, 3, 1, 0, (0, 0, 0)),       # packed, ragged: batched edge kernel
        (70, 50, 33, 3, 2, -1, (3, 5, 1)),      # odd leading dimensions
        (128, 256, 64, 2, 1, 0, (4, 8, 12)),    # whole tiles, 16-byte aligned lines: full-tile kernel
        (128, 256, 64, 2, -3, 2, (4, 8, 12)),   # same through the blending pass
        (256, 128, 352, 1, 1, 1, (0, 0, 0)),    # beta only
        (1, 1, 1, 4, 5, 0, (2, 2, 2)),
        (300, 200, 100, 2, 1, 0, (8, 4, 0)),
    ]
    for (M, N, K, batch, alpha, beta, pads) in cases:
        _announce("strided_batched", M, N, K, batch, alpha, beta, pads, la, lb, lc)
        check_strided_batched_exact(rng, M, N, K, la, lb, lc, batch, alpha, beta, pads)


def test_strided_batched_with_explicit_configs_split_k_and_broadcast():
    rng = np.random.default_rng(77)
    fams = {tuple(f.as_dict()[k] for k in ("macro_m", "macro_n", "k_tile", "stages")): f.as_dict()
            for f in rs.family()}
    for key, split in (((128, 128, 32, 2), 1), ((128, 128, 32, 2), 3), ((256, 128, 16, 0), 2),
                       ((256, 256, 32, 2), 1)):
        cfg = dict(fams[key], split_k=split, group_m=2, wave_slots=0)
        for (la, lb, lc) in ((0, 0, 0), (1, 0, 1), (0, 1, 0)):
            for alpha, beta in ((1, 0), (2, 1)):
                _announce("strided_batched_cfg", key, split, la, lb, lc, alpha, beta)
                check_strided_batched_exact(rng, 256, 256, 352, la, lb, lc, 3, alpha, beta, (4, 4, 4),
                                            config=cfg, broadcast_b=True)
                check_strided_batched_exact(rng, 200, 136, 100, la, lb, lc, 2, alpha, beta, (1, 0, 3),
                                            config=cfg)


def test_general_form_with_defaults_equals_the_plain_entry():
    import torch
    M, N, K = 512, 384, 256
    a, b = oracle.fill_uniform_pair(M, N, K, 0, 1, seed=9)
    dA, dB = to_device(a), to_device(b)
    dC1 = torch.empty(M * N, dtype=torch.float32, device="cuda:0")
    dC2 = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
    _announce("general_defaults", M, N, K)
    rs.gemm(dC1, dA, dB, M, N, K, 0, 0, 1, stream=torch.cuda.current_stream())
    rs.gemm_strided_batched(dC2, dA, dB, M, N, K, layout_b=1, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert torch.equal(dC1, dC2)


# ---- the reference's own GPU kernel as a second oracle --------------------------------------------------

@pytest.mark.parametrize("size", [1024, 4096])
@pytest.mark.parametrize("la,lb,lc", ALL_LAYOUTS, ids=LAYOUT_IDS)
def test_matches_the_reference_gpu_kernel(size, la, lb, lc):
    """oracle/_ref holds the reference's kernel template compiled from the reference's sources with
    the tuned parameters of its own table (oracle/build_ref.py).  On integer-valued inputs both
    libraries must produce the exact product, hence identical bits; on the reference test's
    uniform inputs they may differ by fp32 summation order only (<= 1e-6 scaled)."""
    import torch
    ref = oracle.ref_kernel()
    if ref is None:
        pytest.skip("oracle/_ref/libref_kernel.so has not been built (needs the reference tree)")
    M = N = K = size
    _announce("reference_gpu_kernel", size, la, lb, lc)
    stream = torch.cuda.current_stream()
    rng = np.random.default_rng(size + la * 4 + lb * 2 + lc)
    for kind in ("integers", "uniform"):
        if kind == "integers":
            A = rng.integers(-4, 5, size=(M, K)).astype(np.float32)
            B = rng.integers(-4, 5, size=(K, N)).astype(np.float32)
            a, b = oracle.to_storage(A, la), oracle.to_storage(B, lb)
        else:
            a, b = oracle.fill_uniform(M, K, la, 1), oracle.fill_uniform(K, N, lb, 1)
        dA, dB = to_device(a), to_device(b)
        ours = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
        theirs = torch.full((M * N,), float("nan"), dtype=torch.float32, device="cuda:0")
        rs.gemm(ours, dA, dB, M, N, K, lc, la, lb, stream=stream)
        status = ref.ref_kernel_sgemm(lc, la, lb, theirs.data_ptr(), dA.data_ptr(), dB.data_ptr(), M, N, K,
                                      stream.cuda_stream)
        assert status == 0, "the reference's table has an entry for every layout at this size"
        torch.cuda.synchronize()
        if kind == "integers":
            assert torch.equal(ours.view(torch.int32), theirs.view(torch.int32))
        else:
            amax, bmax = float(np.abs(a).max()), float(np.abs(b).max())
            err = float((ours - theirs).abs().max()) / (K * amax * bmax)
            assert err <= REL_TOL, err


# ---- every tuned entry, at its own size ------------------------------------------------------------------

def test_every_table_entry_is_exact_on_integers_at_its_own_size():
    """Each of the table's (M, N, K, layouts) problems, and its mirror image, through the default
    dispatcher, i.e. under the config tuned for it (tile shape, K split, stream-K tail, band height), on integer-valued
    inputs: bit-exact against the fp64 product.  The tuner's own gate is a sampled check at
    tuning time; this one is complete and runs on the table as shipped."""
    import torch
    g = torch.Generator(device="cuda:0")
    g.manual_seed(11)
    stream = torch.cuda.current_stream()
    table = rs.table()
    assert len(table) > 300
    # and the mirror image of every entry (N, M, K, layouts of A and B exchanged, all three flipped),
    # which the lookup serves with the entry's config, tile shape exchanged
    keys = {key for key, _ in table}
    problems = sorted(keys | {(N, M, K, 1 - lb, 1 - la, 1 - lc) for (M, N, K, la, lb, lc) in keys})
    assert len(problems) > len(keys)
    for (M, N, K, la, lb, lc) in problems:
        cfg = rs.find_config(M, N, K, la, lb, lc)
        _announce("table_entry", M, N, K, la, lb, lc)
        A = torch.randint(-4, 5, (M, K), generator=g, device="cuda:0").float()
        B = torch.randint(-4, 5, (K, N), generator=g, device="cuda:0").float()
        dA = (A if la == 0 else A.t().contiguous()).reshape(-1)
        dB = (B if lb == 0 else B.t().contiguous()).reshape(-1)
        dC = torch.full((M * N,), float("nan"), device="cuda:0")
        rs.gemm(dC, dA, dB, M, N, K, lc, la, lb, stream=stream)
        want = (A.double() @ B.double()).float()
        want = (want if lc == 0 else want.t().contiguous()).reshape(-1)
        torch.cuda.synchronize()
        assert torch.equal(dC, want), (M, N, K, la, lb, lc, cfg)
        del A, B, dA, dB, dC, want


def test_random_mid_and_large_problems_exact_on_integers():
    """600 seeded random problems of the sizes the planner is for (64 ... 6000 per dimension, a third
    multiples of 64, a third multiples of 4, a third arbitrary; all layouts), none of them a table
    entry, so each runs whatever the planner chooses - an inherited or fitted K split, a stream-K
    tail, a tile shape from the cost model: bit-exact against the fp64 product."""
    import random
    import torch
    rnd = random.Random(2024)
    g = torch.Generator(device="cuda:0")
    g.manual_seed(12)
    stream = torch.cuda.current_stream()
    keys = {key for key, _ in rs.table()}
    kinds = set()
    done = 0
    while done < 600:
        step = rnd.choice([64, 4, 1])
        M, N, K = (max(step, int(2 ** rnd.uniform(6, 12.55)) // step * step) for _ in range(3))
        la, lb, lc = (rnd.randint(0, 1) for _ in range(3))
        if 2.0 * M * N * K > 2.0 * 4096 ** 3 or (M, N, K, la, lb, lc) in keys:
            continue
        done += 1
        cfg = rs.find_config(M, N, K, la, lb, lc)
        kinds.add(("split" if cfg.split_k > 1 else "plain", cfg.waves_k > 1, cfg.stages))
        _announce("random_large", M, N, K, la, lb, lc, cfg)
        A = torch.randint(-4, 5, (M, K), generator=g, device="cuda:0").float()
        B = torch.randint(-4, 5, (K, N), generator=g, device="cuda:0").float()
        dA = (A if la == 0 else A.t().contiguous()).reshape(-1)
        dB = (B if lb == 0 else B.t().contiguous()).reshape(-1)
        dC = torch.full((M * N,), float("nan"), device="cuda:0")
        rs.gemm(dC, dA, dB, M, N, K, lc, la, lb, stream=stream)
        want = (A.double() @ B.double()).float()
        want = (want if lc == 0 else want.t().contiguous()).reshape(-1)
        torch.cuda.synchronize()
        assert torch.equal(dC, want), (M, N, K, la, lb, lc, cfg)
    assert len(kinds) >= 4  # the draw exercises K splits, waves along K and several ring depths


# ---- randomised sweep through the default dispatcher ---------------------------------------------------

def test_random_problems_exact_on_integers():
    """120 seeded random problems (sizes 1..700, all layouts, packed or padded leading dimensions,
    1..3 batches, alpha/beta from a small integer set) through the table lookup and whatever
    kernel, split or tail it selects: every one must equal the int64 computation bit for bit."""
    rng = np.random.default_rng(20241125)
    for case in range(120):
        M, N, K = (int(v) for v in rng.integers(1, 701, size=3))
        if case % 6 == 0:  # some whole-tile problems, which take the direct-to-LDS kernels
            M, N, K = 64 * int(rng.integers(1, 9)), 64 * int(rng.integers(1, 9)), 32 * int(rng.integers(1, 24))
        la, lb, lc = (int(v) for v in rng.integers(0, 2, size=3))
        batch = int(rng.integers(1, 4))
        alpha, beta = [(1, 0), (1, 0), (2, 0), (1, 1), (-1, 3)][int(rng.integers(0, 5))]
        pads = tuple(int(v) for v in rng.choice([0, 0, 1, 4, 7], size=3))
        _announce("random", case, M, N, K, la, lb, lc, batch, alpha, beta, pads)
        check_strided_batched_exact(rng, M, N, K, la, lb, lc, batch, alpha, beta, pads)
