"""The allocation-free entry point, rocm_sgemm_f32_no_alloc, against rocm_sgemm_f32.

Both run the same config and the same kernels; only where the partial products of a split-K or
stream-K-tail config live differs (a fixed device array instead of an allocated workspace), so the
outputs must be identical bit for bit, and within the library's tolerance of an fp64 reference.
The calls follow each other on one GPU, the later ones with smaller inputs: the array keeps the
previous call's contents, and nothing of them may reach the next result.
Collected last on purpose (the name sorts after every other test file).
"""

import numpy as np
import pytest

import rocm_sgemm_amd as rs
from helpers import int_matrices, to_device

REL_TOL = 1e-6


def _needs_scratch(M, N, K):
    """Bytes of partial products the planned config of a row-major problem keeps (0 = none)."""
    cfg = rs.find_config(M, N, K)
    k_tiles = -(-K // cfg.k_tile)
    if cfg.split_k > 1:
        split = min(cfg.split_k, k_tiles)
        slice_tiles = -(-k_tiles // split)
        return M * N * -(-k_tiles // slice_tiles) * 4
    return 0


@pytest.mark.gpu
def test_no_alloc_entry_equals_the_allocating_entry_on_calls_in_a_row():
    import torch
    stream = torch.cuda.current_stream()
    # deep K (split-K, 32 MiB of partials), a stream-K tail, then smaller split-K problems (summed
    # by a second kernel, by the launch itself, and ragged)
    shapes = [(1024, 1024, 16384), (2560, 2560, 2560), (512, 512, 8192), (300, 260, 4096), (32, 4096, 4096)]
    assert _needs_scratch(*shapes[0]) > _needs_scratch(*shapes[2]) > 0
    assert _needs_scratch(*shapes[3]) > 0 and _needs_scratch(*shapes[4]) > 0
    for (M, N, K) in shapes:
        print("CASE no_alloc", M, N, K, rs.find_config(M, N, K), flush=True)
        g = torch.Generator(device="cuda:0")
        g.manual_seed(M + N + K)
        dA = torch.rand(M * K, generator=g, device="cuda:0") * 2 - 1
        dB = torch.rand(K * N, generator=g, device="cuda:0") * 2 - 1
        want = torch.full((M * N,), float("nan"), device="cuda:0")
        got = torch.full((M * N,), float("nan"), device="cuda:0")
        rs.gemm(want, dA, dB, M, N, K, stream=stream)
        rs.gemm_no_alloc(got, dA, dB, M, N, K, stream=stream)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (M, N, K)
        ref = (dA.view(M, K).double() @ dB.view(K, N).double()).view(-1)
        scale = K * float(dA.abs().max()) * float(dB.abs().max())
        assert float((got.double() - ref).abs().max()) / scale <= REL_TOL, (M, N, K)
        # integer-valued inputs: every summation order is exact, so the fp64 product bit for bit
        iA = torch.randint(-4, 5, (M * K,), generator=g, device="cuda:0").float()
        iB = torch.randint(-4, 5, (K * N,), generator=g, device="cuda:0").float()
        exact = (iA.view(M, K).double() @ iB.view(K, N).double()).float().view(-1)
        got_i = torch.full((M * N,), float("nan"), device="cuda:0")
        rs.gemm_no_alloc(got_i, iA, iB, M, N, K, stream=stream)
        torch.cuda.synchronize()
        assert torch.equal(got_i, exact), (M, N, K)


@pytest.mark.gpu
def test_no_alloc_entry_in_column_major_layouts_and_on_a_side_stream():
    import torch
    rng = np.random.default_rng(10)
    side = torch.cuda.Stream()
    for (la, lb, lc) in [(1, 1, 1), (0, 1, 0), (1, 0, 1)]:
        M, N, K = 32, 4096, 4096
        print("CASE no_alloc layouts", M, N, K, la, lb, lc, flush=True)
        A, B, C = int_matrices(rng, M, N, K)
        a = A.reshape(-1) if la == 0 else A.T.reshape(-1)
        b = B.reshape(-1) if lb == 0 else B.T.reshape(-1)
        dA, dB = to_device(a), to_device(b)
        got = torch.full((M * N,), float("nan"), device="cuda:0")
        torch.cuda.synchronize()
        rs.gemm_no_alloc(got, dA, dB, M, N, K, lc, la, lb, stream=side)
        side.synchronize()
        want = C.reshape(-1) if lc == 0 else C.T.reshape(-1)
        assert np.array_equal(got.cpu().numpy(), want), (la, lb, lc)


def test_no_alloc_entry_refuses_what_its_scratch_cannot_hold():
    """Host only: the size check comes before any HIP call, so fake (never dereferenced) device
    addresses do.  Looks for a problem whose planned config keeps more partial products than the
    scratch array holds."""
    fake = 0x7F0000000000
    for (M, N, K) in [(5120, 3000, 65536), (3000, 5120, 65536), (4096, 4096, 65536), (8192, 2048, 131072)]:
        if _needs_scratch(M, N, K) > rs.NO_ALLOC_SCRATCH_BYTES:
            with pytest.raises(rs.SgemmError) as e:
                rs.gemm_no_alloc(fake, fake, fake, M, N, K)
            assert e.value.status == rs.STATUS_WORKSPACE_TOO_LARGE
            assert str(rs.NO_ALLOC_SCRATCH_BYTES) in str(e.value)
            return
    pytest.skip("the planner splits K for none of the probed large problems")
