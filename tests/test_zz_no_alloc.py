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
    return rs.workspace_bytes(M, N, K)


def _with_scratch(candidates, count):
    """The first `count` of the candidate problems whose planned config keeps partial products (which
    ones do changes when the table is re-tuned)."""
    chosen = [s for s in candidates if _needs_scratch(*s) > 0][:count]
    assert len(chosen) == count, "too few of the probed problems need a workspace under the current table"
    return chosen


@pytest.mark.gpu
def test_no_alloc_entry_equals_the_allocating_entry_on_calls_in_a_row():
    import torch
    stream = torch.cuda.current_stream()
    # deep K (split-K, 32 MiB of partials), a stream-K tail, then smaller split-K problems (summed
    # by a second kernel, by the launch itself, and ragged)
    shapes = _with_scratch([(1024, 1024, 16384), (2560, 2560, 2560), (512, 512, 8192), (300, 260, 4096),
                            (32, 4096, 4096), (3584, 3584, 3584), (256, 256, 16384), (1536, 1536, 1536),
                            (8, 4096, 4096), (192, 192, 8192)], 4)
    shapes.sort(key=lambda s: -_needs_scratch(*s))  # the later calls use less of the array
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


@pytest.mark.gpu
def test_no_alloc_entry_allocates_nothing_and_replays_from_a_hip_graph():
    """What the entry point is for.  (1) A warmed call leaves the amount of free device memory
    exactly as it was.  (2) Recorded into a HIP graph - where nothing may be allocated - a split-K
    call replays correctly: the counters of the partial tiles it sums inside the launch live in
    the scratch array and must be back at zero after every replay.  Each replay gets fresh
    integer-valued inputs, with eager work (another no-alloc product on the same array) and
    synchronisation in between, and must equal the exact product bit for bit."""
    import torch
    g = torch.Generator(device="cuda:0")
    g.manual_seed(5)
    shapes = _with_scratch([(512, 512, 8192), (32, 4096, 4096), (256, 256, 16384), (300, 260, 4096),
                            (192, 192, 8192), (8, 4096, 4096), (1024, 1024, 16384)], 2)
    for (M, N, K) in shapes:
        print("CASE no_alloc graph", M, N, K, rs.find_config(M, N, K), flush=True)
        dA = torch.randint(-4, 5, (M * K,), generator=g, device="cuda:0").float()
        dB = torch.randint(-4, 5, (K * N,), generator=g, device="cuda:0").float()
        dC = torch.full((M * N,), float("nan"), device="cuda:0")
        other = torch.full((300 * 260,), float("nan"), device="cuda:0")
        oA = torch.randint(-4, 5, (300 * 4096,), generator=g, device="cuda:0").float()
        oB = torch.randint(-4, 5, (4096 * 260,), generator=g, device="cuda:0").float()
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        rs.gemm_no_alloc(dC, dA, dB, M, N, K, stream=stream)  # warm: code object, scratch address
        stream.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        rs.gemm_no_alloc(dC, dA, dB, M, N, K, stream=stream)
        stream.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            rs.gemm_no_alloc(dC, dA, dB, M, N, K, stream=torch.cuda.current_stream())
        for replay in range(3):
            dA.copy_(torch.randint(-4, 5, (M * K,), generator=g, device="cuda:0").float())
            dB.copy_(torch.randint(-4, 5, (K * N,), generator=g, device="cuda:0").float())
            dC.fill_(float("nan"))
            exact = (dA.view(M, K).double() @ dB.view(K, N).double()).float().view(-1)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(dC, exact), (M, N, K, replay)
            # eager work between the replays, on the same scratch array
            rs.gemm_no_alloc(other, oA, oB, 300, 260, 4096, stream=torch.cuda.current_stream())
            torch.cuda.synchronize()
            assert torch.equal(other, (oA.view(300, 4096).double() @ oB.view(4096, 260).double()).float().view(-1))


def test_no_alloc_entry_refuses_what_its_scratch_cannot_hold():
    """Host only: the size check comes before any HIP call, so fake (never dereferenced) device
    addresses do.  Looks for a problem whose planned config keeps more partial products than the
    scratch array holds."""
    fake = 0x7F0000000000
    for (M, N, K) in [(5120, 3000, 65536), (3000, 5120, 65536), (4096, 4096, 65536), (8192, 2048, 131072),
                      (3000, 3000, 131072), (2000, 5000, 262144)]:
        if _needs_scratch(M, N, K) > rs.NO_ALLOC_SCRATCH_BYTES:
            with pytest.raises(rs.SgemmError) as e:
                rs.gemm_no_alloc(fake, fake, fake, M, N, K)
            assert e.value.status == rs.STATUS_WORKSPACE_TOO_LARGE
            assert str(rs.NO_ALLOC_SCRATCH_BYTES) in str(e.value)
            return
    pytest.skip("the planner splits K for none of the probed large problems")
