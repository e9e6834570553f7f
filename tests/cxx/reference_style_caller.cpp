// A caller written the way the reference's own programs are (reference test/gemm/test.cpp:36-96,
// benchmark/gemm/bench.cpp:31-114): it owns a GLOBAL-namespace `m_layout` enum, includes only
// <rocm_sgemm/gemm.hpp>, static_casts its enum to rocm_sgemm::m_layout, passes a named hipStream_t
// by reference and polls hipPeekAtLastError afterwards.  Compiling and linking it against
// librocm_sgemm.so shows the header and the eight exported template instantiations are
// source- and link-compatible; running it checks every layout combination on the GPU against a
// host triple loop.  Exit code 0 = all eight combinations passed.

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include <rocm_sgemm/gemm.hpp>

enum class m_layout
{
    row_major,
    col_major
};

#define HIP_OK(call)                                                                          \
    do                                                                                        \
    {                                                                                         \
        hipError_t e_ = (call);                                                               \
        if(e_ != hipSuccess)                                                                  \
        {                                                                                     \
            std::fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            std::exit(2);                                                                     \
        }                                                                                     \
    } while(0)

static size_t at(m_layout l, size_t rows, size_t cols, size_t i, size_t j)
{
    return l == m_layout::row_major ? i * cols + j : j * rows + i;
}

template<m_layout LA, m_layout LB, m_layout LC>
static bool run_case(size_t M, size_t N, size_t K, hipStream_t& stream)
{
    std::vector<float> hA(M * K), hB(K * N), hC(M * N), ref(M * N);
    std::mt19937                          gen(1);
    std::uniform_real_distribution<float> dis(-1.0f, 1.0f);
    for(size_t i = 0; i < M; ++i)
        for(size_t k = 0; k < K; ++k) hA[at(LA, M, K, i, k)] = dis(gen);
    for(size_t k = 0; k < K; ++k)
        for(size_t j = 0; j < N; ++j) hB[at(LB, K, N, k, j)] = dis(gen);

    float *dA, *dB, *dC;
    HIP_OK(hipMalloc(&dA, hA.size() * sizeof(float)));
    HIP_OK(hipMalloc(&dB, hB.size() * sizeof(float)));
    HIP_OK(hipMalloc(&dC, hC.size() * sizeof(float)));
    HIP_OK(hipMemcpy(dA, hA.data(), hA.size() * sizeof(float), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dB, hB.data(), hB.size() * sizeof(float), hipMemcpyHostToDevice));

    rocm_sgemm::gemm<static_cast<rocm_sgemm::m_layout>(LC),
                     static_cast<rocm_sgemm::m_layout>(LA),
                     static_cast<rocm_sgemm::m_layout>(LB)>(dC, dA, dB, M, N, K, stream);
    HIP_OK(hipPeekAtLastError());
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(hC.data(), dC, hC.size() * sizeof(float), hipMemcpyDeviceToHost));

    double worst = 0.0;
    for(size_t i = 0; i < M; ++i)
        for(size_t j = 0; j < N; ++j)
        {
            float acc = 0.0f;
            for(size_t k = 0; k < K; ++k) acc += hA[at(LA, M, K, i, k)] * hB[at(LB, K, N, k, j)];
            worst = std::fmax(worst, std::fabs(static_cast<double>(acc) - hC[at(LC, M, N, i, j)]));
        }
    HIP_OK(hipFree(dA));
    HIP_OK(hipFree(dB));
    HIP_OK(hipFree(dC));
    const bool ok = worst <= 1e-4; // the reference test's tolerance (test/gemm/test.cpp:82)
    std::printf("A=%d B=%d C=%d  %zux%zux%zu  max abs err %.3g  %s\n", static_cast<int>(LA),
                static_cast<int>(LB), static_cast<int>(LC), M, N, K, worst, ok ? "PASS" : "FAIL");
    return ok;
}

int main()
{
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    constexpr m_layout r = m_layout::row_major, c = m_layout::col_major;
    bool               ok = true;
    ok &= run_case<r, r, r>(320, 512, 512, stream);
    ok &= run_case<r, r, c>(320, 512, 512, stream);
    ok &= run_case<r, c, r>(320, 512, 512, stream);
    ok &= run_case<r, c, c>(320, 512, 512, stream);
    ok &= run_case<c, r, r>(320, 512, 512, stream);
    ok &= run_case<c, r, c>(320, 512, 512, stream);
    ok &= run_case<c, c, r>(320, 512, 512, stream);
    ok &= run_case<c, c, c>(320, 512, 512, stream);
    // zero-sized problem, no try block: like the reference the entry point does not throw for its
    // arguments; nothing is enqueued and the stream stays usable
    {
        float* p = reinterpret_cast<float*>(0x1000);
        rocm_sgemm::gemm<rocm_sgemm::m_layout::row_major, rocm_sgemm::m_layout::row_major,
                         rocm_sgemm::m_layout::row_major>(p, p, p, 0, 4, 4, stream);
        HIP_OK(hipStreamSynchronize(stream));
        std::printf("zero dimension -> returns without launching: PASS\n");
    }
    HIP_OK(hipStreamDestroy(stream));
    return ok ? 0 : 1;
}
