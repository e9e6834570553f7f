// A caller that includes the reference's own host headers next to this library's public header.
//
// Built only where the reference tree is present (its headers are named by path on the compiler's
// command line, nothing of it is copied): <common/matrix.hpp> supplies the GLOBAL ::m_layout and
// matrix<T, Layout>, <common/hip_utils.hpp> supplies HIP_CHECK and gpu_timer, and
// <rocm_sgemm/gemm.hpp> is this repository's header.  What is shown: the two sets of headers
// coexist in one translation unit with no edit to either side (::m_layout and
// rocm_sgemm::m_layout are distinct enums with the same enumerator values, bridged by the same
// static_cast the reference's test and bench use, test/gemm/test.cpp:60-62,
// benchmark/gemm/bench.cpp:77-79), and all eight instantiations run through matrix<T, Layout>
// buffers and agree with a CPU product to the reference test's 1e-4.
// The reference's test driver itself needs GoogleTest, which this environment does not have.

#include <rocm_sgemm/gemm.hpp>

#include <common/hip_utils.hpp>
#include <common/matrix.hpp>

#include <cmath>
#include <cstdio>
#include <random>

static_assert(static_cast<int>(::m_layout::row_major) == static_cast<int>(rocm_sgemm::m_layout::row_major)
                  && static_cast<int>(::m_layout::col_major) == static_cast<int>(rocm_sgemm::m_layout::col_major),
              "the caller's layout enum converts to the library's by value");

namespace
{

// same input stream as the reference test (mt19937(1), uniform(-1, 1), row by row)
template<class T, ::m_layout L>
void fill(matrix<T, L>& x)
{
    std::mt19937                          gen(1);
    std::uniform_real_distribution<float> dis(-1.0f, 1.0f);
    for(size_t i = 0; i < x.m(); ++i)
        for(size_t j = 0; j < x.n(); ++j)
            x(i, j) = static_cast<T>(dis(gen));
}

template<::m_layout LA, ::m_layout LB, ::m_layout LC>
bool run_case(size_t M, size_t N, size_t K, hipStream_t& stream)
{
    matrix<float, LA> h_A(M, K);
    matrix<float, LB> h_B(K, N);
    matrix<float, LC> h_C(M, N);
    fill(h_A);
    fill(h_B);
    float *d_A, *d_B, *d_C;
    HIP_CHECK(hipMalloc(&d_A, h_A.size() * sizeof(float)));
    HIP_CHECK(hipMalloc(&d_B, h_B.size() * sizeof(float)));
    HIP_CHECK(hipMalloc(&d_C, h_C.size() * sizeof(float)));
    HIP_CHECK(hipMemcpy(d_A, h_A.data(), h_A.size() * sizeof(float), hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(d_B, h_B.data(), h_B.size() * sizeof(float), hipMemcpyHostToDevice));
    HIP_CHECK(hipMemset(d_C, 0xFF, h_C.size() * sizeof(float)));

    gpu_timer timer;
    timer.start(stream);
    rocm_sgemm::gemm<static_cast<rocm_sgemm::m_layout>(LC), static_cast<rocm_sgemm::m_layout>(LA),
                     static_cast<rocm_sgemm::m_layout>(LB)>(d_C, d_A, d_B, M, N, K, stream);
    HIP_CHECK(hipPeekAtLastError());
    const float ms = timer.stop(stream);
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipMemcpy(h_C.data(), d_C, h_C.size() * sizeof(float), hipMemcpyDeviceToHost));

    double worst = 0.0;
    bool   finite = true;
    for(size_t i = 0; i < M; ++i)
        for(size_t j = 0; j < N; ++j)
        {
            float acc = 0.0f;
            for(size_t k = 0; k < K; ++k) acc += h_A(i, k) * h_B(k, j);
            const double d = std::fabs(static_cast<double>(acc) - static_cast<double>(h_C(i, j)));
            finite         = finite && d == d;
            worst          = d > worst ? d : worst;
        }
    HIP_CHECK(hipFree(d_A));
    HIP_CHECK(hipFree(d_B));
    HIP_CHECK(hipFree(d_C));
    const bool ok = finite && worst <= 1e-4;
    std::printf("A=%d B=%d C=%d  %zux%zux%zu  max abs err %.3g  %.3f ms  %s\n", static_cast<int>(LA),
                static_cast<int>(LB), static_cast<int>(LC), M, N, K, worst, ms, ok ? "PASS" : "FAIL");
    return ok;
}

} // namespace

int main()
{
    hipStream_t stream;
    HIP_CHECK(hipStreamCreate(&stream));
    constexpr ::m_layout r = ::m_layout::row_major, c = ::m_layout::col_major;
    bool                 ok = true;
    // two of the reference test's shapes (test/gemm/test.cpp:113-176), (A, B, C) in its order
    const size_t shapes[2][3] = {{320, 512, 512}, {256, 1024, 256}};
    for(const auto& s : shapes)
    {
        ok &= run_case<c, c, c>(s[0], s[1], s[2], stream);
        ok &= run_case<r, c, c>(s[0], s[1], s[2], stream);
        ok &= run_case<c, r, c>(s[0], s[1], s[2], stream);
        ok &= run_case<r, r, c>(s[0], s[1], s[2], stream);
        ok &= run_case<c, c, r>(s[0], s[1], s[2], stream);
        ok &= run_case<r, c, r>(s[0], s[1], s[2], stream);
        ok &= run_case<c, r, r>(s[0], s[1], s[2], stream);
        ok &= run_case<r, r, r>(s[0], s[1], s[2], stream);
    }
    HIP_CHECK(hipStreamDestroy(stream));
    std::printf("%s\n", ok ? "ALL PASS" : "FAILED");
    return ok ? 0 : 1;
}
