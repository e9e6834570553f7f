// Sampled correctness check shared by the tuner's trial binary and bench_float: a few hundred
// entries of C (the four corners included) against an fp64-accumulated dot product.  Host only.
//
// The worst error is folded so that a NaN sticks.  Both callers pre-fill C with 0xFF bytes (NaN)
// so that an output that was never written shows up, and std::max(worst, NaN) would return
// `worst` and wave such an output through.
#ifndef ROCM_SGEMM_AMD_SAMPLED_CHECK_HPP
#define ROCM_SGEMM_AMD_SAMPLED_CHECK_HPP

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <limits>

namespace rocm_sgemm
{
namespace check
{

inline size_t element(bool col_major, size_t rows, size_t cols, size_t i, size_t j)
{
    return col_major ? j * rows + i : i * cols + j;
}

// max over the samples of |C(i, j) - sum_k A(i, k) B(k, j)|, NaN if any sampled C(i, j) is not a
// finite number close enough to be compared at all.
inline double worst_sampled_abs_error(const float* C, const float* A, const float* B, size_t M, size_t N,
                                      size_t K, bool a_col, bool b_col, bool c_col, int samples = 256)
{
    uint64_t s     = 12345;
    double   worst = 0.0;
    for(int t = 0; t < samples; ++t)
    {
        s        = s * 6364136223846793005ull + 1442695040888963407ull;
        size_t i = (s >> 33) % M;
        s        = s * 6364136223846793005ull + 1442695040888963407ull;
        size_t j = (s >> 33) % N;
        if(t < 4)
        {
            i = (t & 1) ? M - 1 : 0;
            j = (t & 2) ? N - 1 : 0;
        }
        double ref = 0.0;
        for(size_t k = 0; k < K; ++k)
        {
            ref += static_cast<double>(A[element(a_col, M, K, i, k)])
                   * static_cast<double>(B[element(b_col, K, N, k, j)]);
        }
        const double d = std::fabs(ref - static_cast<double>(C[element(c_col, M, N, i, j)]));
        if(!(d <= worst)) // also true for a NaN d, and from then on for every later sample
        {
            worst = d;
        }
        if(worst != worst)
        {
            return std::numeric_limits<double>::quiet_NaN();
        }
    }
    return worst;
}

// max|C - C_ref| / (K max|A| max|B|) over the samples; NaN (which fails every `<=` test) if a
// sampled output is NaN.
inline double sampled_scaled_error(const float* C, const float* A, const float* B, size_t M, size_t N,
                                   size_t K, bool a_col, bool b_col, bool c_col, int samples = 256)
{
    float amax = 0.0f, bmax = 0.0f;
    for(size_t i = 0; i < M * K; ++i) amax = std::fabs(A[i]) > amax ? std::fabs(A[i]) : amax;
    for(size_t i = 0; i < K * N; ++i) bmax = std::fabs(B[i]) > bmax ? std::fabs(B[i]) : bmax;
    const double worst = worst_sampled_abs_error(C, A, B, M, N, K, a_col, b_col, c_col, samples);
    return worst / (static_cast<double>(K) * amax * bmax);
}

// The gate of a tuner trial and of bench_float --verify.  `!(x <= tol)` so that NaN fails.
inline bool within_tolerance(double scaled_error, double tolerance = 1e-6)
{
    return scaled_error <= tolerance;
}

} // namespace check
} // namespace rocm_sgemm

#endif
