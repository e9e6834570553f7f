// Config selection and kernel dispatch (host side).  Covers what the reference splits over
// src/gemm.cpp:8-41, kernel_launcher.hpp:40-99, kernel_lookup.hpp:39 and the generated
// config_generated.hpp / kernel_lookup.cpp (config/generate_config.py:97-303, 415-545).
#ifndef ROCM_SGEMM_AMD_DISPATCH_HPP
#define ROCM_SGEMM_AMD_DISPATCH_HPP

#include <cstddef>
#include <string>

#include <hip/hip_runtime.h>
#include <rocm_sgemm.h>

namespace rocm_sgemm
{
namespace detail
{

struct tuned_entry
{
    size_t            m, n, k;
    int               layout_a, layout_b, layout_c;
    rocm_sgemm_config config;
};

/// Table lookup with the reference's rule (exact key, else nearest same-layout entry by summed
/// squared log2 ratios, else nearest entry, else default).  Works on any table so the unit tests
/// can feed hand-made ones.
const rocm_sgemm_config& select_config(const tuned_entry*       table,
                                       int                      table_size,
                                       const rocm_sgemm_config& fallback,
                                       size_t                   m,
                                       size_t                   n,
                                       size_t                   k,
                                       int                      layout_a,
                                       int                      layout_b,
                                       int                      layout_c);

/// Config the library runs for `batch` products of one shape: a single product that is itself a
/// table entry gets its entry; anything else the cheapest, by the cost model below, of the
/// nearest entry's config (K split fitted to the problem's own tile count), those of the next
/// three nearest entries and the larger direct-to-LDS shapes of the family at split_k 1, 2, 3, 4, 6, 8 -
/// the nearest entry's config stays unless another is predicted at least 5 % faster.
rocm_sgemm_config plan_config(size_t m, size_t n, size_t k, int layout_a, int layout_b, int layout_c,
                              size_t batch = 1);

/// Cost model behind plan_config: rough duration of `batch` products launched together under a
/// config, in microseconds.
double predict_us(const rocm_sgemm_config& config, size_t m, size_t n, size_t k, size_t batch = 1);

/// Whether a launch deals the last wave of `tiles` tiles out as a stream-K tail (one rule for the
/// launch path and the cost model): over how many slots (*slots_out) and how many tiles that
/// wave holds (*r_out).  `cus` = compute units of the GPU.
bool tail_applies(const rocm_sgemm_config& config, long long tiles, long long k_tiles, size_t k, long long cus,
                  long long* slots_out, long long* r_out);

const tuned_entry*       builtin_table();
int                      builtin_table_size();
/// The tuned table plus the mirror image (N, M, K, !b, !a, !c; tile shape exchanged) of every entry
/// whose mirror was not tuned itself - the same launch, so the same timing; what lookups search.
const tuned_entry*       lookup_table();
int                      lookup_table_size();
const rocm_sgemm_config& builtin_default();

int  family_size();
void family_entry(int index, rocm_sgemm_config* out);

/// One call in its general form: for b in [0, batch)
///   C_b <- alpha * A_b * B_b + beta * C_b,   Z_b = Z + b * stride_z,
/// with leading dimensions lda / ldb / ldc (0 = packed, i.e. the extent of the contiguous dimension).
struct gemm_problem
{
    int          layout_c, layout_a, layout_b;
    float*       C;
    const float* A;
    const float* B;
    size_t       M, N, K;
    size_t       lda, ldb, ldc;
    long long    stride_a, stride_b, stride_c;
    size_t       batch;
    float        alpha, beta;
    /// Partial products go to the fixed scratch array of the GPU instead of an allocated workspace;
    /// a problem that needs more than the array holds is refused.
    bool no_alloc = false;
    /// Query only: when set, run_gemm stores the bytes of workspace the call would need for its
    /// partial products there (0 = none) and returns before any allocation or launch.
    size_t* workspace_bytes_out = nullptr;
};

/// Validates, resolves the kernel and enqueues it.  Returns a ROCM_SGEMM_STATUS_* value and, on
/// failure, a message in `error`.
int run_gemm(const rocm_sgemm_config& config, const gemm_problem& problem, hipStream_t stream,
             std::string& error);

/// The reference's form: packed operands, one product, alpha = 1, beta = 0.
int run_gemm(const rocm_sgemm_config& config,
             int                      layout_c,
             int                      layout_a,
             int                      layout_b,
             float*                   C,
             const float*             A,
             const float*             B,
             size_t                   M,
             size_t                   N,
             size_t                   K,
             hipStream_t              stream,
             std::string&             error);

/// Frees every workspace buffer the library holds (one per device and stream that ever needed
/// one).  Waits for the device; the buffers are re-created on demand.
void release_workspaces();

bool config_supported(const rocm_sgemm_config& config, int layout_c, int layout_a, int layout_b,
                      std::string& error);

} // namespace detail
} // namespace rocm_sgemm

#endif
