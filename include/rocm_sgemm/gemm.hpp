// Public C++ entry point of the MI355X SGEMM library.
//
// Source-compatible with the reference header (reference rocm_sgemm/include/rocm_sgemm/gemm.hpp:51-121):
// same namespace, same enum, same template parameter order (C, A, B), same argument list, and the
// same eight explicit instantiations for float, so a caller written against the reference compiles
// and links unchanged.  The definitions live in librocm_sgemm (csrc/api.cpp) and forward to the C
// ABI in <rocm_sgemm.h>.
//
//   C (M x N)  <-  A (M x K) * B (K x N)      alpha = 1, beta = 0, C is overwritten
//
// All three pointers are device memory owned by the caller, dense and packed in the layout named
// by the template arguments.  The call enqueues on `stream` and returns without synchronising.
// Throws std::runtime_error when no kernel exists for the selected config (as the reference does,
// kernel_launcher.hpp:89-94) and nothing else: like the reference, which does not validate its
// arguments and leaves a failed launch to the caller's hipPeekAtLastError, a call with a zero
// dimension or a null pointer returns normally; it enqueues nothing, and rocm_sgemm_last_error()
// (<rocm_sgemm.h>) says why.  Strict status codes are what the C ABI is for.
#ifndef ROCM_SGEMM_GEMM_HPP
#define ROCM_SGEMM_GEMM_HPP

#include <cstddef>
#include <hip/hip_runtime.h>

#include "layout.hpp"

namespace rocm_sgemm
{

template<m_layout layout_C, m_layout layout_A, m_layout layout_B, class T>
__host__ void gemm(T* C, T* A, T* B, size_t M, size_t N, size_t K, hipStream_t& stream);

#define ROCM_SGEMM_EXTERN_GEMM(LC, LA, LB)                                              \
    extern template void gemm<m_layout::LC, m_layout::LA, m_layout::LB, float>(float*,  \
                                                                               float*,  \
                                                                               float*,  \
                                                                               size_t,  \
                                                                               size_t,  \
                                                                               size_t,  \
                                                                               hipStream_t&);
ROCM_SGEMM_EXTERN_GEMM(row_major, row_major, row_major)
ROCM_SGEMM_EXTERN_GEMM(row_major, row_major, col_major)
ROCM_SGEMM_EXTERN_GEMM(row_major, col_major, row_major)
ROCM_SGEMM_EXTERN_GEMM(row_major, col_major, col_major)
ROCM_SGEMM_EXTERN_GEMM(col_major, row_major, row_major)
ROCM_SGEMM_EXTERN_GEMM(col_major, row_major, col_major)
ROCM_SGEMM_EXTERN_GEMM(col_major, col_major, row_major)
ROCM_SGEMM_EXTERN_GEMM(col_major, col_major, col_major)
#undef ROCM_SGEMM_EXTERN_GEMM

} // namespace rocm_sgemm

#endif // ROCM_SGEMM_GEMM_HPP
