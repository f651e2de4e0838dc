// C++ operator surface with the reference's signatures, forwarding to the C ABI in sspmm.h.
//
// Drop-in for `spmm::SSpMM(...)` of the reference (SSpMM/include/sspmm.cuh:31-53): same
// argument order (m_vec, vec_length, N, K, row_indices, row_offsets, column_indices, values,
// rhs_matrix, output_matrix), device pointers, default stream, returns the launch status
// (hipError_t here, cudaError_t there).  The reference's `float` input overload only prints a
// message and returns success (SSpMM/src/sspmm.cu:651-661); here it reports an invalid value.
#ifndef SSPMM_AMD_SSPMM_HPP
#define SSPMM_AMD_SSPMM_HPP

#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include "sspmm.h"

namespace spmm {

inline hipError_t SSpMM(int m_vec, int vec_length, int N, int K, const int *row_indices, const int *row_offsets,
                        const int *column_indices, const __half *values, const __half *rhs_matrix,
                        float *output_matrix) {
  return static_cast<hipError_t>(sspmm_f16_f32(m_vec, vec_length, N, K, row_indices, row_offsets, column_indices,
                                               reinterpret_cast<const sspmm_half_t *>(values),
                                               reinterpret_cast<const sspmm_half_t *>(rhs_matrix), output_matrix,
                                               nullptr));
}

inline hipError_t SSpMM(int m_vec, int vec_length, int N, int K, const int *row_indices, const int *row_offsets,
                        const int *column_indices, const __half *values, const __half *rhs_matrix,
                        __half *output_matrix) {
  return static_cast<hipError_t>(sspmm_f16_f16(m_vec, vec_length, N, K, row_indices, row_offsets, column_indices,
                                               reinterpret_cast<const sspmm_half_t *>(values),
                                               reinterpret_cast<const sspmm_half_t *>(rhs_matrix),
                                               reinterpret_cast<sspmm_half_t *>(output_matrix), nullptr));
}

inline hipError_t SSpMM(int, int, int, int, const int *, const int *, const int *, const float *, const float *,
                        float *) {
  return hipErrorInvalidValue;  // fp32 inputs are not an implemented path in the reference either
}

// The reference's older-ISA entry point (kernel id 0, SSpMM/include/sspmm.cuh:7-29) computes the
// same product; on gfx950 both names run the same kernels.
template <typename OutT>
inline hipError_t SpMM(int m_vec, int vec_length, int N, int K, const int *row_indices, const int *row_offsets,
                       const int *column_indices, const __half *values, const __half *rhs_matrix,
                       OutT *output_matrix) {
  return SSpMM(m_vec, vec_length, N, K, row_indices, row_offsets, column_indices, values, rhs_matrix, output_matrix);
}

}  // namespace spmm
#endif
