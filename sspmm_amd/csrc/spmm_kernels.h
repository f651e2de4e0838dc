// Launch interface between the C ABI layer and the SpMM kernels.
#ifndef SSPMM_AMD_SPMM_KERNELS_H
#define SSPMM_AMD_SPMM_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sspmm {

struct SpmmArgs {
  int m_vec, N, K, batch;
  const int32_t *row_indices;  // nullable
  const int32_t *row_offsets;
  const int32_t *col_idx;
  const uint16_t *values;
  const uint16_t *B;
  void *C;
  int64_t stride_values, stride_B, stride_C;  // per-batch strides in elements
  // filled by the launcher
  uint32_t n_tiles, total_work, per_xcd;
};

// V must be 8 or 16.  force_generic selects the shape-agnostic kernel even when the MFMA
// kernel's alignment conditions hold (used by tests to cross-check the two).
hipError_t launch_spmm(const SpmmArgs &args, int V, bool out_f16, bool force_generic, hipStream_t stream);

hipError_t launch_sorted_row_swizzle(int m_vec, const int32_t *row_offsets, int32_t *row_indices,
                                     hipStream_t stream);

}  // namespace sspmm
#endif
