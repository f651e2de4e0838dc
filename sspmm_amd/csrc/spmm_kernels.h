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
  // Epilogue of the linear-layer entry point, applied to the fp32 sums before they are rounded and stored:
  // C[r, n] = act(sum + bias[r]).  bias: fp16 per output row (m_vec * V), nullable; act: 0 none, 1 GELU (erf form).
  // Honoured by the scalar, gather and staged gather kernels; launch_spmm keeps to those when either is set.
  const uint16_t *bias;
  int act;
  // Mean number of stored vectors per vector-row when the caller knows it (products with a plan), else 0: the
  // kernel choice then also looks at the density, not only at the shape.
  int mean_row_vectors;
  // filled by the launcher
  uint32_t n_tiles, total_work, per_xcd;
  uint32_t n_slabs, row_blocks, rows_per_block, group_by_batch;  // slab kernel
};

// V must be 8 or 16.  Picks the kernel from the shape: the scalar kernel for widths or alignments
// the MFMA kernels cannot take, the LDS-slab kernel when K is small and the problem is large,
// the gather kernel otherwise.
hipError_t launch_spmm(const SpmmArgs &args, int V, bool out_f16, hipStream_t stream);

// Forces a kernel where its preconditions hold: 0 automatic, 1 scalar, 2 gather, 3 LDS slab, 6 staged gather,
// 7 load-balanced gather (calls with a plan only), 9 LDS slab 128 columns wide.
// Per host thread: meant for tests and tuning.  Returns the previous value.
int set_kernel_override(int which);
// Kernel the latest launch_spmm of the calling thread used (1 scalar, 2 gather, 3 LDS slab; 0 before any launch).
int last_kernel();

// Load-balanced kernel over a schedule (schedule.h), one workgroup per item and column tile.  n_items: the number of
// work items; with device_count an upper bound of it (the kernel reads the count from the schedule's header and
// the workgroups beyond it return at once).
// Only where balanced_kernel_applies (the MFMA kernels' alignment and size conditions).
struct ScheduleView;
bool balanced_kernel_applies(const SpmmArgs &args, int V, bool out_f16);
// bundle_base >= 0: the schedule files its whole rows in bundles, units 0 .. bundle_base - 1 are the panels of cut
// rows (one item each), unit bundle_base + b is bundle b, and n_items counts units.
hipError_t launch_spmm_balanced(const SpmmArgs &args, int V, bool out_f16, const ScheduleView &schedule, int n_items,
                                bool device_count, hipStream_t stream, int bundle_base = -1);
int kernel_override();

hipError_t launch_sorted_row_swizzle(int m_vec, const int32_t *row_offsets, int32_t *row_indices,
                                     hipStream_t stream);
// The same order from a stable radix sort in caller-provided scratch memory (linear in m_vec).
size_t sorted_row_swizzle_workspace_bytes(int m_vec);
hipError_t launch_sorted_row_swizzle_ws(int m_vec, const int32_t *row_offsets, int32_t *row_indices, void *workspace,
                                        size_t workspace_bytes, hipStream_t stream);

}  // namespace sspmm
#endif
