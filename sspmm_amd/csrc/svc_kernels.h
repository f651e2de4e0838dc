// Launch interface between the C ABI layer and the SVC (RowMerge) kernels.
#ifndef SSPMM_AMD_SVC_KERNELS_H
#define SSPMM_AMD_SVC_KERNELS_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace sspmm {

struct SvcArgs {
  int M, K, V;
  long long nnz;                 // entries of col_ind
  const int32_t *row_ptr;
  const int32_t *col_ind;
  int32_t *vec_row_ptr;          // svc_count output
  // workspace views
  int32_t *tmp_cols;             // [nnz]   ordered columns of group g at row_ptr[g*V]
  int32_t *pos;                  // [nnz]   position of every non-zero's column inside its group
  unsigned long long *big_tables;  // [8*nnz] hash tables of groups too large for LDS
  int lds_table_slots;           // filled by the launcher
  // direct mode (svc_direct): set by launch_svc_fill, null otherwise
  const int32_t *scanned;        // the finished vec_row_ptr: group g owns vectors [scanned[g], scanned[g + 1])
  int32_t *vec_col;              // final outputs, written by the merge kernels themselves
  uint16_t *vec_val;
  const uint16_t *csr_val;
  // direct mode: the groups filed by size class (written by svc_count, read by svc_fill)
  int32_t *class_counts;         // [5]
  int32_t *class_lists;          // [5][list_stride]
  int list_stride;
  // a stack of matrices (batched entry points): first row of every group, [groups + 1]; null for a single matrix
  const int32_t *group_rows;
  int groups;
};

// True when svc_count only counts (bitmap pass) and svc_fill runs the merge and writes the outputs directly.
bool svc_direct(int order, int K);

// Total workspace bytes; optional byte offsets of the pos, table and class-list views.
size_t svc_workspace_layout(int64_t nnz, int m_vec, size_t *off_pos, size_t *off_tables, size_t *off_lists);

// group_rows[groups + 1] and mat_groups[count + 1] of a stack of matrices from mat_rows[count + 1] (device arrays).
hipError_t launch_svc_group_rows(int count, int V, int groups, const int32_t *mat_rows, int32_t *group_rows,
                                 int32_t *mat_groups, hipStream_t stream);
hipError_t launch_svc_count(const SvcArgs &a, int order, hipStream_t stream);
hipError_t launch_svc_fill(const SvcArgs &a, int order, const uint16_t *csr_val, const int32_t *vec_row_ptr,
                           int32_t *vec_col, uint16_t *vec_val, hipStream_t stream);

}  // namespace sspmm
#endif
