// Launch interface of the row reordering that runs ahead of the SVC: rows with similar column
// sets are brought next to each other so that merged groups of V rows hold fewer, fuller vectors.
#ifndef SSPMM_AMD_REORDER_KERNELS_H
#define SSPMM_AMD_REORDER_KERNELS_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace sspmm {

// Workspace for either call below (keys, row ids and the sort's / scan's own scratch); 0 on error.
size_t reorder_workspace_bytes(int M);

// perm[i] = the source row that becomes row i: rows ordered by the 64-bit key
// (min-hash 1 << 32 | min-hash 2) of their column sets, ties in source order.
hipError_t launch_minhash_order(int M, const int32_t *row_ptr, const int32_t *col_ind, int32_t *perm, void *workspace,
                                size_t workspace_bytes, hipStream_t stream);

// out row i = source row perm[i]; val / out_val may both be null.
hipError_t launch_permute_csr(int M, const int32_t *perm, const int32_t *row_ptr, const int32_t *col_ind,
                              const uint16_t *val, int32_t *out_row_ptr, int32_t *out_col, uint16_t *out_val,
                              void *workspace, size_t workspace_bytes, hipStream_t stream);

}  // namespace sspmm
#endif
