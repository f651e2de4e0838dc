// Launch interface of the coordinate-list to CSR conversion (the SuiteSparse ingest of the RowMerge tooling).
#ifndef SSPMM_AMD_COO_KERNELS_H
#define SSPMM_AMD_COO_KERNELS_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace sspmm {

size_t coo_workspace_bytes(int64_t n);

// row_ptr[M + 1], col_ind[n]: rows ascending, inside a row the columns ascending, a (row, column) pair that occurs
// several times stored once.  row_ptr[M] is the number of entries that remain.
hipError_t launch_coo_to_csr(int M, int K, int64_t n, const int32_t *coo_row, const int32_t *coo_col, int32_t *row_ptr,
                             int32_t *col_ind, void *workspace, size_t workspace_bytes, hipStream_t stream);

}  // namespace sspmm
#endif
