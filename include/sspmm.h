/*
 * C ABI of libsspmm_amd.so: vector-sparse SpMM and Sparse Vector Compression (RowMerge) on
 * AMD gfx950.  Plain pointers and sizes only; every pointer is a DEVICE pointer owned by the
 * caller unless a comment says otherwise.  All entry points are asynchronous on the given
 * HIP stream (NULL = the default stream), never synchronise, and return 0 on success or a
 * non-zero hipError_t value (1 = invalid value for rejected arguments).
 *
 * The "CVSE" format (reference RowMerge/sparse_matrix_format.py:152-175 and
 * SSpMM/sspmm_test.cpp:28-70):
 *   m_vec                     number of vector-rows, = ceil(M / V); the SpMM treats M = m_vec*V
 *   row_offsets[m_vec+1]      int32, start of each vector-row in col_idx (non-decreasing)
 *   col_idx[nvec]             int32, column of each non-zero V x 1 vector, nvec = row_offsets[m_vec]
 *   values[nvec*V]            fp16, vector-major: values[j*V + v] = A[i*V + v, col_idx[j]]
 *   row_indices[m_vec]        int32 permutation of vector-rows (processing order), may be NULL
 */
#ifndef SSPMM_AMD_SSPMM_H
#define SSPMM_AMD_SSPMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* IEEE binary16 bit pattern (same memory as _Float16 / __half / torch.float16). */
typedef uint16_t sspmm_half_t;

/* Library version, (major << 16) | minor. */
int sspmm_version(void);

/*
 * Testing and tuning hook without a counterpart in the reference: forces one SpMM kernel wherever
 * its preconditions hold.  0 = automatic choice (default), 1 = scalar kernel (any shape),
 * 2 = one-wave gather kernel, 3 = LDS-slab kernel, 6 = the gather kernel's staged form (rows of B
 * fetched whole and passed through LDS; the automatic choice takes it for N <= 64 only) on any
 * width, 7 = the load-balanced gather kernel (products with a plan only; others ignore it), 9 = the
 * LDS-slab kernel with 128-column slabs (K up to about 570).  The setting belongs to the calling host thread
 * (other threads keep the automatic choice).
 * Returns the previous setting, or -1 for an unknown value.
 */
int sspmm_select_kernel(int which);

/* Companion of sspmm_select_kernel (no counterpart in the reference either): the kernel the latest
 * SpMM call of the calling host thread ran, numbered as above, with 4 = the gather kernel's variant for
 * K > 4096 that splits long vector-rows over the waves of a workgroup (selected as 2) and
 * 5 = the LDS-slab kernel with 32-column slabs, for K too tall for 64-column ones (selected
 * as 3); the staged gather kernel reports 6 also where it was chosen automatically, the load-balanced
 * kernel 7, the LDS-slab kernel with 128-column slabs 9 (chosen for fp16 outputs and dense patterns); 0 before any
 * call of this thread. */
int sspmm_last_kernel(void);

/* Static text for a return code of this library. */
const char *sspmm_error_string(int code);

/*
 * C[m_vec*V, N] = A_cvse[m_vec*V, K] * B[K, N]; fp16 inputs, fp32 accumulation, fp32 output.
 * Replaces spmm::SSpMM(..., float* output_matrix), reference SSpMM/include/sspmm.cuh:31-37
 * (launcher SSpMM/src/sspmm.cu:548-587, 626-635).  Argument order m_vec, V, N, K as the
 * reference's callers pass it (SSpMM/sspmm_test.cpp:189).
 *   V must be 8 or 16; any N >= 0 (the reference silently required N % 64 == 0);
 *   B and C are row-major and dense; C is fully overwritten, all-zero vector-rows included;
 *   K*N and nvec*V must be below 2^31.  row_indices may be NULL (natural order); results do
 *   not depend on it.
 */
int sspmm_f16_f32(int m_vec, int V, int N, int K, const int32_t *row_indices, const int32_t *row_offsets,
                  const int32_t *col_idx, const sspmm_half_t *values, const sspmm_half_t *B, float *C,
                  void *hip_stream);

/*
 * Same with fp16 output (the fp32 sum rounded to nearest even).  Replaces
 * spmm::SSpMM(..., half* output_matrix), reference SSpMM/include/sspmm.cuh:39-45
 * (launcher SSpMM/src/sspmm.cu:588-623, 638-648) and the kernel behind sptrans.spmm.spmm,
 * end2end/sspmm_e2e/src/cuda/spmm_kernel.cu:460-514.
 */
int sspmm_f16_f16(int m_vec, int V, int N, int K, const int32_t *row_indices, const int32_t *row_offsets,
                  const int32_t *col_idx, const sspmm_half_t *values, const sspmm_half_t *B, sspmm_half_t *C,
                  void *hip_stream);

/*
 * Batched SpMM with one sparsity pattern shared by the whole batch; per-batch values, B and C
 * at the given element strides.  Replaces batched_spmm_cuda / batchedWmmaSpmmKernel8,
 * reference end2end/sspmm_e2e/src/cuda/spmm_kernel.cu:145-169, 516-586 (strides :532-534).
 */
int sspmm_batched_f16_f16(int batch, int m_vec, int V, int N, int K, const int32_t *row_indices,
                          const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *values,
                          int64_t stride_values, const sspmm_half_t *B, int64_t stride_B, sspmm_half_t *C,
                          int64_t stride_C, void *hip_stream);

/* Batched form with fp32 output (no counterpart kernel in the reference, which only batches the
 * fp16 output; same semantics as sspmm_f16_f32 per batch element). */
int sspmm_batched_f16_f32(int batch, int m_vec, int V, int N, int K, const int32_t *row_indices,
                          const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *values,
                          int64_t stride_values, const sspmm_half_t *B, int64_t stride_B, float *C,
                          int64_t stride_C, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * A linear layer with a vector-sparse weight in one launch: C = act(A_cvse * B + bias), fp16 out.
 * What the reference's model code does with nn.Linear (weight, bias) followed by the activation in
 * torch (reference end2end/sspmm_e2e/end_to_end.py:55-56, 70-73); here bias and activation are
 * applied to the fp32 sums before they are rounded, so C is written once and never re-read.
 *   bias        fp16 device pointer, one value per output row (m_vec * V), or NULL
 *   activation  SSPMM_ACT_NONE, or SSPMM_ACT_GELU = 0.5 x (1 + erf(x / sqrt 2)) (torch's default)
 * With bias == NULL and SSPMM_ACT_NONE the result equals sspmm_f16_f16's.  Other arguments as
 * sspmm_f16_f16 (no row_indices).
 * ---------------------------------------------------------------------------------------- */
#define SSPMM_ACT_NONE 0
#define SSPMM_ACT_GELU 1
int sspmm_linear_f16(int m_vec, int V, int N, int K, const int32_t *row_offsets, const int32_t *col_idx,
                     const sspmm_half_t *values, const sspmm_half_t *B, const sspmm_half_t *bias, int activation,
                     sspmm_half_t *C, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * Plans: what the library can know about a sparsity pattern before its first product.
 *
 * The reference starts one thread block per vector-row whatever its length (reference
 * SSpMM/src/sspmm.cu:558-559); its handle on uneven rows is the permutation of SortedRowSwizzle
 * (reference SSpMM/include/bm_test_utils.h:210-225, applied at end2end/sspmm_e2e/src/cuda/
 * spmm_kernel.cu:48 and commented out at SSpMM/src/sspmm.cu:248).  A plan replaces that
 * permutation for callers that keep a pattern: sspmm_plan_create reads row_offsets on the
 * device, records the number of stored vectors and the longest vector-row, and when some rows
 * are much longer than the rest builds a schedule in which such rows are cut into panels of
 * equal work, processed by different workgroups and added up in a fixed order.  Products with
 * a plan allocate nothing and give the same bits from run to run; a vector-row that was cut
 * may differ from the product without a plan by the re-association of its fp32 sum.
 *
 *   max_N, max_batch  the widest right-hand side and the largest batch the plan will be used
 *                     with (they size its scratch memory; products beyond them run without the
 *                     schedule).
 *   panel_steps       0 lets the library choose; a positive value forces panels of that many
 *                     steps of 32 vectors (tests and tuning).
 * sspmm_plan_create synchronises the stream (it sizes its allocation from what the device
 * found) and must not be called while the stream is being captured; the plan belongs to the
 * device that was current.  One plan serves one product at a time: two products with the same
 * plan must not overlap on the device (use one plan per stream).  The pattern handed to a
 * product must be the one the plan was made from.
 * ---------------------------------------------------------------------------------------- */
typedef struct sspmm_plan sspmm_plan_t;

int sspmm_plan_create(int m_vec, int V, int K, const int32_t *row_offsets, int max_N, int max_batch,
                      int panel_steps, void *hip_stream, sspmm_plan_t **plan);

int sspmm_plan_destroy(sspmm_plan_t *plan);

/* Fills info[0..7] (host memory): stored vectors, steps of the longest vector-row, steps of all
 * vector-rows, steps per panel, vector-rows that were cut, panels of cut rows, work items,
 * bytes of device memory the plan holds. */
int sspmm_plan_info(const sspmm_plan_t *plan, int64_t *info);

/* sspmm_batched_f16_f32 / sspmm_batched_f16_f16 with a plan in place of row_indices (the plan
 * supplies the processing order); batch = 1 with zero strides is the single product. */
int sspmm_plan_batched_f16_f32(const sspmm_plan_t *plan, int batch, int N, const int32_t *row_offsets,
                               const int32_t *col_idx, const sspmm_half_t *values, int64_t stride_values,
                               const sspmm_half_t *B, int64_t stride_B, float *C, int64_t stride_C, void *hip_stream);

int sspmm_plan_batched_f16_f16(const sspmm_plan_t *plan, int batch, int N, const int32_t *row_offsets,
                               const int32_t *col_idx, const sspmm_half_t *values, int64_t stride_values,
                               const sspmm_half_t *B, int64_t stride_B, sspmm_half_t *C, int64_t stride_C,
                               void *hip_stream);

/*
 * sspmm_plan_batched_f16_f32 for one product without a plan and without allocating.  No
 * counterpart in the reference.  It is for callers that cannot allocate device memory and so
 * cannot hold a plan either: code inside a HIP graph capture whose pattern changes from call to
 * call, tight serving loops, harnesses that forbid hipMalloc.  The schedule, its counters and
 * the partial tiles of cut rows live in an array of device memory that is part of the library
 * (9.7 MB on every GPU the library is used on, held until the process ends); every call rebuilds
 * the schedule there on the device from row_offsets, on the caller's stream, before the product.
 *   Limits: m_vec <= 32768 and N <= 4096; beyond them the call returns
 *   SSPMM_ERROR_STATIC_SCRATCH_TOO_SMALL and does nothing.  Other arguments as sspmm_f16_f32.
 *   All calls on one GPU share the array: two calls that overlap on a GPU (different streams,
 *   or threads) race and give wrong results; calls on one stream are safe.
 *   The first call on a device looks the array's address up and must come before any capture:
 *   made on a capturing stream it returns hipErrorInvalidValue and records nothing.  Patterns that
 *   the load-balanced kernel does not cover (N not a multiple of 8, unaligned pointers) take the
 *   kernels of sspmm_f16_f32 and use no scratch.  Same results as sspmm_plan_batched_f16_f32 with a plan of the same pattern, bit
 *   for bit, as long as the plan's panels also fit 8 MB of partial tiles.
 */
#define SSPMM_ERROR_STATIC_SCRATCH_TOO_SMALL 9001
int sspmm_noalloc_f16_f32(int m_vec, int V, int N, int K, const int32_t *row_offsets, const int32_t *col_idx,
                          const sspmm_half_t *values, const sspmm_half_t *B, float *C, void *hip_stream);

/*
 * row_indices = vector-rows ordered by descending length (ties: ascending row).  Replaces
 * SortedRowSwizzle, reference SSpMM/include/bm_test_utils.h:210-225 (a host std::sort there).
 * No scratch memory is needed.
 */
int sspmm_sorted_row_swizzle(int m_vec, const int32_t *row_offsets, int32_t *row_indices, void *hip_stream);

/*
 * The same order (ties included) for patterns of very many vector-rows: the entry above compares every pair of
 * rows in one launch, which suits the 10^2 - 10^4 vector-rows of this format's matrices; this one sorts by
 * length with a stable radix sort in `workspace` (at least sspmm_sorted_row_swizzle_workspace_bytes(m_vec)
 * bytes of device memory, 256-byte aligned), linear in m_vec, several launches on `hip_stream`.
 */
size_t sspmm_sorted_row_swizzle_workspace_bytes(int m_vec);
int sspmm_sorted_row_swizzle_ws(int m_vec, const int32_t *row_offsets, int32_t *row_indices, void *workspace,
                                size_t workspace_bytes, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * The two steps either side of the batched SpMM in the reference's sparse attention block
 * (end2end/sspmm_e2e/spattention.py:167-179), on the same pattern arrays.
 *
 * Sampled dense-dense product: out_values[j*V + v] = sum_f lhs[(i*V + v)*F + f] * rhs[col_idx[j]*F + f]
 * for every stored vector j of every vector-row i; fp16 inputs, fp32 accumulation, fp16 result.
 * Replaces sddmm_cuda / batched_sddmm_cuda, reference end2end/sspmm_e2e/src/cuda/sddmm_kernel.cu:
 * 1161-1226 and 1228-1295 (batch strides m*k, n*k, nnz*V at :1244-1246).
 *   lhs [m_vec*V, F] and rhs [n_rhs, F] row-major, F a multiple of 8 up to 256, 16-byte aligned;
 *   column indices in [0, n_rhs); n_rhs below 2^24 and n_rhs*F below 2^31.
 * ---------------------------------------------------------------------------------------- */
int sspmm_sddmm_f16(int m_vec, int V, int F, int n_rhs, const int32_t *row_indices, const int32_t *row_offsets,
                    const int32_t *col_idx, const sspmm_half_t *lhs, const sspmm_half_t *rhs, sspmm_half_t *out_values,
                    void *hip_stream);

int sspmm_sddmm_batched_f16(int batch, int m_vec, int V, int F, int n_rhs, const int32_t *row_indices,
                            const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *lhs,
                            int64_t stride_lhs, const sspmm_half_t *rhs, int64_t stride_rhs, sspmm_half_t *out_values,
                            int64_t stride_out, void *hip_stream);

/*
 * Row softmax over the stored entries: for dense row i*V + v, over the vectors j of vector-row i,
 * out_values[j*V + v] = exp(values[j*V + v]*scaler - max) / sum, computed in fp32, fp16 result
 * (positions that are not stored count as -infinity).  Replaces csr_softmax_cuda /
 * batched_csr_softmax_cuda, reference end2end/sspmm_e2e/src/cuda/softmax_kernel.cu:202-290
 * (kernel :95-165).  In place (out_values == values) is allowed; 16-byte aligned pointers.
 */
int sspmm_softmax_f16(int m_vec, int V, const int32_t *row_indices, const int32_t *row_offsets,
                      const sspmm_half_t *values, float scaler, sspmm_half_t *out_values, void *hip_stream);

int sspmm_softmax_batched_f16(int batch, int m_vec, int V, const int32_t *row_indices, const int32_t *row_offsets,
                              const sspmm_half_t *values, float scaler, sspmm_half_t *out_values, int64_t stride,
                              void *hip_stream);

/*
 * The three steps of the attention block in one launch, for heads of F = 32, 64 or 128 features:
 * out[b, i*V + v, :] = sum_j softmax_j(scale * q[b, i*V + v, :] . k[b, col_j, :]) * v[b, col_j, :] over the
 * vectors j of vector-row i; a row with no stored vectors gives zeros.  q, out: [batch][m_vec*V][F];
 * k, v: [batch][n_keys][F]; strides in elements.  Stands for the chain bsddmm -> bcsr_softmax -> bspmm of
 * reference end2end/sspmm_e2e/spattention.py:167-179 (which has no single operator for it): the scores and the
 * probabilities stay on the CU, in fp32, and the probabilities enter the product rounded to fp16 before the
 * division by their sum, so results differ from the chain's by fp16 rounding, not bit for bit.
 * Returns invalid-value for any other F; 16-byte aligned pointers, strides multiples of 8, scale > 0.
 */
int sspmm_sparse_attention_f16(int batch, int m_vec, int V, int F, int n_keys, const int32_t *row_indices,
                               const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *q, int64_t stride_q,
                               const sspmm_half_t *k, int64_t stride_k, const sspmm_half_t *v, int64_t stride_v, float scale,
                               sspmm_half_t *out, int64_t stride_out, void *hip_stream);

/*
 * The same launch on operands that hold several heads side by side, so that a model's fused projection can be used
 * where it lies: row r of (batch element e, head h) starts at x + e*stride_x + h*head_x + r*ld_x (elements; 64
 * features each), for x = q, k, v and out.  The mask is shared by all batch * heads pairs.  For the output of a
 * projection [seq][batch][3 * heads * F] (reference spattention.py:151-157 copies q, k and v out of it and into
 * [batch * heads][seq][F] first): q = qkv, k = qkv + heads*F, v = qkv + 2*heads*F, stride = 3*heads*F,
 * head = F, ld = batch*3*heads*F.  Strides non-negative multiples of 8, ld >= F; the caller sees to it that no two
 * rows of out overlap.  No counterpart in the reference.
 */
int sspmm_sparse_attention_heads_f16(int batch, int heads, int m_vec, int V, int F, int n_keys, const int32_t *row_indices,
                                     const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *q,
                                     int64_t stride_q, int64_t head_q, int64_t ld_q, const sspmm_half_t *k, int64_t stride_k,
                                     int64_t head_k, int64_t ld_k, const sspmm_half_t *v, int64_t stride_v, int64_t head_v,
                                     int64_t ld_v, float scale, sspmm_half_t *out, int64_t stride_out, int64_t head_out,
                                     int64_t ld_out, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * Sparse Vector Compression (RowMerge): CSR -> CVSE.  Replaces the Python pass
 * CVSE.__init__, reference RowMerge/sparse_matrix_format.py:94-123 (merge at :110), and adds
 * the value packing its consumers define (SSpMM/sspmm_test.cpp:90).
 *
 * Two phases so the caller can size the outputs:
 *   1. svc_count  writes vec_row_ptr[m_vec+1]; nvec = vec_row_ptr[m_vec] (read it back, or
 *                 skip the read and size the outputs for the bound nvec <= nnz).
 *   2. svc_fill   writes vec_col[nvec] and, when csr_val != NULL, vec_val[nvec*V] (zero filled).
 * Both phases take the same workspace of svc_workspace_bytes(M, nnz, V) bytes and the same
 * `order`; svc_fill consumes what svc_count left in the workspace.  How the work is split
 * between the two is internal: for SVC_ORDER_CPYTHON with K <= 131072 svc_count only counts
 * each group's distinct columns (a few microseconds) and svc_fill runs the merge, every group
 * writing its output in place; otherwise svc_count runs the merge and svc_fill copies.
 *
 * order: SVC_ORDER_CPYTHON reproduces the column order of the reference's output files (the
 * iteration order of CPython's set in `list(set(acc + row))`), bit for bit;
 * SVC_ORDER_SORTED stores each vector-row's columns ascending.
 * Column indices must lie in [0, K) and a CSR row must not repeat a column; a non-zero that breaks
 * the first rule is ignored, rows that break the second give an unspecified column order (every
 * distinct column of the group still once), and neither makes the kernels touch memory outside the
 * arrays named here.
 * ---------------------------------------------------------------------------------------- */
#define SVC_ORDER_CPYTHON 0
#define SVC_ORDER_SORTED 1

size_t svc_workspace_bytes(int M, int64_t nnz, int V);

int svc_count(int M, int K, int V, const int32_t *row_ptr, const int32_t *col_ind, int64_t nnz, int order,
              int32_t *vec_row_ptr, void *workspace, void *hip_stream);

int svc_fill(int M, int K, int V, const int32_t *row_ptr, const int32_t *col_ind, const sspmm_half_t *csr_val,
             int64_t nnz, int order, const int32_t *vec_row_ptr, void *workspace, int32_t *vec_col,
             sspmm_half_t *vec_val, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * The SVC of many matrices in one chain of launches.  The reference's RowMerge job is a loop
 * over a dataset of small matrices, one CVSE per file (generate_CVSE_file, reference
 * RowMerge/sparse_matrix_format.py:190-250: 2688 matrices, driven twice by RowMerge/row_merge.py:
 * 16-18); one matrix at a time leaves a GPU idle behind launch latencies.  Here the matrices are
 * stacked along the rows into one CSR:
 *   mat_rows[count + 1]  device: first row of matrix i in the stack, mat_rows[count] = M_total
 *   row_ptr[M_total + 1] device: row pointer of the stack (entry offsets into col_ind / csr_val of
 *                        the whole stack), col_ind[nnz], csr_val[nnz]
 *   K_max                the largest column count of the stack (column indices of every matrix lie
 *                        below its own K, so below K_max)
 *   groups               sum over the matrices of ceil(rows / V), computed by the caller
 * A matrix whose row count is not a multiple of V ends with a short group, as it does on its own
 * (sparse_matrix_format.py:109), and the next matrix starts a new one.  Outputs, in the stack's order:
 *   mat_groups[count + 1]    first group of matrix i; mat_groups[count] is the group count the device
 *                            arrived at (equal to `groups` unless the caller miscounted)
 *   vec_row_ptr[groups + 1]  over all groups: matrix i's own row pointer is
 *                            vec_row_ptr[mat_groups[i] + j] - vec_row_ptr[mat_groups[i]]
 *   vec_col / vec_val        the matrices' vectors one after the other; sized for the bound nvec <= nnz
 *                            nothing has to be read back between the two phases
 * Workspace of svc_batched_workspace_bytes(count, M_total, nnz, V) bytes, the same for both phases.
 * Results per matrix are those of svc_count / svc_fill on that matrix alone, bit for bit.
 * ---------------------------------------------------------------------------------------- */
size_t svc_batched_workspace_bytes(int count, int M_total, int64_t nnz, int V);

int svc_count_batched(int count, int groups, const int32_t *mat_rows, int M_total, int K_max, int V,
                      const int32_t *row_ptr, const int32_t *col_ind, int64_t nnz, int order, int32_t *mat_groups,
                      int32_t *vec_row_ptr, void *workspace, void *hip_stream);

int svc_fill_batched(int count, int groups, const int32_t *mat_rows, int M_total, int K_max, int V,
                     const int32_t *row_ptr, const int32_t *col_ind, const sspmm_half_t *csr_val, int64_t nnz, int order,
                     const int32_t *vec_row_ptr, void *workspace, int32_t *vec_col, sspmm_half_t *vec_val,
                     void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * Row reordering ahead of the SVC: the step the reference runs as `python row_merge_reorder.py`
 * (reference README.md:36) to write its dataset-v8 / dataset-v16 folders, which the harness
 * reads when its `reorder` argument is 1 (reference SSpMM/sspmm_test.cpp:304, 313-320).  The
 * reference's reorder module itself is absent from its sources (RowMerge/row_merge.py:8 imports
 * it in a comment only), so the ordering method is this library's own: rows are sorted by a
 * 64-bit key of two min-hashes of their column sets, ties in source order, which places rows
 * with equal column sets next to each other and rows with similar ones near each other.
 *
 *   svc_reorder_minhash  writes perm[M]: row i of the reordered matrix is source row perm[i].
 *   svc_permute_csr      writes the reordered CSR arrays (out_row_ptr[M+1], out_col[nnz] and,
 *                        when csr_val != NULL, out_val[nnz]); feed them to svc_count / svc_fill.
 * Both take a workspace of svc_reorder_workspace_bytes(M) bytes (0 = no usable device).
 * perm must be a permutation of 0..M-1; entries outside that range give empty rows, and when an entry
 * repeats, what would not fit into the nnz entries of the output arrays is dropped.
 * ---------------------------------------------------------------------------------------- */
size_t svc_reorder_workspace_bytes(int M);

int svc_reorder_minhash(int M, const int32_t *row_ptr, const int32_t *col_ind, int32_t *perm, void *workspace,
                        size_t workspace_bytes, void *hip_stream);

int svc_permute_csr(int M, const int32_t *perm, const int32_t *row_ptr, const int32_t *col_ind,
                    const sspmm_half_t *csr_val, int32_t *out_row_ptr, int32_t *out_col, sspmm_half_t *out_val,
                    void *workspace, size_t workspace_bytes, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * Residual add + LayerNorm on feature-major activations [H features, T tokens] (the layout the
 * SpMM takes and returns), fp16 in and out, statistics in fp32:
 *   out[h, t] = (s[h, t] - mean_t) / sqrt(var_t + eps) * gamma[h] + beta[h],  s = fp16(x + a).
 * No counterpart among the reference's kernels: its encoder block (reference
 * end2end/sspmm_e2e/end_to_end.py:58-75) calls torch's LayerNorm on token-major tensors; on the
 * SpMM's layout that costs two transposed copies per call.  a, gamma, beta may be NULL (no
 * residual, scale one, shift zero).  T a multiple of 4, H up to 4096, 8-byte aligned pointers.
 * ---------------------------------------------------------------------------------------- */
int sspmm_add_layernorm_f16(int H, int T, const sspmm_half_t *x, const sspmm_half_t *a, const sspmm_half_t *gamma,
                            const sspmm_half_t *beta, float eps, sspmm_half_t *out, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * Dense attention on feature-major activations: out = softmax(Q^T K * scale) V per (batch element,
 * head), the dense attention of the reference's comparison block (reference
 * end2end/sspmm_e2e/end_to_end.py:84-97, attention.py), which runs in torch on token-major tensors.
 * The SpMM leaves q, k, v as [features, tokens]; this entry point reads them in that layout and
 * writes the context in it, which saves the transposed copies either side of a token-major attention.
 *   q, k, v   fp16 [heads * head_dim, batch * seq]: feature f of token t at f * ld + t, token
 *             t = b * seq + s (they may be three row ranges of one fused projection)
 *   out       fp16, same layout with ld_out
 * Supported: head_dim = 64, seq a multiple of 64 up to 16384, ld and ld_out multiples of 8 and at
 * least batch * seq, 16-byte aligned pointers, scale positive and finite; anything else returns
 * hipErrorInvalidValue.
 * ---------------------------------------------------------------------------------------- */
int sspmm_attention_fm_f16(int batch, int heads, int seq, int head_dim, const sspmm_half_t *q, const sspmm_half_t *k,
                           const sspmm_half_t *v, int64_t ld, sspmm_half_t *out, int64_t ld_out, float scale, void *hip_stream);

/* ------------------------------------------------------------------------------------------
 * Coordinate list -> CSR, the step between a Matrix Market file and the RowMerge in the
 * reference's SuiteSparse path: `csr = self.coo.tocsr()` in suite_matrix.coo2csr, reference
 * RowMerge/suit_sparse_matrix.py:109-111 (scipy: rows ascending, inside a row the columns
 * ascending, a (row, column) pair that occurs several times kept once).
 *   coo_row[n], coo_col[n]  zero-based entries in any order; entries outside [0, M) x [0, K) are dropped
 *   row_ptr[M + 1]          row_ptr[M] is the number of entries that remain (read it back)
 *   col_ind[n]              sized for the case that nothing merges
 * workspace of svc_coo_workspace_bytes(n) bytes (0 = no usable device).
 * ---------------------------------------------------------------------------------------- */
size_t svc_coo_workspace_bytes(int64_t n);

int svc_coo_to_csr(int M, int K, int64_t n, const int32_t *coo_row, const int32_t *coo_col, int32_t *row_ptr,
                   int32_t *col_ind, void *workspace, size_t workspace_bytes, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* SSPMM_AMD_SSPMM_H */
