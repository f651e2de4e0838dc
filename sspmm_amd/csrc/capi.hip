// extern "C" boundary of libsspmm_amd.so: argument checks and dispatch to the kernels.
// The declarations and their contracts are in include/sspmm.h.
#include <hip/hip_runtime.h>

#include "../../include/sspmm.h"
#include "attention_kernels.h"
#include "coo_kernels.h"
#include "layer_kernels.h"
#include "plan.h"
#include "reorder_kernels.h"
#include "spmm_kernels.h"
#include "svc_kernels.h"

namespace {

constexpr int kInvalid = (int)hipErrorInvalidValue;

int spmm_entry(int batch, int m_vec, int V, int N, int K, const int32_t *row_indices, const int32_t *row_offsets,
               const int32_t *col_idx, const sspmm_half_t *values, int64_t stride_values, const sspmm_half_t *B,
               int64_t stride_B, void *C, int64_t stride_C, bool out_f16, void *stream,
               const sspmm::Plan *plan = nullptr, const sspmm_half_t *bias = nullptr, int activation = 0) {
  if (V != 8 && V != 16) return kInvalid;
  if (batch < 0 || m_vec < 0 || N < 0 || K < 0) return kInvalid;
  if (batch == 0 || m_vec == 0 || N == 0) return 0;  // nothing to write
  if (!row_offsets || !C) return kInvalid;
  // col_idx / values / B are only dereferenced when some vector-row is non-empty, which the host
  // cannot see (row_offsets is device memory): empty matrices may pass null for them.
  if ((int64_t)K * N >= (1ll << 31)) return kInvalid;
  if ((int64_t)m_vec * V >= (1ll << 31)) return kInvalid;
  const int64_t tiles = ((int64_t)N + 63) / 64;
  if ((int64_t)m_vec * tiles * batch >= (1ll << 31) - 8) return kInvalid;
  if (batch > 1 && (stride_values < 0 || stride_B < 0 || stride_C < (int64_t)m_vec * V * N)) return kInvalid;
  sspmm::SpmmArgs a{};
  a.m_vec = m_vec;
  a.N = N;
  a.K = K;
  a.batch = batch;
  a.row_indices = row_indices;
  a.row_offsets = row_offsets;
  a.col_idx = col_idx;
  a.values = values;
  a.B = B;
  a.C = C;
  a.stride_values = stride_values;
  a.stride_B = stride_B;
  a.stride_C = stride_C;
  a.bias = bias;
  a.act = activation;
  if (plan) return (int)sspmm::launch_spmm_planned(*plan, a, out_f16, static_cast<hipStream_t>(stream));
  return (int)sspmm::launch_spmm(a, V, out_f16, static_cast<hipStream_t>(stream));
}

int plan_entry(const sspmm_plan_t *plan, int batch, int N, const int32_t *row_offsets, const int32_t *col_idx,
               const sspmm_half_t *values, int64_t stride_values, const sspmm_half_t *B, int64_t stride_B, void *C,
               int64_t stride_C, bool out_f16, void *stream) {
  if (!plan) return kInvalid;
  const sspmm::Plan *pl = reinterpret_cast<const sspmm::Plan *>(plan);
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev != pl->device) return kInvalid;  // the plan's memory lives on its device
  return spmm_entry(batch, pl->m_vec, pl->V, N, pl->K, nullptr, row_offsets, col_idx, values, stride_values, B, stride_B,
                    C, stride_C, out_f16, stream, pl);
}

}  // namespace

extern "C" {

int sspmm_version(void) { return (0 << 16) | 1; }

int sspmm_select_kernel(int which) {
  if (which < 0 || (which > 3 && which != 6 && which != 7 && which != 9)) return -1;
  return sspmm::set_kernel_override(which);
}

int sspmm_last_kernel(void) { return sspmm::last_kernel(); }

const char *sspmm_error_string(int code) {
  if (code == 0) return "success";
  if (code == kInvalid) return "invalid argument (unsupported V, negative size, null pointer or index range)";
  if (code == SSPMM_ERROR_STATIC_SCRATCH_TOO_SMALL)
    return "the problem exceeds the static scratch memory of the allocation-free entry point (m_vec <= 32768, N <= 4096)";
  return hipGetErrorString(static_cast<hipError_t>(code));
}

int sspmm_f16_f32(int m_vec, int V, int N, int K, const int32_t *row_indices, const int32_t *row_offsets,
                  const int32_t *col_idx, const sspmm_half_t *values, const sspmm_half_t *B, float *C,
                  void *hip_stream) {
  return spmm_entry(1, m_vec, V, N, K, row_indices, row_offsets, col_idx, values, 0, B, 0, C, 0, false, hip_stream);
}

int sspmm_f16_f16(int m_vec, int V, int N, int K, const int32_t *row_indices, const int32_t *row_offsets,
                  const int32_t *col_idx, const sspmm_half_t *values, const sspmm_half_t *B, sspmm_half_t *C,
                  void *hip_stream) {
  return spmm_entry(1, m_vec, V, N, K, row_indices, row_offsets, col_idx, values, 0, B, 0, C, 0, true, hip_stream);
}

int sspmm_linear_f16(int m_vec, int V, int N, int K, const int32_t *row_offsets, const int32_t *col_idx,
                     const sspmm_half_t *values, const sspmm_half_t *B, const sspmm_half_t *bias, int activation,
                     sspmm_half_t *C, void *hip_stream) {
  if (activation != SSPMM_ACT_NONE && activation != SSPMM_ACT_GELU) return kInvalid;
  return spmm_entry(1, m_vec, V, N, K, nullptr, row_offsets, col_idx, values, 0, B, 0, C, 0, true, hip_stream, nullptr, bias,
                    activation);
}

int sspmm_batched_f16_f16(int batch, int m_vec, int V, int N, int K, const int32_t *row_indices,
                          const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *values,
                          int64_t stride_values, const sspmm_half_t *B, int64_t stride_B, sspmm_half_t *C,
                          int64_t stride_C, void *hip_stream) {
  return spmm_entry(batch, m_vec, V, N, K, row_indices, row_offsets, col_idx, values, stride_values, B, stride_B, C,
                    stride_C, true, hip_stream);
}

int sspmm_batched_f16_f32(int batch, int m_vec, int V, int N, int K, const int32_t *row_indices,
                          const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *values,
                          int64_t stride_values, const sspmm_half_t *B, int64_t stride_B, float *C,
                          int64_t stride_C, void *hip_stream) {
  return spmm_entry(batch, m_vec, V, N, K, row_indices, row_offsets, col_idx, values, stride_values, B, stride_B, C,
                    stride_C, false, hip_stream);
}

int sspmm_plan_create(int m_vec, int V, int K, const int32_t *row_offsets, int max_N, int max_batch, int panel_steps,
                      void *hip_stream, sspmm_plan_t **plan) {
  if (!plan) return kInvalid;
  *plan = nullptr;
  if (V != 8 && V != 16) return kInvalid;
  if (m_vec < 0 || K < 0 || max_N < 0 || max_batch < 0 || panel_steps < 0) return kInvalid;
  if (m_vec > 0 && !row_offsets) return kInvalid;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    return kInvalid;
  }
  if (capturing != hipStreamCaptureStatusNone) return kInvalid;  // it allocates and synchronises
  sspmm::Plan *pl = nullptr;
  const hipError_t e = sspmm::plan_create(m_vec, V, K, row_offsets, max_N, max_batch, panel_steps, stream, &pl);
  *plan = reinterpret_cast<sspmm_plan_t *>(pl);
  return (int)e;
}

int sspmm_plan_destroy(sspmm_plan_t *plan) { return (int)sspmm::plan_destroy(reinterpret_cast<sspmm::Plan *>(plan)); }

int sspmm_plan_info(const sspmm_plan_t *plan, int64_t *info) {
  if (!plan || !info) return kInvalid;
  const sspmm::Plan *pl = reinterpret_cast<const sspmm::Plan *>(plan);
  info[0] = pl->header[sspmm::kHdrNvec];
  info[1] = pl->header[sspmm::kHdrMaxSteps];
  info[2] = pl->header[sspmm::kHdrTotalSteps];
  info[3] = pl->header[sspmm::kHdrBudget];
  info[4] = pl->header[sspmm::kHdrSplitRows];
  info[5] = pl->header[sspmm::kHdrSlots];
  info[6] = pl->header[sspmm::kHdrItems];
  info[7] = (int64_t)pl->bytes;
  return 0;
}

int sspmm_plan_batched_f16_f32(const sspmm_plan_t *plan, int batch, int N, const int32_t *row_offsets,
                               const int32_t *col_idx, const sspmm_half_t *values, int64_t stride_values,
                               const sspmm_half_t *B, int64_t stride_B, float *C, int64_t stride_C, void *hip_stream) {
  return plan_entry(plan, batch, N, row_offsets, col_idx, values, stride_values, B, stride_B, C, stride_C, false, hip_stream);
}

int sspmm_plan_batched_f16_f16(const sspmm_plan_t *plan, int batch, int N, const int32_t *row_offsets,
                               const int32_t *col_idx, const sspmm_half_t *values, int64_t stride_values,
                               const sspmm_half_t *B, int64_t stride_B, sspmm_half_t *C, int64_t stride_C,
                               void *hip_stream) {
  return plan_entry(plan, batch, N, row_offsets, col_idx, values, stride_values, B, stride_B, C, stride_C, true, hip_stream);
}

int sspmm_noalloc_f16_f32(int m_vec, int V, int N, int K, const int32_t *row_offsets, const int32_t *col_idx,
                          const sspmm_half_t *values, const sspmm_half_t *B, float *C, void *hip_stream) {
  if (V != 8 && V != 16) return kInvalid;
  if (m_vec < 0 || N < 0 || K < 0) return kInvalid;
  if (!sspmm::static_spmm_fits(m_vec, N)) return SSPMM_ERROR_STATIC_SCRATCH_TOO_SMALL;
  if (m_vec == 0 || N == 0) return 0;  // nothing to write
  if (!row_offsets || !C) return kInvalid;
  if ((int64_t)K * N >= (1ll << 31)) return kInvalid;
  sspmm::SpmmArgs a{};
  a.m_vec = m_vec;
  a.N = N;
  a.K = K;
  a.batch = 1;
  a.row_offsets = row_offsets;
  a.col_idx = col_idx;
  a.values = values;
  a.B = B;
  a.C = C;
  return (int)sspmm::launch_spmm_static(a, V, false, static_cast<hipStream_t>(hip_stream));
}

int sspmm_sorted_row_swizzle(int m_vec, const int32_t *row_offsets, int32_t *row_indices, void *hip_stream) {
  if (m_vec < 0) return kInvalid;
  if (m_vec == 0) return 0;
  if (!row_offsets || !row_indices) return kInvalid;
  return (int)sspmm::launch_sorted_row_swizzle(m_vec, row_offsets, row_indices, static_cast<hipStream_t>(hip_stream));
}

size_t sspmm_sorted_row_swizzle_workspace_bytes(int m_vec) {
  return m_vec < 0 ? 0 : sspmm::sorted_row_swizzle_workspace_bytes(m_vec);
}

int sspmm_sorted_row_swizzle_ws(int m_vec, const int32_t *row_offsets, int32_t *row_indices, void *workspace,
                                size_t workspace_bytes, void *hip_stream) {
  if (m_vec < 0) return kInvalid;
  if (m_vec == 0) return 0;
  if (!row_offsets || !row_indices || !workspace) return kInvalid;
  return (int)sspmm::launch_sorted_row_swizzle_ws(m_vec, row_offsets, row_indices, workspace, workspace_bytes,
                                                  static_cast<hipStream_t>(hip_stream));
}

int sspmm_sddmm_batched_f16(int batch, int m_vec, int V, int F, int n_rhs, const int32_t *row_indices,
                            const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *lhs,
                            int64_t stride_lhs, const sspmm_half_t *rhs, int64_t stride_rhs, sspmm_half_t *out_values,
                            int64_t stride_out, void *hip_stream) {
  if (V != 8 && V != 16) return kInvalid;
  if (batch < 0 || m_vec < 0 || F < 0 || n_rhs < 0) return kInvalid;
  if (F % 8 != 0 || F > 256) return kInvalid;
  if (batch == 0 || m_vec == 0) return 0;
  if (!row_offsets) return kInvalid;
  // (the kernel forms a row's byte offset with a 24-bit multiply of the column index)
  if ((int64_t)n_rhs * F >= (1ll << 31) || n_rhs >= (1 << 24) || (int64_t)m_vec * batch >= (1ll << 31) - 8) return kInvalid;
  if (reinterpret_cast<uintptr_t>(lhs) % 16 || reinterpret_cast<uintptr_t>(rhs) % 16 ||
      reinterpret_cast<uintptr_t>(out_values) % 8 || stride_lhs % 8 || stride_rhs % 8 || stride_out % 4)
    return kInvalid;
  if (batch > 1 && (stride_lhs < 0 || stride_rhs < 0 || stride_out < 0)) return kInvalid;
  sspmm::SddmmArgs a{};
  a.m_vec = m_vec;
  a.F = F;
  a.n_rhs = n_rhs;
  a.batch = batch;
  a.row_indices = row_indices;
  a.row_offsets = row_offsets;
  a.col_idx = col_idx;
  a.lhs = lhs;
  a.rhs = rhs;
  a.out = out_values;
  a.stride_lhs = stride_lhs;
  a.stride_rhs = stride_rhs;
  a.stride_out = stride_out;
  return (int)sspmm::launch_sddmm(a, V, static_cast<hipStream_t>(hip_stream));
}

int sspmm_sddmm_f16(int m_vec, int V, int F, int n_rhs, const int32_t *row_indices, const int32_t *row_offsets,
                    const int32_t *col_idx, const sspmm_half_t *lhs, const sspmm_half_t *rhs, sspmm_half_t *out_values,
                    void *hip_stream) {
  return sspmm_sddmm_batched_f16(1, m_vec, V, F, n_rhs, row_indices, row_offsets, col_idx, lhs, 0, rhs, 0, out_values, 0,
                                 hip_stream);
}

int sspmm_softmax_batched_f16(int batch, int m_vec, int V, const int32_t *row_indices, const int32_t *row_offsets,
                              const sspmm_half_t *values, float scaler, sspmm_half_t *out_values, int64_t stride,
                              void *hip_stream) {
  if (V != 8 && V != 16) return kInvalid;
  if (batch < 0 || m_vec < 0) return kInvalid;
  if (batch == 0 || m_vec == 0) return 0;
  if (!row_offsets) return kInvalid;
  if ((int64_t)m_vec * batch >= (1ll << 31) - 8) return kInvalid;
  if (reinterpret_cast<uintptr_t>(values) % 16 || reinterpret_cast<uintptr_t>(out_values) % 16 || stride % 8 ||
      (batch > 1 && stride < 0))
    return kInvalid;
  sspmm::SoftmaxArgs a{};
  a.m_vec = m_vec;
  a.batch = batch;
  a.row_indices = row_indices;
  a.row_offsets = row_offsets;
  a.values = values;
  a.out = out_values;
  a.stride = stride;
  a.scaler = scaler;
  return (int)sspmm::launch_softmax(a, V, static_cast<hipStream_t>(hip_stream));
}

int sspmm_softmax_f16(int m_vec, int V, const int32_t *row_indices, const int32_t *row_offsets,
                      const sspmm_half_t *values, float scaler, sspmm_half_t *out_values, void *hip_stream) {
  return sspmm_softmax_batched_f16(1, m_vec, V, row_indices, row_offsets, values, scaler, out_values, 0, hip_stream);
}

int sspmm_sparse_attention_heads_f16(int batch, int heads, int m_vec, int V, int F, int n_keys, const int32_t *row_indices,
                                     const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *q,
                                     int64_t stride_q, int64_t head_q, int64_t ld_q, const sspmm_half_t *k, int64_t stride_k,
                                     int64_t head_k, int64_t ld_k, const sspmm_half_t *v, int64_t stride_v, int64_t head_v,
                                     int64_t ld_v, float scale, sspmm_half_t *out, int64_t stride_out, int64_t head_out,
                                     int64_t ld_out, void *hip_stream) {
  if (V != 8 && V != 16) return kInvalid;
  if (F != 32 && F != 64 && F != 128) return kInvalid;
  if (batch < 0 || heads < 1 || m_vec < 0 || n_keys < 0) return kInvalid;
  if (!(scale > 0.f) || !std::isfinite(scale)) return kInvalid;
  if (batch == 0 || m_vec == 0) return 0;
  if (!row_offsets || !col_idx || !q || !k || !v || !out) return kInvalid;
  if ((int64_t)m_vec * batch * heads >= (1ll << 31) - 8) return kInvalid;
  const int64_t strides[] = {stride_q, head_q, ld_q, stride_k, head_k, ld_k, stride_v, head_v, ld_v, stride_out, head_out, ld_out};
  for (int64_t x : strides)
    if (x % 8 || x < 0) return kInvalid;
  if (ld_q < F || ld_k < F || ld_v < F || ld_out < F) return kInvalid;
  if (ld_k >= (1 << 23) || ld_v >= (1 << 23) || n_keys >= (1 << 24)) return kInvalid;  // (24-bit multiplies of column by row pitch)
  // one buffer descriptor spans the rows of an (element, head) pair
  const int64_t rows_q = (int64_t)m_vec * V, limit = (1ll << 31) - 256;
  if (n_keys > 0 && ((n_keys - 1) * ld_k * 2 >= limit || (n_keys - 1) * ld_v * 2 >= limit)) return kInvalid;
  if ((rows_q - 1) * ld_q * 2 >= limit) return kInvalid;
  if (reinterpret_cast<uintptr_t>(q) % 16 || reinterpret_cast<uintptr_t>(k) % 16 || reinterpret_cast<uintptr_t>(v) % 16 ||
      reinterpret_cast<uintptr_t>(out) % 16)
    return kInvalid;
  sspmm::AttentionArgs a{};
  a.m_vec = m_vec;
  a.n_keys = n_keys;
  a.batch = batch * heads;
  a.heads = heads;
  a.row_indices = row_indices;
  a.row_offsets = row_offsets;
  a.col_idx = col_idx;
  a.q = q;
  a.k = k;
  a.v = v;
  a.out = out;
  a.stride_q = stride_q;
  a.stride_k = stride_k;
  a.stride_v = stride_v;
  a.stride_out = stride_out;
  a.head_q = head_q;
  a.head_k = head_k;
  a.head_v = head_v;
  a.head_out = head_out;
  a.ld_q = ld_q;
  a.ld_k = ld_k;
  a.ld_v = ld_v;
  a.ld_out = ld_out;
  a.scale = scale;
  return (int)sspmm::launch_sparse_attention(a, V, F, static_cast<hipStream_t>(hip_stream));
}

int sspmm_sparse_attention_f16(int batch, int m_vec, int V, int F, int n_keys, const int32_t *row_indices,
                               const int32_t *row_offsets, const int32_t *col_idx, const sspmm_half_t *q, int64_t stride_q,
                               const sspmm_half_t *k, int64_t stride_k, const sspmm_half_t *v, int64_t stride_v, float scale,
                               sspmm_half_t *out, int64_t stride_out, void *hip_stream) {
  if (batch > 1 && stride_out < (int64_t)m_vec * V * F) return kInvalid;  // (the batch elements' outputs must not overlap)
  return sspmm_sparse_attention_heads_f16(batch, 1, m_vec, V, F, n_keys, row_indices, row_offsets, col_idx, q, stride_q, 0, F,
                                          k, stride_k, 0, F, v, stride_v, 0, F, scale, out, stride_out, 0, F, hip_stream);
}

size_t svc_workspace_bytes(int M, int64_t nnz, int V) {
  if (M < 0 || V < 1) return 0;
  return sspmm::svc_workspace_layout(nnz, (M + V - 1) / V, nullptr, nullptr, nullptr);
}

static int svc_args(int M, int K, int V, const int32_t *row_ptr, const int32_t *col_ind, int64_t nnz, void *workspace,
                    sspmm::SvcArgs *a) {
  if (M < 0 || K < 0 || V < 1 || V > 64 || nnz < 0 || nnz >= (1ll << 28)) return kInvalid;
  if (!row_ptr || !workspace || (nnz > 0 && !col_ind)) return kInvalid;
  size_t off_pos, off_tables, off_lists;
  const int m_vec = (M + V - 1) / V;
  sspmm::svc_workspace_layout(nnz, m_vec, &off_pos, &off_tables, &off_lists);
  unsigned char *w = static_cast<unsigned char *>(workspace);
  a->M = M;
  a->K = K;
  a->V = V;
  a->nnz = nnz;
  a->row_ptr = row_ptr;
  a->col_ind = col_ind;
  a->tmp_cols = reinterpret_cast<int32_t *>(w);
  a->pos = reinterpret_cast<int32_t *>(w + off_pos);
  a->big_tables = reinterpret_cast<unsigned long long *>(w + off_tables);
  a->lds_table_slots = 0;
  a->class_counts = reinterpret_cast<int32_t *>(w + off_lists);
  a->class_lists = a->class_counts + 64;
  a->list_stride = m_vec > 0 ? m_vec : 1;
  return 0;
}

int svc_count(int M, int K, int V, const int32_t *row_ptr, const int32_t *col_ind, int64_t nnz, int order,
              int32_t *vec_row_ptr, void *workspace, void *hip_stream) {
  sspmm::SvcArgs a{};
  if (order != SVC_ORDER_CPYTHON && order != SVC_ORDER_SORTED) return kInvalid;
  if (!vec_row_ptr) return kInvalid;
  const int rc = svc_args(M, K, V, row_ptr, col_ind, nnz, workspace, &a);
  if (rc) return rc;
  a.vec_row_ptr = vec_row_ptr;
  return (int)sspmm::launch_svc_count(a, order, static_cast<hipStream_t>(hip_stream));
}

int svc_fill(int M, int K, int V, const int32_t *row_ptr, const int32_t *col_ind, const sspmm_half_t *csr_val,
             int64_t nnz, int order, const int32_t *vec_row_ptr, void *workspace, int32_t *vec_col,
             sspmm_half_t *vec_val, void *hip_stream) {
  sspmm::SvcArgs a{};
  if (order != SVC_ORDER_CPYTHON && order != SVC_ORDER_SORTED) return kInvalid;
  if (!vec_row_ptr) return kInvalid;
  if (csr_val && !vec_val) return kInvalid;
  const int rc = svc_args(M, K, V, row_ptr, col_ind, nnz, workspace, &a);
  if (rc) return rc;
  if (M == 0) return 0;
  return (int)sspmm::launch_svc_fill(a, order, csr_val, vec_row_ptr, vec_col, vec_val,
                                     static_cast<hipStream_t>(hip_stream));
}

// A stack of matrices: the single-matrix workspace for the stacked CSR with room for one short group per matrix,
// then the table of every group's first row.
static size_t svc_batched_layout(int count, int M_total, int64_t nnz, int V, size_t *off_group_rows) {
  const int groups_bound = M_total / V + count;
  const size_t base = sspmm::svc_workspace_layout(nnz, groups_bound, nullptr, nullptr, nullptr);
  if (off_group_rows) *off_group_rows = base;
  return base + (((size_t)groups_bound + 2) * 4 + 255) / 256 * 256;
}

size_t svc_batched_workspace_bytes(int count, int M_total, int64_t nnz, int V) {
  if (count < 0 || M_total < 0 || V < 1) return 0;
  return svc_batched_layout(count, M_total, nnz, V, nullptr);
}

static int svc_batched_args(int count, int groups, const int32_t *mat_rows, int M_total, int K_max, int V,
                            const int32_t *row_ptr, const int32_t *col_ind, int64_t nnz, void *workspace,
                            sspmm::SvcArgs *a, int32_t **group_rows) {
  if (count < 0 || groups < 0 || groups > M_total / (V > 0 ? V : 1) + count || !mat_rows) return kInvalid;
  const int rc = svc_args(M_total, K_max, V, row_ptr, col_ind, nnz, workspace, a);
  if (rc) return rc;
  // (the views of the single-matrix layout, laid out for the most groups the stack can have)
  size_t off_pos, off_tables, off_lists, off_group_rows;
  const int groups_bound = M_total / V + count;
  sspmm::svc_workspace_layout(nnz, groups_bound, &off_pos, &off_tables, &off_lists);
  svc_batched_layout(count, M_total, nnz, V, &off_group_rows);
  unsigned char *w = static_cast<unsigned char *>(workspace);
  a->class_counts = reinterpret_cast<int32_t *>(w + off_lists);
  a->class_lists = a->class_counts + 64;
  a->list_stride = groups_bound > 0 ? groups_bound : 1;
  *group_rows = reinterpret_cast<int32_t *>(w + off_group_rows);
  a->group_rows = *group_rows;
  a->groups = groups;
  return 0;
}

int svc_count_batched(int count, int groups, const int32_t *mat_rows, int M_total, int K_max, int V,
                      const int32_t *row_ptr, const int32_t *col_ind, int64_t nnz, int order, int32_t *mat_groups,
                      int32_t *vec_row_ptr, void *workspace, void *hip_stream) {
  sspmm::SvcArgs a{};
  int32_t *group_rows = nullptr;
  if (order != SVC_ORDER_CPYTHON && order != SVC_ORDER_SORTED) return kInvalid;
  if (!vec_row_ptr || !mat_groups) return kInvalid;
  const int rc = svc_batched_args(count, groups, mat_rows, M_total, K_max, V, row_ptr, col_ind, nnz, workspace, &a, &group_rows);
  if (rc) return rc;
  a.vec_row_ptr = vec_row_ptr;
  hipStream_t stream = static_cast<hipStream_t>(hip_stream);
  const hipError_t e = sspmm::launch_svc_group_rows(count, V, groups, mat_rows, group_rows, mat_groups, stream);
  if (e != hipSuccess) return (int)e;
  return (int)sspmm::launch_svc_count(a, order, stream);
}

int svc_fill_batched(int count, int groups, const int32_t *mat_rows, int M_total, int K_max, int V,
                     const int32_t *row_ptr, const int32_t *col_ind, const sspmm_half_t *csr_val, int64_t nnz, int order,
                     const int32_t *vec_row_ptr, void *workspace, int32_t *vec_col, sspmm_half_t *vec_val,
                     void *hip_stream) {
  sspmm::SvcArgs a{};
  int32_t *group_rows = nullptr;
  if (order != SVC_ORDER_CPYTHON && order != SVC_ORDER_SORTED) return kInvalid;
  if (!vec_row_ptr) return kInvalid;
  if (csr_val && !vec_val) return kInvalid;
  const int rc = svc_batched_args(count, groups, mat_rows, M_total, K_max, V, row_ptr, col_ind, nnz, workspace, &a, &group_rows);
  if (rc) return rc;
  if (groups == 0) return 0;
  return (int)sspmm::launch_svc_fill(a, order, csr_val, vec_row_ptr, vec_col, vec_val, static_cast<hipStream_t>(hip_stream));
}

size_t svc_reorder_workspace_bytes(int M) { return sspmm::reorder_workspace_bytes(M); }

int svc_reorder_minhash(int M, const int32_t *row_ptr, const int32_t *col_ind, int32_t *perm, void *workspace,
                        size_t workspace_bytes, void *hip_stream) {
  if (M < 0) return kInvalid;
  if (M == 0) return 0;
  if (!row_ptr || !perm || !workspace) return kInvalid;
  return (int)sspmm::launch_minhash_order(M, row_ptr, col_ind, perm, workspace, workspace_bytes,
                                          static_cast<hipStream_t>(hip_stream));
}

int svc_permute_csr(int M, const int32_t *perm, const int32_t *row_ptr, const int32_t *col_ind,
                    const sspmm_half_t *csr_val, int32_t *out_row_ptr, int32_t *out_col, sspmm_half_t *out_val,
                    void *workspace, size_t workspace_bytes, void *hip_stream) {
  if (M < 0 || !out_row_ptr) return kInvalid;
  if (M > 0 && (!perm || !row_ptr || !workspace)) return kInvalid;
  if (csr_val && !out_val) return kInvalid;
  return (int)sspmm::launch_permute_csr(M, perm, row_ptr, col_ind, csr_val, out_row_ptr, out_col,
                                        csr_val ? out_val : nullptr, workspace, workspace_bytes,
                                        static_cast<hipStream_t>(hip_stream));
}

int sspmm_add_layernorm_f16(int H, int T, const sspmm_half_t *x, const sspmm_half_t *a, const sspmm_half_t *gamma,
                            const sspmm_half_t *beta, float eps, sspmm_half_t *out, void *hip_stream) {
  if (H < 0 || T < 0 || T % 4 != 0 || H > 4096) return kInvalid;
  if (H == 0 || T == 0) return 0;
  if (!x || !out) return kInvalid;
  if (reinterpret_cast<uintptr_t>(x) % 8 || reinterpret_cast<uintptr_t>(a) % 8 || reinterpret_cast<uintptr_t>(out) % 8)
    return kInvalid;
  return (int)sspmm::launch_add_layernorm(H, T, x, a, gamma, beta, eps, out, static_cast<hipStream_t>(hip_stream));
}

int sspmm_attention_fm_f16(int batch, int heads, int seq, int head_dim, const sspmm_half_t *q, const sspmm_half_t *k,
                           const sspmm_half_t *v, int64_t ld, sspmm_half_t *out, int64_t ld_out, float scale, void *hip_stream) {
  if (batch < 0 || heads < 0 || seq < 0 || head_dim <= 0) return kInvalid;
  if (batch == 0 || heads == 0 || seq == 0) return 0;
  // (the kernel's running maximum is taken of the unscaled scores, which orders the scaled ones only for scale > 0)
  if (!(scale > 0.0f) || !(scale <= 3.0e38f)) return kInvalid;
  if (!q || !k || !v || !out || ld < (int64_t)batch * seq || ld_out < (int64_t)batch * seq) return kInvalid;
  if (!sspmm::attention_fm_applies(batch, heads, seq, head_dim, q, k, v, ld, out, ld_out)) return kInvalid;
  return (int)sspmm::launch_attention_fm(batch, heads, seq, q, k, v, ld, out, ld_out, scale, static_cast<hipStream_t>(hip_stream));
}

size_t svc_coo_workspace_bytes(int64_t n) { return sspmm::coo_workspace_bytes(n); }

int svc_coo_to_csr(int M, int K, int64_t n, const int32_t *coo_row, const int32_t *coo_col, int32_t *row_ptr,
                   int32_t *col_ind, void *workspace, size_t workspace_bytes, void *hip_stream) {
  if (M < 0 || K < 0 || n < 0 || n >= (1ll << 31) - 1 || !row_ptr) return kInvalid;
  if (n > 0 && (!coo_row || !coo_col || !col_ind || !workspace)) return kInvalid;
  return (int)sspmm::launch_coo_to_csr(M, K, n, coo_row, coo_col, row_ptr, col_ind, workspace, workspace_bytes,
                                       static_cast<hipStream_t>(hip_stream));
}

}  // extern "C"
