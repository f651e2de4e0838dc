// Launch interface of the two steps that sit either side of the batched SpMM in a sparse
// attention block: the sampled dense-dense product and the row softmax over stored entries.
#ifndef SSPMM_AMD_ATTENTION_KERNELS_H
#define SSPMM_AMD_ATTENTION_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sspmm {

struct SddmmArgs {
  int m_vec, F, n_rhs, batch;
  const int32_t *row_indices;  // nullable
  const int32_t *row_offsets;
  const int32_t *col_idx;
  const uint16_t *lhs;  // [batch][m_vec*V][F]
  const uint16_t *rhs;  // [batch][n_rhs][F]
  uint16_t *out;        // [batch][nvec*V]
  int64_t stride_lhs, stride_rhs, stride_out;  // per-batch strides in elements
  uint32_t total_work, per_xcd;                // filled by the launcher
  int pair_stores;                             // filled by the launcher: out and stride_out allow 16-byte stores
};

struct SoftmaxArgs {
  int m_vec, batch;
  const int32_t *row_indices;  // nullable
  const int32_t *row_offsets;
  const uint16_t *values;  // [batch][nvec*V]
  uint16_t *out;           // [batch][nvec*V]
  int64_t stride;          // per-batch stride in elements
  float scaler;
  uint32_t total_work, per_xcd;
};

struct AttentionArgs {
  int m_vec, n_keys, batch, heads;  // batch counts (batch element, head) pairs: element = index / heads, head = index % heads
  const int32_t *row_indices;  // nullable
  const int32_t *row_offsets;
  const int32_t *col_idx;
  const uint16_t *q;  // row r of (element e, head h) at q + e * stride_q + h * head_q + r * ld_q, F features each
  const uint16_t *k;  // n_keys rows per (element, head), addressed the same way
  const uint16_t *v;
  uint16_t *out;      // m_vec * V rows per (element, head)
  int64_t stride_q, stride_k, stride_v, stride_out;  // between batch elements, in elements
  int64_t head_q, head_k, head_v, head_out;          // between the heads of an element
  int64_t ld_q, ld_k, ld_v, ld_out;                  // between rows
  float scale;
  uint32_t total_work, per_xcd;  // filled by the launcher
};

// V must be 8 or 16; F a multiple of 8 up to 256; 16-byte aligned operands and strides.
hipError_t launch_sddmm(const SddmmArgs &args, int V, hipStream_t stream);
hipError_t launch_softmax(const SoftmaxArgs &args, int V, hipStream_t stream);
// sddmm, softmax and the product with v in one kernel, for F = 32, 64 or 128 features per row of q, k and v.  16-byte aligned
// operands and strides; the rows of one (element, head) span less than 2 GiB.
hipError_t launch_sparse_attention(const AttentionArgs &args, int V, int F, hipStream_t stream);

}  // namespace sspmm
#endif
