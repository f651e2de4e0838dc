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
  int m_vec, n_keys, batch;
  const int32_t *row_indices;  // nullable
  const int32_t *row_offsets;
  const int32_t *col_idx;
  const uint16_t *q;  // [batch][m_vec*V][64]
  const uint16_t *k;  // [batch][n_keys][64]
  const uint16_t *v;  // [batch][n_keys][64]
  uint16_t *out;      // [batch][m_vec*V][64]
  int64_t stride_q, stride_k, stride_v, stride_out;  // per-batch strides in elements
  float scale;
  uint32_t total_work, per_xcd;  // filled by the launcher
};

// V must be 8 or 16; F a multiple of 8 up to 256; 16-byte aligned operands and strides.
hipError_t launch_sddmm(const SddmmArgs &args, int V, hipStream_t stream);
hipError_t launch_softmax(const SoftmaxArgs &args, int V, hipStream_t stream);
// sddmm, softmax and the product with v in one kernel, for 64 features per row of q, k and v.  16-byte aligned
// operands and strides; n_keys * 128 bytes below 2 GiB.
hipError_t launch_sparse_attention(const AttentionArgs &args, int V, hipStream_t stream);

}  // namespace sspmm
#endif
