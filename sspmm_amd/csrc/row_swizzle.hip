// Device version of the harness helper that orders vector-rows by descending length
// (reference SSpMM/include/bm_test_utils.h:210-225, a host std::sort there).
//
// rank(i) = #{ j : len_j > len_i  or  (len_j == len_i and j < i) } is a stable argsort position,
// so row_indices[rank(i)] = i needs no scratch memory and no atomics.  Lengths are streamed
// through LDS in tiles of 1024; the cost is O(m_vec^2) compares, which for the few thousand
// vector-rows of the matrices this format is used on is a few microseconds.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace sspmm {

static constexpr int kSwizzleThreads = 256;
static constexpr int kSwizzleTile = 1024;

__global__ __launch_bounds__(kSwizzleThreads) void row_swizzle_kernel(int m_vec, const int32_t *row_offsets,
                                                                       int32_t *row_indices) {
  __shared__ int32_t tile_len[kSwizzleTile];
  const int i = blockIdx.x * kSwizzleThreads + threadIdx.x;
  const bool live = i < m_vec;
  const int32_t my_len = live ? row_offsets[i + 1] - row_offsets[i] : 0;
  int32_t rank = 0;
  for (int base = 0; base < m_vec; base += kSwizzleTile) {
    const int cnt = min(kSwizzleTile, m_vec - base);
    __syncthreads();
    for (int t = threadIdx.x; t < cnt; t += kSwizzleThreads)
      tile_len[t] = row_offsets[base + t + 1] - row_offsets[base + t];
    __syncthreads();
    if (live) {
      for (int t = 0; t < cnt; ++t) {
        const int32_t l = tile_len[t];
        rank += (l > my_len) || (l == my_len && base + t < i);
      }
    }
  }
  if (live) row_indices[rank] = i;
}

hipError_t launch_sorted_row_swizzle(int m_vec, const int32_t *row_offsets, int32_t *row_indices,
                                     hipStream_t stream) {
  const int blocks = (m_vec + kSwizzleThreads - 1) / kSwizzleThreads;
  hipLaunchKernelGGL(row_swizzle_kernel, dim3(blocks), dim3(kSwizzleThreads), 0, stream, m_vec, row_offsets,
                     row_indices);
  return hipGetLastError();
}

}  // namespace sspmm
