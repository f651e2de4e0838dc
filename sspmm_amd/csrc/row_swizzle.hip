// Device version of the harness helper that orders vector-rows by descending length
// (reference SSpMM/include/bm_test_utils.h:210-225, a host std::sort there).
//
// rank(i) = #{ j : len_j > len_i  or  (len_j == len_i and j < i) } is a stable argsort position,
// so row_indices[rank(i)] = i needs no scratch memory and no atomics.  Lengths are streamed
// through LDS in tiles of 1024; the cost is O(m_vec^2) compares, spread over 16 threads per vector-row.
//
// For patterns of 10^5 vector-rows and more the same order comes from a stable radix sort by length
// (rocPRIM) in caller-provided scratch memory: linear in m_vec, several launches.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <rocprim/device/device_radix_sort.hpp>

#include "spmm_kernels.h"

namespace sspmm {

static constexpr int kSwizzleThreads = 256;
static constexpr int kSwizzleTile = 1024;
static constexpr int kSwizzleRows = 16;                               // vector-rows ranked by a workgroup
static constexpr int kSwizzleParts = kSwizzleThreads / kSwizzleRows;  // threads that share the comparisons of a row

// Thread (row = tid % 16, part = tid / 16) compares its row with every 16th row of the matrix; the 16 counts of a
// row are added up through LDS.  (One thread per row walking all of m_vec, as this kernel first did, is a serial chain
// of m_vec steps on a sixteenth of the workgroups: 124 us for 2048 vector-rows.)
__global__ __launch_bounds__(kSwizzleThreads) void row_swizzle_kernel(int m_vec, const int32_t *row_offsets,
                                                                       int32_t *row_indices) {
  __shared__ int32_t tile_len[kSwizzleTile];
  __shared__ int32_t part_rank[kSwizzleParts][kSwizzleRows];
  const int row = threadIdx.x % kSwizzleRows, part = threadIdx.x / kSwizzleRows;
  const int i = blockIdx.x * kSwizzleRows + row;
  const bool live = i < m_vec;
  const int32_t my_len = live ? row_offsets[i + 1] - row_offsets[i] : 0;
  int32_t rank = 0;
  for (int base = 0; base < m_vec; base += kSwizzleTile) {
    const int cnt = min(kSwizzleTile, m_vec - base);
    __syncthreads();
    for (int t = threadIdx.x; t < cnt; t += kSwizzleThreads)
      tile_len[t] = row_offsets[base + t + 1] - row_offsets[base + t];
    __syncthreads();
    for (int t = part; t < cnt; t += kSwizzleParts) {
      const int32_t l = tile_len[t];
      rank += (l > my_len) || (l == my_len && base + t < i);
    }
  }
  part_rank[part][row] = rank;
  __syncthreads();
  if (part == 0 && live) {
    int32_t r = 0;
#pragma unroll
    for (int q = 0; q < kSwizzleParts; ++q) r += part_rank[q][row];
    row_indices[r] = i;
  }
}

hipError_t launch_sorted_row_swizzle(int m_vec, const int32_t *row_offsets, int32_t *row_indices,
                                     hipStream_t stream) {
  const int blocks = (m_vec + kSwizzleRows - 1) / kSwizzleRows;
  hipLaunchKernelGGL(row_swizzle_kernel, dim3(blocks), dim3(kSwizzleThreads), 0, stream, m_vec, row_offsets,
                     row_indices);
  return hipGetLastError();
}

// ---- with scratch memory: keys (lengths), sorted keys, row numbers, rocPRIM's own temporary storage
namespace {

struct SwizzleLayout {
  size_t keys_in, keys_out, rows_in, lib_temp, lib_bytes, total;
};

SwizzleLayout swizzle_layout(int m_vec) {
  const size_t m = (size_t)(m_vec > 0 ? m_vec : 1);
  const auto up = [](size_t x) { return (x + 255) & ~(size_t)255; };
  SwizzleLayout l{};
  l.keys_in = 0;
  l.keys_out = up(l.keys_in + 4 * m);
  l.rows_in = up(l.keys_out + 4 * m);
  l.lib_temp = up(l.rows_in + 4 * m);
  (void)rocprim::radix_sort_pairs_desc(nullptr, l.lib_bytes, (uint32_t *)nullptr, (uint32_t *)nullptr, (int32_t *)nullptr,
                                       (int32_t *)nullptr, m, 0, 32, (hipStream_t)0);
  l.total = l.lib_temp + up(l.lib_bytes);
  return l;
}

__global__ __launch_bounds__(256) void swizzle_keys_kernel(int m_vec, const int32_t *row_offsets, uint32_t *keys, int32_t *rows) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < m_vec) {
    keys[i] = (uint32_t)(row_offsets[i + 1] - row_offsets[i]);
    rows[i] = i;
  }
}

}  // namespace

size_t sorted_row_swizzle_workspace_bytes(int m_vec) { return swizzle_layout(m_vec).total; }

hipError_t launch_sorted_row_swizzle_ws(int m_vec, const int32_t *row_offsets, int32_t *row_indices, void *workspace,
                                        size_t workspace_bytes, hipStream_t stream) {
  const SwizzleLayout l = swizzle_layout(m_vec);
  if (workspace_bytes < l.total) return hipErrorInvalidValue;
  unsigned char *w = static_cast<unsigned char *>(workspace);
  uint32_t *keys_in = reinterpret_cast<uint32_t *>(w + l.keys_in), *keys_out = reinterpret_cast<uint32_t *>(w + l.keys_out);
  int32_t *rows_in = reinterpret_cast<int32_t *>(w + l.rows_in);
  hipLaunchKernelGGL(swizzle_keys_kernel, dim3((m_vec + 255) / 256), dim3(256), 0, stream, m_vec, row_offsets, keys_in, rows_in);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  // (a radix sort is stable: rows of one length stay in ascending order)
  size_t temp = l.lib_bytes;
  return rocprim::radix_sort_pairs_desc(w + l.lib_temp, temp, keys_in, keys_out, rows_in, row_indices, (size_t)m_vec, 0, 32, stream);
}

}  // namespace sspmm
