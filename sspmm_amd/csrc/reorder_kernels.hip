// Row reordering ahead of the SVC (the role of the reference's row_merge_reorder.py step, reference
// README.md:36, whose reorder module is not part of the reference's sources: the method here is this
// library's own).
//
// Merging V consecutive rows pays off when those rows name the same columns.  Every row gets a
// 64-bit key made of two min-hashes of its column set; two rows agree on a min-hash with a
// probability equal to the Jaccard similarity of their column sets, so a stable sort by key lays
// rows with similar column sets next to each other, and rows with equal column sets always.
// The passes are integer work bound by HBM: one read of the column indices for the keys, a radix
// sort of M (key, row) pairs, and one read + one write of the CSR arrays to apply the order.
#include "reorder_kernels.h"

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/functional.hpp>

namespace sspmm {

static constexpr int kRowLanes = 16;  // lanes that share one CSR row
static constexpr int kReorderThreads = 256;
static constexpr uint32_t kSeed1 = 0x9e3779b9u, kSeed2 = 0x7f4a7c15u;

// Finaliser of MurmurHash3: a bijection on 32-bit words, so distinct columns never tie.
__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x85ebca6bu;
  x ^= x >> 13;
  x *= 0xc2b2ae35u;
  x ^= x >> 16;
  return x;
}

__global__ __launch_bounds__(kReorderThreads) void minhash_key_kernel(int M, const int32_t *row_ptr,
                                                                       const int32_t *col_ind,
                                                                       unsigned long long *keys, int32_t *ids) {
  const int64_t t = (int64_t)blockIdx.x * kReorderThreads + threadIdx.x;
  const int row = (int)(t / kRowLanes);
  const int lane = (int)(t % kRowLanes);
  uint32_t h1 = ~0u, h2 = ~0u;  // an empty row keeps the largest key and sorts last
  if (row < M) {
    const int e1 = row_ptr[row + 1];
    for (int e = row_ptr[row] + lane; e < e1; e += kRowLanes) {
      const uint32_t c = (uint32_t)col_ind[e];
      h1 = min(h1, mix32(c ^ kSeed1));
      h2 = min(h2, mix32(c ^ kSeed2));
    }
  }
  for (int d = kRowLanes / 2; d >= 1; d >>= 1) {
    h1 = min(h1, (uint32_t)__shfl_xor((int)h1, d, kRowLanes));
    h2 = min(h2, (uint32_t)__shfl_xor((int)h2, d, kRowLanes));
  }
  if (row < M && lane == 0) {
    keys[row] = ((unsigned long long)h1 << 32) | h2;
    ids[row] = row;
  }
}

__global__ __launch_bounds__(kReorderThreads) void permuted_length_kernel(int M, const int32_t *perm,
                                                                           const int32_t *row_ptr,
                                                                           int32_t *lengths) {
  const int i = blockIdx.x * kReorderThreads + threadIdx.x;
  if (i >= M) return;
  const int src = perm[i];
  lengths[i] = (src >= 0 && src < M) ? row_ptr[src + 1] - row_ptr[src] : 0;
}

__global__ __launch_bounds__(kReorderThreads) void permute_rows_kernel(int M, const int32_t *perm,
                                                                        const int32_t *row_ptr,
                                                                        const int32_t *col_ind, const uint16_t *val,
                                                                        const int32_t *out_row_ptr, int32_t *out_col,
                                                                        uint16_t *out_val) {
  const int64_t t = (int64_t)blockIdx.x * kReorderThreads + threadIdx.x;
  const int i = (int)(t / kRowLanes);
  const int lane = (int)(t % kRowLanes);
  if (i >= M) return;
  const int src = perm[i];
  if (src < 0 || src >= M) return;
  // A permutation keeps the number of non-zeros; when `perm` repeats a row the lengths add up to more, and whatever
  // would land beyond the source's non-zero count (the size of the output arrays) is dropped.
  const int total = row_ptr[M];
  const int s0 = row_ptr[src], d0 = out_row_ptr[i];
  const int n = min(row_ptr[src + 1] - s0, total - d0);
  for (int e = lane; e < n; e += kRowLanes) {
    out_col[d0 + e] = col_ind[s0 + e];
    if (val) out_val[d0 + e] = val[s0 + e];
  }
}

__global__ void zero_first_kernel(int32_t *p) {
  if (threadIdx.x == 0 && blockIdx.x == 0) p[0] = 0;
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct ReorderLayout {
  size_t keys_in, keys_out, ids, lengths, lib_temp, lib_temp_bytes, total;
};

static hipError_t reorder_layout(int M, ReorderLayout *l) {
  size_t sort_bytes = 0, scan_bytes = 0;
  const size_t n = (size_t)(M > 0 ? M : 1);
  hipError_t e = rocprim::radix_sort_pairs(nullptr, sort_bytes, (unsigned long long *)nullptr,
                                           (unsigned long long *)nullptr, (int32_t *)nullptr, (int32_t *)nullptr, n,
                                           0, 64, (hipStream_t)0);
  if (e != hipSuccess) return e;
  e = rocprim::inclusive_scan(nullptr, scan_bytes, (int32_t *)nullptr, (int32_t *)nullptr, n,
                              rocprim::plus<int32_t>(), (hipStream_t)0);
  if (e != hipSuccess) return e;
  size_t off = 0;
  l->keys_in = off, off += align256(n * 8);
  l->keys_out = off, off += align256(n * 8);
  l->ids = off, off += align256(n * 4);
  l->lengths = off, off += align256(n * 4);
  l->lib_temp = off;
  l->lib_temp_bytes = align256(sort_bytes > scan_bytes ? sort_bytes : scan_bytes);
  l->total = off + l->lib_temp_bytes;
  return hipSuccess;
}

size_t reorder_workspace_bytes(int M) {
  ReorderLayout l;
  if (M < 0 || reorder_layout(M, &l) != hipSuccess) return 0;
  return l.total;
}

static int blocks_for(int64_t threads) { return (int)((threads + kReorderThreads - 1) / kReorderThreads); }

hipError_t launch_minhash_order(int M, const int32_t *row_ptr, const int32_t *col_ind, int32_t *perm, void *workspace,
                                size_t workspace_bytes, hipStream_t stream) {
  if (M == 0) return hipSuccess;
  ReorderLayout l;
  hipError_t e = reorder_layout(M, &l);
  if (e != hipSuccess) return e;
  if (workspace_bytes < l.total) return hipErrorInvalidValue;
  unsigned char *w = static_cast<unsigned char *>(workspace);
  auto *keys_in = reinterpret_cast<unsigned long long *>(w + l.keys_in);
  auto *keys_out = reinterpret_cast<unsigned long long *>(w + l.keys_out);
  auto *ids = reinterpret_cast<int32_t *>(w + l.ids);
  hipLaunchKernelGGL(minhash_key_kernel, dim3(blocks_for((int64_t)M * kRowLanes)), dim3(kReorderThreads), 0, stream,
                     M, row_ptr, col_ind, keys_in, ids);
  if ((e = hipGetLastError()) != hipSuccess) return e;
  size_t temp_bytes = l.lib_temp_bytes;
  // LSD radix sort: stable, so rows with equal keys keep their source order
  return rocprim::radix_sort_pairs(w + l.lib_temp, temp_bytes, keys_in, keys_out, ids, perm, (size_t)M, 0, 64,
                                   stream);
}

hipError_t launch_permute_csr(int M, const int32_t *perm, const int32_t *row_ptr, const int32_t *col_ind,
                              const uint16_t *val, int32_t *out_row_ptr, int32_t *out_col, uint16_t *out_val,
                              void *workspace, size_t workspace_bytes, hipStream_t stream) {
  hipLaunchKernelGGL(zero_first_kernel, dim3(1), dim3(64), 0, stream, out_row_ptr);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || M == 0) return e;
  ReorderLayout l;
  if ((e = reorder_layout(M, &l)) != hipSuccess) return e;
  if (workspace_bytes < l.total) return hipErrorInvalidValue;
  unsigned char *w = static_cast<unsigned char *>(workspace);
  auto *lengths = reinterpret_cast<int32_t *>(w + l.lengths);
  hipLaunchKernelGGL(permuted_length_kernel, dim3(blocks_for(M)), dim3(kReorderThreads), 0, stream, M, perm, row_ptr,
                     lengths);
  if ((e = hipGetLastError()) != hipSuccess) return e;
  size_t temp_bytes = l.lib_temp_bytes;
  e = rocprim::inclusive_scan(w + l.lib_temp, temp_bytes, lengths, out_row_ptr + 1, (size_t)M,
                              rocprim::plus<int32_t>(), stream);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(permute_rows_kernel, dim3(blocks_for((int64_t)M * kRowLanes)), dim3(kReorderThreads), 0, stream,
                     M, perm, row_ptr, col_ind, val, out_row_ptr, out_col, out_val);
  return hipGetLastError();
}

}  // namespace sspmm
