// Coordinate list -> CSR on the device, the step between a Matrix Market file and the RowMerge in the
// reference's SuiteSparse path (`csr = self.coo.tocsr()`, reference RowMerge/suit_sparse_matrix.py:109-111,
// whose result has the rows' columns ascending and repeated entries merged).
//
// Integer work bound by HBM: every entry becomes a 64-bit key (row in the high word, column in the low
// word); a radix sort over the bits that can differ orders them, equal neighbours are dropped, and the row
// pointer is read off the places where the high word changes.  12 * n bytes per digit pass of the sort,
// 8 * n read + 4 * n written by the split.
#include "coo_kernels.h"

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_select.hpp>

namespace sspmm {

static constexpr int kCooThreads = 256;
static constexpr unsigned long long kCooInvalid = ~0ull;  // an entry outside the matrix: sorts last, never stored

__global__ __launch_bounds__(kCooThreads) void coo_key_kernel(int M, int K, long long n, const int32_t *__restrict__ row,
                                                              const int32_t *__restrict__ col,
                                                              unsigned long long *__restrict__ keys) {
  const long long i = (long long)blockIdx.x * kCooThreads + threadIdx.x;
  if (i >= n) return;
  const int r = row[i], c = col[i];
  keys[i] = (r >= 0 && r < M && c >= 0 && c < K) ? ((unsigned long long)(uint32_t)r << 32) | (uint32_t)c : kCooInvalid;
}

// keys[0 .. *count): distinct and ascending.  Entry i goes to col_ind[i]; where the row changes between i - 1
// and i, the rows in between (empty ones included) start at i.
__global__ __launch_bounds__(kCooThreads) void coo_split_kernel(int M, long long n, const unsigned long long *__restrict__ keys,
                                                                const unsigned long long *__restrict__ count,
                                                                int32_t *__restrict__ row_ptr, int32_t *__restrict__ col_ind) {
  const long long i = (long long)blockIdx.x * kCooThreads + threadIdx.x;
  long long valid = (long long)*count;
  if (valid > 0 && keys[valid - 1] == kCooInvalid) --valid;  // (all entries outside the matrix collapse into one key)
  if (i > valid || i > n) return;
  const int row_here = i < valid ? (int)(keys[i] >> 32) : M;            // (the end acts as row M)
  const int row_before = i > 0 ? (int)(keys[i - 1] >> 32) : -1;
  if (i < valid) col_ind[i] = (int32_t)(uint32_t)keys[i];
  for (int r = row_before + 1; r <= row_here; ++r) row_ptr[r] = (int32_t)i;
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct CooLayout {
  size_t keys_in, keys_out, count, lib_temp, lib_temp_bytes, total;
};

static hipError_t coo_layout(int64_t n, CooLayout *l) {
  const size_t m = (size_t)(n > 0 ? n : 1);
  size_t sort_bytes = 0, unique_bytes = 0;
  hipError_t e = rocprim::radix_sort_keys(nullptr, sort_bytes, (unsigned long long *)nullptr, (unsigned long long *)nullptr, m, 0,
                                          64, (hipStream_t)0);
  if (e != hipSuccess) return e;
  e = rocprim::unique(nullptr, unique_bytes, (unsigned long long *)nullptr, (unsigned long long *)nullptr,
                      (unsigned long long *)nullptr, m, rocprim::equal_to<unsigned long long>(), (hipStream_t)0);
  if (e != hipSuccess) return e;
  size_t off = 0;
  l->keys_in = off, off += align256(m * 8);
  l->keys_out = off, off += align256(m * 8);
  l->count = off, off += 256;
  l->lib_temp = off;
  l->lib_temp_bytes = align256(sort_bytes > unique_bytes ? sort_bytes : unique_bytes);
  l->total = off + l->lib_temp_bytes;
  return hipSuccess;
}

size_t coo_workspace_bytes(int64_t n) {
  CooLayout l;
  if (n < 0 || coo_layout(n, &l) != hipSuccess) return 0;
  return l.total;
}

__global__ void coo_empty_kernel(int M, int32_t *row_ptr) {
  for (int r = threadIdx.x + blockIdx.x * blockDim.x; r <= M; r += blockDim.x * gridDim.x) row_ptr[r] = 0;
}

hipError_t launch_coo_to_csr(int M, int K, int64_t n, const int32_t *coo_row, const int32_t *coo_col, int32_t *row_ptr,
                             int32_t *col_ind, void *workspace, size_t workspace_bytes, hipStream_t stream) {
  if (n == 0) {
    hipLaunchKernelGGL(coo_empty_kernel, dim3(64), dim3(256), 0, stream, M, row_ptr);
    return hipGetLastError();
  }
  CooLayout l;
  hipError_t e = coo_layout(n, &l);
  if (e != hipSuccess) return e;
  if (workspace_bytes < l.total) return hipErrorInvalidValue;
  unsigned char *w = static_cast<unsigned char *>(workspace);
  auto *keys_in = reinterpret_cast<unsigned long long *>(w + l.keys_in);
  auto *keys_out = reinterpret_cast<unsigned long long *>(w + l.keys_out);
  auto *count = reinterpret_cast<unsigned long long *>(w + l.count);
  const int blocks = (int)((n + kCooThreads - 1) / kCooThreads);
  hipLaunchKernelGGL(coo_key_kernel, dim3(blocks), dim3(kCooThreads), 0, stream, M, K, (long long)n, coo_row, coo_col, keys_in);
  if ((e = hipGetLastError()) != hipSuccess) return e;
  size_t temp = l.lib_temp_bytes;
  if ((e = rocprim::radix_sort_keys(w + l.lib_temp, temp, keys_in, keys_out, (size_t)n, 0, 64, stream)) != hipSuccess) return e;
  temp = l.lib_temp_bytes;
  if ((e = rocprim::unique(w + l.lib_temp, temp, keys_out, keys_in, count, (size_t)n, rocprim::equal_to<unsigned long long>(),
                           stream)) != hipSuccess)
    return e;
  // one thread per position 0 .. n (position `valid` closes the last rows)
  const int blocks1 = (int)((n + 1 + kCooThreads - 1) / kCooThreads);
  hipLaunchKernelGGL(coo_split_kernel, dim3(blocks1), dim3(kCooThreads), 0, stream, M, (long long)n, keys_in, count, row_ptr,
                     col_ind);
  return hipGetLastError();
}

}  // namespace sspmm
