// Diagnostic kernels: what the memory system of the device sustains for the access pattern of the gather kernels,
// measured with nothing else in the loop.  They are not part of any product; the benchmark reports their rates
// beside the kernels' so that a kernel's distance from the hardware's ceiling can be read off.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "probe.h"

namespace sspmm {

typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));

// Every wave issues `steps` rounds of eight 16-byte loads per lane.  A 16-lane group reads 256 contiguous bytes
// (columns 128 * tile .. + 127) of a pseudo-random row of the [rows x row_bytes] matrix, as the gather kernel's lanes
// do for the rows of B a chunk of vectors names; the eight loads of a round are in flight together.
__global__ __launch_bounds__(256) void probe_gather_kernel(const uintx4 *__restrict__ b, uint32_t rows, uint32_t row_pieces,
                                                            int steps, uintx4 *__restrict__ sink) {
  const uint32_t lane = threadIdx.x & 63u, wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const uint32_t m = lane & 15u, g = lane >> 4;
  const uint32_t tile = wave % (row_pieces / 16u);
  uint32_t state = wave * 0x9E3779B9u + g * 0x85EBCA6Bu + 1u;
  uintx4 acc = {0u, 0u, 0u, 0u};
  for (int s = 0; s < steps; ++s) {
    uintx4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      state = state * 1664525u + 1013904223u;
      const uint32_t row = __umulhi(state, rows);
      v[u] = b[(size_t)row * row_pieces + tile * 16u + m];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  if (acc[0] == 0x9E3779B9u && acc[1] == 0x85EBCA6Bu && acc[2] == 1u) sink[wave] = acc;  // (keeps the loads alive)
}

hipError_t launch_probe_gather(const void *matrix, int rows, int row_bytes, int waves, int steps, void *sink,
                               hipStream_t stream) {
  const unsigned blocks = (unsigned)((waves + 3) / 4);
  hipLaunchKernelGGL(probe_gather_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<const uintx4 *>(matrix),
                     (uint32_t)rows, (uint32_t)row_bytes / 16u, steps, static_cast<uintx4 *>(sink));
  return hipGetLastError();
}

}  // namespace sspmm
