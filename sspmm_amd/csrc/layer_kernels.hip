// Residual add + LayerNorm on feature-major activations, the glue between the sparse products of the
// encoder-layer configuration (the reference's model code keeps these in torch on token-major tensors,
// reference end2end/sspmm_e2e/end_to_end.py:58-75; the SpMM wants and returns [features, tokens], and
// normalising that layout through torch costs two transposed copies per LayerNorm).
//
//   out[h, t] = (s[h, t] - mean_t) * rsqrt(var_t + eps) * gamma[h] + beta[h],   s = fp16(x + a)
//
// with mean and (biased) variance over the H features of token t, in fp32.  HBM-bound: x and a read once, out
// written once (6 * H * T bytes); a workgroup owns 64 tokens, keeps their H x 64 sums in LDS as fp16 and makes
// its three passes (mean, variance, result) over LDS.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layer_kernels.h"

namespace sspmm {

static constexpr int kLnThreads = 1024;
static constexpr int kLnTokens = 64;           // tokens per workgroup: kLnLanes lanes x 4 tokens
static constexpr int kLnLanes = kLnTokens / 4;
static constexpr int kLnRowGroups = kLnThreads / kLnLanes;

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Sum over the workgroup's row groups of one value per token group: across the row groups of a wave with lane
// exchanges, across the waves through LDS.  Contains barriers.
__device__ __forceinline__ floatx4 block_sum_per_token(floatx4 v, floatx4 *red, int tl) {
#pragma unroll
  for (int d = kLnLanes; d < 64; d <<= 1)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += __shfl_xor(v[i], d, 64);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();  // red may still be read from the call before
  if (lane < kLnLanes) red[wave * kLnLanes + tl] = v;
  __syncthreads();
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < kLnThreads / 64; ++w) s += red[w * kLnLanes + tl];
  return s;
}

__global__ __launch_bounds__(kLnThreads) void add_layernorm_kernel(int H, int T, const _Float16 *__restrict__ x,
                                                                    const _Float16 *__restrict__ a,
                                                                    const _Float16 *__restrict__ gamma,
                                                                    const _Float16 *__restrict__ beta, float eps,
                                                                    _Float16 *__restrict__ out) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  half4 *sums = reinterpret_cast<half4 *>(lds_raw);                         // [H][kLnLanes] groups of four tokens
  floatx4 *red = reinterpret_cast<floatx4 *>(lds_raw + (size_t)H * kLnTokens * 2);  // [waves][kLnLanes]
  const int tl = threadIdx.x % kLnLanes, rg = threadIdx.x / kLnLanes;
  const int t0 = blockIdx.x * kLnTokens + 4 * tl;
  const bool live = t0 < T;  // (T is a multiple of 4: a group of four tokens is inside or outside as a whole)
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  // (four rows per trip, their loads issued together: one row per trip would leave a single load per operand in
  // flight per thread, and the kernel is bound by how many bytes its workgroups keep in flight)
  constexpr int kRowsPerTrip = 4;
  for (int h0 = rg; h0 < H; h0 += kLnRowGroups * kRowsPerTrip) {
    half4 xs[kRowsPerTrip], as[kRowsPerTrip];
#pragma unroll
    for (int u = 0; u < kRowsPerTrip; ++u) {
      const int h = h0 + u * kLnRowGroups;
      xs[u] = half4{0, 0, 0, 0};
      as[u] = half4{0, 0, 0, 0};
      if (live && h < H) {
        xs[u] = *reinterpret_cast<const half4 *>(x + (size_t)h * T + t0);
        if (a) as[u] = *reinterpret_cast<const half4 *>(a + (size_t)h * T + t0);
      }
    }
#pragma unroll
    for (int u = 0; u < kRowsPerTrip; ++u) {
      const int h = h0 + u * kLnRowGroups;
      if (h < H) {
        const half4 s = xs[u] + as[u];  // fp16 sum, as the unfused add gives
        sums[h * kLnLanes + tl] = s;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += (float)s[i];
      }
    }
  }
  floatx4 mean = block_sum_per_token(acc, red, tl);
  mean *= 1.0f / (float)H;
  acc = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int h = rg; h < H; h += kLnRowGroups) {
    const half4 s = sums[h * kLnLanes + tl];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float d = (float)s[i] - mean[i];
      acc[i] += d * d;
    }
  }
  floatx4 rstd = block_sum_per_token(acc, red, tl);
#pragma unroll
  for (int i = 0; i < 4; ++i) rstd[i] = rsqrtf(rstd[i] / (float)H + eps);
  if (!live) return;
  for (int h = rg; h < H; h += kLnRowGroups) {
    const half4 s = sums[h * kLnLanes + tl];
    const float w = gamma ? (float)gamma[h] : 1.0f, b = beta ? (float)beta[h] : 0.0f;
    half4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (_Float16)(((float)s[i] - mean[i]) * rstd[i] * w + b);
    *reinterpret_cast<half4 *>(out + (size_t)h * T + t0) = o;
  }
}

size_t add_layernorm_lds_bytes(int H) { return (size_t)H * kLnTokens * 2 + (size_t)(kLnThreads / 64) * kLnLanes * 16; }

hipError_t launch_add_layernorm(int H, int T, const uint16_t *x, const uint16_t *a, const uint16_t *gamma,
                                const uint16_t *beta, float eps, uint16_t *out, hipStream_t stream) {
  const size_t lds = add_layernorm_lds_bytes(H);
  auto kern = add_layernorm_kernel;
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
  }
  const int blocks = (T + kLnTokens - 1) / kLnTokens;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(kLnThreads), lds, stream, H, T, reinterpret_cast<const _Float16 *>(x),
                     reinterpret_cast<const _Float16 *>(a), reinterpret_cast<const _Float16 *>(gamma),
                     reinterpret_cast<const _Float16 *>(beta), eps, reinterpret_cast<_Float16 *>(out));
  return hipGetLastError();
}

}  // namespace sspmm
