// Launch interface of the model-side glue kernels (feature-major residual add + LayerNorm).
#ifndef SSPMM_AMD_LAYER_KERNELS_H
#define SSPMM_AMD_LAYER_KERNELS_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace sspmm {

// LDS bytes a workgroup needs for H features (the caller checks it against the 160 KB of a CU).

// out[H, T] = LayerNorm over the H features of every token of fp16(x + a) (a may be null), fp16 in and out.
// T must be a multiple of 4 and the pointers 8-byte aligned.
hipError_t launch_add_layernorm(int H, int T, const uint16_t *x, const uint16_t *a, const uint16_t *gamma,
                                const uint16_t *beta, float eps, uint16_t *out, hipStream_t stream);

// Dense attention softmax(Q^T K * scale) V on feature-major activations: q, k, v are [heads * 64, batch * seq] with
// `ld` elements between consecutive features, out likewise with ld_out; fp16, fp32 accumulation.  Applies to a head
// size of 64, seq a multiple of 64 up to 16384, ld and ld_out multiples of 8 and 16-byte aligned pointers.
bool attention_fm_applies(int batch, int heads, int seq, int head_dim, const void *q, const void *k, const void *v,
                          long long ld, const void *out, long long ld_out);
hipError_t launch_attention_fm(int batch, int heads, int seq, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                               long long ld, uint16_t *out, long long ld_out, float scale, hipStream_t stream);

}  // namespace sspmm
#endif
