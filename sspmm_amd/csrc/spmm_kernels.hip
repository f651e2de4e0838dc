// Vector-sparse SpMM kernels for gfx950 (wave64, MFMA 16x16x32 f16).
//
// C[m_vec*V, N] = A_cvse * B with fp16 inputs and fp32 accumulation.  Same arithmetic as the
// reference kernels SSpMM_V8 / SSpMM_V16 (reference SSpMM/src/sspmm.cu:222-439): per vector-row,
// the sum over its non-zero V x 1 vectors of value-vector (x) gathered row of B.
//
// Mapping to the hardware (not the reference's warp tiling):
//   * one wavefront owns one (vector-row, 128-column tile of B/C) work item;
//   * per step it contracts 32 non-zero vectors with one v_mfma_f32_16x16x32_f16 per 16 output
//     columns.  The MFMA "A" operand (16 rows x 32 k) carries the value vectors, rows = the V
//     entries of a vector (V = 16 fills it, V = 8 uses the lower half); the "B" operand
//     (32 k x 16 columns) carries the gathered rows of the dense matrix;
//   * lane (m = lane % 16, g = lane / 16) gathers, for its eight k slots 8g..8g+7, 16 bytes
//     (8 consecutive columns n0 + 8m .. +7) of each indexed row of B with one
//     buffer_load_dwordx4 each: a 16-lane group reads 256 contiguous bytes of one row.
//     Eight byte-permutes per output column pair turn the "8 columns of one k" registers into
//     "8 k of one column" MFMA operands; accumulator q of a lane then holds column n0 + 8m + q for
//     rows 4g..4g+3, so a lane stores 8 consecutive columns (32 B fp32 / 16 B fp16) per row and
//     a 16-lane group writes a contiguous 512 B / 256 B run of C;
//   * out-of-range k slots and columns are redirected past the end of the buffer descriptor,
//     where buffer loads return zero, so there are no divergent branches in the loop.
//
// Workgroups are 64 threads.  Linear block ids are dealt round-robin to the 8 XCDs by the
// hardware; the block->work mapping gives each XCD one contiguous range of the (tile-major)
// work list so that the waves resident on one XCD gather from the same 128-column slab of B
// and share it in that XCD's L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace sspmm {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));

// Raw buffer descriptor word 3 for gfx9-family targets: 32-bit raw (untyped) buffer.
static constexpr uint32_t kSrdWord3 = 0x00020000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_srd(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, (int)kSrdWord3);
}

__device__ __forceinline__ uint32_t pack_lo(uint32_t x, uint32_t y) { return (x & 0xffffu) | (y << 16); }
__device__ __forceinline__ uint32_t pack_hi(uint32_t x, uint32_t y) { return (x >> 16) | (y & 0xffff0000u); }

union Half8Bits {
  half8 h;
  uint32_t u[4];
};

template <typename OutT>
struct Store8;

template <>
struct Store8<float> {
  static __device__ __forceinline__ void run(float *p, const float (&v)[8]) {
    floatx4 a = {v[0], v[1], v[2], v[3]};
    floatx4 b = {v[4], v[5], v[6], v[7]};
    *reinterpret_cast<floatx4 *>(p) = a;
    *reinterpret_cast<floatx4 *>(p + 4) = b;
  }
};

template <>
struct Store8<_Float16> {
  static __device__ __forceinline__ void run(_Float16 *p, const float (&v)[8]) {
    half8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (_Float16)v[i];  // v_cvt_f16_f32: round to nearest even
    *reinterpret_cast<half8 *>(p) = h;
  }
};

// One chunk = 32 consecutive non-zero vectors of a vector-row.
struct Chunk {
  uintx4 raw[8];     // raw[j] = 8 halfs (columns n0+8m..+7) of the row of B named by k slot 8g+j
  uint16_t a16[8];   // a16[j] = values[(k slot 8g+j), v = m]
};

template <int V>
__device__ __forceinline__ void load_chunk(Chunk &c, int kc, int end, int g, __amdgpu_buffer_rsrc_t srd_cols,
                                           __amdgpu_buffer_rsrc_t srd_vals, __amdgpu_buffer_rsrc_t srd_b,
                                           uint32_t lane_n2, uint32_t lane_col_off, uint32_t b_bytes,
                                           uint32_t vals_lane_off) {
  const int kb = kc + 8 * g;
  // srd_cols / srd_vals end at this vector-row's last vector: slots past it read as zero.
  const uintx4 c0 = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_cols, kb * 4, 0, 0));
  const uintx4 c1 = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_cols, kb * 4 + 16, 0, 0));
  const uint32_t voff = (uint32_t)kb * (V * 2) + vals_lane_off;
#pragma unroll
  for (int j = 0; j < 8; ++j)
    c.a16[j] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(srd_vals, voff + j * V * 2, 0, 0);
  uint32_t off[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t col = j < 4 ? c0[j] : c1[j - 4];
    off[j] = __umul24(col, lane_n2) + lane_col_off;
  }
  if (kc + 32 > end) {  // wave-uniform: only the last chunk of a vector-row can be partial
#pragma unroll
    for (int j = 0; j < 8; ++j) off[j] = (kb + j < end) ? off[j] : b_bytes;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j)
    c.raw[j] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_b, off[j], 0, 0));
}

__device__ __forceinline__ void mac_chunk(const Chunk &c, floatx4 (&acc)[8]) {
  Half8Bits a;
#pragma unroll
  for (int d = 0; d < 4; ++d) a.u[d] = (uint32_t)c.a16[2 * d] | ((uint32_t)c.a16[2 * d + 1] << 16);
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    Half8Bits b;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t x = c.raw[2 * d][q >> 1], y = c.raw[2 * d + 1][q >> 1];
      b.u[d] = (q & 1) ? pack_hi(x, y) : pack_lo(x, y);
    }
    acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, acc[q], 0, 0, 0);
  }
}

template <int V, typename OutT>
__global__ __launch_bounds__(64) void spmm_gather_kernel(const SpmmArgs p) {
  const uint32_t id = blockIdx.x;
  const uint32_t w = (id & 7u) * p.per_xcd + (id >> 3);
  if (w >= p.total_work) return;
  const uint32_t r = w % (uint32_t)p.m_vec;
  const uint32_t t = w / (uint32_t)p.m_vec;
  const uint32_t tile = t % p.n_tiles;
  const uint32_t batch = t / p.n_tiles;
  const int row = p.row_indices ? p.row_indices[r] : (int)r;

  const int lane = threadIdx.x;
  const int m = lane & 15, g = lane >> 4;
  const int beg = p.row_offsets[row], end = p.row_offsets[row + 1];

  const uint16_t *vals = p.values + (int64_t)batch * p.stride_values;
  const uint16_t *bmat = p.B + (int64_t)batch * p.stride_B;
  const uint32_t b_bytes = (uint32_t)p.K * (uint32_t)p.N * 2u;
  const __amdgpu_buffer_rsrc_t srd_cols = make_srd(p.col_idx, (uint32_t)end * 4u);
  const __amdgpu_buffer_rsrc_t srd_vals = make_srd(vals, (uint32_t)end * (V * 2u));
  const __amdgpu_buffer_rsrc_t srd_b = make_srd(bmat, b_bytes);

  const int ncol = (int)tile * 128 + m * 8;
  const bool col_ok = ncol < p.N;
  // Lanes whose columns lie beyond N aim every gather at the first byte past B.
  const uint32_t lane_n2 = col_ok ? (uint32_t)p.N * 2u : 0u;
  const uint32_t lane_col_off = col_ok ? (uint32_t)ncol * 2u : b_bytes;
  const uint32_t vals_lane_off = (uint32_t)m * 2u;

  floatx4 acc[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};

  if (beg < end) {
    // Two chunk buffers used alternately: the gathers of the next 32 vectors are in flight while
    // the current 32 are contracted.
    Chunk c0, c1;
    load_chunk<V>(c0, beg, end, g, srd_cols, srd_vals, srd_b, lane_n2, lane_col_off, b_bytes, vals_lane_off);
    int kc = beg + 32;
    for (;;) {
      if (kc >= end) {
        mac_chunk(c0, acc);
        break;
      }
      load_chunk<V>(c1, kc, end, g, srd_cols, srd_vals, srd_b, lane_n2, lane_col_off, b_bytes, vals_lane_off);
      mac_chunk(c0, acc);
      kc += 32;
      if (kc >= end) {
        mac_chunk(c1, acc);
        break;
      }
      load_chunk<V>(c0, kc, end, g, srd_cols, srd_vals, srd_b, lane_n2, lane_col_off, b_bytes, vals_lane_off);
      mac_chunk(c1, acc);
      kc += 32;
    }
  }

  if (col_ok) {
    OutT *cbase = reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int v = 4 * g + rr;
      if (v < V) {
        float o[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) o[q] = acc[q][rr];
        Store8<OutT>::run(cbase + ((int64_t)row * V + v) * p.N + ncol, o);
      }
    }
  }
}

// Shape-agnostic kernel: any N, any alignment.  One thread per output column, scalar gathers,
// accumulation in ascending vector order (the order of the reference's host check loop,
// reference SSpMM/sspmm_test.cpp:82-94).
template <int V, typename OutT>
__global__ __launch_bounds__(64) void spmm_generic_kernel(const SpmmArgs p) {
  const uint32_t w = blockIdx.x;
  const uint32_t r = w % (uint32_t)p.m_vec;
  const uint32_t t = w / (uint32_t)p.m_vec;
  const uint32_t tile = t % p.n_tiles;
  const uint32_t batch = t / p.n_tiles;
  const int row = p.row_indices ? p.row_indices[r] : (int)r;
  const int n = (int)tile * 64 + threadIdx.x;
  if (n >= p.N) return;
  const _Float16 *vals = reinterpret_cast<const _Float16 *>(p.values) + (int64_t)batch * p.stride_values;
  const _Float16 *bmat = reinterpret_cast<const _Float16 *>(p.B) + (int64_t)batch * p.stride_B;
  float acc[V];
#pragma unroll
  for (int v = 0; v < V; ++v) acc[v] = 0.f;
  const int beg = p.row_offsets[row], end = p.row_offsets[row + 1];
  for (int j = beg; j < end; ++j) {
    const float b = (float)bmat[(int64_t)p.col_idx[j] * p.N + n];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] += (float)vals[(int64_t)j * V + v] * b;
  }
  OutT *cbase = reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C;
#pragma unroll
  for (int v = 0; v < V; ++v) cbase[((int64_t)row * V + v) * p.N + n] = (OutT)acc[v];
}

template <int V, typename OutT>
static hipError_t launch_v(const SpmmArgs &a, bool fast, hipStream_t stream) {
  SpmmArgs p = a;
  if (fast) {
    p.n_tiles = (uint32_t)((a.N + 127) / 128);
    p.total_work = (uint32_t)a.m_vec * p.n_tiles * (uint32_t)a.batch;
    p.per_xcd = (p.total_work + 7u) / 8u;
    hipLaunchKernelGGL((spmm_gather_kernel<V, OutT>), dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
  } else {
    p.n_tiles = (uint32_t)((a.N + 63) / 64);
    p.total_work = (uint32_t)a.m_vec * p.n_tiles * (uint32_t)a.batch;
    p.per_xcd = 0;
    hipLaunchKernelGGL((spmm_generic_kernel<V, OutT>), dim3(p.total_work), dim3(64), 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_spmm(const SpmmArgs &a, int V, bool out_f16, bool force_generic, hipStream_t stream) {
  // The MFMA kernel needs 16-byte row segments of B and C: N % 8 == 0 and aligned bases/strides;
  // 24-bit multiplies bound K and 2N; one buffer descriptor must span B.
  const uint64_t b_bytes = (uint64_t)a.K * (uint64_t)a.N * 2u;
  const int out_size = out_f16 ? 2 : 4;
  bool fast = !force_generic && (a.N % 8 == 0) && (reinterpret_cast<uintptr_t>(a.B) % 16 == 0) &&
              (reinterpret_cast<uintptr_t>(a.C) % 16 == 0) && (a.stride_B % 8 == 0) &&
              ((a.stride_C * out_size) % 16 == 0) && (a.K < (1 << 24)) && (a.N < (1 << 23)) &&
              (b_bytes + 16 <= 0xffffffffull);
  if (V == 8) return out_f16 ? launch_v<8, _Float16>(a, fast, stream) : launch_v<8, float>(a, fast, stream);
  return out_f16 ? launch_v<16, _Float16>(a, fast, stream) : launch_v<16, float>(a, fast, stream);
}

}  // namespace sspmm
