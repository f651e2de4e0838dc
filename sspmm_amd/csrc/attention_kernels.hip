// The two steps either side of the batched SpMM in a sparse attention block, in the same
// vector-sparse format, for gfx950 (wave64, MFMA 16x16x32 f16).
//
//   sddmm:   out[j*V + v] = lhs[i*V + v, :] . rhs[col_j, :]   for the vectors j of vector-row i
//            (reference end2end/sspmm_e2e/src/cuda/sddmm_kernel.cu:1161-1295: `sddmm`, `bsddmm`);
//   softmax: per dense row, over its stored entries, exp(x*scaler - max) / sum
//            (reference end2end/sspmm_e2e/src/cuda/softmax_kernel.cu:95-290: `csr_softmax`, `bcsr_softmax`).
//
// Both are bound by memory traffic: the sddmm by the gathers of rows of rhs (F*2 bytes per stored
// vector) and the writes of the values, the softmax by one read and one write of the values.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "attention_kernels.h"
#include "lane_ops.h"

namespace sspmm {

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));

static constexpr uint32_t kSrdWord3 = 0x00020000u;  // 32-bit raw (untyped) buffer, gfx9 family

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_srd(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, (int)kSrdWord3);
}

// Linear block ids are dealt round-robin to the 8 XCDs by the hardware; each XCD gets one
// contiguous range of the work list so that neighbouring work shares an L2.
__device__ __forceinline__ uint32_t xcd_work_index(uint32_t per_xcd) {
  const uint32_t id = blockIdx.x;
  return (id & 7u) * per_xcd + (id >> 3);
}

}  // namespace

// ------------------------------------------------------------------------------------ sddmm
// One wave per (vector-row, batch element).  The V rows of lhs are the MFMA's first operand and
// stay in registers (lane (m, g) holds features 32c + 8g .. + 7 of row m, c = 0 .. NC-1).  Per
// group of 16 stored vectors the 16 rows of rhs they name are needed in the same layout, lane
// (m, g) holding features 32c + 8g .. of the row of vector m.  Loaded that way, neighbouring
// lanes would read 16 bytes each of sixteen different rows; instead the rows are fetched with
// neighbouring lanes on neighbouring 16-byte pieces of one row (whole 128-byte lines for 64
// features), written to a small LDS stage, and read back in the operand layout.  Rows of the
// stage are padded by 16 bytes so that the sixteen rows a read touches spread over the banks.
// NC MFMAs contract the features, and the lane ends up with rows 4g .. 4g+3 of vector m: eight
// contiguous bytes of the output.  The column indices run two groups ahead of the arithmetic, the
// rows of rhs one group (two stages, used alternately).
template <int V, int NC>
__global__ __launch_bounds__(64) void sddmm_kernel(const SddmmArgs p) {
  constexpr uint32_t kStageRow = NC * 64u + 16u;  // bytes: room for 32 * NC features, and the padding
  __shared__ __align__(16) unsigned char stage[2][16 * kStageRow];
  const uint32_t w = xcd_work_index(p.per_xcd);
  if (w >= p.total_work) return;
  const uint32_t r = w % (uint32_t)p.m_vec;
  const uint32_t batch = w / (uint32_t)p.m_vec;
  const int row = p.row_indices ? p.row_indices[r] : (int)r;
  const int beg = p.row_offsets[row], end = p.row_offsets[row + 1];
  if (beg == end) return;

  const int lane = threadIdx.x, m = lane & 15, g = lane >> 4;
  const uint32_t F = (uint32_t)p.F;
  const uint16_t *lhs = p.lhs + (int64_t)batch * p.stride_lhs + (int64_t)row * V * F;
  const __amdgpu_buffer_rsrc_t srd_lhs = make_srd(lhs, (uint32_t)V * F * 2u);
  const uint32_t rhs_bytes = (uint32_t)p.n_rhs * F * 2u;
  const __amdgpu_buffer_rsrc_t srd_rhs = make_srd(p.rhs + (int64_t)batch * p.stride_rhs, rhs_bytes);
  const __amdgpu_buffer_rsrc_t srd_cols = make_srd(p.col_idx, (uint32_t)end * 4u);  // past the row: reads 0
  uint16_t *out = p.out + (int64_t)batch * p.stride_out;

  // operand side: feature offsets of this lane's 16-byte pieces; pieces past F (or rows past V) are zeros
  uint32_t op_off[NC];
  bool op_ok[NC];
  half8 a[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const uint32_t f0 = 32u * c + 8u * g;
    op_ok[c] = f0 < F;
    op_off[c] = (uint32_t)m * kStageRow + f0 * 2u;
    const uint32_t off = (m < V && f0 < F) ? ((uint32_t)m * F + f0) * 2u : 0xfffffff0u;
    a[c] = __builtin_bit_cast(half8, __builtin_amdgcn_raw_buffer_load_b128(srd_lhs, off, 0, 0));
  }
  // fetch side: piece lane + 64 i of the group's 16 * F / 8 pieces, row-major (piece = 8 features of one row)
  const uint32_t chunks = F / 8u;
  uint32_t ld_row[NC], ld_src[NC], ld_dst[NC];
  bool ld_ok[NC];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const uint32_t piece = (uint32_t)lane + 64u * i;
    ld_row[i] = piece / chunks;
    const uint32_t ch = piece - ld_row[i] * chunks;
    ld_ok[i] = ld_row[i] < 16u;
    ld_src[i] = ch * 16u;
    ld_dst[i] = ld_row[i] * kStageRow + ch * 16u;
  }

  struct Cols {
    uint32_t c[NC];
  };
  struct Pieces {
    uintx4 d[NC];
  };
  // The column indices come in blocks of 64 (four groups), one per lane in one fully coalesced load, a block
  // ahead; the lanes that fetch a row then pick its column out of the block with a lane permute.  (A load per
  // group, eight lanes asking for the same index, costs the memory pipeline sixteen quarter-wave passes for 64
  // bytes, and this kernel is bound by that pipeline.)
  int blk_base = beg;
  uint32_t blk0 = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(srd_cols, (beg + lane) * 4, 0, 0);
  uint32_t blk1 = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(srd_cols, (beg + 64 + lane) * 4, 0, 0);
  auto load_cols = [&](int kc) {  // (called with kc rising by 16 from beg)
    if (kc - blk_base >= 64) {
      blk_base += 64;
      blk0 = blk1;
      blk1 = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(srd_cols, (blk_base + 64 + lane) * 4, 0, 0);
    }
    Cols x;
#pragma unroll
    for (int i = 0; i < NC; ++i)
      x.c[i] = (uint32_t)__builtin_amdgcn_ds_bpermute((kc - blk_base + (int)ld_row[i]) * 4, (int)blk0);
    return x;
  };
  auto load_rows = [&](Pieces &b, const Cols &x) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const uint32_t off = ld_ok[i] ? __umul24(x.c[i], F * 2u) + ld_src[i] : 0xfffffff0u;
      b.d[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_rhs, off, 0, 0));
    }
  };
  auto to_stage = [&](const Pieces &b, unsigned char *st) {
#pragma unroll
    for (int i = 0; i < NC; ++i)
      if (ld_ok[i]) *reinterpret_cast<uintx4 *>(st + ld_dst[i]) = b.d[i];
  };
  // the group's 16 x V products: lane (m, g) gets rows 4g .. 4g+3 of stored vector kc + m, as four halfs
  auto products = [&](const unsigned char *st) {
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      half8 b = {0, 0, 0, 0, 0, 0, 0, 0};
      if (op_ok[c]) b = *reinterpret_cast<const half8 *>(st + op_off[c]);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[c], b, acc, 0, 0, 0);
    }
    const half4 h = {(_Float16)acc[0], (_Float16)acc[1], (_Float16)acc[2], (_Float16)acc[3]};  // round to nearest even
    return __builtin_bit_cast(uintx2, h);
  };
  auto store_group = [&](uintx2 h, int kc) {
    if (kc + m < end && 4 * g < V) *reinterpret_cast<uintx2 *>(out + ((int64_t)(kc + m) * V + 4 * g)) = h;
  };
  // Two groups in one store instruction (a store costs the address unit the same sixteen cycles whether its lanes
  // carry 8 or 16 bytes, and this kernel is bound by that unit): the lane groups g and g + 1 exchange halves, so
  // that g even holds rows 8 (g / 2) .. + 7 of vector kc + m and g odd those of vector kc + 16 + m.
  auto store_two_groups = [&](uintx2 first, uintx2 second, int kc) {
    const auto w0 = __builtin_amdgcn_permlane16_swap(first[0], second[0], false, false);
    const auto w1 = __builtin_amdgcn_permlane16_swap(first[1], second[1], false, false);
    const uintx4 v = {(uint32_t)w0[0], (uint32_t)w1[0], (uint32_t)w0[1], (uint32_t)w1[1]};
    const int vec = kc + m + 16 * (g & 1);
    if (vec < end && 8 * (g >> 1) < V) *reinterpret_cast<uintx4 *>(out + ((int64_t)vec * V + 8 * (g >> 1))) = v;
  };
  const bool pair_stores = p.pair_stores != 0;

  // The LDS operations of a wave execute in order, so a stage can be rewritten right after the reads of the group
  // that used it have been issued; no barrier is involved (one wave per workgroup).
  Pieces b0, b1;
  const Cols c_first = load_cols(beg);
  Cols c_next = load_cols(beg + 16);
  load_rows(b0, c_first);
  to_stage(b0, stage[0]);
  int kc = beg;
  for (;;) {
    // stage[0] holds group kc; c_next the columns of group kc + 16
    if (kc + 16 >= end) {
      store_group(products(stage[0]), kc);
      break;
    }
    Cols c_after = load_cols(kc + 32);
    load_rows(b1, c_next);
    const uintx2 first = products(stage[0]);
    if (!pair_stores) store_group(first, kc);
    to_stage(b1, stage[1]);
    kc += 16;
    if (kc + 16 >= end) {
      const uintx2 second = products(stage[1]);
      if (pair_stores) store_two_groups(first, second, kc - 16);
      else store_group(second, kc);
      break;
    }
    c_next = load_cols(kc + 32);
    load_rows(b0, c_after);
    const uintx2 second = products(stage[1]);
    if (pair_stores) store_two_groups(first, second, kc - 16);
    else store_group(second, kc);
    to_stage(b0, stage[0]);
    kc += 16;
  }
}

template <int V, int NC>
static hipError_t launch_sddmm_nc(const SddmmArgs &a, hipStream_t stream) {
  SddmmArgs p = a;
  p.pair_stores = reinterpret_cast<uintptr_t>(a.out) % 16 == 0 && a.stride_out % 8 == 0;
  p.total_work = (uint32_t)a.m_vec * (uint32_t)a.batch;
  p.per_xcd = (p.total_work + 7u) / 8u;
  if (p.total_work == 0) return hipSuccess;
  hipLaunchKernelGGL((sddmm_kernel<V, NC>), dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
  return hipGetLastError();
}

template <int V>
static hipError_t launch_sddmm_v(const SddmmArgs &a, hipStream_t stream) {
  const int nc = (a.F + 31) / 32;
  if (nc <= 1) return launch_sddmm_nc<V, 1>(a, stream);
  if (nc <= 2) return launch_sddmm_nc<V, 2>(a, stream);
  if (nc <= 4) return launch_sddmm_nc<V, 4>(a, stream);
  return launch_sddmm_nc<V, 8>(a, stream);
}

hipError_t launch_sddmm(const SddmmArgs &a, int V, hipStream_t stream) {
  return V == 8 ? launch_sddmm_v<8>(a, stream) : launch_sddmm_v<16>(a, stream);
}

// ---------------------------------------------------------------------------------- softmax
namespace {

__device__ __forceinline__ float wave_max(float x) { return wave_max_all(x); }
__device__ __forceinline__ float wave_sum(float x) { return wave_sum_all(x); }

template <int V>
struct VecLoad;  // the V halfs of one stored vector
template <>
struct VecLoad<8> {
  static __device__ __forceinline__ void load(const uint16_t *p, _Float16 (&x)[8]) {
    const half8 h = *reinterpret_cast<const half8 *>(p);
#pragma unroll
    for (int v = 0; v < 8; ++v) x[v] = h[v];
  }
  static __device__ __forceinline__ void store(uint16_t *p, const _Float16 (&x)[8]) {
    half8 h;
#pragma unroll
    for (int v = 0; v < 8; ++v) h[v] = x[v];
    // (streamed out: ordinary stores would push the values still to be read out of the L2; measured 75 -> 60 us)
    __builtin_nontemporal_store(h, reinterpret_cast<half8 *>(p));
  }
};
template <>
struct VecLoad<16> {
  static __device__ __forceinline__ void load(const uint16_t *p, _Float16 (&x)[16]) {
    const half8 lo = *reinterpret_cast<const half8 *>(p), hi = *reinterpret_cast<const half8 *>(p + 8);
#pragma unroll
    for (int v = 0; v < 8; ++v) {
      x[v] = lo[v];
      x[8 + v] = hi[v];
    }
  }
  static __device__ __forceinline__ void store(uint16_t *p, const _Float16 (&x)[16]) {
    half8 lo, hi;
#pragma unroll
    for (int v = 0; v < 8; ++v) {
      lo[v] = x[v];
      hi[v] = x[8 + v];
    }
    __builtin_nontemporal_store(lo, reinterpret_cast<half8 *>(p));
    __builtin_nontemporal_store(hi, reinterpret_cast<half8 *>(p + 8));
  }
};

}  // namespace

// One wave per (vector-row, batch element); lane l takes the stored vectors l, l + 64, ... of the
// row, V dense rows at a time.  Three passes over the row's values (maximum, sum of exponentials,
// result).  The first kSoftmaxCached vectors of every lane (512 / 256 vectors of the row for V = 8 / 16) are
// loaded once, all loads in flight together, and stay in registers for the three passes; only the
// rest of a longer row is read again (from the caches).
template <int V>
struct SoftmaxCached {
  static constexpr int value = V == 8 ? 8 : 4;
};

template <int V>
__global__ __launch_bounds__(64) void softmax_kernel(const SoftmaxArgs p) {
  constexpr int KC = SoftmaxCached<V>::value;
  const uint32_t w = xcd_work_index(p.per_xcd);
  if (w >= p.total_work) return;
  const uint32_t r = w % (uint32_t)p.m_vec;
  const uint32_t batch = w / (uint32_t)p.m_vec;
  const int row = p.row_indices ? p.row_indices[r] : (int)r;
  const int beg = p.row_offsets[row], end = p.row_offsets[row + 1];
  if (beg == end) return;
  const int lane = threadIdx.x;
  const uint16_t *in = p.values + (int64_t)batch * p.stride;
  uint16_t *out = p.out + (int64_t)batch * p.stride;
  const float s = p.scaler;
  const int tail = beg + lane + 64 * KC;  // the lane's first vector that is not held in registers

  _Float16 cached[KC][V];
#pragma unroll
  for (int i = 0; i < KC; ++i) {
    const int j = beg + lane + 64 * i;
    if (j < end) {
      VecLoad<V>::load(in + (int64_t)j * V, cached[i]);
    } else {
#pragma unroll
      for (int v = 0; v < V; ++v) cached[i][v] = (_Float16)0;  // never used: the passes below skip these slots
    }
  }

  float mx[V], sum[V];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    mx[v] = -INFINITY;
    sum[v] = 0.f;
  }
#pragma unroll
  for (int i = 0; i < KC; ++i)
    if (beg + lane + 64 * i < end) {
#pragma unroll
      for (int v = 0; v < V; ++v) mx[v] = fmaxf(mx[v], (float)cached[i][v] * s);
    }
  for (int j = tail; j < end; j += 64) {
    _Float16 x[V];
    VecLoad<V>::load(in + (int64_t)j * V, x);
#pragma unroll
    for (int v = 0; v < V; ++v) mx[v] = fmaxf(mx[v], (float)x[v] * s);
  }
#pragma unroll
  for (int v = 0; v < V; ++v) mx[v] = wave_max(mx[v]);
#pragma unroll
  for (int i = 0; i < KC; ++i)
    if (beg + lane + 64 * i < end) {
#pragma unroll
      for (int v = 0; v < V; ++v) sum[v] += __expf((float)cached[i][v] * s - mx[v]);
    }
  for (int j = tail; j < end; j += 64) {
    _Float16 x[V];
    VecLoad<V>::load(in + (int64_t)j * V, x);
#pragma unroll
    for (int v = 0; v < V; ++v) sum[v] += __expf((float)x[v] * s - mx[v]);
  }
#pragma unroll
  for (int v = 0; v < V; ++v) sum[v] = 1.0f / wave_sum(sum[v]);
#pragma unroll
  for (int i = 0; i < KC; ++i) {
    const int j = beg + lane + 64 * i;
    if (j < end) {
      _Float16 y[V];
#pragma unroll
      for (int v = 0; v < V; ++v) y[v] = (_Float16)(__expf((float)cached[i][v] * s - mx[v]) * sum[v]);
      VecLoad<V>::store(out + (int64_t)j * V, y);
    }
  }
  for (int j = tail; j < end; j += 64) {
    _Float16 x[V], y[V];
    VecLoad<V>::load(in + (int64_t)j * V, x);
#pragma unroll
    for (int v = 0; v < V; ++v) y[v] = (_Float16)(__expf((float)x[v] * s - mx[v]) * sum[v]);
    VecLoad<V>::store(out + (int64_t)j * V, y);
  }
}

hipError_t launch_softmax(const SoftmaxArgs &a, int V, hipStream_t stream) {
  SoftmaxArgs p = a;
  p.total_work = (uint32_t)a.m_vec * (uint32_t)a.batch;
  p.per_xcd = (p.total_work + 7u) / 8u;
  if (p.total_work == 0) return hipSuccess;
  if (V == 8)
    hipLaunchKernelGGL(softmax_kernel<8>, dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
  else
    hipLaunchKernelGGL(softmax_kernel<16>, dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
  return hipGetLastError();
}

}  // namespace sspmm
