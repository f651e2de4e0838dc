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

// ---------------------------------------------------------------------- the three steps in one
// softmax(mask(q k^T) * scale) v per vector-row without the scores ever leaving the CU, for heads of 32, 64 or 128
// features (described for 64)
// (the three launches of the block, reference end2end/sspmm_e2e/spattention.py:167-179, move the scores and the
// probabilities through memory twice each: 2 * V bytes per stored vector four times over).
//
// One wave per (vector-row, batch element), a step is 32 stored vectors.  The rows of k and of v the step names
// are fetched as in the staged SpMM kernel (eight lanes on the eight 16-byte pieces of one 128-byte row, lane
// (j, pc) = rows of k slots 4j .. 4j+3, piece pc) and written to two LDS stages with padded rows.
//   scores:  the staged rows of k are the MFMA's first operand (lane (n, g): features 32c + 8g .. of staged row
//            16t + n), the V rows of q the second, held in registers for the whole row; the lane ends up with the
//            scores of query n against staged rows 16t + 4g + r, r = 0 .. 3, t = 0, 1.
//   softmax: running maximum and running sum per query in base 2 (the scale carries log2 e); a query's scores
//            sit in the four lanes n, n + 16, n + 32, n + 48, which exchange their maxima with two lane swaps.
//            When the maximum moves, the sums so far are scaled down by 2^(old - new).
//   product: the eight probabilities of a lane are, in this order, the second operand's k slots 8g .. 8g+7 of
//            query n; the first operand is the transpose read of the staged rows of v in the matching order
//            (rows 4g .. 4g+3, then 16 + 4g .. 16 + 4g + 3).  Lane (n, g) accumulates features 16u + 4g + r of
//            query n, u = 0 .. 3, divides by the sum at the end and stores four times 8 bytes.
// The probabilities enter the product rounded to fp16 before the division by the sum (the three launches round
// after it); sums are fp32 throughout.
// The launch is bound by the stream of gathered rows from the L2 into the CUs (256 bytes per stored vector and batch
// element; measured 21 TB/s on 4096 keys, 90 % masked, 48 heads), not by waves in flight: two waves per SIMD with
// the registers that allows measured 2-7 % faster than three, and four (which spills) 75 % slower.  Column indices
// fetched in blocks of 64 with one coalesced load and handed out with lane permutes, as the sddmm kernel does, take
// 11 % of the address unit's work away and cost 10 % in time here (124 -> 137 us): the permutes queue in the LDS pipe
// behind the stage's writes and reads.  One index per lane of a quad (a 4-byte load) passed round with DPP moves
// measures the same as the 16-byte load, run against it on one box (128.6 and 128.7 us): it is the 64 bytes a
// cycle of the cache's data path that bound the launch, not the count of load instructions.
namespace {

typedef short shortx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uintx2 lds_read_tr(const unsigned char *p) {
  const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) shortx4 *)p);
  return __builtin_bit_cast(uintx2, v);
}

// max / sum over the four lanes n, n + 16, n + 32, n + 48, in each of them
__device__ __forceinline__ float quad_rows_max(float x) {
  const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_rows_sum(float x) {
  const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}


}  // namespace

// F: features per row of q, k and v (32, 64 or 128).  A row is F * 2 bytes = LPR 16-byte pieces, a load instruction
// brings 64 / LPR rows, a step of 32 rows takes L = LPR / 2 of them per operand; lane (jr, pc) fetches piece pc of the
// rows of k slots L * jr .. L * jr + L - 1, whose column indices it reads as L consecutive ints.
template <int V, int F>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(F == 32 ? 4 : 2, F == 32 ? 4 : 2))) void sparse_attention_kernel(const AttentionArgs p) {
  constexpr int LPR = F / 8, L = LPR / 2, NC = F / 32, NT = F / 16;
  constexpr uint32_t kRowBytes = F * 2u, kPitch = kRowBytes + 16u;  // staged rows padded by 16 bytes against bank conflicts
  __shared__ __align__(16) unsigned char stage_k[32 * kPitch];
  __shared__ __align__(16) unsigned char stage_v[32 * kPitch];
  const uint32_t w = xcd_work_index(p.per_xcd);
  if (w >= p.total_work) return;
  const uint32_t r = w % (uint32_t)p.m_vec;
  const uint32_t batch = w / (uint32_t)p.m_vec;
  const int row = __builtin_amdgcn_readfirstlane(p.row_indices ? p.row_indices[r] : (int)r);
  const int beg = p.row_offsets[row], end = p.row_offsets[row + 1];
  const int lane = threadIdx.x, n = lane & 15, g = lane >> 4, jr = lane / LPR, pc = lane % LPR;

  const uint32_t elem = batch / (uint32_t)p.heads, head = batch % (uint32_t)p.heads;
  uint16_t *out = p.out + (int64_t)elem * p.stride_out + (int64_t)head * p.head_out + ((int64_t)row * V + n) * p.ld_out + 4 * g;
  if (beg == end) {  // a query that attends to nothing: zeros, as the product with no stored vectors gives
    if (n < V) {
#pragma unroll
      for (int u = 0; u < NT; ++u) *reinterpret_cast<uintx2 *>(out + 16 * u) = uintx2{0u, 0u};
    }
    return;
  }
  // (descriptors end with the last row's bytes; between the rows of a strided operand lies what belongs to other heads)
  const uint32_t q_row = (uint32_t)p.ld_q * 2u, k_row = (uint32_t)p.ld_k * 2u, v_row = (uint32_t)p.ld_v * 2u;
  const __amdgpu_buffer_rsrc_t srd_q = make_srd(p.q + (int64_t)elem * p.stride_q + (int64_t)head * p.head_q + (int64_t)row * V * p.ld_q,
                                                (uint32_t)(V - 1) * q_row + kRowBytes);
  // (no keys at all: descriptors of zero bytes, whatever a pattern then names reads as zeros)
  const uint32_t k_bytes = p.n_keys > 0 ? (uint32_t)(p.n_keys - 1) * k_row + kRowBytes : 0u;
  const uint32_t v_bytes = p.n_keys > 0 ? (uint32_t)(p.n_keys - 1) * v_row + kRowBytes : 0u;
  const __amdgpu_buffer_rsrc_t srd_k = make_srd(p.k + (int64_t)elem * p.stride_k + (int64_t)head * p.head_k, k_bytes);
  const __amdgpu_buffer_rsrc_t srd_v = make_srd(p.v + (int64_t)elem * p.stride_v + (int64_t)head * p.head_v, v_bytes);
  const __amdgpu_buffer_rsrc_t srd_cols = make_srd(p.col_idx, (uint32_t)end * 4u);  // past the row: reads 0

  half8 q[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c)  // (rows past V: beyond the descriptor, zeros)
    q[c] = __builtin_bit_cast(half8, __builtin_amdgcn_raw_buffer_load_b128(srd_q, n < V ? (uint32_t)n * q_row + (32u * c + 8u * g) * 2u : 0xfffffff0u, 0, 0));

  unsigned char *const k_dst = stage_k + (uint32_t)(L * jr) * kPitch + (uint32_t)pc * 16u;
  unsigned char *const v_dst = stage_v + (uint32_t)(L * jr) * kPitch + (uint32_t)pc * 16u;
  const unsigned char *const k_rd = stage_k + (uint32_t)n * kPitch + (uint32_t)g * 16u;
  const unsigned char *const v_rd = stage_v + (uint32_t)(4 * g + (n >> 2)) * kPitch + (uint32_t)(n & 3) * 8u;
  const uint32_t piece_off = (uint32_t)pc * 16u;
  const float scale2 = p.scale * 1.4426950408889634f;

  struct Head {
    uint32_t c[L];
  };
  struct Body {
    uintx4 k[L], v[L];
  };
  const auto load_head = [&](int kc) {
    Head h;
    const int at = (kc + L * jr) * 4;
    if (L == 2) {
      const uintx2 x = __builtin_bit_cast(uintx2, __builtin_amdgcn_raw_buffer_load_b64(srd_cols, at, 0, 0));
      h.c[0] = x[0]; h.c[1] = x[1];
    } else {
#pragma unroll
      for (int i = 0; i < L; i += 4) {
        const uintx4 x = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_cols, at + 4 * i, 0, 0));
#pragma unroll
        for (int e = 0; e < 4; ++e) h.c[(i + e) % L] = x[e];
      }
    }
    return h;
  };
  const auto load_body = [&](Body &b, const Head &h, int kc) {
    uint32_t ok[L], ov[L];
#pragma unroll
    for (int i = 0; i < L; ++i) {
      ok[i] = __umul24(h.c[i], k_row) + piece_off;  // (both factors below 2^24: the launcher's caller checks the row pitch)
      ov[i] = __umul24(h.c[i], v_row) + piece_off;
    }
    if (kc + 32 > end) {  // (uniform) the row's last step: slots past its end fetch zeros
#pragma unroll
      for (int i = 0; i < L; ++i) {
        const bool live = kc + L * jr + i < end;
        ok[i] = live ? ok[i] : k_bytes;
        ov[i] = live ? ov[i] : v_bytes;
      }
    }
#pragma unroll
    for (int i = 0; i < L; ++i) b.k[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_k, ok[i], 0, 0));
#pragma unroll
    for (int i = 0; i < L; ++i) b.v[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_v, ov[i], 0, 0));
  };

  floatx4 acc[NT];
#pragma unroll
  for (int u = 0; u < NT; ++u) acc[u] = floatx4{0.f, 0.f, 0.f, 0.f};
  float run_max = -INFINITY, run_sum = 0.f;  // of query n; the sum only over this lane's share of the keys

  const auto contract = [&](const Body &b, int kc) {
    // (LDS operations of a wave execute in order: these writes land behind the previous step's reads)
#pragma unroll
    for (int i = 0; i < L; ++i) *reinterpret_cast<uintx4 *>(k_dst + i * kPitch) = b.k[i];
#pragma unroll
    for (int i = 0; i < L; ++i) *reinterpret_cast<uintx4 *>(v_dst + i * kPitch) = b.v[i];
    float x[8];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const half8 a = *reinterpret_cast<const half8 *>(k_rd + (uint32_t)t * (16u * kPitch) + (uint32_t)c * 64u);
        s = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, q[c], s, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) x[4 * t + i] = s[i] * scale2;
    }
    if (kc + 32 > end) {  // (uniform)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (kc + 16 * t + 4 * g + i >= end) x[4 * t + i] = -INFINITY;
    }
    float mx = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
    mx = quad_rows_max(mx);  // finite: the step's first slot is always a stored vector
    const float new_max = fmaxf(run_max, mx);
    if (__builtin_amdgcn_ballot_w64(new_max > run_max)) {  // (uniform) some query's maximum moved
      const float alpha = __builtin_amdgcn_exp2f(run_max - new_max);
      run_sum *= alpha;
#pragma unroll
      for (int u = 0; u < NT; ++u) acc[u] *= alpha;
      run_max = new_max;
    }
    float e[8], sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      e[i] = __builtin_amdgcn_exp2f(x[i] - run_max);
      sum += e[i];
    }
    run_sum += sum;
    const half8 pb = {(_Float16)e[0], (_Float16)e[1], (_Float16)e[2], (_Float16)e[3],
                      (_Float16)e[4], (_Float16)e[5], (_Float16)e[6], (_Float16)e[7]};
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const uintx2 lo = lds_read_tr(v_rd + 32u * u);
      const uintx2 hi = lds_read_tr(v_rd + 16u * kPitch + 32u * u);
      const uintx4 a = {lo[0], lo[1], hi[0], hi[1]};
      acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), pb, acc[u], 0, 0, 0);
    }
  };

  // Column indices run two steps ahead of the arithmetic, the rows of k and v one (two sets, used alternately).
  Body b0, b1;
  Head h0 = load_head(beg), h1 = load_head(beg + 32);
  load_body(b0, h0, beg);
  int kc = beg;  // the step held in b0
  for (;;) {
    if (kc + 32 >= end) {
      contract(b0, kc);
      break;
    }
    h0 = load_head(kc + 64);
    load_body(b1, h1, kc + 32);
    contract(b0, kc);
    kc += 32;
    if (kc + 32 >= end) {
      contract(b1, kc);
      break;
    }
    h1 = load_head(kc + 64);
    load_body(b0, h0, kc + 32);
    contract(b1, kc);
    kc += 32;
  }

  const float inv = 1.0f / quad_rows_sum(run_sum);
  if (n < V) {
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const half4 h = {(_Float16)(acc[u][0] * inv), (_Float16)(acc[u][1] * inv), (_Float16)(acc[u][2] * inv), (_Float16)(acc[u][3] * inv)};
      *reinterpret_cast<uintx2 *>(out + 16 * u) = __builtin_bit_cast(uintx2, h);
    }
  }
}

template <int V>
static void launch_sparse_attention_v(const AttentionArgs &p, int F, hipStream_t stream) {
  const dim3 grid(p.per_xcd * 8u), block(64);
  if (F == 32) hipLaunchKernelGGL((sparse_attention_kernel<V, 32>), grid, block, 0, stream, p);
  else if (F == 64) hipLaunchKernelGGL((sparse_attention_kernel<V, 64>), grid, block, 0, stream, p);
  else hipLaunchKernelGGL((sparse_attention_kernel<V, 128>), grid, block, 0, stream, p);
}

hipError_t launch_sparse_attention(const AttentionArgs &a, int V, int F, hipStream_t stream) {
  if (F != 32 && F != 64 && F != 128) return hipErrorInvalidValue;
  AttentionArgs p = a;
  p.total_work = (uint32_t)a.m_vec * (uint32_t)a.batch;
  p.per_xcd = (p.total_work + 7u) / 8u;
  if (p.total_work == 0) return hipSuccess;
  if (V == 8) launch_sparse_attention_v<8>(p, F, stream);
  else launch_sparse_attention_v<16>(p, F, stream);
  return hipGetLastError();
}

}  // namespace sspmm
