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

#include "schedule.h"
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

// v_perm_b32 picks each result byte from the 8 bytes {y (bytes 4-7), x (bytes 0-3)}.
// pack_lo = low half of x | low half of y << 16; pack_hi the same with the high halves.
__device__ __forceinline__ uint32_t pack_lo(uint32_t x, uint32_t y) {
  return __builtin_amdgcn_perm(y, x, 0x05040100u);
}
__device__ __forceinline__ uint32_t pack_hi(uint32_t x, uint32_t y) {
  return __builtin_amdgcn_perm(y, x, 0x07060302u);
}

union Half8Bits {
  half8 h;
  uint32_t u[4];
};

// erf with an absolute error below 2e-7 (Abramowitz and Stegun 7.1.26): a reciprocal, an exponential and five
// multiply-adds, where the library's erff spends three times as many instructions on bits an fp16 result drops.
__device__ __forceinline__ float erf_fast(float x) {
  const float ax = __builtin_fabsf(x);
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, ax, 1.0f));
  float poly = __builtin_fmaf(1.061405429f, t, -1.453152027f);
  poly = __builtin_fmaf(poly, t, 1.421413741f);
  poly = __builtin_fmaf(poly, t, -0.284496736f);
  poly = __builtin_fmaf(poly, t, 0.254829592f);
  const float e = __builtin_amdgcn_exp2f(-1.4426950408889634f * ax * ax);
  return __builtin_copysignf(__builtin_fmaf(-poly * t, e, 1.0f), x);
}
// The linear-layer epilogue on one fp32 sum: bias, then the activation (1 = GELU, 0.5 x (1 + erf(x / sqrt 2))).
__device__ __forceinline__ float epilogue_value(float x, float bias, int act) {
  x += bias;
  if (act == 1) x = 0.5f * x * (1.0f + erf_fast(x * 0.70710678118654752f));
  return x;
}
__device__ __forceinline__ bool has_epilogue(const SpmmArgs &p) { return p.bias != nullptr || p.act != 0; }
__device__ __forceinline__ float bias_of_row(const SpmmArgs &p, int64_t out_row) {
  return p.bias ? (float)reinterpret_cast<const _Float16 *>(p.bias)[out_row] : 0.0f;
}

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
    // (non-temporal: the rows of B the grid keeps gathering stay in the L2; measured 1-10 % on fp16 outputs.  fp32
    // tiles of 128 columns do not come through here: they go out as whole lines, see store_tile_f32_lines)
    __builtin_nontemporal_store(h, reinterpret_cast<half8 *>(p));
  }
};

template <typename OutT, int CPL>
struct StoreRow;
template <typename OutT>
struct StoreRow<OutT, 8> {
  static __device__ __forceinline__ void run(OutT *p, const float (&v)[8]) { Store8<OutT>::run(p, v); }
};
template <>
struct StoreRow<float, 4> {
  static __device__ __forceinline__ void run(float *p, const float (&v)[4]) {
    *reinterpret_cast<floatx4 *>(p) = floatx4{v[0], v[1], v[2], v[3]};
  }
};
template <>
struct StoreRow<_Float16, 4> {
  static __device__ __forceinline__ void run(_Float16 *p, const float (&v)[4]) {
    typedef _Float16 half4v __attribute__((ext_vector_type(4)));
    const half4v h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};  // round to nearest even
    *reinterpret_cast<half4v *>(p) = h;
  }
};

// The value tile of a step: 32 vectors x V halfs as they lie in memory (vector-major), written to LDS with one
// 8- or 16-byte store per lane and read back as the MFMA operand (lane (v, g): k = 8g .. 8g+7 of row v) by two
// ds_read_b64_tr_b16.  The V = 8 transpose read touches 16 bytes past its 512.
static constexpr int val_tile_bytes(int V) { return V == 8 ? 528 : 1024; }

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;

// The same read at an absolute LDS byte address (saves adding the base of the dynamic LDS array,
// which the compiler does not fold, to every address).
__device__ __forceinline__ uintx2 lds_read_tr_abs(uint32_t lds_addr) {
  const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4 *)(uintptr_t)lds_addr);
  return __builtin_bit_cast(uintx2, v);
}
__device__ __forceinline__ uint32_t lds_address(const unsigned char *p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char *)p;
}
__device__ __forceinline__ uintx2 lds_read_tr(const unsigned char *lds_base, uint32_t byte_off) {
  const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4 *)(lds_base + byte_off));
  return __builtin_bit_cast(uintx2, v);
}

template <int V>
struct SlabVals;  // the 32 x V halfs of a step, spread over the 64 lanes
template <>
struct SlabVals<8> {
  typedef uintx2 type;  // 8 bytes per lane
  static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t srd, uint32_t off) {
    return __builtin_bit_cast(uintx2, __builtin_amdgcn_raw_buffer_load_b64(srd, off, 0, 0));
  }
};
template <>
struct SlabVals<16> {
  typedef uintx4 type;  // 16 bytes per lane
  static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t srd, uint32_t off) {
    return __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd, off, 0, 0));
  }
};

// One chunk = 32 consecutive non-zero vectors of a vector-row.  Its loads form a chain of two
// memory round trips (column indices, then the rows of B they name), so they are issued in two
// stages, one step apart: while chunk s is contracted, the gathers of chunk s + 1 and the column
// indices of chunk s + 2 are in flight.
// SHARED_COLS: the column indices come as one dword per lane and the lanes that need one fetch it from there with a
// lane permute (the address unit takes sixteen cycles for a load instruction of a wave whatever it carries: the
// eight indices a lane needs, loaded by the lane itself, cost two of them).  Pays where that unit bounds the kernel
// (one wave per vector-row, many in flight); where a single long row is the critical path (the split-row kernel)
// the permutes' latency costs more than the instruction saves.
template <int V, bool SHARED_COLS = true>
struct ChunkHead {   // stage 1: what does not depend on other loads
  uint32_t cols;     // SHARED_COLS: column index of k slot lane % 32
  uintx4 c0, c1;     // otherwise: column indices of k slots 8g .. 8g+7
  typename SlabVals<V>::type vraw;  // the lane's share of the chunk's 32 x V values, as they lie in memory
  int kc;            // first vector of the chunk
};
// CPL = columns per lane: 8 (a wave covers 128 columns) or, for narrow right-hand sides such as attention heads
// of 64 features, 4 (64 columns: all sixteen lanes of a row group stay useful).
template <int CPL>
struct ChunkRaw;
template <>
struct ChunkRaw<8> {
  typedef uintx4 type;
  static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t srd, uint32_t off) {
    return __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd, off, 0, 0));
  }
};
template <>
struct ChunkRaw<4> {
  typedef uintx2 type;
  static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t srd, uint32_t off) {
    return __builtin_bit_cast(uintx2, __builtin_amdgcn_raw_buffer_load_b64(srd, off, 0, 0));
  }
};
template <int CPL = 8>
struct Chunk {
  typename ChunkRaw<CPL>::type raw[8];  // raw[j] = CPL halfs (columns n0+CPL*m..) of the row of B named by k slot 8g+j
};

template <int V, bool SHARED_COLS>
__device__ __forceinline__ void load_head(ChunkHead<V, SHARED_COLS> &h, int kc, int g, __amdgpu_buffer_rsrc_t srd_cols,
                                          __amdgpu_buffer_rsrc_t srd_vals, uint32_t vals_lane_off) {
  h.kc = kc;
  // srd_cols / srd_vals end at this vector-row's last vector: slots past it read as zero.
  if (SHARED_COLS) {
    h.cols = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(srd_cols, (kc + (int)(threadIdx.x & 31)) * 4, 0, 0);
  } else {
    const int kb = kc + 8 * g;
    h.c0 = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_cols, kb * 4, 0, 0));
    h.c1 = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_cols, kb * 4 + 16, 0, 0));
  }
  // one coalesced load of the chunk's values (vals_lane_off = lane * V bytes); vectors past the row read as zero
  h.vraw = SlabVals<V>::load(srd_vals, (uint32_t)kc * (V * 2) + vals_lane_off);
}

// (also sends the chunk's values to the value tile `tile_lane` points into: the lane's slot of the tile)
template <int CPL, int V, bool SHARED_COLS>
__device__ __forceinline__ void load_body(Chunk<CPL> &c, const ChunkHead<V, SHARED_COLS> &h, int end, int g, __amdgpu_buffer_rsrc_t srd_b,
                                          uint32_t lane_n2, uint32_t lane_col_off, uint32_t b_bytes,
                                          unsigned char *tile_lane) {
  const int kb = h.kc + 8 * g;
  uint32_t off[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t col = SHARED_COLS ? (uint32_t)__builtin_amdgcn_ds_bpermute((8 * g + j) * 4, (int)h.cols)
                                     : (j < 4 ? h.c0[j] : h.c1[j - 4]);
    off[j] = __umul24(col, lane_n2) + lane_col_off;
  }
  if (h.kc + 32 > end) {  // wave-uniform: only the last chunk of a vector-row can be partial
#pragma unroll
    for (int j = 0; j < 8; ++j) off[j] = (kb + j < end) ? off[j] : b_bytes;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    c.raw[j] = ChunkRaw<CPL>::load(srd_b, off[j]);
  }
  *reinterpret_cast<typename SlabVals<V>::type *>(tile_lane) = h.vraw;
}

// tile_op: the lane's address for the transpose reads of the chunk's value tile
template <int CPL, int V>
__device__ __forceinline__ void mac_chunk(const Chunk<CPL> &c, floatx4 (&acc)[CPL], const unsigned char *tile_op) {
  Half8Bits a;
  {
    const uintx2 lo = lds_read_tr(tile_op, 0);
    const uintx2 hi = lds_read_tr(tile_op, 4u * (V * 2u));
    a.u[0] = lo[0]; a.u[1] = lo[1]; a.u[2] = hi[0]; a.u[3] = hi[1];
  }
#pragma unroll
  for (int q = 0; q < CPL; ++q) {
    Half8Bits b;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t x = c.raw[2 * d][q >> 1], y = c.raw[2 * d + 1][q >> 1];
      b.u[d] = (q & 1) ? pack_hi(x, y) : pack_lo(x, y);
    }
    acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.h, b.h, acc[q], 0, 0, 0);
  }
}

// fp32 rows of 128 columns: a lane's eight columns are 32 bytes, so a store instruction of the layout the MFMAs
// leave would write 16-byte pieces 32 bytes apart.  The V x 128 tile passes through LDS instead (`ctile`, private to
// the wave: LDS operations of a wave execute in order, no barrier) and goes out as whole lines, two rows of 512
// bytes per instruction, non-temporal.  Launches of few vectors per row are mostly these stores: measured up to
// 2.2x at 95-98 % sparsity, 0.85-0.9x the time over a sweep of shapes at 90 %.
// acc[q][rr] = C[row 4g + rr][column 8m + q] of the tile; crow = the tile's first row of C, at column 0.
template <int V>
__device__ __forceinline__ void store_tile_f32_lines(float (*ctile)[128 + 4], const floatx4 (&acc)[8], int lane, float *crow,
                                                     int N, int tile) {
  const int m = lane & 15, g = lane >> 4;
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int v = 4 * g + rr;
    if (v < V) {
      *reinterpret_cast<floatx4 *>(&ctile[v][8 * m]) = floatx4{acc[0][rr], acc[1][rr], acc[2][rr], acc[3][rr]};
      *reinterpret_cast<floatx4 *>(&ctile[v][8 * m + 4]) = floatx4{acc[4][rr], acc[5][rr], acc[6][rr], acc[7][rr]};
    }
  }
  const int c4 = (lane & 31) * 4, gcol = tile * 128 + c4;
  if (gcol < N) {
#pragma unroll
    for (int i = 0; i < V / 2; ++i) {
      const int v = 2 * i + (lane >> 5);
      const floatx4 x = *reinterpret_cast<const floatx4 *>(&ctile[v][c4]);
      __builtin_nontemporal_store(x, reinterpret_cast<floatx4 *>(crow + (int64_t)v * N + gcol));
    }
  }
}

// WPE: waves per SIMD the register allocation aims at.  The loop fits 168 registers, three waves per SIMD, without
// spilling; a launch with more waves than two per SIMD can hold at once runs 6-8 % faster that way (more gathers in
// flight per CU), one that fits anyway runs level or a few per cent slower, so the launcher picks by the grid.
// (Three chunk buffers in rotation, two chunks of gathers in flight per wave, were measured as well: 15-30 % slower.)
template <int V, typename OutT, int CPL, int WPE = 2>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void spmm_gather_kernel(const SpmmArgs p) {
  __shared__ __align__(16) unsigned char val_tiles[2][val_tile_bytes(V)];  // the value tiles of two chunks in turn
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

  const int ncol = (int)tile * (16 * CPL) + m * CPL;
  const bool col_ok = ncol < p.N;
  // Lanes whose columns lie beyond N aim every gather at the first byte past B.
  const uint32_t lane_n2 = col_ok ? (uint32_t)p.N * 2u : 0u;
  const uint32_t lane_col_off = col_ok ? (uint32_t)ncol * 2u : b_bytes;
  constexpr uint32_t kLaneBytes = V * 2u * 32u / 64u;
  const uint32_t vals_lane_off = (uint32_t)lane * kLaneBytes;
  // where the lane writes its share of a value tile, and where its transpose reads start (rows 8g + m/4 of the tile)
  unsigned char *const tw0 = val_tiles[0] + lane * kLaneBytes, *const tw1 = val_tiles[1] + lane * kLaneBytes;
  const uint32_t a_off = (uint32_t)(8 * g + (m >> 2)) * (V * 2u) + (uint32_t)(m & 3) * 8u;
  const unsigned char *const tr0 = val_tiles[0] + a_off, *const tr1 = val_tiles[1] + a_off;

  floatx4 acc[CPL];
#pragma unroll
  for (int q = 0; q < CPL; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the bias of the lane's four output rows, fetched before the loop so that the row's end does not wait for it
  _Float16 bias4[4] = {0, 0, 0, 0};
  if (p.bias) {
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) bias4[rr] = reinterpret_cast<const _Float16 *>(p.bias)[(int64_t)row * V + ((4 * g + rr) & (V - 1))];
  }

  if (beg < end) {
    // Heads run two chunks ahead of the arithmetic, bodies one (two buffers of each, used alternately).
    // A head past the end of the row reads zeros and is never turned into a body.
    ChunkHead<V> h0, h1;
    Chunk<CPL> c0, c1;
    load_head(h0, beg, g, srd_cols, srd_vals, vals_lane_off);
    load_head(h1, beg + 32, g, srd_cols, srd_vals, vals_lane_off);
    load_body(c0, h0, end, g, srd_b, lane_n2, lane_col_off, b_bytes, tw0);
    int kc = beg + 32;  // first vector of the chunk whose body is loaded next
    for (;;) {
      if (kc >= end) {
        mac_chunk<CPL, V>(c0, acc, tr0);
        break;
      }
      load_head(h0, kc + 32, g, srd_cols, srd_vals, vals_lane_off);
      load_body(c1, h1, end, g, srd_b, lane_n2, lane_col_off, b_bytes, tw1);
      mac_chunk<CPL, V>(c0, acc, tr0);
      kc += 32;
      if (kc >= end) {
        mac_chunk<CPL, V>(c1, acc, tr1);
        break;
      }
      load_head(h1, kc + 32, g, srd_cols, srd_vals, vals_lane_off);
      load_body(c0, h0, end, g, srd_b, lane_n2, lane_col_off, b_bytes, tw0);
      mac_chunk<CPL, V>(c1, acc, tr1);
      kc += 32;
    }
  }

  if (has_epilogue(p)) {  // (uniform) acc[q][rr] belongs to output row 4g + rr of the vector-row
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
#pragma unroll
      for (int q = 0; q < CPL; ++q) acc[q][rr] = epilogue_value(acc[q][rr], (float)bias4[rr], p.act);
    }
  }
  if constexpr (std::is_same<OutT, float>::value && CPL == 8) {
    __shared__ __align__(16) float ctile[V][128 + 4];
    store_tile_f32_lines<V>(ctile, acc, lane, reinterpret_cast<float *>(p.C) + (int64_t)batch * p.stride_C + (int64_t)row * V * p.N,
                            p.N, (int)tile);
  } else if (col_ok) {
    OutT *cbase = reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int v = 4 * g + rr;
      if (v < V) {
        float o[CPL];
#pragma unroll
        for (int q = 0; q < CPL; ++q) o[q] = acc[q][rr];
        StoreRow<OutT, CPL>::run(cbase + ((int64_t)row * V + v) * p.N + ncol, o);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Gather kernel for wide matrices (K above kSplitMinK), where a vector-row may hold thousands of
// vectors: the merged rows of an unstructured matrix with power-law row lengths do, and one wave
// per vector-row would keep a few waves busy long after the rest of the grid has drained.
//
// A workgroup of kSplitWaves waves owns as many consecutive vector-rows of one 128-column tile.
// Each wave computes and stores its own row as the kernel above does, unless the row has more
// than kLongRowSteps steps.  Such a row is left for a second phase in which all waves of the
// group take a contiguous share of its steps and add their partial tiles up in LDS in wave order,
// so the result does not depend on timing.  Every wave reads the extents of all rows of its group,
// so a group without a long row never meets at a barrier.
static constexpr int kSplitWaves = 4;
static constexpr int kLongRowSteps = 16;
static constexpr int kSplitMinK = 4096;

// The partial V x 128 tile of vectors [beg, sub_end) of a vector-row that ends at `end`.
template <int V>
__device__ __forceinline__ void gather_accumulate(floatx4 (&acc)[8], const SpmmArgs &p, uint32_t batch, int beg,
                                                  int sub_end, int end, int lane, int ncol, bool col_ok,
                                                  unsigned char (*val_tiles)[val_tile_bytes(V)]) {
  const int m = lane & 15, g = lane >> 4;
  const uint16_t *vals = p.values + (int64_t)batch * p.stride_values;
  const uint16_t *bmat = p.B + (int64_t)batch * p.stride_B;
  const uint32_t b_bytes = (uint32_t)p.K * (uint32_t)p.N * 2u;
  const __amdgpu_buffer_rsrc_t srd_cols = make_srd(p.col_idx, (uint32_t)end * 4u);
  const __amdgpu_buffer_rsrc_t srd_vals = make_srd(vals, (uint32_t)end * (V * 2u));
  const __amdgpu_buffer_rsrc_t srd_b = make_srd(bmat, b_bytes);
  const uint32_t lane_n2 = col_ok ? (uint32_t)p.N * 2u : 0u;
  const uint32_t lane_col_off = col_ok ? (uint32_t)ncol * 2u : b_bytes;
  constexpr uint32_t kLaneBytes = V * 2u * 32u / 64u;
  const uint32_t vals_lane_off = (uint32_t)lane * kLaneBytes;
  unsigned char *const tw0 = val_tiles[0] + lane * kLaneBytes, *const tw1 = val_tiles[1] + lane * kLaneBytes;
  const uint32_t a_off = (uint32_t)(8 * g + (m >> 2)) * (V * 2u) + (uint32_t)(m & 3) * 8u;
  const unsigned char *const tr0 = val_tiles[0] + a_off, *const tr1 = val_tiles[1] + a_off;
#pragma unroll
  for (int q = 0; q < 8; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};
  if (beg >= sub_end) return;
  ChunkHead<V, false> h0, h1;
  Chunk<8> c0, c1;
  load_head(h0, beg, g, srd_cols, srd_vals, vals_lane_off);
  load_head(h1, beg + 32, g, srd_cols, srd_vals, vals_lane_off);
  load_body(c0, h0, end, g, srd_b, lane_n2, lane_col_off, b_bytes, tw0);
  int kc = beg + 32;  // first vector of the chunk whose body is loaded next
  for (;;) {
    if (kc >= sub_end) {
      mac_chunk<8, V>(c0, acc, tr0);
      break;
    }
    load_head(h0, kc + 32, g, srd_cols, srd_vals, vals_lane_off);
    load_body(c1, h1, end, g, srd_b, lane_n2, lane_col_off, b_bytes, tw1);
    mac_chunk<8, V>(c0, acc, tr0);
    kc += 32;
    if (kc >= sub_end) {
      mac_chunk<8, V>(c1, acc, tr1);
      break;
    }
    load_head(h1, kc + 32, g, srd_cols, srd_vals, vals_lane_off);
    load_body(c0, h0, end, g, srd_b, lane_n2, lane_col_off, b_bytes, tw0);
    mac_chunk<8, V>(c1, acc, tr1);
    kc += 32;
  }
}

template <int V, typename OutT>
__global__ __launch_bounds__(64 * kSplitWaves) void spmm_gather_split_kernel(const SpmmArgs p) {
  __shared__ floatx4 part[4][2][64];  // the tile being added up: part[rr][half][lane] = acc[4 * half .. + 3][rr]
  __shared__ __align__(16) unsigned char val_tiles_all[kSplitWaves][2][val_tile_bytes(V)];  // per wave: value tiles of two chunks
  const uint32_t id = blockIdx.x;
  const uint32_t w = (id & 7u) * p.per_xcd + (id >> 3);
  if (w >= p.total_work) return;
  const uint32_t n_groups = ((uint32_t)p.m_vec + kSplitWaves - 1u) / kSplitWaves;
  const uint32_t grp = w % n_groups;
  const uint32_t t = w / n_groups;
  const uint32_t tile = t % p.n_tiles;
  const uint32_t batch = t / p.n_tiles;

  const int lane = threadIdx.x & 63, m = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  // the rows of the group and their extents (the same in every wave)
  int g_row[kSplitWaves], g_beg[kSplitWaves], g_end[kSplitWaves];
  bool any_long = false;
#pragma unroll
  for (int j = 0; j < kSplitWaves; ++j) {
    const int rj = (int)grp * kSplitWaves + j;
    const bool have = rj < p.m_vec;
    g_row[j] = have ? (p.row_indices ? p.row_indices[rj] : rj) : -1;
    g_beg[j] = have ? p.row_offsets[g_row[j]] : 0;
    g_end[j] = have ? p.row_offsets[g_row[j] + 1] : 0;
    any_long = any_long || (g_end[j] - g_beg[j] > 32 * kLongRowSteps);
  }
  int row = -1, beg = 0, end = 0;
#pragma unroll
  for (int j = 0; j < kSplitWaves; ++j)
    if (j == wave) {
      row = g_row[j];
      beg = g_beg[j];
      end = g_end[j];
    }
  const bool is_long = end - beg > 32 * kLongRowSteps;
  const int ncol = (int)tile * 128 + m * 8;
  const bool col_ok = ncol < p.N;
  OutT *cbase = reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C;

  floatx4 acc[8];
  if (row >= 0 && !is_long) {
    gather_accumulate<V>(acc, p, batch, beg, end, end, lane, ncol, col_ok, val_tiles_all[wave]);
    if constexpr (std::is_same<OutT, float>::value) {
      __shared__ __align__(16) float ctile_all[kSplitWaves][V][128 + 4];
      store_tile_f32_lines<V>(ctile_all[wave], acc, lane, reinterpret_cast<float *>(cbase) + (int64_t)row * V * p.N, p.N, (int)tile);
    } else if (col_ok) {
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
  if (!any_long) return;  // uniform over the workgroup
  // (one copy of the loop body: the extents are read again rather than indexed out of registers)
#pragma nounroll
  for (int j = 0; j < kSplitWaves; ++j) {
    const int rj = (int)grp * kSplitWaves + j;
    if (rj >= p.m_vec) break;
    const int lrow = p.row_indices ? p.row_indices[rj] : rj;
    const int lbeg = p.row_offsets[lrow], lend = p.row_offsets[lrow + 1];
    if (lend - lbeg <= 32 * kLongRowSteps) continue;  // uniform over the workgroup
    const int steps = (lend - lbeg + 31) >> 5;
    const int per = (steps + kSplitWaves - 1) / kSplitWaves;
    const int my_beg = min(lend, lbeg + wave * per * 32);
    const int my_end = min(lend, my_beg + per * 32);
    gather_accumulate<V>(acc, p, batch, my_beg, my_end, lend, lane, ncol, col_ok, val_tiles_all[wave]);
    for (int turn = 0; turn < kSplitWaves; ++turn) {
      if (wave == turn) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            floatx4 x = {acc[4 * h][rr], acc[4 * h + 1][rr], acc[4 * h + 2][rr], acc[4 * h + 3][rr]};
            if (turn > 0) x = part[rr][h][lane] + x;
            part[rr][h][lane] = x;
          }
      }
      __syncthreads();
    }
    if (col_ok && wave < 4) {  // wave rr stores output row 4g + rr
      const int v = 4 * g + wave;
      if (v < V) {
        const floatx4 lo = part[wave][0][lane], hi = part[wave][1][lane];
        const float o[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        Store8<OutT>::run(cbase + ((int64_t)lrow * V + v) * p.N + ncol, o);
      }
    }
    __syncthreads();  // part is rewritten for the next long row
  }
}

// ------------------------------------------------------------------------------------------
// Slab kernel: B resident in LDS, operands formed by LDS transpose reads.
//
// When K is small enough that a 64-column slab of B (K rows x 128 bytes) fits in the 160 KB of
// LDS, a workgroup copies the slab into LDS with coalesced 16-byte loads and then walks a block of
// vector-rows against it, so HBM/L2 only see each slab once per row block, the value vectors, the
// column indices and the stores of C.
//
// The kernel is persistent: one workgroup of 16 waves per CU walks a list of work items
// (slab, row block).  Where two slabs fit in LDS the next item's slab and row table are fetched
// into registers while the current item is computed and are written to the other LDS buffer when
// the item is done, so the copy of B never stalls the CU after its first item; larger K runs the
// same loop with one buffer.  Items that follow each other on the same slab reuse it.
//
// ds_read_b64_tr_b16 is what makes the inner loop cheap.  Within 16 lanes, lane n receives element n of the
// four 32-byte runs addressed by lanes 0-3, 4-7, 8-11, 12-15: four rows that are contiguous in the
// column direction come back as "four k of one column", which is the MFMA operand layout.  Per
// step of 32 vectors a wave therefore issues
//   * 2 transpose reads of its value tile (32 vectors x V halfs, written to LDS with one
//     16-byte store per lane from one coalesced 16-byte global load per lane), and
//   * 8 transpose reads of the slab (two k halves x four 16-column tiles), addressed by just
//     two column indices per lane,
// and 4 MFMAs, with no byte shuffling in registers.  A 16-lane group of a slab read touches four
// different rows of B at the same column offset; the 32-byte segments of slab row c are stored
// XOR-swizzled by (c >> 1) & 3 so that those rows spread over the LDS banks.
// The waves claim the vector-rows of a row block one at a time, and the loads of a step are
// issued a few steps ahead (across vector-row boundaries).  Row K of the slab is all
// zeros: unused k slots of a partial step point there.
static constexpr int kSlabWaves = 16;
static constexpr int kSlabThreads = kSlabWaves * 64;
// A slab is NQ tiles of 16 columns wide: 4 (64 columns, 128-byte rows) where K lets it fit in LDS, 2 (32 columns,
// 64-byte rows) for matrices up to twice as tall, 8 (128 columns, 256-byte rows, one buffer) for K up to about 570.
static constexpr int slab_row_bytes(int NQ) { return 32 * NQ; }
// How a 64-column slab lies in LDS.  With 128-byte rows the 32-byte segments of a row are XOR-swizzled (see
// slab_unit_dst) and every read address needs the swizzle applied in registers; where LDS allows, rows are padded
// instead, which spreads the banks the same way and leaves the four tiles of a row at the immediate offsets
// 0 / 32 / 64 / 96 of one address: a dozen vector-ALU instructions fewer per step, in a loop whose speed follows
// its instruction count.  Padded and double-buffered, the rows of the two slabs alternate (A, B, 32 bytes of
// padding: 288 bytes per row pair), which costs no more LDS than two unpadded slabs plus the padding.
enum SlabLayout { kXorSingle = 0, kXorDouble = 1, kPadSingle = 2, kPadDouble = 3 };
static constexpr bool layout_double(int L) { return L == kXorDouble || L == kPadDouble; }
static constexpr bool layout_pad(int L) { return L == kPadSingle || L == kPadDouble; }
static constexpr uint32_t layout_row_bytes(int L, int NQ) { return L == kPadSingle ? 160u : L == kPadDouble ? 288u : 32u * NQ; }
// bytes of LDS taken by the slab(s), K rows and the zero row
static constexpr uint32_t layout_slab_region(int L, int NQ, uint32_t rows) {
  return rows * layout_row_bytes(L, NQ) * (L == kXorDouble ? 2u : 1u);
}
// offset of buffer `sel` (0 / 1) inside the region
static constexpr uint32_t layout_buffer_off(int L, int NQ, uint32_t rows, uint32_t sel) {
  return L == kPadDouble ? sel * 128u : sel * rows * layout_row_bytes(L, NQ);
}
// Per-wave LDS: the value tile of a step (32 vectors x V halfs; the V = 8 transpose read touches 16
// bytes past its 512).
static constexpr int wave_lds_bytes(int V) { return val_tile_bytes(V); }

// steps whose loads are in flight or waiting in registers (bounded by the 128 registers a lane has
// with 16 waves per CU)
static constexpr int slab_ring(int V) { return V == 8 ? 6 : 5; }

template <int V>
struct SlabLoads {    // what the head records for a step; the step consumes it slab_ring(V) - 1 steps later
  uint32_t col[2];    // column index of k slots 8g + m/4 and 8g + 4 + m/4
  typename SlabVals<V>::type vraw;
  int row, left;      // (wave-uniform) vector-row and its vectors from this step on
  int valid;          // (wave-uniform) 0 once the wave has run out of steps
};

// Walks one wave's sequence of steps.  The (vector-row, first vector, end vector) triples of the
// row block are copied into a table in LDS when the workgroup starts, and the waves claim its
// positions one at a time from a counter in LDS: the waves of a workgroup do not run at the same
// speed (the older waves of a SIMD win the arbitration for the memory pipeline, and finish a
// fixed share of rows a third sooner than the younger ones), so a fixed deal of rows would leave
// the fast waves idle at the end of every item.  A vector-row of n vectors is ceil(n / 32) steps,
// and an empty vector-row is one step without vectors (its zeros still have to be written).  The
// cursor runs slab_ring(V) - 1 steps ahead of the arithmetic: it issues the loads of a step and
// records the step's vector-row and length in the ring slot that receives them.  Both LDS round
// trips behind a new row are off the critical path: the claim of a position is issued two rows
// ahead and the read of its table entry one row ahead.
typedef int intx4 __attribute__((ext_vector_type(4)));
struct SlabCursor {
  int row, kc, end;  // current step: vectors [kc, min(kc + 32, end)) of vector-row `row`
  int valid;  // flags are ints: wave-uniform 0 / 1 that stay in scalar registers
  intx4 next;        // table entry of the following vector-row (still in vector registers)
  int claim;         // what the counter returned for the row after that (still in a vector register)
};

struct SlabRows {      // what the cursors need to find rows
  const intx4 *table;  // LDS: n_rows entries (row, first vector, end vector, 1) and an all-zero entry behind them
  int *counter;        // LDS: the number of positions claimed so far (in the entry behind the table's last)
  int n_rows, lane;
};

// Lane 0 takes the next position (the append instruction that would do it for a whole wave addresses only the
// first 64 KB of LDS, and the tables lie above that).
// (`spent` is a value the caller no longer needs: what the other lanes return, so that no register has to be cleared)
__device__ __forceinline__ int cursor_claim(const SlabRows &rows, int spent) {
  int t = spent;
  if (rows.lane == 0) t = __hip_atomic_fetch_add(rows.counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  return t;
}

__device__ __forceinline__ void cursor_prefetch(SlabCursor &c, const SlabRows &rows) {
  const int idx = __builtin_amdgcn_readfirstlane(c.claim);
  c.next = rows.table[min(idx, rows.n_rows)];  // positions beyond the block read the all-zero entry: not valid
  c.claim = cursor_claim(rows, c.claim);
}

__device__ __forceinline__ void cursor_take_next(SlabCursor &c, const SlabRows &rows) {
  c.row = __builtin_amdgcn_readfirstlane(c.next[0]);
  c.kc = __builtin_amdgcn_readfirstlane(c.next[1]);
  c.end = __builtin_amdgcn_readfirstlane(c.next[2]);
  c.valid = __builtin_amdgcn_readfirstlane(c.next[3]);
  cursor_prefetch(c, rows);
}

__device__ __forceinline__ void cursor_advance(SlabCursor &c, const SlabRows &rows) {
  c.kc += 32;
  if (c.kc >= c.end) cursor_take_next(c, rows);
}

template <int V>
__device__ __forceinline__ void slab_issue(SlabLoads<V> &r, int row, int kc, int end, int valid, int lane, uint32_t slot0,
                                           __amdgpu_buffer_rsrc_t srd_cols, const uint16_t *vals) {
  r.row = row;
  r.left = end - kc;
  r.valid = valid;
  r.col[0] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(srd_cols, (kc + (int)slot0) * 4, 0, 0);
  r.col[1] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(srd_cols, (kc + (int)slot0) * 4 + 16, 0, 0);
  // The value descriptor ends with the vector-row: vectors past it read as zero.
  const __amdgpu_buffer_rsrc_t srd_vals = make_srd(vals, (uint32_t)end * (V * 2u));
  constexpr uint32_t kLaneBytes = V * 2u * 32u / 64u;
  r.vraw = SlabVals<V>::load(srd_vals, (uint32_t)kc * (V * 2u) + (uint32_t)lane * kLaneBytes);
}

// The store of one 16-byte piece of C per lane.  A wave's vector-memory counter counts loads and
// stores together and guarantees order only within each kind, so a compiler that sees a store in
// flight must drain the whole counter wherever the wave waits for a load; that would serialise
// every step of the main loop behind its own loads.  The store is therefore issued from inline
// assembly, which keeps it out of the compiler's count: the waits it computes for the loads of the
// ring are then "at most n operations outstanding" with n the number of younger loads.  Loads
// return in order among themselves, so while an awaited load is outstanding so are its n younger
// loads, and the wait cannot pass early whatever the stores do; stores in flight only make it
// pass later.  The trailing s_nop covers the cycles in which the store still reads its data registers.
__device__ __forceinline__ void slab_store_line(uintx4 line, __amdgpu_buffer_rsrc_t srd, uint32_t voff, uint32_t soff) {
  asm volatile("buffer_store_dwordx4 %0, %1, %2, %3 offen nt\n\ts_nop 1" ::"v"(line), "v"(voff), "s"(srd), "s"(soff));
}

// Writing a finished V x 64 tile of C.  The MFMAs run with the slab as their first operand, so
// accumulator q of lane (m, g) holds C[row m][n0 + 16q + 4g .. + 3]: four consecutive columns of
// one row.  Lanes are then regrouped in registers so that each lane owns 16 contiguous bytes and a
// store instruction writes whole 128-byte lines:
//   * fp32: the 16 bytes are the lane's own four columns.  With V = 8 only lanes m < 8 hold rows;
//     lanes m >= 8 take tile q + 1 of row m - 8 (a DPP shift by 8 inside the 16-lane row), so one
//     instruction writes 8 rows x (64 + 64) bytes.  With V = 16 the same exchange runs in both
//     directions and two instructions write rows 0..7 and 8..15.
//   * fp16: a lane's four columns are 8 bytes; v_permlane16_swap pairs lane groups g and g + 1 of
//     two tiles so that a lane owns eight consecutive columns, then the DPP exchange as above
//     gathers all four tiles of a row into one instruction.
template <int V, typename OutT, int NQ>
struct SlabStore;
// Lanes whose columns lie beyond N carry this offset instead of a mask: it is outside every buffer the kernel is
// launched on (C of one batch element is at most 2 GiB), and the hardware drops stores outside the buffer.  The
// stores of a tile then need no branch and no change of the execution mask.
static constexpr uint32_t kSlabDropStore = 0x80000000u;

__device__ __forceinline__ uint32_t dpp_from_m_minus_8(uint32_t keep, uint32_t src) {  // lanes m >= 8 take src of lane m - 8
  return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)src, 0x118, 0xf, 0xc, false);
}
__device__ __forceinline__ uint32_t dpp_from_m_plus_8(uint32_t keep, uint32_t src) {  // lanes m < 8 take src of lane m + 8
  return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)src, 0x108, 0xf, 0x3, false);
}

template <int V, int NQ>
struct SlabStore<V, float, NQ> {
  uint32_t voff[V / 8][NQ / 2];         // byte offset of the lane's 16 bytes per row half and tile pair
  __device__ __forceinline__ void init(int lane, int n0, int N) {
    const int m = lane & 15, g = lane >> 4;
#pragma unroll
    for (int h = 0; h < V / 8; ++h) {
      const int row = 8 * h + (m & 7);
      const int tile = h == 0 ? (m >> 3) : 1 - (m >> 3);
#pragma unroll
      for (int qp = 0; qp < NQ / 2; ++qp) {
        const int col = n0 + 32 * qp + 16 * tile + 4 * g;
        voff[h][qp] = col < N ? ((uint32_t)row * (uint32_t)N + (uint32_t)col) * 4u : kSlabDropStore;
      }
    }
  }
  __device__ __forceinline__ void store(const floatx4 (&acc)[NQ], __amdgpu_buffer_rsrc_t srd, uint32_t crow) const {
#pragma unroll
    for (int qp = 0; qp < NQ / 2; ++qp) {
#pragma unroll
      for (int h = 0; h < V / 8; ++h) {
        uintx4 line;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // (copied to scalars first: a bit cast applied directly to a vector element reads element 0)
          const float fx = acc[2 * qp][r], fy = acc[2 * qp + 1][r];
          const uint32_t x = __builtin_bit_cast(uint32_t, fx), y = __builtin_bit_cast(uint32_t, fy);
          line[r] = h == 0 ? dpp_from_m_minus_8(x, y) : dpp_from_m_plus_8(x, y);
        }
        slab_store_line(line, srd, voff[h][qp], crow);
      }
    }
  }
};

template <int V>
struct SlabStore<V, _Float16, 4> {
  uint32_t voff[V / 8];
  __device__ __forceinline__ void init(int lane, int n0, int N) {
    const int m = lane & 15, g = lane >> 4;
#pragma unroll
    for (int h = 0; h < V / 8; ++h) {
      const int row = 8 * h + (m & 7);
      const int pair = h == 0 ? (m >> 3) : 1 - (m >> 3);
      const int col = n0 + 32 * pair + 16 * (g & 1) + 8 * (g >> 1);
      voff[h] = col < N ? ((uint32_t)row * (uint32_t)N + (uint32_t)col) * 2u : kSlabDropStore;
    }
  }
  __device__ __forceinline__ void store(const floatx4 (&acc)[4], __amdgpu_buffer_rsrc_t srd, uint32_t crow) const {
    // pr[pair][0..3]: after the swaps, lane (m, g) holds columns 8 * (g >> 1) .. + 7 of tile
    // 2 * pair + (g & 1), row m
    uint32_t pr[2][4];
#pragma unroll
    for (int pair = 0; pair < 2; ++pair) {
      uint32_t pk[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          typedef _Float16 half2v __attribute__((ext_vector_type(2)));
          const half2v hv = {(_Float16)acc[2 * pair + t][2 * w], (_Float16)acc[2 * pair + t][2 * w + 1]};  // round to nearest even
          pk[t][w] = __builtin_bit_cast(uint32_t, hv);
        }
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        // odd rows of the first operand <-> even rows of the second
        const auto sw = __builtin_amdgcn_permlane16_swap(pk[0][w], pk[1][w], false, false);
        pr[pair][w] = sw[0];      // lane group g: columns 4 * (g & ~1) .. + 3 of tile 2 * pair + (g & 1)
        pr[pair][2 + w] = sw[1];  // and the four columns after them
      }
    }
#pragma unroll
    for (int h = 0; h < V / 8; ++h) {
      uintx4 line;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        line[r] = h == 0 ? dpp_from_m_minus_8(pr[0][r], pr[1][r]) : dpp_from_m_plus_8(pr[0][r], pr[1][r]);
      slab_store_line(line, srd, voff[h], crow);
    }
  }
};

// fp16 with a 128-column slab: two 64-column halves.
template <int V>
struct SlabStore<V, _Float16, 8> {
  SlabStore<V, _Float16, 4> half_lo, half_hi;
  __device__ __forceinline__ void init(int lane, int n0, int N) {
    half_lo.init(lane, n0, N);
    half_hi.init(lane, n0 + 64, N);
  }
  __device__ __forceinline__ void store(const floatx4 (&acc)[8], __amdgpu_buffer_rsrc_t srd, uint32_t crow) const {
    const floatx4 a[4] = {acc[0], acc[1], acc[2], acc[3]}, b[4] = {acc[4], acc[5], acc[6], acc[7]};
    half_lo.store(a, srd, crow);
    half_hi.store(b, srd, crow);
  }
};

// fp16 with a 32-column slab: after the swap a lane owns eight consecutive columns of row m, four lanes make a
// row's 64 bytes, and one instruction writes the V rows (with V = 8 the lanes m >= 8 have nothing to write).
template <int V>
struct SlabStore<V, _Float16, 2> {
  uint32_t voff;
  __device__ __forceinline__ void init(int lane, int n0, int N) {
    const int m = lane & 15, g = lane >> 4;
    const int col = n0 + 16 * (g & 1) + 8 * (g >> 1);
    voff = (m < V && col < N) ? ((uint32_t)m * (uint32_t)N + (uint32_t)col) * 2u : kSlabDropStore;
  }
  __device__ __forceinline__ void store(const floatx4 (&acc)[2], __amdgpu_buffer_rsrc_t srd, uint32_t crow) const {
    uint32_t pk[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        const half2v hv = {(_Float16)acc[t][2 * w], (_Float16)acc[t][2 * w + 1]};  // round to nearest even
        pk[t][w] = __builtin_bit_cast(uint32_t, hv);
      }
    uintx4 line;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      const auto sw = __builtin_amdgcn_permlane16_swap(pk[0][w], pk[1][w], false, false);
      line[w] = sw[0];
      line[2 + w] = sw[1];
    }
    slab_store_line(line, srd, voff, crow);
  }
};

// Per-lane constants of the inner loop and the operands of the current work item.
template <int V, typename OutT>
struct SlabCtx {
  int lane;
  uint32_t slot0, a_off, b_lane_off, zero_row;
  unsigned char *val_tile, *val_dst;
  __amdgpu_buffer_rsrc_t srd_cols;
  uint32_t c_vrow_bytes;
};

// One wave's share of a work item: the vector-rows it claims from the item's row table,
// against the slab at byte offset slab_base of LDS.
template <int V, typename OutT, int NQ, int L>
__device__ __forceinline__ void slab_process_item(const SlabCtx<V, OutT> &x, unsigned char *lds, uint32_t slab_base,
                                                  const SlabRows &rows, const uint16_t *vals,
                                                  __amdgpu_buffer_rsrc_t srd_c, const SlabStore<V, OutT, NQ> &out) {
  SlabCursor head;  // issues loads
  head.claim = cursor_claim(rows, 0);
  cursor_prefetch(head, rows);
  cursor_take_next(head, rows);
  if (!head.valid) return;

  constexpr int R = slab_ring(V);
  SlabLoads<V> ld[R];
#pragma unroll
  for (int i = 0; i < R - 1; ++i) {
    // Loads are issued whether or not the head still has a step (an exhausted head has kc = end = 0:
    // the value load is out of bounds and returns zeros), so that the number of loads in flight
    // behind any ring slot is a compile-time constant and the waits below can be exact.
    slab_issue<V>(ld[i], head.row, head.kc, head.end, head.valid, x.lane, x.slot0, x.srd_cols, vals);
    if (head.valid) cursor_advance(head, rows);
  }
  // the value tile of the first step
  *reinterpret_cast<typename SlabVals<V>::type *>(x.val_dst) = ld[0].vraw;

  const uint32_t lane_base = x.b_lane_off + slab_base + lds_address(lds);  // slab_base is a multiple of 32 (128 for swizzled rows), the LDS base of 128
  // Accumulators are cleared by an MFMA of two zero operands: four instructions on the otherwise
  // idle matrix pipe instead of sixteen register moves on the vector ALU, which the loop saturates.
  Half8Bits zero_op;
  zero_op.u[0] = zero_op.u[1] = zero_op.u[2] = zero_op.u[3] = 0u;
  asm volatile("" : "+v"(zero_op.u[0]), "+v"(zero_op.u[1]), "+v"(zero_op.u[2]), "+v"(zero_op.u[3]));  // keep it in registers
  const floatx4 zero_c = {0.f, 0.f, 0.f, 0.f};
  floatx4 acc[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(zero_op.h, zero_op.h, zero_c, 0, 0, 0);
  for (;;) {
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int cur = u, nxt = (u + 1) % R, fill = (u + R - 1) % R;
      slab_issue<V>(ld[fill], head.row, head.kc, head.end, head.valid, x.lane, x.slot0, x.srd_cols, vals);
      if (head.valid) cursor_advance(head, rows);
      const int left = ld[cur].left;

      // A operand: this step's value tile
      Half8Bits a;
      {
        const uintx2 lo = lds_read_tr(x.val_tile, x.a_off);
        const uintx2 hi = lds_read_tr(x.val_tile, x.a_off + 4u * (V * 2u));
        a.u[0] = lo[0]; a.u[1] = lo[1]; a.u[2] = hi[0]; a.u[3] = hi[1];
      }
      // B operands: two column indices per lane; unused k slots of a partial step read the zero row
      uint32_t addr[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t c = ((int)x.slot0 + 4 * h < left) ? ld[cur].col[h] : x.zero_row;
        // row c of the slab, and the swizzle of its 32-byte segments (see slab_unit_dst)
        addr[h] = layout_pad(L) ? __umul24(c, layout_row_bytes(L, NQ)) + lane_base
                  : NQ == 8     ? (((c << 8) + lane_base) | ((c << 5) & 0xe0u))
                  : NQ == 4     ? (((c << 7) + lane_base) | ((c << 4) & 0x60u))
                                : (((c << 6) + lane_base) | ((c << 3) & 0x20u));
      }
      Half8Bits b[NQ];
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        // (padded rows: an immediate offset of the read; swizzled rows: the segment index XORed in)
        const uintx2 lo = layout_pad(L) ? lds_read_tr_abs(addr[0] + ((uint32_t)q << 5)) : lds_read_tr_abs(addr[0] ^ ((uint32_t)q << 5));
        const uintx2 hi = layout_pad(L) ? lds_read_tr_abs(addr[1] + ((uint32_t)q << 5)) : lds_read_tr_abs(addr[1] ^ ((uint32_t)q << 5));
        b[q].u[0] = lo[0]; b[q].u[1] = lo[1]; b[q].u[2] = hi[0]; b[q].u[3] = hi[1];
      }
      // the next step's value tile goes to LDS behind the reads above (LDS operations of a wave
      // execute in order; unconditionally: after the last step it is zeros that nobody reads)
      *reinterpret_cast<typename SlabVals<V>::type *>(x.val_dst) = ld[nxt].vraw;

#pragma unroll
      for (int q = 0; q < NQ; ++q) acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[q].h, a.h, acc[q], 0, 0, 0);
      if (left <= 32) {  // last step of the vector-row: write its V x 64 tile of C and start over from zero
        out.store(acc, srd_c, (uint32_t)ld[cur].row * x.c_vrow_bytes);
#pragma unroll
        for (int q = 0; q < NQ; ++q) acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(zero_op.h, zero_op.h, zero_c, 0, 0, 0);
      }
      if (!ld[nxt].valid) return;
    }
  }
}

// A work item of the slab kernel.
struct SlabItem {
  uint32_t batch, tile, rb;
};

// Item `it` of XCD `xcd`: slabs are dealt to the XCDs so that workgroups sharing an L2 share
// operands.  With at least 8 batch elements a batch element (all its column tiles and row blocks)
// stays on one XCD: its value vectors, read once per column tile, then come from that L2 after
// the first touch.  With fewer batch elements the slabs are dealt round-robin.
__device__ __forceinline__ SlabItem slab_item(const SpmmArgs &p, uint32_t xcd, uint32_t it) {
  SlabItem r;
  const uint32_t q = it / p.row_blocks;
  r.rb = it % p.row_blocks;
  if (p.group_by_batch) {
    r.batch = (q / p.n_tiles) * 8u + xcd;
    r.tile = q % p.n_tiles;
  } else {
    const uint32_t slab_id = q * 8u + xcd;
    r.tile = slab_id % p.n_tiles;
    r.batch = slab_id / p.n_tiles;
  }
  return r;
}

// The slab of an item on its way from global memory to LDS.  Unit u = 16 bytes = columns
// n0 + 8 * (u % 8) .. + 7 of row u / 8; the 32-byte segment (u % 8) / 2 of row c lands at segment
// ((u % 8) / 2) ^ ((c >> 1) & 3).
static constexpr int kSlabFetchUnits = 4;  // 16-byte units per thread held in registers (double-buffered mode)
struct SlabFetch {
  uintx4 d[kSlabFetchUnits];
  intx4 entry;
};

template <int NQ>
__device__ __forceinline__ uint32_t slab_unit_src(const SpmmArgs &p, uint32_t u, uint32_t units, uint32_t n0, uint32_t b_bytes) {
  constexpr uint32_t kPerRow = 2u * NQ;  // 16-byte units per slab row
  const uint32_t col = n0 + (u % kPerRow) * 8u;
  return (u < units && col < (uint32_t)p.N) ? __umul24(u / kPerRow, (uint32_t)p.N * 2u) + col * 2u : b_bytes;  // b_bytes: out of bounds, reads zeros
}
// A 16-lane group of a slab read touches four rows at the same segment; rows 256 bytes apart share banks, so the
// segment index is XORed with the row bits above that distance: c & 7 for 256-byte rows, (c >> 1) & 3 for 128-byte
// rows, (c >> 2) & 1 for 64-byte rows.  Rows then collide only when they agree modulo 8.
template <int NQ, int L>
__device__ __forceinline__ uint32_t slab_unit_dst(uint32_t u) {
  constexpr uint32_t kPerRow = 2u * NQ;
  const uint32_t c = u / kPerRow;
  if (layout_pad(L)) return c * layout_row_bytes(L, NQ) + (u % kPerRow) * 16u;
  const uint32_t swz = NQ == 8 ? (c & 7u) : NQ == 4 ? ((c >> 1) & 3u) : ((c >> 2) & 1u);
  return c * slab_row_bytes(NQ) + (((u % kPerRow) * 16u) ^ (swz << 5));
}

__device__ __forceinline__ intx4 slab_table_fetch(const SpmmArgs &p, const int32_t *__restrict__ row_offsets,
                                                  const int32_t *__restrict__ row_indices, uint32_t rb, int tid) {
  const int row_lo = (int)(rb * p.rows_per_block);
  const int n_rows = min(p.m_vec, row_lo + (int)p.rows_per_block) - row_lo;
  intx4 e = {0, 0, 0, 0};
  if (tid < n_rows) {
    e[0] = row_indices ? row_indices[row_lo + tid] : row_lo + tid;
    e[1] = row_offsets[e[0]];
    e[2] = row_offsets[e[0] + 1];
    e[3] = 1;
  }
  return e;
}

template <int V, typename OutT, int L, int NQ>
__global__ __launch_bounds__(kSlabThreads) void spmm_slab_kernel(const SpmmArgs p,
                                                                 const int32_t *__restrict__ row_offsets,
                                                                 const int32_t *__restrict__ row_indices) {
  extern __shared__ __align__(256) unsigned char lds[];
  // The hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each with its own L2.
  const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, wgs_per_xcd = gridDim.x >> 3;
  const uint32_t slabs_x = p.group_by_batch ? (((uint32_t)p.batch + 7u - xcd) / 8u) * p.n_tiles : (p.n_slabs + 7u - xcd) / 8u;
  const uint32_t items_x = slabs_x * p.row_blocks;
  uint32_t it = (uint32_t)(((uint64_t)slot * items_x) / wgs_per_xcd);
  const uint32_t it_end = (uint32_t)(((uint64_t)(slot + 1u) * items_x) / wgs_per_xcd);
  if (it >= it_end) return;

  const int tid = threadIdx.x, lane = tid & 63, m = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // tell the compiler it is wave-uniform
  const uint32_t b_bytes = (uint32_t)p.K * (uint32_t)p.N * 2u;
  constexpr bool DOUBLE = layout_double(L);
  constexpr bool ONE_TABLE = L == kPadDouble;  // (what fits beside the padded pair of slabs)
  static_assert(!layout_pad(L) || NQ == 4, "padded rows are for the 64-column slab");
  constexpr uint32_t kSlabRowBytes = layout_row_bytes(L, NQ);
  const uint32_t units = (uint32_t)p.K * (2u * NQ);

  // ---- LDS: slab 0, [slab 1] (their rows alternating when padded), value tiles, row table 0, [row table 1]
  const uint32_t zero_row = (uint32_t)p.K;
  const uint32_t tiles_off = layout_slab_region(L, NQ, zero_row + 1u);
  const uint32_t table_off = tiles_off + kSlabWaves * wave_lds_bytes(V);
  const uint32_t table_bytes = (p.rows_per_block + 2u) * 16u;
  if (tid < 2 * NQ) {
    *reinterpret_cast<uintx4 *>(lds + zero_row * kSlabRowBytes + tid * 16) = uintx4{0u, 0u, 0u, 0u};
    if (DOUBLE)
      *reinterpret_cast<uintx4 *>(lds + layout_buffer_off(L, NQ, zero_row + 1u, 1u) + zero_row * kSlabRowBytes + tid * 16) =
          uintx4{0u, 0u, 0u, 0u};
  }

  SlabCtx<V, OutT> x;
  x.lane = lane;
  x.val_tile = lds + tiles_off + wave * wave_lds_bytes(V);
  constexpr uint32_t kLaneBytes = V * 2u * 32u / 64u;
  x.val_dst = x.val_tile + lane * kLaneBytes;
  // value tile rows are V*2 bytes; transpose read h picks rows 8g + 4h + m/4
  x.a_off = (uint32_t)(8 * g + (m >> 2)) * (V * 2u) + (uint32_t)(m & 3) * 8u;
  x.slot0 = (uint32_t)(8 * g + (m >> 2));
  x.b_lane_off = (uint32_t)(m & 3) * 8u;
  x.zero_row = zero_row;
  x.c_vrow_bytes = (uint32_t)V * (uint32_t)p.N * (uint32_t)sizeof(OutT);
  const uint32_t nvec = (uint32_t)row_offsets[p.m_vec];
  x.srd_cols = make_srd(p.col_idx, nvec * 4u);

  // ---- first item: fetch and commit its slab and table
  SlabItem cur = slab_item(p, xcd, it);
  {
    const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.B + (int64_t)cur.batch * p.stride_B, b_bytes);
    const intx4 e = slab_table_fetch(p, row_offsets, row_indices, cur.rb, tid);
    for (uint32_t u0 = 0; u0 < units; u0 += kSlabThreads * 4) {
      uintx4 d[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        d[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(
                                              srd_b, slab_unit_src<NQ>(p, u0 + i * kSlabThreads + tid, units, cur.tile * (16u * NQ), b_bytes), 0, 0));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t u = u0 + i * kSlabThreads + tid;
        if (u < units) *reinterpret_cast<uintx4 *>(lds + slab_unit_dst<NQ, L>(u)) = d[i];
      }
    }
    if ((uint32_t)tid <= p.rows_per_block + 1u) *reinterpret_cast<intx4 *>(lds + table_off + tid * 16) = e;
  }
  __syncthreads();

  uint32_t slab_sel = 0, table_sel = 0;
  for (;;) {
    const bool has_next = it + 1u < it_end;
    const SlabItem nxt = has_next ? slab_item(p, xcd, it + 1u) : cur;
    const bool new_slab = nxt.batch != cur.batch || nxt.tile != cur.tile;
    SlabFetch f;
    // (a copy of the thread index the compiler cannot see through: the address arithmetic of the
    // fetch would otherwise be hoisted out of the item loop and held in registers across it)
    int ftid = tid;
    asm volatile("" : "+v"(ftid));
    if (DOUBLE && has_next) {
      // the next item's table and slab start their way to registers now and are written to LDS
      // when this item's rows are done
      f.entry = slab_table_fetch(p, row_offsets, row_indices, nxt.rb, ftid);
      if (new_slab) {
        const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.B + (int64_t)nxt.batch * p.stride_B, b_bytes);
#pragma unroll
        for (int i = 0; i < kSlabFetchUnits; ++i)
          f.d[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(
                                                  srd_b, slab_unit_src<NQ>(p, i * kSlabThreads + ftid, units, nxt.tile * (16u * NQ), b_bytes), 0, 0));
      }
    }

    {
      const int row_lo = (int)(cur.rb * p.rows_per_block);
      SlabRows rows;
      rows.table = reinterpret_cast<const intx4 *>(lds + table_off + table_sel * table_bytes);
      rows.n_rows = min(p.m_vec, row_lo + (int)p.rows_per_block) - row_lo;
      // (the entries at rows_per_block and behind it are rewritten, all zeros, with every table)
      rows.counter = reinterpret_cast<int *>(lds + table_off + table_sel * table_bytes + (p.rows_per_block + 1u) * 16u);
      rows.lane = lane;
      SlabStore<V, OutT, NQ> out;
      out.init(lane, (int)cur.tile * (16 * NQ), p.N);
      // One buffer descriptor spans this batch element's C (the launcher checks it is at most 2 GiB).
      const __amdgpu_buffer_rsrc_t srd_c = make_srd(reinterpret_cast<OutT *>(p.C) + (int64_t)cur.batch * p.stride_C,
                                                    (uint32_t)p.m_vec * x.c_vrow_bytes);
      slab_process_item<V, OutT, NQ, L>(x, lds, layout_buffer_off(L, NQ, zero_row + 1u, slab_sel), rows, p.values + (int64_t)cur.batch * p.stride_values,
                                 srd_c, out);
    }
    if (!has_next) break;

    int ctid = tid;
    asm volatile("" : "+v"(ctid));
    if (DOUBLE) {
      // The other buffers were last read during the previous item, which every wave has left.
      if (new_slab) {
        slab_sel ^= 1u;
#pragma unroll
        for (int i = 0; i < kSlabFetchUnits; ++i) {
          const uint32_t u = i * kSlabThreads + ctid;
          if (u < units)
            *reinterpret_cast<uintx4 *>(lds + layout_buffer_off(L, NQ, zero_row + 1u, slab_sel) + slab_unit_dst<NQ, L>(u)) = f.d[i];
        }
      }
      if (ONE_TABLE) {
        __syncthreads();  // every wave is done with the table
      } else {
        table_sel ^= 1u;
      }
      if ((uint32_t)ctid <= p.rows_per_block + 1u) *reinterpret_cast<intx4 *>(lds + table_off + table_sel * table_bytes + ctid * 16) = f.entry;
      __syncthreads();
    } else {
      __syncthreads();  // every wave is done with the slab and the table
      const intx4 e = slab_table_fetch(p, row_offsets, row_indices, nxt.rb, ctid);
      if (new_slab) {
        const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.B + (int64_t)nxt.batch * p.stride_B, b_bytes);
        for (uint32_t u0 = 0; u0 < units; u0 += kSlabThreads * 4) {
          uintx4 d[4];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            d[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(
                                                  srd_b, slab_unit_src<NQ>(p, u0 + i * kSlabThreads + ctid, units, nxt.tile * (16u * NQ), b_bytes), 0, 0));
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t u = u0 + i * kSlabThreads + ctid;
            if (u < units) *reinterpret_cast<uintx4 *>(lds + slab_unit_dst<NQ, L>(u)) = d[i];
          }
        }
      }
      if ((uint32_t)ctid <= p.rows_per_block + 1u) *reinterpret_cast<intx4 *>(lds + table_off + ctid * 16) = e;
      __syncthreads();
    }
    cur = nxt;
    ++it;
  }
}

// ------------------------------------------------------------------------------------------
// Gather kernel for right-hand sides of at most 64 columns (an attention head's features), where a
// row of B is 128 bytes or less.  Fetching such rows in the MFMA's operand layout means 8 bytes per
// lane, and the vector memory pipeline works through a wave's load four lanes at a time whatever
// their width: half of its byte rate.  Here eight neighbouring lanes fetch the eight 16-byte pieces
// of one row (a load instruction brings 8 whole rows, a step's 32 rows take 4 of them instead of 8),
// the rows are staged in a per-wave tile in LDS and come back as MFMA operands through the
// transpose reads of the slab kernel, whose accumulator layout and store of C are shared too.  No
// byte shuffling in registers.  Rows of the tile are 144 bytes apart so that the four consecutive
// rows a 16-lane group reads fall into different banks.
static constexpr uint32_t kStagePitch = 144;

template <int V>
struct StageHead {  // what does not depend on other loads
  uintx4 cols;      // column indices of k slots 4j .. 4j+3, j = lane / 8
  typename SlabVals<V>::type vraw;
  int kc;
};
template <int V>
struct StageBody {
  uintx4 piece[4];  // piece[i] = 16 bytes (columns 8 * (lane % 8) ..) of the row of B named by k slot 4j + i
  typename SlabVals<V>::type vraw;
};

// Per-lane constants of the staged gather: where the lane writes its share of the staged rows and of the value
// tile, and where its transpose reads start.
template <int V>
struct StageLane {
  int j, pc;            // the lane fetches 16-byte piece pc of the rows named by k slots 4j .. 4j+3
  uint32_t vals_lane_off, a_off, b_rd;
  unsigned char *tile_dst, *stage_dst;
  const unsigned char *val_tile;
  __device__ __forceinline__ void init(int lane, unsigned char *stage, unsigned char *tile) {
    const int m = lane & 15, g = lane >> 4;
    j = lane >> 3;
    pc = lane & 7;
    constexpr uint32_t kLaneBytes = V * 2u * 32u / 64u;
    vals_lane_off = (uint32_t)lane * kLaneBytes;
    val_tile = tile;
    tile_dst = tile + lane * kLaneBytes;
    stage_dst = stage + (uint32_t)(4 * j) * kStagePitch + (uint32_t)pc * 16u;
    // transpose reads: k slots 8g + m/4 (and + 4) of the value tile and of the staged rows
    a_off = (uint32_t)(8 * g + (m >> 2)) * (V * 2u) + (uint32_t)(m & 3) * 8u;
    b_rd = lds_address(stage) + (uint32_t)(8 * g + (m >> 2)) * kStagePitch + (uint32_t)(m & 3) * 8u;
  }
};

// acc += the V x 64 tile of vectors [beg, end) of a vector-row against columns ncol0 .. of B.  srd_cols and
// srd_vals end at vector `end`: slots past it read as zero.  Lane (m, g) ends up with columns 16q + 4g .. + 3 of
// output row m in acc[q] (the staged rows are the MFMA's first operand, as the slab is in the slab kernel).
template <int V>
__device__ __forceinline__ void stage_accumulate(floatx4 (&acc)[4], const StageLane<V> &x, __amdgpu_buffer_rsrc_t srd_cols,
                                                 __amdgpu_buffer_rsrc_t srd_vals, __amdgpu_buffer_rsrc_t srd_b, int beg,
                                                 int end, uint32_t lane_n2, uint32_t lane_col_off, uint32_t b_bytes) {
  const auto load_head = [&](StageHead<V> &h, int kc) {
    h.kc = kc;
    h.cols = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_cols, (kc + 4 * x.j) * 4, 0, 0));
    h.vraw = SlabVals<V>::load(srd_vals, (uint32_t)kc * (V * 2u) + x.vals_lane_off);
  };
  const auto load_body = [&](StageBody<V> &c, const StageHead<V> &h) {
    uint32_t off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) off[i] = __umul24(h.cols[i], lane_n2) + lane_col_off;
    if (h.kc + 32 > end) {  // wave-uniform: only the last chunk of a vector-row can be partial
#pragma unroll
      for (int i = 0; i < 4; ++i) off[i] = (h.kc + 4 * x.j + i < end) ? off[i] : b_bytes;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      c.piece[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_b, off[i], 0, 0));
    c.vraw = h.vraw;
  };
  const auto contract = [&](const StageBody<V> &c) {
    // (LDS operations of a wave execute in order: these writes land behind the previous chunk's reads)
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uintx4 *>(x.stage_dst + i * kStagePitch) = c.piece[i];
    *reinterpret_cast<typename SlabVals<V>::type *>(x.tile_dst) = c.vraw;
    Half8Bits a;
    {
      const uintx2 lo = lds_read_tr(x.val_tile, x.a_off);
      const uintx2 hi = lds_read_tr(x.val_tile, x.a_off + 4u * (V * 2u));
      a.u[0] = lo[0]; a.u[1] = lo[1]; a.u[2] = hi[0]; a.u[3] = hi[1];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      Half8Bits b;
      const uintx2 lo = lds_read_tr_abs(x.b_rd + 32u * q);
      const uintx2 hi = lds_read_tr_abs(x.b_rd + 4u * kStagePitch + 32u * q);
      b.u[0] = lo[0]; b.u[1] = lo[1]; b.u[2] = hi[0]; b.u[3] = hi[1];
      acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b.h, a.h, acc[q], 0, 0, 0);
    }
  };
  if (beg >= end) return;
  // Heads run two chunks ahead of the arithmetic, bodies one (two of each, used alternately).
  StageHead<V> h0, h1;
  StageBody<V> c0, c1;
  load_head(h0, beg);
  load_head(h1, beg + 32);
  load_body(c0, h0);
  int kc = beg + 32;  // first vector of the chunk whose body is loaded next
  for (;;) {
    if (kc >= end) {
      contract(c0);
      break;
    }
    load_head(h0, kc + 32);
    load_body(c1, h1);
    contract(c0);
    kc += 32;
    if (kc >= end) {
      contract(c1);
      break;
    }
    load_head(h1, kc + 32);
    load_body(c0, h0);
    contract(c1);
    kc += 32;
  }
}

// The same pipeline over a bundle of whole vector-rows (items first .. first + count - 1 of a schedule, count <= 64):
// the steps of all the rows are one stream, so that the column indices of a row's first step and the rows of B they
// name are in flight while the row before it is contracted, and a row's V x 64 tile of C is stored when its last
// step has been.  A row of no vectors is one step of zeros.  Each row's sums are formed exactly as stage_accumulate
// forms them (same steps, same order).
template <int V, typename OutT>
__device__ __forceinline__ void stage_stream(const StageLane<V> &x, const int32_t *col_idx, const uint16_t *vals,
                                             __amdgpu_buffer_rsrc_t srd_b, uint32_t lane_n2, uint32_t lane_col_off, uint32_t b_bytes,
                                             const void *first_item, int count, int lane, const SlabStore<V, OutT, 4> &out,
                                             __amdgpu_buffer_rsrc_t srd_c, uint32_t c_vrow_bytes) {
  // the bundle's items, one per lane (row, first vector, end): a uniform index reads one back without memory
  const uintx4 mine = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(
                                                     make_srd(first_item, (uint32_t)count * 32u), (uint32_t)lane * 32u, 0, 0));
  struct Step {  // (uniform)
    int row, kc, end;
    bool valid;
  };
  int j = 0;
  Step cur;
  cur.row = __builtin_amdgcn_readlane((int)mine[0], 0);
  cur.kc = __builtin_amdgcn_readlane((int)mine[1], 0);
  cur.end = __builtin_amdgcn_readlane((int)mine[2], 0);
  cur.valid = true;
  const auto next = [&]() {
    const Step d = cur;
    if (cur.valid) {
      cur.kc += 32;
      if (cur.kc >= cur.end) {
        ++j;
        cur.valid = j < count;
        const int jj = cur.valid ? j : 0;
        cur.row = __builtin_amdgcn_readlane((int)mine[0], jj);
        cur.kc = __builtin_amdgcn_readlane((int)mine[1], jj);
        cur.end = __builtin_amdgcn_readlane((int)mine[2], jj);
      }
    }
    return d;
  };
  // (a step past the bundle's end has no vectors to its name: descriptors of zero bytes, every load reads zeros)
  const auto load_head = [&](StageHead<V> &h, const Step &d) {
    const uint32_t recs = d.valid ? (uint32_t)d.end : 0u;
    h.kc = d.kc;
    h.cols = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(make_srd(col_idx, recs * 4u), (d.kc + 4 * x.j) * 4, 0, 0));
    h.vraw = SlabVals<V>::load(make_srd(vals, recs * (V * 2u)), (uint32_t)d.kc * (V * 2u) + x.vals_lane_off);
  };
  const auto load_body = [&](StageBody<V> &c, const StageHead<V> &h, const Step &d) {
    uint32_t off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) off[i] = __umul24(h.cols[i], lane_n2) + lane_col_off;
    if (h.kc + 32 > d.end) {  // wave-uniform: only the last step of a vector-row can be partial
#pragma unroll
      for (int i = 0; i < 4; ++i) off[i] = (h.kc + 4 * x.j + i < d.end) ? off[i] : b_bytes;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      c.piece[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_b, off[i], 0, 0));
    c.vraw = h.vraw;
  };
  floatx4 acc[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};
  const auto contract = [&](const StageBody<V> &c, const Step &d) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uintx4 *>(x.stage_dst + i * kStagePitch) = c.piece[i];
    *reinterpret_cast<typename SlabVals<V>::type *>(x.tile_dst) = c.vraw;
    Half8Bits a;
    {
      const uintx2 lo = lds_read_tr(x.val_tile, x.a_off);
      const uintx2 hi = lds_read_tr(x.val_tile, x.a_off + 4u * (V * 2u));
      a.u[0] = lo[0]; a.u[1] = lo[1]; a.u[2] = hi[0]; a.u[3] = hi[1];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      Half8Bits b;
      const uintx2 lo = lds_read_tr_abs(x.b_rd + 32u * q);
      const uintx2 hi = lds_read_tr_abs(x.b_rd + 4u * kStagePitch + 32u * q);
      b.u[0] = lo[0]; b.u[1] = lo[1]; b.u[2] = hi[0]; b.u[3] = hi[1];
      acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b.h, a.h, acc[q], 0, 0, 0);
    }
    if (d.kc + 32 >= d.end) {  // the row's last step: its tile of C, and the next row starts from zero
      out.store(acc, srd_c, (uint32_t)d.row * c_vrow_bytes);
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
  };
  // Heads run two steps ahead of the arithmetic, bodies one; loads are only issued on the paths that use them, so
  // that the waits in front of every use count exactly the loads behind it.
  StageHead<V> h0, h1;
  StageBody<V> c0, c1;
  Step d0 = next();
  load_head(h0, d0);
  Step d1 = next();
  load_head(h1, d1);
  load_body(c0, h0, d0);
  for (;;) {
    if (!d1.valid) {
      contract(c0, d0);
      break;
    }
    const Step d2 = next();
    load_head(h0, d2);
    load_body(c1, h1, d1);
    contract(c0, d0);
    if (!d2.valid) {
      contract(c1, d1);
      break;
    }
    const Step d3 = next();
    load_head(h1, d3);
    load_body(c0, h0, d2);
    contract(c1, d1);
    d0 = d2;
    d1 = d3;
  }
}

template <int V, typename OutT>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(V == 8 ? 5 : 4, V == 8 ? 5 : 4))) void spmm_stage_kernel(const SpmmArgs p) {
  __shared__ __align__(16) unsigned char stage[32 * kStagePitch];
  __shared__ __align__(16) unsigned char val_tile[val_tile_bytes(V)];
  const uint32_t id = blockIdx.x;
  const uint32_t w = (id & 7u) * p.per_xcd + (id >> 3);
  if (w >= p.total_work) return;
  const uint32_t r = w % (uint32_t)p.m_vec;
  const uint32_t t = w / (uint32_t)p.m_vec;
  const uint32_t tile = t % p.n_tiles;  // 64 columns
  const uint32_t batch = t / p.n_tiles;
  const int row = __builtin_amdgcn_readfirstlane(p.row_indices ? p.row_indices[r] : (int)r);

  const int lane = threadIdx.x;
  StageLane<V> x;
  x.init(lane, stage, val_tile);
  const int beg = p.row_offsets[row], end = p.row_offsets[row + 1];

  const uint16_t *vals = p.values + (int64_t)batch * p.stride_values;
  const uint32_t b_bytes = (uint32_t)p.K * (uint32_t)p.N * 2u;
  // the descriptors of the pattern and the values end at this vector-row's last vector: slots past it read as zero
  const __amdgpu_buffer_rsrc_t srd_cols = make_srd(p.col_idx, (uint32_t)end * 4u);
  const __amdgpu_buffer_rsrc_t srd_vals = make_srd(vals, (uint32_t)end * (V * 2u));
  const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.B + (int64_t)batch * p.stride_B, b_bytes);

  // Lanes whose columns lie beyond N aim every gather at the first byte past B, where loads return zero.
  const int ncol = (int)tile * 64 + 8 * x.pc;
  const bool col_ok = ncol < p.N;
  const uint32_t lane_n2 = col_ok ? (uint32_t)p.N * 2u : 0u;
  const uint32_t lane_col_off = col_ok ? (uint32_t)ncol * 2u : b_bytes;
  floatx4 acc[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};
  // (the bias of the lane's output row is fetched before the loop so that the row's end does not wait for it)
  const float b = bias_of_row(p, (int64_t)row * V + (lane & (V - 1)));
  stage_accumulate<V>(acc, x, srd_cols, srd_vals, srd_b, beg, end, lane_n2, lane_col_off, b_bytes);
  if (has_epilogue(p)) {  // (uniform) every accumulator of lane (m, g) belongs to output row m of the vector-row
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[q][r] = epilogue_value(acc[q][r], b, p.act);
  }

  SlabStore<V, OutT, 4> out;
  out.init(lane, (int)tile * 64, p.N);
  const uint32_t c_vrow_bytes = (uint32_t)V * (uint32_t)p.N * (uint32_t)sizeof(OutT);
  // One buffer descriptor spans this batch element's C (the launcher checks it is at most 2 GiB).
  const __amdgpu_buffer_rsrc_t srd_c = make_srd(reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C,
                                                (uint32_t)p.m_vec * c_vrow_bytes);
  out.store(acc, srd_c, (uint32_t)row * c_vrow_bytes);
}

// ------------------------------------------------------------------------------------------
// Load-balanced kernel: the work list is a schedule (schedule.h) instead of the vector-rows.
//
// One wave per (work item, 64-column tile).  An item is at most `budget` steps of one vector-row, so
// every wave of the grid has about the same amount to do whatever the row lengths are, and the
// hardware's workgroup dispatcher hands items to CUs as waves retire.  The panels of a cut row leave
// their accumulators in scratch memory as they lie in registers; each then counts itself in on the
// row's counter, and the wave that finds all the others counted adds the partial tiles up in panel
// order (its own from memory too, so that the sum has one order whichever wave does it), stores the
// row of C and puts the counter back to zero for the next launch.  No wave ever waits for another.
//
// The inner loop is the staged gather's (rows of B fetched as whole 128-byte lines by eight lanes each,
// passed through a per-wave LDS tile to the transpose reads): its 100 registers instead of the
// register-path kernel's 190 keep twice as many waves on a CU.  (Deeper prefetch was measured and
// does not pay: a grid of panels is bound by the rate at which the CUs' address units take load
// instructions, 16 cycles per 16-byte load of a wave, and every load issued past the end of a short
// row costs that too.)
//
// Work id -> (batch element, item, column tile) with the tile index fastest and the tile count padded
// to 1, 2, 4 or a multiple of 8 (padding tiles return at once): workgroup ids go round-robin to the 8
// XCDs, so an XCD sees only the column tiles congruent to it and keeps their slab of B in its L2,
// while the items are dealt evenly over the XCDs that share a tile.
struct BalancedArgs {
  const int32_t *header;
  const ScheduleItem *items;
  int32_t *counters;
  unsigned char *partials;
  int n_items;            // units the grid covers: the schedule's count, or an upper bound of it
  uint32_t tiles_padded;
  const int32_t *bundles; // first item of every bundle of whole rows, or null: every item is a unit
  int bundle_base;        // with bundles: units below this are single items (the panels of cut rows)
};

// Partial tiles travel between workgroups that may sit on different XCDs, each with an L2 of its own.  They are
// written and read with device-scope accesses (the sc1 bit, what a device-scope atomic store or load carries:
// stores go through to memory and are complete when the wave's store counter says so, loads are served from
// there), as the counter's atomics are.  Release and acquire fences in their place write back and invalidate a
// whole L2 for every panel (measured on 2048 rows with 1000 panels: 35 us per launch for the former, 5 us for the
// latter, in a kernel of 18 us).
static constexpr int kDeviceScope = 16;  // cache-policy bit sc1 of the buffer instructions

// acc[q] of lane (m, g) = columns 16q + 4g .. + 3 of output row m; with V = 8 the lanes m >= 8 hold nothing.
template <int V>
struct PartialTile {
  static constexpr uint32_t kLanes = V == 8 ? 32u : 64u;
  static __device__ __forceinline__ uint32_t lane_offset(int lane) {
    const int m = lane & 15, g = lane >> 4;
    if (V == 8) return m < 8 ? (uint32_t)(g * 8 + m) * 16u : 0x80000000u;  // (beyond the descriptor: dropped / zeros)
    return (uint32_t)lane * 16u;
  }
  static __device__ __forceinline__ void store(__amdgpu_buffer_rsrc_t srd, uint32_t tile_off, const floatx4 (&acc)[4], int lane) {
    const uint32_t off = tile_off + lane_offset(lane);
#pragma unroll
    for (int q = 0; q < 4; ++q)
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uintx4, acc[q]), srd, off + (uint32_t)q * (kLanes * 16u), 0, kDeviceScope);
  }
  static __device__ __forceinline__ void add(__amdgpu_buffer_rsrc_t srd, uint32_t tile_off, floatx4 (&acc)[4], int lane) {
    const uint32_t off = tile_off + lane_offset(lane);
    floatx4 x[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
      x[q] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(srd, off + (uint32_t)q * (kLanes * 16u), 0, kDeviceScope));
#pragma unroll
    for (int q = 0; q < 4; ++q) acc[q] += x[q];
  }
};
static_assert(PartialTile<8>::kLanes * 64u == partial_tile_bytes(8) && PartialTile<16>::kLanes * 64u == partial_tile_bytes(16),
              "a partial tile is four 16-byte pieces per lane that holds rows");

// DEVICE_COUNT: the number of items is only known on the device; the grid covers an upper bound of it and the
// workgroups beyond the schedule's end return at once.
template <int V, typename OutT, bool DEVICE_COUNT>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 4))) void spmm_balanced_kernel(const SpmmArgs p, const BalancedArgs s) {
  __shared__ __align__(16) unsigned char stage[32 * kStagePitch];
  __shared__ __align__(16) unsigned char val_tile[val_tile_bytes(V)];
  const int lane = threadIdx.x;
  StageLane<V> x;
  x.init(lane, stage, val_tile);
  // s.n_items: the schedule's item count, or with DEVICE_COUNT the bound the grid was sized for
  const uint32_t per_batch = (uint32_t)s.n_items * s.tiles_padded;
  const uint32_t b_bytes = (uint32_t)p.K * (uint32_t)p.N * 2u;
  const uint32_t c_vrow_bytes = (uint32_t)V * (uint32_t)p.N * (uint32_t)sizeof(OutT);
  {
    const uint32_t id = blockIdx.x;
    const uint32_t batch = id / per_batch, rem = id % per_batch;
    const uint32_t tile = rem % s.tiles_padded, unit = rem / s.tiles_padded;
    if (tile >= p.n_tiles) return;
    if (DEVICE_COUNT && unit >= (uint32_t)s.header[kHdrItems]) return;
    uint32_t item = unit;
    if (!DEVICE_COUNT && s.bundles != nullptr && unit >= (uint32_t)s.bundle_base) {
      // a bundle of rows that stay whole: one stream of steps
      const int32_t *bp = s.bundles + (unit - (uint32_t)s.bundle_base);
      const int first = __builtin_amdgcn_readfirstlane(bp[0]), last = __builtin_amdgcn_readfirstlane(bp[1]);
      const int ncol = (int)tile * 64 + 8 * x.pc;
      const bool col_ok = ncol < p.N;
      SlabStore<V, OutT, 4> out;
      out.init(lane, (int)tile * 64, p.N);
      stage_stream<V, OutT>(x, p.col_idx, p.values + (int64_t)batch * p.stride_values,
                            make_srd(p.B + (int64_t)batch * p.stride_B, b_bytes), col_ok ? (uint32_t)p.N * 2u : 0u,
                            col_ok ? (uint32_t)ncol * 2u : b_bytes, b_bytes, s.items + first, last - first, lane, out,
                            make_srd(reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C, (uint32_t)p.m_vec * c_vrow_bytes),
                            c_vrow_bytes);
      return;
    }
    const ScheduleItem *ip = s.items + item;
    // (the item is the same for the whole wave: scalar registers)
    const int row = __builtin_amdgcn_readfirstlane(ip->row), kbeg = __builtin_amdgcn_readfirstlane(ip->kbeg),
              kend = __builtin_amdgcn_readfirstlane(ip->kend), split_id = __builtin_amdgcn_readfirstlane(ip->split_id);

    // the descriptors of the pattern and the values end at the panel's last vector: slots past it read as zero
    const __amdgpu_buffer_rsrc_t srd_cols = make_srd(p.col_idx, (uint32_t)kend * 4u);
    const __amdgpu_buffer_rsrc_t srd_vals = make_srd(p.values + (int64_t)batch * p.stride_values, (uint32_t)kend * (V * 2u));
    const __amdgpu_buffer_rsrc_t srd_b = make_srd(p.B + (int64_t)batch * p.stride_B, b_bytes);
    // Lanes whose columns lie beyond N aim every gather at the first byte past B, where loads return zero.
    const int ncol = (int)tile * 64 + 8 * x.pc;
    const bool col_ok = ncol < p.N;
    const uint32_t lane_n2 = col_ok ? (uint32_t)p.N * 2u : 0u;
    const uint32_t lane_col_off = col_ok ? (uint32_t)ncol * 2u : b_bytes;
    floatx4 acc[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};
    stage_accumulate<V>(acc, x, srd_cols, srd_vals, srd_b, kbeg, kend, lane_n2, lane_col_off, b_bytes);

    if (split_id >= 0) {
      const uint32_t n_slots = (uint32_t)s.header[kHdrSlots], n_split = (uint32_t)s.header[kHdrSplitRows];
      const int first_slot = __builtin_amdgcn_readfirstlane(ip->first_slot), pieces = __builtin_amdgcn_readfirstlane(ip->pieces),
                piece = __builtin_amdgcn_readfirstlane(ip->piece);
      const size_t unit = (size_t)batch * p.n_tiles + tile;
      // the partial tiles of this row for this column tile and batch element (one descriptor)
      const __amdgpu_buffer_rsrc_t srd_part =
          make_srd(s.partials + (unit * n_slots + (uint32_t)first_slot) * partial_tile_bytes(V),
                   (uint32_t)pieces * (uint32_t)partial_tile_bytes(V));
      PartialTile<V>::store(srd_part, (uint32_t)piece * (uint32_t)partial_tile_bytes(V), acc, lane);
      // the tile has reached memory before the panel counts itself in
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      int32_t *counter = s.counters + unit * n_split + (uint32_t)split_id;
      int seen = 0;
      if (lane == 0) seen = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      seen = __builtin_amdgcn_readfirstlane(seen);
      if (seen != pieces - 1) return;  // other panels of the row are still out: the last one adds up
      asm volatile("" ::: "memory");  // the loads below stay behind the count
      if (lane == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[q] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
      for (int pc = 0; pc < pieces; ++pc)
        PartialTile<V>::add(srd_part, (uint32_t)pc * (uint32_t)partial_tile_bytes(V), acc, lane);
    }
    SlabStore<V, OutT, 4> out;
    out.init(lane, (int)tile * 64, p.N);
    // One buffer descriptor spans this batch element's C (the launcher checks it is at most 2 GiB).
    const __amdgpu_buffer_rsrc_t srd_c = make_srd(reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C,
                                                  (uint32_t)p.m_vec * c_vrow_bytes);
    out.store(acc, srd_c, (uint32_t)row * c_vrow_bytes);
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
  if (has_epilogue(p)) {
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = epilogue_value(acc[v], bias_of_row(p, (int64_t)row * V + v), p.act);
  }
  OutT *cbase = reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C;
#pragma unroll
  for (int v = 0; v < V; ++v) cbase[((int64_t)row * V + v) * p.N + n] = (OutT)acc[v];
}

// Test and tuning hooks.  Both are per host thread: a thread that forces a kernel changes what its own calls
// run and nobody else's, and the launch path shares no mutable state between threads.
static thread_local int g_kernel_override = 0;  // 0 auto, 1 generic, 2 gather, 3 slab, 6 staged gather

static thread_local int g_last_kernel = 0;  // kernel of this thread's latest launch
int last_kernel() { return g_last_kernel; }

int kernel_override() { return g_kernel_override; }

int set_kernel_override(int which) {
  const int old = g_kernel_override;
  g_kernel_override = which;
  return old;
}

static constexpr uint32_t kSlabLds = 160u * 1024u;
static constexpr uint32_t kSlabMaxRows = 512;  // vector-rows per work item (one row table entry per thread, tables of 8 KB)
static constexpr uint32_t kSlabMinRows = 32;   // keeps the copy of the slab a small part of an item's traffic

// LDS bytes of a workgroup: slabs (+ zero rows), value tiles, two row tables.
static uint32_t slab_lds_bytes(int K, int V, uint32_t rows, int layout, int NQ) {
  return layout_slab_region(layout, NQ, (uint32_t)K + 1u) + kSlabWaves * wave_lds_bytes(V) +
         (layout == kPadDouble ? 1u : 2u) * 16u * (rows + 2u);
}
// Largest K the slab kernel takes (one slab, smallest row tables).
static bool slab_fits(int K, int V, int NQ) { return slab_lds_bytes(K, V, kSlabMinRows, kXorSingle, NQ) <= kSlabLds; }

static constexpr int kMaxDevices = 64;
static int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
  return dev;
}

static uint32_t device_cus() {  // of the current device
  static uint32_t cus[kMaxDevices] = {};
  const int dev = current_device();
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8) n = 256;
    cus[dev] = (uint32_t)n;
  }
  return cus[dev];
}

template <int V, typename OutT, int L, int NQ>
static hipError_t launch_slab_kernel(const SpmmArgs &p, uint32_t grid, uint32_t lds, hipStream_t stream) {
  auto kern = spmm_slab_kernel<V, OutT, L, NQ>;
  static bool raised[kMaxDevices] = {};  // per instantiation and device
  const int dev = current_device();
  if (!raised[dev]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSlabLds);
    if (e != hipSuccess) return e;
    raised[dev] = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kSlabThreads), lds, stream, p, p.row_offsets, p.row_indices);
  return hipGetLastError();
}

template <int V, typename OutT, int NQ>
static hipError_t launch_slab(const SpmmArgs &a, hipStream_t stream) {
  SpmmArgs p = a;
  p.n_tiles = (uint32_t)((a.N + 16 * NQ - 1) / (16 * NQ));
  p.n_slabs = p.n_tiles * (uint32_t)a.batch;
  p.group_by_batch = a.batch >= 8 ? 1u : 0u;
  const uint32_t wgs_per_xcd = device_cus() / 8u;
  // Aim at two or more items per workgroup (so that fetching a slab overlaps computing on the
  // previous one), within kSlabMinRows .. kSlabMaxRows vector-rows per item.
  const uint32_t slabs_per_xcd = p.group_by_batch ? (((uint32_t)a.batch + 7u) / 8u) * p.n_tiles : (p.n_slabs + 7u) / 8u;
  uint32_t row_blocks = (2u * wgs_per_xcd + slabs_per_xcd - 1u) / slabs_per_xcd;
  const uint32_t max_blocks = ((uint32_t)a.m_vec + kSlabMinRows - 1u) / kSlabMinRows;
  const uint32_t min_blocks = ((uint32_t)a.m_vec + kSlabMaxRows - 1u) / kSlabMaxRows;
  if (row_blocks > max_blocks) row_blocks = max_blocks;
  if (row_blocks < min_blocks) row_blocks = min_blocks;
  uint32_t rows = ((uint32_t)a.m_vec + row_blocks - 1u) / row_blocks;
  // Layout: double-buffered where the next slab fits into the registers of one fetch and both slabs into LDS,
  // padded rows where they fit (64-column slabs only).
  const bool can_dbl = (uint32_t)a.K * (2u * NQ) <= (uint32_t)kSlabFetchUnits * kSlabThreads;
  int layout = kXorSingle;
  if (NQ == 4 && can_dbl && slab_lds_bytes(a.K, V, rows, kPadDouble, NQ) <= kSlabLds) layout = kPadDouble;
  else if (NQ != 8 && can_dbl && slab_lds_bytes(a.K, V, rows, kXorDouble, NQ) <= kSlabLds) layout = kXorDouble;
  else if (NQ == 4 && slab_lds_bytes(a.K, V, rows, kPadSingle, NQ) <= kSlabLds) layout = kPadSingle;
  while (layout == kXorSingle && slab_lds_bytes(a.K, V, rows, kXorSingle, NQ) > kSlabLds && rows > kSlabMinRows)
    rows = (rows + 1u) / 2u;  // smaller tables for a tall slab
  p.rows_per_block = rows;
  p.row_blocks = ((uint32_t)a.m_vec + rows - 1u) / rows;
  const uint32_t lds = slab_lds_bytes(a.K, V, rows, layout, NQ);
  const uint32_t grid = 8u * wgs_per_xcd;
  if (NQ == 4) {
    if (layout == kPadDouble) return launch_slab_kernel<V, OutT, kPadDouble, 4>(p, grid, lds, stream);
    if (layout == kPadSingle) return launch_slab_kernel<V, OutT, kPadSingle, 4>(p, grid, lds, stream);
  }
  if (NQ == 8) return launch_slab_kernel<V, OutT, kXorSingle, NQ>(p, grid, lds, stream);  // (128-column slabs: one buffer)
  return layout == kXorDouble ? launch_slab_kernel<V, OutT, kXorDouble, NQ == 8 ? 4 : NQ>(p, grid, lds, stream)
                              : launch_slab_kernel<V, OutT, kXorSingle, NQ>(p, grid, lds, stream);
}

template <int V, typename OutT>
static hipError_t launch_v(const SpmmArgs &a, int which, hipStream_t stream) {
  SpmmArgs p = a;
  if (which == 3) return launch_slab<V, OutT, 4>(a, stream);
  if (which == 5) return launch_slab<V, OutT, 2>(a, stream);
  if (which == 9) return launch_slab<V, OutT, 8>(a, stream);
  if (which == 2) {
    p.n_tiles = (uint32_t)((a.N + 127) / 128);
    p.total_work = (uint32_t)a.m_vec * p.n_tiles * (uint32_t)a.batch;
    p.per_xcd = (p.total_work + 7u) / 8u;
    // (the staged kernel addresses one batch element's C through a 32-bit buffer descriptor, as the slab kernel does)
    const bool c_ok = (uint64_t)a.m_vec * V * (uint64_t)a.N * sizeof(OutT) <= (uint64_t)kSlabDropStore;
    // The staged kernel: forced (tuning) on any width, 64 columns per wave; chosen for N <= 64 whatever K is (rows of
    // 64 columns leave half of the split-row kernel's lanes idle: measured 1.5-2x on 8192 and 16384 columns).
    // Also where the register-path kernel would start fewer than two waves per CU: 64 columns per wave make twice
    // as many (about 10 % on launches of 4-5 us; from two to four waves per CU the register path is 10-20 % faster).
    // (Not for K above 3072: where such a matrix is denser than 90 % its long rows cost the staged form 1.5x.)
    const bool few_waves = a.K <= 3072 && p.total_work <= 2u * device_cus();
    const bool epilogue = a.bias != nullptr || a.act != 0;  // (the split-row kernel does not apply one)
    if ((g_kernel_override == 6 || a.N <= 64 || (few_waves && g_kernel_override == 0)) && c_ok) {
      p.n_tiles = (uint32_t)((a.N + 63) / 64);
      p.total_work = (uint32_t)a.m_vec * p.n_tiles * (uint32_t)a.batch;
      p.per_xcd = (p.total_work + 7u) / 8u;
      g_last_kernel = 6;
      hipLaunchKernelGGL((spmm_stage_kernel<V, OutT>), dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
    } else if (a.K > kSplitMinK && !epilogue) {
      g_last_kernel = 4;
      static_assert(kSplitWaves >= 4, "wave rr < 4 stores output row 4g + rr");
      p.total_work = (((uint32_t)a.m_vec + kSplitWaves - 1u) / kSplitWaves) * p.n_tiles * (uint32_t)a.batch;
      p.per_xcd = (p.total_work + 7u) / 8u;
      hipLaunchKernelGGL((spmm_gather_split_kernel<V, OutT>), dim3(p.per_xcd * 8u), dim3(64 * kSplitWaves), 0, stream, p);
    } else if (a.N <= 64) {
      p.n_tiles = 1;
      p.total_work = (uint32_t)a.m_vec * (uint32_t)a.batch;
      p.per_xcd = (p.total_work + 7u) / 8u;
      if (c_ok) {
        g_last_kernel = 6;
        hipLaunchKernelGGL((spmm_stage_kernel<V, OutT>), dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
      } else {
        hipLaunchKernelGGL((spmm_gather_kernel<V, OutT, 4>), dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
      }
    } else if (p.total_work > 8u * device_cus()) {
      // more waves than the chip holds at two per SIMD: three per SIMD (the first feed-forward product of the encoder
      // layer, 3072 x 768 at N = 4096, 10.6 -> 9.9 us)
      hipLaunchKernelGGL((spmm_gather_kernel<V, OutT, 8, 3>), dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
    } else {
      hipLaunchKernelGGL((spmm_gather_kernel<V, OutT, 8>), dim3(p.per_xcd * 8u), dim3(64), 0, stream, p);
    }
  } else {
    p.n_tiles = (uint32_t)((a.N + 63) / 64);
    p.total_work = (uint32_t)a.m_vec * p.n_tiles * (uint32_t)a.batch;
    p.per_xcd = 0;
    hipLaunchKernelGGL((spmm_generic_kernel<V, OutT>), dim3(p.total_work), dim3(64), 0, stream, p);
  }
  return hipGetLastError();
}

// The MFMA kernels need 16-byte row segments of B and C: N % 8 == 0 and aligned bases/strides;
// 24-bit multiplies bound K and 2N; one buffer descriptor must span B.
static bool mfma_kernels_apply(const SpmmArgs &a, bool out_f16) {
  const uint64_t b_bytes = (uint64_t)a.K * (uint64_t)a.N * 2u;
  const int out_size = out_f16 ? 2 : 4;
  // The value vectors are fetched with 8-byte (V = 8) or 16-byte (V = 16) loads per lane.
  return (a.N % 8 == 0) && (reinterpret_cast<uintptr_t>(a.B) % 16 == 0) &&
         (reinterpret_cast<uintptr_t>(a.C) % 16 == 0) && (a.stride_B % 8 == 0) &&
         (reinterpret_cast<uintptr_t>(a.values) % 16 == 0) && (a.stride_values % 8 == 0) &&
         ((a.stride_C * out_size) % 16 == 0) && (a.K < (1 << 24)) && (a.N < (1 << 23)) &&
         (b_bytes + 16 <= 0xffffffffull);
}

static uint32_t padded_tiles(uint32_t t) { return t <= 1u ? 1u : t <= 2u ? 2u : t <= 4u ? 4u : (t + 7u) & ~7u; }

bool balanced_kernel_applies(const SpmmArgs &a, int V, bool out_f16) {
  // (one batch element's C is addressed through a 32-bit buffer descriptor, and lanes that must not store carry an
  // offset of 2 GiB)
  return mfma_kernels_apply(a, out_f16) && (uint64_t)a.m_vec * (uint64_t)V * (uint64_t)a.N * (out_f16 ? 2u : 4u) <= 0x80000000ull;
}

template <int V, typename OutT>
static void launch_balanced_v(const SpmmArgs &p, const BalancedArgs &s, uint32_t grid, bool device_count, hipStream_t stream) {
  if (!device_count) hipLaunchKernelGGL((spmm_balanced_kernel<V, OutT, false>), dim3(grid), dim3(64), 0, stream, p, s);
  else hipLaunchKernelGGL((spmm_balanced_kernel<V, OutT, true>), dim3(grid), dim3(64), 0, stream, p, s);
}

hipError_t launch_spmm_balanced(const SpmmArgs &a, int V, bool out_f16, const ScheduleView &sv, int n_items,
                                bool device_count, hipStream_t stream, int bundle_base) {
  SpmmArgs p = a;
  p.n_tiles = (uint32_t)((a.N + 63) / 64);
  BalancedArgs s;
  s.header = sv.header;
  s.items = sv.items;
  s.counters = sv.counters;
  s.partials = sv.partials;
  s.n_items = n_items;
  s.tiles_padded = padded_tiles(p.n_tiles);
  s.bundles = bundle_base >= 0 ? sv.bundles : nullptr;
  s.bundle_base = bundle_base;
  const uint64_t units = (uint64_t)n_items * s.tiles_padded * (uint64_t)a.batch;
  if (units >= (1ull << 31)) return hipErrorInvalidValue;
  if (units == 0) return hipSuccess;
  const uint32_t grid = (uint32_t)units;
  g_last_kernel = 7;
  if (V == 8) {
    if (out_f16) launch_balanced_v<8, _Float16>(p, s, grid, device_count, stream);
    else launch_balanced_v<8, float>(p, s, grid, device_count, stream);
  } else {
    if (out_f16) launch_balanced_v<16, _Float16>(p, s, grid, device_count, stream);
    else launch_balanced_v<16, float>(p, s, grid, device_count, stream);
  }
  return hipGetLastError();
}

hipError_t launch_spmm(const SpmmArgs &a, int V, bool out_f16, hipStream_t stream) {
  const int out_size = out_f16 ? 2 : 4;
  const bool fast = mfma_kernels_apply(a, out_f16);
  int which = 1;
  if (fast) {
    // The slab kernel pays off when enough vector-rows share a slab and there are enough
    // workgroups to fill the chip; otherwise one wave per (vector-row, 128 columns).
    const uint64_t slabs = (uint64_t)((a.N + 63) / 64) * (uint64_t)a.batch;
    const uint64_t blocks = slabs * (uint64_t)((a.m_vec + 31) / 32);
    // The slab kernel addresses one batch element's C through a 32-bit buffer descriptor, and marks the lanes
    // that must not store with an offset of 2 GiB.
    const bool c_ok = (uint64_t)a.m_vec * (V == 8 ? 8u : 16u) * (uint64_t)a.N * out_size <= (uint64_t)kSlabDropStore;
    const bool slab_ok = slab_fits(a.K, V, 4) && c_ok;
    // Matrices too tall for a 64-column slab can take slabs 32 columns wide, twice as many.  A tall slab is not
    // double-buffered, so it pays only where many vector-rows share it, and only for V = 8: with V = 16 a
    // gathered row of B already serves 16 output rows (measured: 1.2-1.3x over the gather kernel for V = 8 from
    // 256 vector-rows on, 0.8-0.9x for V = 16, 0.5-0.7x with 64 vector-rows at 90 % sparsity and above).
    const bool narrow_ok = !slab_ok && slab_fits(a.K, V, 2) && c_ok;
    // (measured on a sweep of shapes at 90 % sparsity: with V = 8 the slab kernel is 1.15-1.4x faster than the gather
    // kernel from 512 such blocks on, with V = 16 from 1024 (fp16 C) or 2048 (fp32 C, where the gather kernel's
    // whole-line stores keep it level with the slab kernel for longer); below that the two tie or the gather kernel
    // wins)
    // (N <= 64: the alternative is the staged gather kernel, which the slab kernel beats by 1.2-1.3x from 512 on)
    const uint32_t enough = (V == 8 || a.N <= 64) ? 512u : out_f16 ? 1024u : 2048u;
    // With the density known (a plan carries the pattern's vector count), a block of 32 vector-rows is counted by
    // the work in it: the thresholds above were measured at 90 % sparsity, and at 70 % the slab kernel pays from a
    // third of the blocks on (measured 1.1-1.28x over the gather kernels on shapes just below the thresholds).
    uint64_t weighted = blocks;
    if (a.mean_row_vectors > 0 && a.K > 0) {
      const uint64_t percent = ((uint64_t)a.mean_row_vectors * 100u) / (uint64_t)a.K;  // density in percent (vectors per row / K)
      if (percent > 10u) weighted = blocks * (percent < 40u ? percent : 40u) / 10u;
    }
    which = (slab_ok && a.m_vec >= 64 && weighted >= enough) ? 3 : 2;
    if (narrow_ok && V == 8 && a.m_vec >= 256 && 2u * blocks >= 1024) which = 5;
    // (known to be at least 30 % dense, a slab's rows are used often enough from half as many vector-rows on:
    // 1.3-1.45x over the gather kernel on 1024 x 2048 at 50 and 70 % sparsity, level at 80 %)
    if (narrow_ok && V == 8 && a.m_vec >= 128 && 2u * blocks >= 1024 && a.mean_row_vectors > 0 &&
        (int64_t)a.mean_row_vectors * 10 >= (int64_t)a.K * 3)
      which = 5;
    // Very sparse patterns with V = 16 and fp32 C: a vector-row is one step, the slab kernel's per-row work (claim,
    // table entry, store set-up) outweighs it, and the gather kernels win (measured at 95 and 98 % sparsity up to 32
    // vectors per row: 1.13-1.18x; with V = 8 the two tie, and between the gather kernels the density changes nothing).
    if (which == 3 && !out_f16 && V == 16 && a.mean_row_vectors > 0 && a.mean_row_vectors <= 32) which = 2;
    // Slabs 128 columns wide where they fit (K up to about 570, one buffer): a step then feeds eight MFMAs, and the
    // work around them (cursor, loads, value tile, addresses) is spent once per 128 columns.  Measured on K = 256 and
    // 512: 4-13 % on fp16 outputs from two such column tiles on, 7-15 % at 70 % sparsity whatever the output; level
    // on fp32 outputs at 90 % and above (there the stores bound the kernel), where the double-buffered 64-column slab stays.
    const bool wide_ok = which == 3 && slab_fits(a.K, V, 8) && a.N >= 192;
    const bool dense_known = a.mean_row_vectors > 0 && (int64_t)a.mean_row_vectors * 5 >= (int64_t)a.K;  // 20 % and denser
    if (wide_ok && (out_f16 || dense_known)) which = 9;
    if (g_kernel_override == 2 || g_kernel_override == 6) which = 2;
    if (g_kernel_override == 3 && slab_ok) which = 3;
    if (g_kernel_override == 9 && slab_fits(a.K, V, 8) && c_ok && a.m_vec >= 64) which = 9;
    if (g_kernel_override == 3 && narrow_ok) which = 5;
    if (a.bias != nullptr || a.act != 0) which = 2;  // the kernels that apply the linear-layer epilogue
  }
  if (g_kernel_override == 1) which = 1;
  g_last_kernel = which;
  if (V == 8) return out_f16 ? launch_v<8, _Float16>(a, which, stream) : launch_v<8, float>(a, which, stream);
  return out_f16 ? launch_v<16, _Float16>(a, which, stream) : launch_v<16, float>(a, which, stream);
}

}  // namespace sspmm
