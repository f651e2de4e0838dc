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

// ------------------------------------------------------------------------------------------
// Slab kernel: B resident in LDS, operands formed by LDS transpose reads.
//
// When K is small enough that a 64-column slab of B (K rows x 128 bytes) fits in the 160 KB of
// LDS, a workgroup of 8 waves copies the slab into LDS once with coalesced 16-byte loads and
// then walks a block of vector-rows against it, so HBM/L2 only see each slab once per row
// block, the value vectors, the column indices and the stores of C.
//
// ds_read_b64_tr_b16 is what makes this cheap.  Within 16 lanes, lane n receives element n of the
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
// The vector-rows of a row block are dealt to the waves round-robin, and the loads of a step are
// issued kSlabRing - 1 steps ahead (across vector-row boundaries).  Row K of the slab is all
// zeros: unused k slots of a partial step point there.
static constexpr int kSlabWaves = 8;
static constexpr int kSlabThreads = kSlabWaves * 64;
static constexpr int kSlabRowBytes = 128;       // 64 columns of fp16
// Per-wave LDS: the value tile of a step (32 vectors x V halfs; the V = 8 transpose read touches 16
// bytes past its 512).
static constexpr int val_tile_bytes(int V) { return V == 8 ? 528 : 1024; }
static constexpr int wave_lds_bytes(int V) { return val_tile_bytes(V); }

static constexpr int kSlabRing = 8;  // steps whose loads are in flight or waiting in registers

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;

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

template <int V>
struct SlabLoads {
  uint32_t col[2];  // column index of k slots 8g + m/4 and 8g + 4 + m/4
  typename SlabVals<V>::type vraw;
};

// Walks one wave's sequence of steps.  The (vector-row, first vector, end vector) triples of the
// row block are copied into a table in LDS when the workgroup starts; wave w takes the positions
// w, w + 8, w + 16, ... of the block, so finding the next vector-row is one broadcast LDS read and
// no scalar-memory or atomic round trip sits in the main loop.  A vector-row of n vectors is
// ceil(n / 32) steps, and an empty vector-row is one step without vectors (its zeros still have
// to be written).  Two cursors run over the same sequence: the head issues the loads of a step,
// the tail, kSlabRing - 1 steps behind it, consumes them.  Either cursor reads the table entry of
// its following vector-row one row ahead, so that the LDS latency is off the critical path.
typedef int intx4 __attribute__((ext_vector_type(4)));
struct SlabCursor {
  int row, kc, end;  // current step: vectors [kc, min(kc + 32, end)) of vector-row `row`
  bool valid;
  intx4 next;        // table entry of the following vector-row (still in vector registers)
  bool next_valid;
  int count;         // rows requested so far
};

struct SlabRows {      // what the cursors need to find rows
  const intx4 *table;  // LDS: n_rows entries (row, first vector, end vector, -) and an all-zero entry behind them
  int n_rows, wave;
};

__device__ __forceinline__ void cursor_prefetch(SlabCursor &c, const SlabRows &rows) {
  const int idx = rows.wave + kSlabWaves * c.count;
  ++c.count;
  c.next_valid = idx < rows.n_rows;
  c.next = rows.table[min(idx, rows.n_rows)];
}

__device__ __forceinline__ void cursor_take_next(SlabCursor &c, const SlabRows &rows) {
  c.row = __builtin_amdgcn_readfirstlane(c.next[0]);
  c.kc = __builtin_amdgcn_readfirstlane(c.next[1]);
  c.end = __builtin_amdgcn_readfirstlane(c.next[2]);
  c.valid = c.next_valid;
  cursor_prefetch(c, rows);
}

__device__ __forceinline__ void cursor_advance(SlabCursor &c, const SlabRows &rows) {
  c.kc += 32;
  if (c.kc >= c.end) cursor_take_next(c, rows);
}

template <int V>
__device__ __forceinline__ void slab_issue(SlabLoads<V> &r, int kc, int end, int lane, uint32_t slot0,
                                           __amdgpu_buffer_rsrc_t srd_cols, const uint16_t *vals) {
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
template <int V, typename OutT>
struct SlabStore;

__device__ __forceinline__ uint32_t dpp_from_m_minus_8(uint32_t keep, uint32_t src) {  // lanes m >= 8 take src of lane m - 8
  return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)src, 0x118, 0xf, 0xc, false);
}
__device__ __forceinline__ uint32_t dpp_from_m_plus_8(uint32_t keep, uint32_t src) {  // lanes m < 8 take src of lane m + 8
  return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)src, 0x108, 0xf, 0x3, false);
}

template <int V>
struct SlabStore<V, float> {
  static constexpr int kInstr = V / 4;  // 2 tile pairs x (V / 8) row halves
  uint32_t voff[V / 8];                 // byte offset of the lane's 16 bytes for tile pair 0, per row half
  int col[V / 8];                       // its first column
  __device__ __forceinline__ void init(int lane, int n0, int N) {
    const int m = lane & 15, g = lane >> 4;
#pragma unroll
    for (int h = 0; h < V / 8; ++h) {
      const int row = 8 * h + (m & 7);
      const int tile = h == 0 ? (m >> 3) : 1 - (m >> 3);
      col[h] = n0 + 16 * tile + 4 * g;
      voff[h] = ((uint32_t)row * (uint32_t)N + (uint32_t)col[h]) * 4u;
    }
  }
  __device__ __forceinline__ void store(const floatx4 (&acc)[4], __amdgpu_buffer_rsrc_t srd, uint32_t crow, int N) const {
#pragma unroll
    for (int qp = 0; qp < 2; ++qp) {
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
        if (col[h] + 32 * qp < N) slab_store_line(line, srd, voff[h] + 128u * qp, crow);
      }
    }
  }
};

template <int V>
struct SlabStore<V, _Float16> {
  uint32_t voff[V / 8];
  int col[V / 8];
  __device__ __forceinline__ void init(int lane, int n0, int N) {
    const int m = lane & 15, g = lane >> 4;
#pragma unroll
    for (int h = 0; h < V / 8; ++h) {
      const int row = 8 * h + (m & 7);
      const int pair = h == 0 ? (m >> 3) : 1 - (m >> 3);
      col[h] = n0 + 32 * pair + 16 * (g & 1) + 8 * (g >> 1);
      voff[h] = ((uint32_t)row * (uint32_t)N + (uint32_t)col[h]) * 2u;
    }
  }
  __device__ __forceinline__ void store(const floatx4 (&acc)[4], __amdgpu_buffer_rsrc_t srd, uint32_t crow, int N) const {
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
      if (col[h] < N) slab_store_line(line, srd, voff[h], crow);
    }
  }
};

template <int V, typename OutT>
__global__ __launch_bounds__(kSlabThreads) void spmm_slab_kernel(const SpmmArgs p,
                                                                 const int32_t *__restrict__ row_offsets,
                                                                 const int32_t *__restrict__ row_indices) {
  extern __shared__ __align__(16) unsigned char lds[];
  const uint32_t id = blockIdx.x;
  // The hardware deals consecutive block ids round-robin to the 8 XCDs, each with its own L2, so
  // blocks whose ids are equal modulo 8 share an L2.  With at least 8 batch elements, all blocks of
  // one batch element (every column tile and row block) are given the same residue: the value
  // vectors, read once per column tile, and the slab, read once per row block, then come from
  // that L2 after the first touch.  With fewer batch elements the residue is taken from the slab.
  const uint32_t xcd = id & 7u, qd = id >> 3;
  uint32_t rb, tile, batch;
  if (p.group_by_batch) {
    const uint32_t per_batch = p.n_tiles * p.row_blocks;
    const uint32_t rem = qd % per_batch;
    batch = (qd / per_batch) * 8u + xcd;
    tile = rem / p.row_blocks;
    rb = rem % p.row_blocks;
    if (batch >= (uint32_t)p.batch) return;
  } else {
    rb = qd % p.row_blocks;
    const uint32_t slab_id = (qd / p.row_blocks) * 8u + xcd;
    if (slab_id >= p.n_slabs) return;
    tile = slab_id % p.n_tiles;
    batch = slab_id / p.n_tiles;
  }

  const int tid = threadIdx.x, lane = tid & 63, m = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // tell the compiler it is wave-uniform
  const int n0 = (int)tile * 64;
  const uint16_t *vals = p.values + (int64_t)batch * p.stride_values;
  const uint16_t *bmat = p.B + (int64_t)batch * p.stride_B;
  const uint32_t b_bytes = (uint32_t)p.K * (uint32_t)p.N * 2u;
  const __amdgpu_buffer_rsrc_t srd_b = make_srd(bmat, b_bytes);
  uint32_t touch_sink = 0;  // keeps the destination register of the warming loads reserved

  // ---- the row table of this block: thread i fetches entry i (kSlabMaxRows < kSlabThreads).  The
  // loads go out first so that they do not queue behind the slab and the warming loads.
  const int row_lo = (int)(rb * p.rows_per_block);
  const int row_hi = min(p.m_vec, row_lo + (int)p.rows_per_block);
  const int n_rows = row_hi - row_lo;
  intx4 table_entry = {0, 0, 0, 0};
  if (tid < n_rows) {
    table_entry[0] = row_indices ? row_indices[row_lo + tid] : row_lo + tid;
    table_entry[1] = row_offsets[table_entry[0]];
    table_entry[2] = row_offsets[table_entry[0] + 1];
  }
  // ---- stage the slab: unit u = 16 bytes = columns n0 + 8*(u % 8) .. +7 of row u / 8; the
  // 32-byte segment (u % 8) / 2 of row c lands at segment ((u % 8) / 2) ^ ((c >> 1) & 3).
  const uint32_t units = (uint32_t)p.K * 8u;
  const uint32_t n2 = (uint32_t)p.N * 2u;
  for (uint32_t u0 = 0; u0 < units; u0 += kSlabThreads * 8) {
    uintx4 d[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t u = u0 + i * kSlabThreads + tid;
      const uint32_t col = (uint32_t)n0 + (u & 7u) * 8u;
      const uint32_t off = (u < units && col < (uint32_t)p.N) ? __umul24(u >> 3, n2) + col * 2u : b_bytes;
      d[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(srd_b, off, 0, 0));
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t u = u0 + i * kSlabThreads + tid;
      const uint32_t c = u >> 3;
      const uint32_t dst = c * kSlabRowBytes + (((u & 7u) * 16u) ^ (((c >> 1) & 3u) << 5));
      if (u < units) *reinterpret_cast<uintx4 *>(lds + dst) = d[i];
    }
  }
  // ---- warm the L2 with this block's value vectors.  Under a saturating stream of C stores an
  // HBM read takes several microseconds, far more than the register ring of the main loop covers,
  // so every 128-byte line of the block's (contiguous) value range is touched once now, behind the
  // loads of the slab; nothing ever waits for these loads, and the main loop then finds the
  // lines in the L2 or on their way to it.  One 4-byte load per lane touches 64 lines per instruction.
  if (row_indices == nullptr) {
    const uint32_t lo = (uint32_t)row_offsets[row_lo] * (V * 2u), hi = (uint32_t)row_offsets[row_hi] * (V * 2u);
    const __amdgpu_buffer_rsrc_t srd_touch = make_srd(vals, hi);
    uint32_t sink = 0;
    for (uint32_t off = (lo & ~127u) + (uint32_t)tid * 128u; off < hi; off += kSlabThreads * 128u)
      asm volatile("buffer_load_dword %0, %1, %2, 0 offen" : "+v"(sink) : "v"(off), "s"(srd_touch) : "memory");
    touch_sink = sink;
  }

  const uint32_t zero_row = (uint32_t)p.K;
  if (tid < 8) *reinterpret_cast<uintx4 *>(lds + zero_row * kSlabRowBytes + tid * 16) = uintx4{0u, 0u, 0u, 0u};
  const uint32_t tiles_off = (zero_row + 1u) * kSlabRowBytes;
  intx4 *table = reinterpret_cast<intx4 *>(lds + tiles_off + kSlabWaves * wave_lds_bytes(V));
  if (tid <= n_rows) table[tid] = table_entry;
  __syncthreads();

  // ---- per-lane constants
  unsigned char *val_tile = lds + tiles_off + wave * wave_lds_bytes(V);
  constexpr uint32_t kLaneBytes = V * 2u * 32u / 64u;
  unsigned char *val_dst = val_tile + lane * kLaneBytes;
  // value tile rows are V*2 bytes; transpose read h picks rows 8g + 4h + m/4
  const uint32_t a_off = (uint32_t)(8 * g + (m >> 2)) * (V * 2u) + (uint32_t)(m & 3) * 8u;
  const uint32_t slot0 = (uint32_t)(8 * g + (m >> 2));
  const uint32_t b_lane_off = (uint32_t)(m & 3) * 8u;
  SlabStore<V, OutT> out;
  out.init(lane, n0, p.N);
  // One buffer descriptor spans this batch element's C (the launcher checks it is below 4 GiB).
  const uint32_t c_vrow_bytes = (uint32_t)V * (uint32_t)p.N * (uint32_t)sizeof(OutT);
  const __amdgpu_buffer_rsrc_t srd_c = make_srd(reinterpret_cast<OutT *>(p.C) + (int64_t)batch * p.stride_C,
                                                (uint32_t)p.m_vec * c_vrow_bytes);
  const uint32_t nvec = (uint32_t)row_offsets[p.m_vec];
  const __amdgpu_buffer_rsrc_t srd_cols = make_srd(p.col_idx, nvec * 4u);

  // ---- this wave's stream of steps
  SlabRows rows;
  rows.table = table;
  rows.n_rows = n_rows;
  rows.wave = wave;
  SlabCursor head;  // issues loads
  head.count = 0;
  cursor_prefetch(head, rows);
  cursor_take_next(head, rows);
  if (!head.valid) return;
  SlabCursor tail;  // consumes them
  tail.count = 0;
  cursor_prefetch(tail, rows);
  cursor_take_next(tail, rows);

  SlabLoads<V> ld[kSlabRing];
#pragma unroll
  for (int i = 0; i < kSlabRing - 1; ++i) {
    // Loads are issued whether or not the head still has a step (an exhausted head has kc = end = 0:
    // the value load is out of bounds and returns zeros), so that the number of loads in flight
    // behind any ring slot is a compile-time constant and the waits below can be exact.
    slab_issue<V>(ld[i], head.kc, head.end, lane, slot0, srd_cols, vals);
    if (head.valid) cursor_advance(head, rows);
  }
  // the value tile of the first step
  *reinterpret_cast<typename SlabVals<V>::type *>(val_dst) = ld[0].vraw;

  floatx4 acc[4];
  bool first = true;  // first step of a vector-row: accumulate onto zero
  for (;;) {
#pragma unroll
    for (int u = 0; u < kSlabRing; ++u) {
      constexpr int R = kSlabRing;
      const int cur = u, nxt = (u + 1) % R, fill = (u + R - 1) % R;
      slab_issue<V>(ld[fill], head.kc, head.end, lane, slot0, srd_cols, vals);
      if (head.valid) cursor_advance(head, rows);
      const int row = tail.row;
      const int left = tail.end - tail.kc;  // vectors of this vector-row from this step on
      cursor_advance(tail, rows);

      // A operand: this step's value tile
      Half8Bits a;
      {
        const uintx2 lo = lds_read_tr(val_tile, a_off);
        const uintx2 hi = lds_read_tr(val_tile, a_off + 4u * (V * 2u));
        a.u[0] = lo[0]; a.u[1] = lo[1]; a.u[2] = hi[0]; a.u[3] = hi[1];
      }
      // B operands: two column indices per lane; unused k slots of a partial step read the zero row
      uint32_t addr[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t c = ((int)slot0 + 4 * h < left) ? ld[cur].col[h] : zero_row;
        const uint32_t t = c << 4;
        addr[h] = (t << 3) | ((t & 0x60u) | b_lane_off);
      }
      Half8Bits b[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uintx2 lo = lds_read_tr(lds, addr[0] ^ ((uint32_t)q << 5));
        const uintx2 hi = lds_read_tr(lds, addr[1] ^ ((uint32_t)q << 5));
        b[q].u[0] = lo[0]; b[q].u[1] = lo[1]; b[q].u[2] = hi[0]; b[q].u[3] = hi[1];
      }
      // the next step's value tile goes to LDS behind the reads above (LDS operations of a wave
      // execute in order)
      if (tail.valid) *reinterpret_cast<typename SlabVals<V>::type *>(val_dst) = ld[nxt].vraw;

      if (first) {
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[q].h, a.h, zero, 0, 0, 0);
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[q].h, a.h, acc[q], 0, 0, 0);
      }
      first = left <= 32;
      if (first) {  // last step of the vector-row: write its V x 64 tile of C
        out.store(acc, srd_c, (uint32_t)row * c_vrow_bytes, p.N);
      }
      if (!tail.valid) {
        asm volatile("" ::"v"(touch_sink));  // the warming loads may still be writing this register
        return;
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

static int g_kernel_override = 0;  // 0 auto, 1 generic, 2 gather, 3 slab (tests and tuning)

int set_kernel_override(int which) {
  const int old = g_kernel_override;
  g_kernel_override = which;
  return old;
}

static constexpr uint32_t kSlabMaxRows = 255;  // vector-rows per workgroup (row table of 256 entries)
static constexpr int kSlabMaxK = 1180;  // slab + zero row + 8 value tiles + row table must fit in 160 KB of LDS

template <int V, typename OutT>
static hipError_t launch_slab(const SpmmArgs &a, hipStream_t stream) {
  SpmmArgs p = a;
  p.n_tiles = (uint32_t)((a.N + 63) / 64);
  p.n_slabs = p.n_tiles * (uint32_t)a.batch;
  // Aim at ~4 workgroups per CU, but keep at least 32 vector-rows per workgroup so that the copy
  // of the slab into LDS stays a small part of the workgroup's traffic, and at most kSlabMaxRows
  // (the row table in LDS).
  const uint32_t rb_target = p.n_slabs >= 1024u ? 1u : 1024u / p.n_slabs;
  uint32_t rows = ((uint32_t)a.m_vec + rb_target - 1u) / rb_target;
  if (rows < 32u) rows = 32u;
  if (rows > kSlabMaxRows) {
    const uint32_t blocks = ((uint32_t)a.m_vec + kSlabMaxRows - 1u) / kSlabMaxRows;
    rows = ((uint32_t)a.m_vec + blocks - 1u) / blocks;
  }
  p.rows_per_block = rows;
  p.row_blocks = ((uint32_t)a.m_vec + rows - 1u) / rows;
  const size_t lds = (size_t)(a.K + 1) * kSlabRowBytes + kSlabWaves * wave_lds_bytes(V) + 16 * (rows + 1);
  auto kern = spmm_slab_kernel<V, OutT>;
  static size_t lds_allowed = 64 * 1024;  // per instantiation
  if (lds > lds_allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    lds_allowed = 160 * 1024;
  }
  p.group_by_batch = a.batch >= 8 ? 1u : 0u;
  const uint32_t grid = p.group_by_batch ? (((uint32_t)a.batch + 7u) / 8u) * 8u * p.n_tiles * p.row_blocks
                                         : ((p.n_slabs + 7u) / 8u) * 8u * p.row_blocks;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kSlabThreads), lds, stream, p, a.row_offsets, a.row_indices);
  return hipGetLastError();
}

template <int V, typename OutT>
static hipError_t launch_v(const SpmmArgs &a, int which, hipStream_t stream) {
  SpmmArgs p = a;
  if (which == 3) return launch_slab<V, OutT>(a, stream);
  if (which == 2) {
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

hipError_t launch_spmm(const SpmmArgs &a, int V, bool out_f16, hipStream_t stream) {
  // The MFMA kernels need 16-byte row segments of B and C: N % 8 == 0 and aligned bases/strides;
  // 24-bit multiplies bound K and 2N; one buffer descriptor must span B.
  const uint64_t b_bytes = (uint64_t)a.K * (uint64_t)a.N * 2u;
  const int out_size = out_f16 ? 2 : 4;
  const bool fast = (a.N % 8 == 0) && (reinterpret_cast<uintptr_t>(a.B) % 16 == 0) &&
                    (reinterpret_cast<uintptr_t>(a.C) % 16 == 0) && (a.stride_B % 8 == 0) &&
                    ((a.stride_C * out_size) % 16 == 0) && (a.K < (1 << 24)) && (a.N < (1 << 23)) &&
                    (b_bytes + 16 <= 0xffffffffull);
  int which = 1;
  if (fast) {
    // The slab kernel pays off when enough vector-rows share a slab and there are enough
    // workgroups to fill the chip; otherwise one wave per (vector-row, 128 columns).
    const uint64_t slabs = (uint64_t)((a.N + 63) / 64) * (uint64_t)a.batch;
    const uint64_t blocks = slabs * (uint64_t)((a.m_vec + 31) / 32);
    // The slab kernel addresses one batch element's C through a 32-bit buffer descriptor.
    const bool slab_ok = a.K <= kSlabMaxK && (uint64_t)a.m_vec * (V == 8 ? 8u : 16u) * (uint64_t)a.N * out_size < 0xffffffffull;
    which = (slab_ok && a.m_vec >= 64 && blocks >= 1024) ? 3 : 2;
    if (g_kernel_override == 2) which = 2;
    if (g_kernel_override == 3 && slab_ok) which = 3;
  }
  if (g_kernel_override == 1) which = 1;
  if (V == 8) return out_f16 ? launch_v<8, _Float16>(a, which, stream) : launch_v<8, float>(a, which, stream);
  return out_f16 ? launch_v<16, _Float16>(a, which, stream) : launch_v<16, float>(a, which, stream);
}

}  // namespace sspmm
