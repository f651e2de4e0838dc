// Residual add + LayerNorm on feature-major activations, the glue between the sparse products of the
// encoder-layer configuration (the reference's model code keeps these in torch on token-major tensors,
// reference end2end/sspmm_e2e/end_to_end.py:58-75; the SpMM wants and returns [features, tokens], and
// normalising that layout through torch costs two transposed copies per LayerNorm).
//
//   out[h, t] = (s[h, t] - mean_t) * rsqrt(var_t + eps) * gamma[h] + beta[h],   s = fp16(x + a)
//
// with mean and (biased) variance over the H features of token t, in fp32.  HBM-bound: x and a read once, out
// written once (6 * H * T bytes); a workgroup of eight waves owns 16 tokens (32 bytes of every row), has the loads of
// six rows per thread in flight together, keeps the H x 16 sums in LDS as fp16 and makes its passes (mean,
// variance, result) over LDS.  The four workgroups that share the 128-byte lines of 64 consecutive tokens get
// workgroup ids that the hardware's round-robin deal puts on one XCD, so a line crosses the fabric once.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "layer_kernels.h"

namespace sspmm {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// TOK tokens per workgroup (TOK / 4 lanes of four tokens each), THREADS threads, TRIP rows per thread whose loads are
// in flight together.
template <int TOK, int THREADS, int TRIP>
struct LnShape {
  static constexpr int kLanes = TOK / 4;
  static constexpr int kRowGroups = THREADS / kLanes;
  static constexpr int kParts = 64 / TOK;  // workgroups that share the 128-byte lines of 64 consecutive tokens
};

// Sum over the workgroup's row groups of one value per token group: across the row groups of a wave with lane
// exchanges, across the waves through LDS.  Contains barriers.
template <int LANES, int THREADS>
__device__ __forceinline__ floatx4 block_sum_per_token(floatx4 v, floatx4 *red, int tl) {
#pragma unroll
  for (int d = LANES; d < 64; d <<= 1)
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += __shfl_xor(v[i], d, 64);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();  // red may still be read from the call before
  if (lane < LANES) red[wave * LANES + tl] = v;
  __syncthreads();
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < THREADS / 64; ++w) s += red[w * LANES + tl];
  return s;
}

template <int TOK, int THREADS, int TRIP, bool NT = true>
__global__ __launch_bounds__(THREADS) void add_layernorm_kernel(int H, int T, const _Float16 *__restrict__ x,
                                                                 const _Float16 *__restrict__ a,
                                                                 const _Float16 *__restrict__ gamma,
                                                                 const _Float16 *__restrict__ beta, float eps,
                                                                 _Float16 *__restrict__ out) {
  typedef LnShape<TOK, THREADS, TRIP> S;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  half4 *sums = reinterpret_cast<half4 *>(lds_raw);                            // [H][S::kLanes] groups of four tokens
  floatx4 *red = reinterpret_cast<floatx4 *>(lds_raw + (size_t)H * TOK * 2);  // [waves][S::kLanes]
  const int tl = threadIdx.x % S::kLanes, rg = threadIdx.x / S::kLanes;
  // workgroup id -> token group: ids congruent modulo 8 share an XCD, and the parts of a 64-token line group go to
  // ids 8 apart, so the workgroups that share 128-byte lines share an L2
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int first = (((idx / S::kParts) * 8 + xcd) * S::kParts + (idx % S::kParts)) * TOK;
  if (first >= T) return;  // (the whole workgroup: the grid is padded to eight line groups)
  const int t0 = first + 4 * tl;
  const bool live = t0 < T;  // (T is a multiple of 4: a group of four tokens is inside or outside as a whole)
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  // (the loads of TRIP rows are issued together: the kernel is bound by how many bytes its workgroups keep in flight)
  for (int h0 = rg; h0 < H; h0 += S::kRowGroups * TRIP) {
    half4 xs[TRIP], as[TRIP];
#pragma unroll
    for (int u = 0; u < TRIP; ++u) {
      const int h = h0 + u * S::kRowGroups;
      xs[u] = half4{0, 0, 0, 0};
      as[u] = half4{0, 0, 0, 0};
      if (live && h < H) {
        if (NT) {
          xs[u] = __builtin_nontemporal_load(reinterpret_cast<const half4 *>(x + (size_t)h * T + t0));
          if (a) as[u] = __builtin_nontemporal_load(reinterpret_cast<const half4 *>(a + (size_t)h * T + t0));
        } else {
          xs[u] = *reinterpret_cast<const half4 *>(x + (size_t)h * T + t0);
          if (a) as[u] = *reinterpret_cast<const half4 *>(a + (size_t)h * T + t0);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < TRIP; ++u) {
      const int h = h0 + u * S::kRowGroups;
      if (h < H) {
        const half4 s = xs[u] + as[u];  // fp16 sum, as the unfused add gives
        sums[h * S::kLanes + tl] = s;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += (float)s[i];
      }
    }
  }
  floatx4 mean = block_sum_per_token<S::kLanes, THREADS>(acc, red, tl);
  mean *= 1.0f / (float)H;
  acc = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int h = rg; h < H; h += S::kRowGroups) {
    const half4 s = sums[h * S::kLanes + tl];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float d = (float)s[i] - mean[i];
      acc[i] += d * d;
    }
  }
  floatx4 rstd = block_sum_per_token<S::kLanes, THREADS>(acc, red, tl);
#pragma unroll
  for (int i = 0; i < 4; ++i) rstd[i] = rsqrtf(rstd[i] / (float)H + eps);
  if (!live) return;
  for (int h = rg; h < H; h += S::kRowGroups) {
    const half4 s = sums[h * S::kLanes + tl];
    const float w = gamma ? (float)gamma[h] : 1.0f, b = beta ? (float)beta[h] : 0.0f;
    half4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (_Float16)(((float)s[i] - mean[i]) * rstd[i] * w + b);
    *reinterpret_cast<half4 *>(out + (size_t)h * T + t0) = o;
  }
}

template <int TOK, int THREADS, int TRIP, bool NT = true>
static hipError_t launch_ln(int H, int T, const uint16_t *x, const uint16_t *a, const uint16_t *gamma, const uint16_t *beta,
                            float eps, uint16_t *out, hipStream_t stream) {
  const size_t lds = (size_t)H * TOK * 2 + (size_t)(THREADS / 64) * (TOK / 4) * 16;
  auto kern = add_layernorm_kernel<TOK, THREADS, TRIP, NT>;
  if (lds > 64 * 1024) {
    // the runtime is told once per device and size
    static int raised[16] = {};
    static std::mutex raised_mutex;
    std::lock_guard<std::mutex> lock(raised_mutex);
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) dev = -1;
    if (dev < 0 || raised[dev] < (int)lds) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return e;
      if (dev >= 0) raised[dev] = (int)lds;
    }
  }
  const int line_groups = (T + 63) / 64;
  const int blocks = ((line_groups + 7) / 8) * 8 * (64 / TOK);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(THREADS), lds, stream, H, T, reinterpret_cast<const _Float16 *>(x),
                     reinterpret_cast<const _Float16 *>(a), reinterpret_cast<const _Float16 *>(gamma),
                     reinterpret_cast<const _Float16 *>(beta), eps, reinterpret_cast<_Float16 *>(out));
  return hipGetLastError();
}

hipError_t launch_add_layernorm(int H, int T, const uint16_t *x, const uint16_t *a, const uint16_t *gamma,
                                const uint16_t *beta, float eps, uint16_t *out, hipStream_t stream) {
  // 16 tokens and eight waves per workgroup, six rows per thread in flight (measured on 768 x 4096 against 32 and 64
  // tokens, 4 to 16 waves, 3 to 12 rows: 8.5 us against 9-15)
  return launch_ln<16, 512, 6>(H, T, x, a, gamma, beta, eps, out, stream);
}

// ------------------------------------------------------------------------------------------
// Dense softmax(Q^T K / sqrt(d)) attention on feature-major activations (the dense attention of the
// reference's comparison block, reference end2end/sspmm_e2e/end_to_end.py:84-97, which runs it in torch on
// token-major tensors).  The SpMM that produces q, k, v leaves them as [features, tokens]; torch's attention
// wants [batch, heads, tokens, head size] with the head size contiguous, which costs one transposed copy of all
// three before it and one of the context behind it.  Here a workgroup of four waves owns 64 queries of one
// (batch element, head): its 64 columns of Q go to LDS once, and the head's K and V pass through LDS in blocks of
// 64 keys (64 features x 64 tokens each, as they lie in memory; two buffers, the next block's loads in flight in
// registers while the current one is computed, one barrier per block), 45 KB of LDS in all, so three workgroups
// share a CU.  Each wave computes for 32 queries (two sets of 16) and half of every block's keys
//     scores^T[key, query] = sum_d K[d, key] Q[d, query]          (MFMA; both operands by transpose reads)
//     out[d, query]        = sum_key V[d, key] P[query, key]       (MFMA; V read directly, P from registers)
// per block with the running maximum and sum of the usual one-pass softmax.  The scores come out of the first
// product with a query per lane and four consecutive keys per accumulator, which is the second product's operand
// layout once its contraction slots are numbered accordingly (slots 0-3 and 4-7 of lane group g = keys 4g .. 4g+3
// of two neighbouring 16-key tiles; V is read with the same numbering), so the probabilities never leave the
// registers.  The context goes back through LDS and is written feature-major in whole 128-byte lines.  Bound by
// HBM in bytes (q, k, v read once, out written once: 8 * hidden * tokens bytes; a head's K and V are re-read by its
// seq / 64 workgroups from L2), by the exponentials and the LDS reads in time.
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef uint32_t uintx2 __attribute__((ext_vector_type(2)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;

static constexpr int kAttThreads = 256;
static constexpr int kAttD = 64;          // head size
static constexpr int kAttQueries = 64;    // per workgroup, 16 per wave
static constexpr int kAttKeys = 64;       // per block of the softmax
// Row pitches in bytes, chosen so that the rows one LDS pass touches fall into different banks.  Q and K are read by
// transpose reads, 32 lanes = eight consecutive rows of 32 bytes per pass: 160-byte rows put them at bank offsets
// 0, 40, 16, 56, 32, 8, 48, 24 (of 64 four-byte banks), each eight banks wide.  V is read eight bytes per lane from
// sixteen consecutive rows: 144-byte rows put those at sixteen different multiples of four banks.
static constexpr uint32_t kAttPitchK = 64 * 2 + 32;
static constexpr uint32_t kAttPitchV = 64 * 2 + 16;
static constexpr uint32_t kAttTileK = kAttD * kAttPitchK, kAttTileV = kAttD * kAttPitchV;
static constexpr size_t kAttLds = 3 * (size_t)kAttTileK + 2 * (size_t)kAttTileV;  // Q, two K blocks, two V blocks
static constexpr int kAttMaxSeq = 16384;

union AttOperand {
  half8 h;
  uint32_t u[4];
};

// Within 16 lanes, lane n receives element n of the four 32-byte runs addressed by lanes 0-3, 4-7, 8-11, 12-15.
__device__ __forceinline__ uintx2 att_read_tr(const unsigned char *p) {
  const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4 *)p);
  return __builtin_bit_cast(uintx2, v);
}

__device__ __forceinline__ uint32_t att_pack(float lo, float hi) {
  typedef _Float16 half2v __attribute__((ext_vector_type(2)));
  const half2v h = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, h);
}

struct AttentionArgs {
  const _Float16 *q, *k, *v;
  _Float16 *out;
  long long ld, ld_out;  // elements between consecutive features
  int S, heads, units;  // units = batch elements x heads
  float scale_log2e;
};

__global__ __launch_bounds__(kAttThreads, 3) void attention_fm_kernel(const AttentionArgs p) {
  __shared__ __align__(16) unsigned char lds[kAttLds];
  const int S = p.S, qblocks = S / kAttQueries, blocks = S / kAttKeys;
  // Workgroup ids go round-robin to the 8 XCDs, each with its own L2: the query blocks of one (batch element, head)
  // take ids 8 apart, so that the head's K and V are fetched from memory once and found in that L2 by the others.
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int qb = idx % qblocks, unit = (idx / qblocks) * 8 + xcd;
  if (unit >= p.units) return;  // (the grid is padded to a multiple of eight units)
  const int head = unit % p.heads, b = unit / p.heads;
  const int tid = threadIdx.x, lane = tid & 63, m = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned char *const q_tile = lds;
  unsigned char *const k_tiles = lds + kAttTileK;      // buffer i at k_tiles + i * kAttTileK
  unsigned char *const v_tiles = lds + 3 * kAttTileK;  // buffer i at v_tiles + i * kAttTileV
  const long long tok0 = (long long)b * S;
  const _Float16 *qg = p.q + (long long)(head * kAttD) * p.ld + tok0 + qb * kAttQueries;
  const _Float16 *kg = p.k + (long long)(head * kAttD) * p.ld + tok0;
  const _Float16 *vg = p.v + (long long)(head * kAttD) * p.ld + tok0;

  // A 64 x 64 fp16 tile is 512 pieces of 16 bytes, two per thread: rows r0 and r0 + 32, piece pc.
  const int r0 = tid >> 3, pc = tid & 7;
  const long long g0 = (long long)r0 * p.ld + pc * 8, g1 = g0 + 32 * p.ld;
  const uint32_t l0 = r0 * kAttPitchK + pc * 16, l1 = l0 + 32 * kAttPitchK;    // in a Q or K tile
  const uint32_t lv0 = r0 * kAttPitchV + pc * 16, lv1 = lv0 + 32 * kAttPitchV;  // in a V tile
  uintx4 kk[2], vv[2];
  kk[0] = *reinterpret_cast<const uintx4 *>(kg + g0);
  kk[1] = *reinterpret_cast<const uintx4 *>(kg + g1);
  vv[0] = *reinterpret_cast<const uintx4 *>(vg + g0);
  vv[1] = *reinterpret_cast<const uintx4 *>(vg + g1);
  *reinterpret_cast<uintx4 *>(q_tile + l0) = *reinterpret_cast<const uintx4 *>(qg + g0);
  *reinterpret_cast<uintx4 *>(q_tile + l1) = *reinterpret_cast<const uintx4 *>(qg + g1);
  *reinterpret_cast<uintx4 *>(k_tiles + l0) = kk[0];
  *reinterpret_cast<uintx4 *>(k_tiles + l1) = kk[1];
  *reinterpret_cast<uintx4 *>(v_tiles + lv0) = vv[0];
  *reinterpret_cast<uintx4 *>(v_tiles + lv1) = vv[1];
  __syncthreads();

  // ---- Wave w works on queries 32 * (w / 2) .. + 31 of the workgroup's 64 (two sets of 16) against keys
  // 32 * (w % 2) .. + 31 of every block: an operand read of K or V then serves two products (the two query sets),
  // which halves the LDS reads per product, and the two waves that share queries merge their softmax states at the end.
  // The contraction slots of the first product are numbered so that a transpose read of 32 lanes touches eight
  // consecutive rows: slots 0-3 of lane group g are features 32u + 4g .. + 3, slots 4-7 features 32u + 16 + 4g .. + 3
  // (the same numbering for Q and K).
  const int qhalf = wave >> 1, khalf = wave & 1;
  AttOperand qop[2][2];  // [query set][u]: lane (m, g) holds its slots of query 32 * qhalf + 16 * set + m
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const unsigned char *a = q_tile + (32 * u + 4 * g + (m >> 2)) * kAttPitchK + (32 * qhalf + 16 * j) * 2 + (m & 3) * 8;
      const uintx2 lo = att_read_tr(a), hi = att_read_tr(a + 16 * kAttPitchK);
      qop[j][u].u[0] = lo[0]; qop[j][u].u[1] = lo[1]; qop[j][u].u[2] = hi[0]; qop[j][u].u[3] = hi[1];
    }

  const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
  floatx4 o[2][4] = {{zero, zero, zero, zero}, {zero, zero, zero, zero}};  // [set][dt], lane (m, g): features 16dt + 4g .. + 3 of query m
  // per query set, of query m: the largest raw score so far, and this lane's share of the sum of
  // 2^((score - max) * scale_log2e), over the keys of this wave
  float run_max[2] = {-3.0e38f, -3.0e38f}, run_sum[2] = {0.f, 0.f};
  const float c = p.scale_log2e;  // > 0: the largest scaled score is the scaled largest score
  const uint32_t k_rd = (4 * g + (m >> 2)) * kAttPitchK + (m & 3) * 8 + (32 * khalf) * 2;
  const uint32_t v_rd = m * kAttPitchV + (4 * g) * 2 + (32 * khalf) * 2;
  for (int kb = 0; kb < blocks; ++kb) {
    const unsigned char *const k_tile = k_tiles + (kb & 1) * kAttTileK;
    const unsigned char *const v_tile = v_tiles + (kb & 1) * kAttTileV;
    const bool more = kb + 1 < blocks;  // uniform
    if (more) {
      const int off = (kb + 1) * kAttKeys;
      kk[0] = *reinterpret_cast<const uintx4 *>(kg + g0 + off);
      kk[1] = *reinterpret_cast<const uintx4 *>(kg + g1 + off);
      vv[0] = *reinterpret_cast<const uintx4 *>(vg + g0 + off);
      vv[1] = *reinterpret_cast<const uintx4 *>(vg + g1 + off);
    }
    // scores^T: s[set][kt], lane (m, g): keys 32 * khalf + 16kt + 4g .. + 3 of the block against query m of the set
    floatx4 s[2][2] = {{zero, zero}, {zero, zero}};
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const unsigned char *a = k_tile + k_rd + (32 * u) * kAttPitchK + (16 * kt) * 2;
        const uintx2 lo = att_read_tr(a), hi = att_read_tr(a + 16 * kAttPitchK);
        AttOperand kop;
        kop.u[0] = lo[0]; kop.u[1] = lo[1]; kop.u[2] = hi[0]; kop.u[3] = hi[1];
#pragma unroll
        for (int j = 0; j < 2; ++j) s[j][kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop.h, qop[j][u].h, s[j][kt], 0, 0, 0);
      }
    }
    AttOperand pop[2];  // per set: contraction slots 0-3 = keys 4g .. + 3 of tile 0, slots 4-7 = the same keys of tile 1
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float mx = s[j][0][0];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[j][kt][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // The reference point of the exponentials moves only when some query's maximum has grown by more than 8 in
      // the base-2 domain (a wave-uniform decision): until then the probabilities are at most 2^8 times too large,
      // which fp16 holds, the running sums and the context stay consistent with the old reference point, and the
      // rescaling of the accumulators, which after the first block is nearly always by 1, is skipped.
      const float new_max = fmaxf(run_max[j], mx);
      if (__ballot((new_max - run_max[j]) * c > 8.0f) != 0) {
        const float alpha = __builtin_amdgcn_exp2f(fmaxf((run_max[j] - new_max) * c, -126.0f));
        run_max[j] = new_max;
        run_sum[j] *= alpha;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) o[j][dt] *= alpha;
      }
      const float shift = -run_max[j] * c;
      float part = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          s[j][kt][r] = __builtin_amdgcn_exp2f(fmaf(s[j][kt][r], c, shift));
          part += s[j][kt][r];
        }
      run_sum[j] += part;
      pop[j].u[0] = att_pack(s[j][0][0], s[j][0][1]);
      pop[j].u[1] = att_pack(s[j][0][2], s[j][0][3]);
      pop[j].u[2] = att_pack(s[j][1][0], s[j][1][1]);
      pop[j].u[3] = att_pack(s[j][1][2], s[j][1][3]);
    }
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
      const unsigned char *a = v_tile + v_rd + (16 * dt) * kAttPitchV;
      const uintx2 lo = *reinterpret_cast<const uintx2 *>(a), hi = *reinterpret_cast<const uintx2 *>(a + 32);
      AttOperand vop;
      vop.u[0] = lo[0]; vop.u[1] = lo[1]; vop.u[2] = hi[0]; vop.u[3] = hi[1];
#pragma unroll
      for (int j = 0; j < 2; ++j) o[j][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vop.h, pop[j].h, o[j][dt], 0, 0, 0);
    }
    if (more) {  // the other buffer: every wave finished reading it before the barrier that ended the previous block
      unsigned char *const kn = k_tiles + ((kb + 1) & 1) * kAttTileK, *const vn = v_tiles + ((kb + 1) & 1) * kAttTileV;
      *reinterpret_cast<uintx4 *>(kn + l0) = kk[0];
      *reinterpret_cast<uintx4 *>(kn + l1) = kk[1];
      *reinterpret_cast<uintx4 *>(vn + lv0) = vv[0];
      *reinterpret_cast<uintx4 *>(vn + lv1) = vv[1];
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    run_sum[j] += __shfl_xor(run_sum[j], 16, 64);
    run_sum[j] += __shfl_xor(run_sum[j], 32, 64);
  }

  // ---- The two waves of a query half merge: the one with the upper keys leaves its state in LDS (over the K tiles:
  // the loop's last barrier is behind every read of them), the other adds it to its own.
  floatx4 *const xo = reinterpret_cast<floatx4 *>(k_tiles) + qhalf * (2 * 4 * 64);  // [set][dt][lane]
  float *const xs = reinterpret_cast<float *>(k_tiles + 2 * (2 * 4 * 64) * 16) + qhalf * (2 * 2 * 64);  // [set][max, sum][lane]
  if (khalf == 1) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) xo[(j * 4 + dt) * 64 + lane] = o[j][dt];
      xs[(j * 2 + 0) * 64 + lane] = run_max[j];
      xs[(j * 2 + 1) * 64 + lane] = run_sum[j];
    }
  }
  __syncthreads();
  if (khalf == 0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const float m1 = xs[(j * 2 + 0) * 64 + lane], l1 = xs[(j * 2 + 1) * 64 + lane];
      const float mm = fmaxf(run_max[j], m1);
      const float a0 = __builtin_amdgcn_exp2f(fmaxf((run_max[j] - mm) * c, -126.0f));
      const float a1 = __builtin_amdgcn_exp2f(fmaxf((m1 - mm) * c, -126.0f));
      const float inv = 1.0f / (run_sum[j] * a0 + l1 * a1);
      // the context through LDS (over the query tile: every wave read its queries before the first barrier of the
      // loop) and out in whole lines
#pragma unroll
      for (int dt = 0; dt < 4; ++dt) {
        const floatx4 other = xo[(j * 4 + dt) * 64 + lane];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          *reinterpret_cast<_Float16 *>(q_tile + (16 * dt + 4 * g + r) * kAttPitchK + (32 * qhalf + 16 * j + m) * 2) =
              (_Float16)((o[j][dt][r] * a0 + other[r] * a1) * inv);
      }
    }
  }
  __syncthreads();
  _Float16 *og = p.out + (long long)(head * kAttD) * p.ld_out + tok0 + qb * kAttQueries;
  *reinterpret_cast<uintx4 *>(og + (long long)r0 * p.ld_out + pc * 8) = *reinterpret_cast<const uintx4 *>(q_tile + l0);
  *reinterpret_cast<uintx4 *>(og + (long long)(r0 + 32) * p.ld_out + pc * 8) = *reinterpret_cast<const uintx4 *>(q_tile + l1);
}

bool attention_fm_applies(int batch, int heads, int seq, int head_dim, const void *q, const void *k, const void *v,
                          long long ld, const void *out, long long ld_out) {
  const auto aligned = [](const void *x) { return (reinterpret_cast<uintptr_t>(x) & 15u) == 0; };
  return batch > 0 && heads > 0 && head_dim == kAttD && seq >= kAttQueries && seq % kAttQueries == 0 && seq <= kAttMaxSeq &&
         ld % 8 == 0 && ld_out % 8 == 0 && aligned(q) && aligned(k) && aligned(v) && aligned(out) &&
         ((long long)batch * heads + 7) * (seq / kAttQueries) <= 0x7fffffffLL;
}

hipError_t launch_attention_fm(int batch, int heads, int seq, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                               long long ld, uint16_t *out, long long ld_out, float scale, hipStream_t stream) {
  AttentionArgs a;
  a.q = reinterpret_cast<const _Float16 *>(q);
  a.k = reinterpret_cast<const _Float16 *>(k);
  a.v = reinterpret_cast<const _Float16 *>(v);
  a.out = reinterpret_cast<_Float16 *>(out);
  a.ld = ld;
  a.ld_out = ld_out;
  a.S = seq;
  a.heads = heads;
  a.units = batch * heads;
  a.scale_log2e = scale * 1.4426950408889634f;
  const long long units_padded = (((long long)batch * heads + 7) / 8) * 8;
  const unsigned blocks = (unsigned)(units_padded * (seq / kAttQueries));
  hipLaunchKernelGGL(attention_fm_kernel, dim3(blocks), dim3(kAttThreads), 0, stream, a);
  return hipGetLastError();
}

}  // namespace sspmm
