// Sparse Vector Compression (RowMerge) on the GPU: CSR -> CVSE.
//
// The reference does this in Python (reference RowMerge/sparse_matrix_format.py:94-123): for every
// group of V consecutive rows it folds  acc = list(set(acc + row))  over the member rows, so the
// column order of a vector-row is the iteration order of a CPython set, rebuilt from an empty
// table once per member row.  SVC_ORDER_CPYTHON reproduces that order bit for bit.
//
// How a set construction is replayed in parallel.  For non-negative int keys hash(k) = k, and a
// CPython set (Objects/setobject.c, 3.7 - 3.12) is an open-addressed table: look at slot
// i = k & mask, then, when i + 9 <= mask, at the nine slots after it; if none is free continue
// with perturb >>= 5, i = (5 i + 1 + perturb) & mask.  The table starts with 8 slots and, as
// soon as 5 * fill >= 3 * mask after an insert, is rebuilt into the smallest power of two above
// 4 * fill (2 * fill beyond 50 000 keys) by re-inserting the keys in slot order.  Inserting a key
// that is present changes nothing, so duplicates are dropped first; after that the number of
// keys alone fixes where the rebuilds happen, and a construction is a short sequence of phases:
//     phase with S slots: keys[0 .. min(n, thr(S))) are inserted into an empty S-slot table,
//     where keys[0 .. thr(previous S)) have been put into the previous table's slot order.
// Within a phase the final table is the unique first-come-first-served placement: every key sits
// in the first slot of its probe sequence not held by an earlier key.  That fixed point is
// reached by any interleaving of threads that claim slots with a 64-bit atomic min on
// (insertion index << 32 | key): a later key that is displaced by an earlier one resumes its own
// probe sequence behind that slot.  So one thread per key inserts a whole phase at once.
//
// One workgroup owns one vector-row group.  The list and the table live in LDS (64-thread groups
// for up to 306 keys, 256 threads up to 1228, 1024 threads up to 4914) or, beyond that, in the
// caller's workspace.
//
// Which phase does what.  The caller sizes the outputs from svc_count's row pointer, so the count
// must come first, but the count of a group (its distinct columns) needs no order: for column
// indices of up to 17 bits svc_count is a bitmap pass plus the prefix sum, a few microseconds,
// and svc_fill runs the replay with every group already knowing its size class exactly and its
// final offset, so the workgroup that has ordered a group writes the group's columns and
// zero-filled value vectors straight to their place ("direct" mode; nothing waits behind the
// longest group but its own output).  The prefix-sum kernel also files every group under its size
// class, so a class kernel walks a list of exactly its groups with a grid sized for the chip: the
// largest groups start at once instead of behind thousands of workgroups that look at a group and
// leave, and a class without groups costs an empty launch of a few workgroups.  Wider matrices and SVC_ORDER_SORTED keep the older split:
// svc_count runs the merge and leaves the ordered columns and every non-zero's position in the
// workspace; svc_fill copies them to their final offsets and scatters the values.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "lane_ops.h"
#include "svc_kernels.h"

namespace sspmm {

typedef unsigned long long u64;
static constexpr u64 kEmpty = ~0ull;

// Size classes by a group's number of columns: the largest sets CPython keeps in tables of 512, 2048, 8192 and
// 32768 slots, and everything beyond.
static constexpr int kSmallKeys = 306, kMediumKeys = 1228, kLargeKeys = 4914, kXLargeKeys = 19660;
static constexpr int kClasses = 5, kClassBeyond = 4;

__device__ __forceinline__ void probe_start(uint32_t key, uint32_t mask, uint32_t &i, uint32_t &perturb,
                                            uint32_t &lin) {
  i = key & mask;
  perturb = key;
  lin = 0;
}

// (written with selects: lanes of a wave are at different points of their probe sequences, and a
// branch here would make every wave walk both sides)
__device__ __forceinline__ void probe_next(uint32_t mask, uint32_t &i, uint32_t &perturb, uint32_t &lin) {
  const bool in_window = (lin < 9u) & (i + 9u <= mask);
  const uint32_t shifted = perturb >> 5;
  const uint32_t jumped = (i * 5u + 1u + shifted) & mask;
  lin = in_window ? lin + 1u : 0u;
  perturb = in_window ? perturb : shifted;
  i = in_window ? i : jumped;
}

// Slot that holds `key`, or -1.  The table always keeps free slots, so the walk ends.
__device__ __forceinline__ int find_slot(const u64 *table, uint32_t mask, uint32_t key) {
  uint32_t i, perturb, lin;
  probe_start(key, mask, i, perturb, lin);
  for (;;) {
    const u64 x = table[i + lin];
    if (x == kEmpty) return -1;
    if ((uint32_t)x == key) return (int)(i + lin);
    probe_next(mask, i, perturb, lin);
  }
}

// First-come-first-served placement of (order, key) by atomic min; see the file header.
__device__ __forceinline__ void place(u64 *table, uint32_t mask, uint32_t key, uint32_t order) {
  u64 mine = ((u64)order << 32) | key;
  uint32_t i, perturb, lin;
  probe_start(key, mask, i, perturb, lin);
  for (;;) {
    const uint32_t s = i + lin;
    const u64 old = atomicMin(&table[s], mine);
    if (old == kEmpty) return;
    // The same key twice can only come from a CSR row that repeats a column (invalid input):
    // keep one copy so the output stays a valid pattern.
    if ((uint32_t)old == (uint32_t)mine) return;
    if (old > mine) {
      // An entry inserted later than mine was sitting here: it moves on.  It reached this slot
      // on the first visit of its own probe sequence, so replay that sequence up to here.
      mine = old;
      key = (uint32_t)old;
      probe_start(key, mask, i, perturb, lin);
      while (i + lin != s) probe_next(mask, i, perturb, lin);
    }
    probe_next(mask, i, perturb, lin);
  }
}

// Exclusive prefix sum of one int per thread over the workgroup; *total = sum.  `scratch` holds
// THREADS / 64 + 1 ints of LDS.  Contains barriers: every thread of the group must call it.
template <int THREADS>
__device__ __forceinline__ int block_exclusive_scan(int x, int *total, int *scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int incl = (int)wave_inclusive_sum((uint32_t)x);
  constexpr int WAVES = THREADS / 64;
  if (WAVES == 1) {
    *total = (int)from_last_lane((uint32_t)incl);
    return incl - x;
  }
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  int base = 0, sum = 0;
#pragma unroll
  for (int wv = 0; wv < WAVES; ++wv) {
    const int t = scratch[wv];
    if (wv < wave) base += t;
    sum += t;
  }
  *total = sum;
  return base + incl - x;
}

// The same for a flag per thread, for loops that call it every trip: the rank comes from the wave's ballot, and
// consecutive calls alternate between two halves of `scratch` (2 x THREADS / 64 ints; `turn` is the caller's
// counter, starting anywhere), so that one barrier per call is enough: a wave that comes round to a half again
// has passed the barrier of the call in between, which every wave reaches only after it has read that half.
template <int THREADS>
__device__ __forceinline__ int block_rank_of_flag(bool flag, int *total, int *scratch, int &turn) {
  constexpr int WAVES = THREADS / 64;
  const unsigned long long m = __ballot(flag);
  const int in_wave = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
  if (WAVES == 1) {
    *total = (int)__popcll(m);
    return in_wave;
  }
  const int wave = threadIdx.x >> 6;
  int *mine = scratch + (turn & 1) * WAVES;
  ++turn;
  if ((threadIdx.x & 63) == 0) mine[wave] = (int)__popcll(m);
  __syncthreads();
  int base = 0, sum = 0;
#pragma unroll
  for (int wv = 0; wv < WAVES; ++wv) {
    const int t = mine[wv];
    if (wv < wave) base += t;
    sum += t;
  }
  *total = sum;
  return base + in_wave;
}

__device__ __forceinline__ uint32_t resize_threshold(uint32_t slots) { return (3u * (slots - 1u) + 4u) / 5u; }

__device__ __forceinline__ uint32_t resized_slots(uint32_t fill) {
  const uint32_t minused = fill > 50000u ? fill * 2u : fill * 4u;
  uint32_t s = 8;
  while (s <= minused) s <<= 1;
  return s;
}

// Writes the keys of table[0..slots) to list[0..) in slot order; when `final` also replaces each
// entry's insertion index by its position in that order.
template <int THREADS>
__device__ __forceinline__ int extract_slot_order(u64 *table, uint32_t slots, int *list, bool final, int *scratch) {
  const uint32_t per = (slots + THREADS - 1) / THREADS;
  const uint32_t lo = min(slots, threadIdx.x * per), hi = min(slots, lo + per);
  int mine = 0;
  for (uint32_t s = lo; s < hi; ++s) mine += table[s] != kEmpty;
  int total;
  int at = block_exclusive_scan<THREADS>(mine, &total, scratch);
  for (uint32_t s = lo; s < hi; ++s) {
    const u64 x = table[s];
    if (x != kEmpty) {
      list[at] = (int)(uint32_t)x;
      if (final) table[s] = ((u64)(uint32_t)at << 32) | (uint32_t)x;
      ++at;
    }
  }
  return total;
}

// list(set(list[0..n))) for distinct keys: on return list holds the set's iteration order and
// table (slot count returned) maps each key to its position.  n is updated to the number of keys
// in the table (it only changes for invalid input with repeated keys).
template <int THREADS>
__device__ __forceinline__ uint32_t rebuild_set(u64 *table, int *list, int &n, int *scratch) {
  uint32_t slots = 8;
  for (;;) {
    const uint32_t thr = resize_threshold(slots);
    const int cnt = min(n, (int)thr);
    for (uint32_t s = threadIdx.x; s < slots; s += THREADS) table[s] = kEmpty;
    __syncthreads();
    for (int idx = threadIdx.x; idx < cnt; idx += THREADS) place(table, slots - 1u, (uint32_t)list[idx], (uint32_t)idx);
    __syncthreads();
    const bool final = n < (int)thr;
    const int kept = extract_slot_order<THREADS>(table, slots, list, final, scratch);
    __syncthreads();
    if (final) {
      n = kept;
      return slots;
    }
    slots = resized_slots(thr);
  }
}

// First member row of group grp (grp = number of groups: one past the last row).  A single matrix's groups are V
// rows each, the last one what is left; a stack of matrices (the batched entry points) brings a table, because a
// matrix whose row count is not a multiple of V ends with a short group and the next one starts a new group.
__device__ __forceinline__ int group_first_row(const SvcArgs &a, int grp) {
  return a.group_rows ? a.group_rows[grp] : min(a.M, grp * a.V);
}

// The table of a stack of `count` matrices: mat_rows[i] is the first row of matrix i in the stack (mat_rows[count]
// the total), group_rows[g] the first row of group g, group_rows[groups] the total, mat_groups[i] the first group of
// matrix i.  One workgroup; matrices in tiles of 1024.
__global__ __launch_bounds__(1024) void svc_group_rows_kernel(int count, int V, int groups, const int32_t *mat_rows,
                                                              int32_t *group_rows, int32_t *mat_groups) {
  __shared__ int scratch[32];
  int carry = 0;
  for (int base = 0; base < count; base += 1024) {
    const int i = base + (int)threadIdx.x;
    const int r0 = i < count ? mat_rows[i] : 0, r1 = i < count ? mat_rows[i + 1] : 0;
    const int n = (r1 - r0 + V - 1) / V;
    int total;
    const int first = carry + block_exclusive_scan<1024>(n, &total, scratch);
    if (i < count) {
      mat_groups[i] = first;
      // (never past the table the caller sized for `groups` groups: a wrong count shows in mat_groups[count])
      for (int g = 0; g < n && first + g < groups; ++g) group_rows[first + g] = r0 + g * V;
    }
    carry += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    mat_groups[count] = carry;
    group_rows[groups] = mat_rows[count];
  }
}

// Class of a vector-row group by its key bound: which kernel instance handles it.
__device__ __forceinline__ bool in_class(int bound, int lo, int hi) { return bound > lo && bound <= hi; }

// Direct mode: number of distinct columns of every group, from a K-bit occupancy bitmap in LDS.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void svc_count_distinct_kernel(const SvcArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int grp = blockIdx.x;
  const int r0 = group_first_row(a, grp), r1 = group_first_row(a, grp + 1);
  const int e0 = a.row_ptr[r0], e1 = a.row_ptr[r1];
  if (e1 - e0 <= 1) {  // nothing to deduplicate
    if (threadIdx.x == 0) a.vec_row_ptr[grp + 1] = e1 - e0;
    return;
  }
  int *scratch = reinterpret_cast<int *>(smem);
  uint32_t *bits = reinterpret_cast<uint32_t *>(smem + 128);
  const int words = (a.K + 31) / 32;
  for (int w = threadIdx.x; w < words; w += THREADS) bits[w] = 0;
  __syncthreads();
  // a thread counts the bits it is the first to set: no second pass over the bitmap
  int mine = 0;
  for (int idx = e0 + (int)threadIdx.x; idx < e1; idx += THREADS) {
    const uint32_t c = (uint32_t)a.col_ind[idx], bit = 1u << (c & 31u);
    if (c < (uint32_t)a.K) mine += (atomicOr(&bits[c >> 5], bit) & bit) ? 0 : 1;  // (a column outside [0, K) is ignored)
  }
  int total;
  block_exclusive_scan<THREADS>(mine, &total, scratch);
  if (threadIdx.x == 0) a.vec_row_ptr[grp + 1] = total;
}

// The first entries of a group's member rows, fetched once: lane j of every wave holds the start of member row j
// (the end of the last row behind them), and a uniform index reads it back without touching memory again.
// Groups of 64 rows, one boundary more than a wave has lanes, read the row pointer each time.
struct RowBounds {
  const int32_t *row_ptr;
  int r0, count;  // first row, number of rows
  int mine;
  bool in_lanes;
  __device__ __forceinline__ RowBounds(const SvcArgs &a, int first, int last) : row_ptr(a.row_ptr), r0(first), count(last - first) {
    in_lanes = count < 64;
    mine = a.row_ptr[first + min((int)(threadIdx.x & 63), count)];
  }
  __device__ __forceinline__ int start(int j) const {  // j uniform, 0 .. count
    return in_lanes ? __builtin_amdgcn_readlane(mine, j) : row_ptr[r0 + j];
  }
  __device__ __forceinline__ int row_of(int idx) const {  // member row (0-based) of entry idx of the group
    int r = 0;
    for (int j = 1; j < count; ++j) r += idx >= start(j) ? 1 : 0;
    return r;
  }
};

// Direct mode: a group's ordered columns and value vectors go to their final place.  list[0 .. n) are the
// ordered columns; position_of(column) is the column's index in that list.  The group owns
// scanned[grp + 1] - scanned[grp] vectors; n equals that count unless a CSR row repeats a column (invalid
// input), in which case surplus vectors stay zero with column 0.
template <int THREADS, typename PositionOf>
__device__ __forceinline__ void write_group_output(const SvcArgs &a, int grp, const RowBounds &rows, const int *list, int n,
                                                   PositionOf position_of) {
  const int v0 = a.scanned[grp], n_out = a.scanned[grp + 1] - v0;
  if (a.vec_col)
    for (int p = threadIdx.x; p < n_out; p += THREADS) a.vec_col[v0 + p] = p < n ? list[p] : 0;
  if (!a.vec_val) return;
  // The value region starts at v0 * V halfs and holds n_out * V of them: whole 16-byte pieces when V is a
  // multiple of 8 (and vec_val is 16-byte aligned), 4-byte pieces whenever V is even.
  const int64_t halfs = (int64_t)n_out * a.V;
  uint16_t *out = a.vec_val + (int64_t)v0 * a.V;
  if ((a.V & 7) == 0 && (reinterpret_cast<uintptr_t>(a.vec_val) & 15) == 0) {
    uint4 *out128 = reinterpret_cast<uint4 *>(out);
    for (int64_t t = threadIdx.x; t < halfs / 8; t += THREADS) out128[t] = uint4{0u, 0u, 0u, 0u};
  } else if ((a.V & 1) == 0 && (reinterpret_cast<uintptr_t>(a.vec_val) & 3) == 0) {
    uint32_t *out32 = reinterpret_cast<uint32_t *>(out);
    for (int64_t t = threadIdx.x; t < halfs / 2; t += THREADS) out32[t] = 0u;
  } else {
    for (int64_t t = threadIdx.x; t < halfs; t += THREADS) out[t] = 0;
  }
  __syncthreads();
  if (n == 0) return;
  // the member rows' entries are one contiguous run of the CSR arrays: one pass over it, the row found from the
  // boundaries in registers, so that no load waits for another
  const int e_end = rows.start(rows.count);
  for (int idx = rows.start(0) + (int)threadIdx.x; idx < e_end; idx += THREADS) {
    const uint32_t c = (uint32_t)a.col_ind[idx];
    const uint16_t value = a.csr_val[idx];
    const int r = rows.row_of(idx);
    const int p = c < (uint32_t)a.K ? position_of(c) : -1;
    if (p >= 0 && p < n_out) out[(int64_t)p * a.V + r] = value;
  }
}

template <int THREADS, bool IN_LDS>
__global__ __launch_bounds__(THREADS) void svc_merge_cpython_kernel(const SvcArgs a, int class_lo, int class_hi,
                                                                    int list_cap) {
  extern __shared__ __align__(16) unsigned char smem[];
  // Direct mode walks the list of the groups of its class (kClassBeyond); otherwise there is one workgroup per
  // group, which leaves unless the group's bound on its columns falls into the launch's class.
  const bool listed = a.scanned != nullptr;
  const int n_groups = listed ? a.class_counts[kClassBeyond] : (a.group_rows ? a.groups : (a.M + a.V - 1) / a.V);
  for (int li = blockIdx.x; li < n_groups; li += gridDim.x) {
  const int grp = listed ? a.class_lists[(int64_t)kClassBeyond * a.list_stride + li] : li;
  const int r0 = group_first_row(a, grp), r1 = group_first_row(a, grp + 1);
  const int e0 = a.row_ptr[r0], e1 = a.row_ptr[r1];
  const int bound = listed ? a.scanned[grp + 1] - a.scanned[grp] : min(e1 - e0, a.K);
  if (!listed && !in_class(bound, class_lo, class_hi)) continue;  // uniform over the group

  int *scratch = reinterpret_cast<int *>(smem);  // 32 ints
  int *list;
  u64 *table;
  if (IN_LDS) {
    table = reinterpret_cast<u64 *>(smem + 128);
    list = reinterpret_cast<int *>(smem + 128 + (size_t)a.lds_table_slots * 8);
  } else {
    list_cap = listed ? bound : e1 - e0;
    list = a.tmp_cols + e0;
    table = a.big_tables + (int64_t)e0 * 8;
  }

  int n = 0;
  uint32_t slots = 0;
  for (int r = r0; r < r1; ++r) {
    const int b = a.row_ptr[r], e = a.row_ptr[r + 1];
    // acc + row: append the row's columns that are not in acc yet, in row order.
    int appended = 0;
    for (int base = b; base < e; base += THREADS) {
      const int idx = base + (int)threadIdx.x;
      bool is_new = false;
      int key = 0;
      if (idx < e) {
        key = a.col_ind[idx];
        is_new = (uint32_t)key < (uint32_t)a.K && ((slots == 0) || find_slot(table, slots - 1u, (uint32_t)key) < 0);
      }
      int total;
      const int rank = block_exclusive_scan<THREADS>(is_new ? 1 : 0, &total, scratch);
      if (is_new && n + appended + rank < list_cap) list[n + appended + rank] = key;
      appended += total;
    }
    n = min(n + appended, list_cap);  // the cap only bites for invalid input (repeated columns)
    __syncthreads();
    slots = rebuild_set<THREADS>(table, list, n, scratch);
  }

  if (listed) {
    write_group_output<THREADS>(a, grp, RowBounds(a, r0, r1), list, n, [&](uint32_t key) {
      const int s = find_slot(table, slots - 1u, key);
      return s >= 0 ? (int)(table[s] >> 32) : -1;
    });
    __syncthreads();  // the next group reuses the table
    continue;
  }
  if (threadIdx.x == 0) a.vec_row_ptr[grp + 1] = n;
  if (IN_LDS)
    for (int p = threadIdx.x; p < n; p += THREADS) a.tmp_cols[e0 + p] = list[p];
  if (n > 0)
    for (int idx = e0 + (int)threadIdx.x; idx < e1; idx += THREADS) {
      const uint32_t c = (uint32_t)a.col_ind[idx];
      const int s = c < (uint32_t)a.K ? find_slot(table, slots - 1u, c) : -1;
      a.pos[idx] = s >= 0 ? (int)(table[s] >> 32) : -1;  // s < 0 only for invalid input: the fill skips it
    }
  }
}

// ------------------------------------------------------------------------------------------
// The same replay on 32-bit table entries.
//
// When the column indices fit in 17 bits (K <= 131 072) a table entry is
// (insertion index << key_bits | key) in 32 bits, key_bits = bits of K - 1, which leaves at least 15
// bits of insertion index: enough for 19 660 keys, the largest set CPython keeps in a 32 768-slot
// table.  Halving the entries brings groups of up to 19 660 keys into LDS (a 128 KB table; their
// key list stays in the workspace) and makes the atomics 32-bit.  The compaction of a phase is done
// one 64-slot word per wave iteration: a ballot gives the occupancy mask; every wave takes a contiguous
// run of words and counts its keys in a first pass, the counts of the waves before it give its starting
// rank (one barrier), and a second pass writes list[running count + rank in word] = key, so nothing
// is scanned per thread.
static constexpr uint32_t kEmpty32 = 0xffffffffu;

struct Table32 {
  uint32_t *slots;  // LDS
  uint32_t key_bits, key_mask;
};

__device__ __forceinline__ int find_slot32(const Table32 &t, uint32_t mask, uint32_t key) {
  uint32_t i, perturb, lin;
  probe_start(key, mask, i, perturb, lin);
  for (;;) {
    const uint32_t x = t.slots[i + lin];
    if (x == kEmpty32) return -1;
    if ((x & t.key_mask) == key) return (int)(i + lin);
    probe_next(mask, i, perturb, lin);
  }
}

// First-come-first-served placement of one key, as in place() above, on 32-bit entries.
// A function of its own on purpose: inlined into the eight-fold unrolled loops of every phase variant it made the
// merge kernels 150 KB of code, more than twice the instruction cache that two CUs share, and a construction is
// a walk through all of it.  The table comes as an LDS pointer so that the atomic stays an LDS instruction.
typedef __attribute__((address_space(3))) uint32_t lds_u32;
__device__ __attribute__((noinline)) void place32_lds(lds_u32 *slots, uint32_t key_bits, uint32_t mask, uint32_t key, uint32_t order) {
  const uint32_t key_mask = (1u << key_bits) - 1u;
  uint32_t mine = (order << key_bits) | key;
  uint32_t i, perturb, lin;
  probe_start(key, mask, i, perturb, lin);
  for (;;) {
    const uint32_t s0 = i + lin;
    const uint32_t old = __hip_atomic_fetch_min(slots + s0, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (old == kEmpty32 || ((old ^ mine) & key_mask) == 0) return;  // placed, or a repeated key (invalid row)
    if (old > mine) {
      // a later entry sat here: carry it on from this slot of its own probe sequence
      mine = old;
      probe_start(old & key_mask, mask, i, perturb, lin);
      // nearly always it lost a slot of its first window: no walk needed then
      const uint32_t d = s0 - i;
      if ((d <= 9u) & ((i + 9u <= mask) | (d == 0u)))
        lin = d;
      else
        while (i + lin != s0) probe_next(mask, i, perturb, lin);
    }
    probe_next(mask, i, perturb, lin);
  }
}
__device__ __forceinline__ void place32(const Table32 &t, uint32_t mask, uint32_t key, uint32_t order) {
  place32_lds((lds_u32 *)t.slots, t.key_bits, mask, key, order);
}
// The same placement inlined, for keys that come from LDS (two call sites per phase): alone on its SIMD a wave
// pays every instruction in full, the call and its register shuffling included, and with four waves per SIMD a round
// of placements is bound by the instructions the waves issue, not by the LDS.
//
// Together with its attempt on a slot a key reads the three slots behind it: an entry only ever gets smaller
// (atomic min), so a slot that holds an earlier key now is lost to this key for good and can be passed without an
// atomic; if the attempt fails, the next one goes to the first of the three that is free or holds a later key, or to
// the slot behind them.  The reads are in flight with the atomic and add nothing to the round trip; rounds, and
// with them the wave-rounds a phase costs, come down to about half.  Passing over slots unseen would also pass
// over an earlier copy of the same key, which only a row that repeats a column (invalid input) can bring:
// `safe` = true switches the passing off and the test for the same key on (the caller falls back to it when a
// group turns out to hold more keys than distinct columns).
__device__ __forceinline__ void place32_inline(const Table32 &t, uint32_t mask, uint32_t key, uint32_t order, bool safe) {
  uint32_t mine = (order << t.key_bits) | key;
  uint32_t i, perturb, lin;
  probe_start(key, mask, i, perturb, lin);
  for (;;) {
    const uint32_t s0 = i + lin;
    const uint32_t old = __hip_atomic_fetch_min(t.slots + s0, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    // (slots behind the table's end are read and not used: every table is followed by other LDS of the group)
    const uint32_t x1 = t.slots[s0 + 1u], x2 = t.slots[s0 + 2u], x3 = t.slots[s0 + 3u];
    if (old == kEmpty32) return;
    if (safe && ((old ^ mine) & t.key_mask) == 0) return;  // a repeated key (invalid row)
    if (old > mine) {
      // a later entry sat here: carry it on from this slot of its own probe sequence
      mine = old;
      probe_start(old & t.key_mask, mask, i, perturb, lin);
      const uint32_t d = s0 - i;
      if ((d <= 9u) & ((i + 9u <= mask) | (d == 0u)))
        lin = d;
      else
        while (i + lin != s0) probe_next(mask, i, perturb, lin);
    }
    // slots s0 + 1 .. s0 + 3 are the next three of the sequence, and the one behind them the fourth, if they are
    // inside the window of ten
    const bool can = (lin <= 5u) & (i + 9u <= mask) & !safe;
    uint32_t k = x3 < mine ? 3u : 2u;
    k = x2 < mine ? k : 1u;
    k = x1 < mine ? k : 0u;
    lin += can ? k : 0u;
    probe_next(mask, i, perturb, lin);
  }
}

// The key list lives in LDS, or in the workspace where other waves of the group wrote it: those
// accesses go past the L1.
template <bool IN_LDS>
__device__ __forceinline__ int list_load(const int *list, int idx) {
  return IN_LDS ? list[idx] : __hip_atomic_load(list + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool IN_LDS>
__device__ __forceinline__ void list_store(int *list, int idx, int v) {
  if (IN_LDS) list[idx] = v;
  else __hip_atomic_store(list + idx, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Writes the keys of a table to list[] in slot order and returns their number; with `final`, the
// table entries are rewritten as (rank, key).  wcount: one word of LDS per wave.  Contains
// barriers; the table must be complete (a barrier behind the last insert) on entry.
// check (optional): compares the new order with the list as it was (the construction's input) and with the input
// of the construction before (check->before, if kept), and leaves the old list there for the next comparison.
struct OrderCheck {
  bool on;            // off: nothing is compared or kept (both answers "no")
  int *before;        // LDS copy of the previous construction's input, or null
  int *wave_words;    // LDS, one int per wave, free between the barriers inside a compaction
  bool same_as_input;   // out: every key landed on the list entry that already held it
  bool same_as_before;  // out: ... on the entry of `before` that held it (meaningful when `before` was that input)
};
template <int THREADS, bool LIST_IN_LDS>
__device__ __forceinline__ int compact_table32(const Table32 &t, uint32_t slots, uint32_t *wcount, int *list, bool final,
                                               OrderCheck *check = nullptr) {
  constexpr int WAVES = THREADS / 64;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t words = slots >= 64u ? slots / 64u : 1u;
  // A wave takes a contiguous run of 64-slot words, so that the number of keys before its first word is a sum over
  // the waves before it: one barrier, and no wave scans the words' counts for the others.
  const uint32_t per_wave = (words + WAVES - 1u) / WAVES;
  const uint32_t w_beg = min(words, (uint32_t)wave * per_wave), w_end = min(words, w_beg + per_wave);
  // (four words per trip, their loads in flight together: these passes are chains of LDS round trips)
  uint32_t in_wave = 0;
  for (uint32_t w0 = w_beg; w0 < w_end; w0 += 4) {
    uint32_t x[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t s = (w0 + j) * 64u + lane;
      x[j] = (w0 + j < w_end && s < slots) ? t.slots[s] : kEmpty32;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) in_wave += (uint32_t)__popcll(__ballot(x[j] != kEmpty32));
  }
  uint32_t running = 0, kept_u = in_wave;  // keys before this wave's words; keys in the table
  if (WAVES > 1) {
    if (lane == 0) wcount[wave] = in_wave;
    __syncthreads();
    kept_u = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const uint32_t c = wcount[w];
      if (w < wave) running += c;
      kept_u += c;
    }
  }
  int moved = 0, moved_before = 0;
  for (uint32_t w0 = w_beg; w0 < w_end; w0 += 4) {
    uint32_t x[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t s = (w0 + j) * 64u + lane;
      x[j] = (w0 + j < w_end && s < slots) ? t.slots[s] : kEmpty32;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t s = (w0 + j) * 64u + lane;
      const bool occ = x[j] != kEmpty32;
      const unsigned long long m = __ballot(occ);
      const uint32_t rank = running + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
      running += (uint32_t)__popcll(m);
      if (occ) {
        // (entry `rank` of either list is written by this thread alone, so what it reads here is the old content)
        if (check) {
          const int key = (int)(x[j] & t.key_mask), was = list_load<LIST_IN_LDS>(list, (int)rank);
          moved |= was != key;
          if (check->before) {
            moved_before |= check->before[rank] != key;
            check->before[rank] = was;
          }
        }
        list_store<LIST_IN_LDS>(list, (int)rank, (int)(x[j] & t.key_mask));
        if (final) t.slots[s] = (rank << t.key_bits) | (x[j] & t.key_mask);
      }
    }
  }
  const int kept = (int)kept_u;
  if (check) {
    // both answers through one word per wave (the library's workgroup-wide "or" is three barriers per answer)
    const int mine = (__ballot(moved) != 0 ? 1 : 0) | (__ballot(moved_before) != 0 ? 2 : 0);
    if (lane == 0) check->wave_words[wave] = mine;
    __syncthreads();
    int any = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) any |= check->wave_words[w];
    check->same_as_input = (any & 1) == 0;
    check->same_as_before = check->before != nullptr && (any & 2) == 0;
  }
  __syncthreads();  // (also: the wave words may be written again)
  return kept;
}

// The two table regions of a group: consecutive phases of a construction alternate between them,
// so that a phase can re-insert the previous phase's table straight from its slots.
struct TableRegions {
  uint32_t *a, *b;        // LDS
  uint32_t cap_a, cap_b;  // in slots; cap_a = the largest table of the class
};

// The inserts of one phase by STRIDE cooperating threads, `me` the caller's index among them: either
// list[0 .. cnt) (insertion index = list index), or the previous table's keys, indexed by their
// slot, and the list keys [prev_cnt, cnt) behind them.  A thread inserts its keys in order
// (me, me + STRIDE, ...), so the threads work through the keys in chunks and a later key rarely
// arrives before an earlier one; keys are fetched eight at a time ahead of the inserts.
template <int STRIDE, bool LIST_IN_LDS>
__device__ __forceinline__ void phase_insert(const Table32 &t, uint32_t mask, const int *list, int cnt, const uint32_t *old_table,
                                             uint32_t old_slots, int prev_cnt, int me, bool safe) {
  if (LIST_IN_LDS) {
    // every key comes from LDS: nothing to fetch ahead, and two inlined placements instead of sixteen calls
    uint32_t first = 0;
    if (old_table != nullptr) {
      first = old_slots;
#pragma unroll 1
      for (uint32_t s = me; s < old_slots; s += STRIDE) {
        const uint32_t x = old_table[s];
        if (x != kEmpty32) place32_inline(t, mask, x & t.key_mask, s, safe);
      }
    }
    me = (me + STRIDE - (int)(first % (uint32_t)STRIDE)) % STRIDE;
#pragma unroll 1
    for (int idx = prev_cnt + me; idx < cnt; idx += STRIDE)
      place32_inline(t, mask, (uint32_t)list[idx], first + (uint32_t)(idx - prev_cnt), safe);
    return;
  }
  if (old_table != nullptr) {
    for (uint32_t base = me; base < old_slots; base += 8 * STRIDE) {
      uint32_t x8[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t s = base + j * STRIDE;
        x8[j] = s < old_slots ? old_table[s] : kEmpty32;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (x8[j] != kEmpty32) place32(t, mask, x8[j] & t.key_mask, base + j * STRIDE);
    }
  }
  const uint32_t first_index = old_table != nullptr ? old_slots : 0u;
  // the list's keys start with the thread behind the last one that holds a slot of the previous table, so that as few
  // threads as possible have a key of both kinds to place one after the other
  me = (me + STRIDE - (int)(first_index % (uint32_t)STRIDE)) % STRIDE;
  for (int base = prev_cnt + me; base < cnt; base += 8 * STRIDE) {
    int k8[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = base + j * STRIDE;
      k8[j] = idx < cnt ? list_load<LIST_IN_LDS>(list, idx) : 0;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int idx = base + j * STRIDE;
      if (idx < cnt) place32(t, mask, (uint32_t)k8[j], first_index + (uint32_t)(idx - prev_cnt));
    }
  }
}

// The same inserts by one wave on its own (tables of up to kSoloSlots slots: a lane has a key or two).
template <bool LIST_IN_LDS>
__device__ __forceinline__ void phase_insert_solo(const Table32 &t, uint32_t mask, const int *list, int cnt,
                                                  const uint32_t *old_table, uint32_t old_slots, int prev_cnt, int lane,
                                                  bool safe) {
  uint32_t first_index = 0;
  if (old_table != nullptr) {
    first_index = old_slots;
#pragma unroll 1
    for (uint32_t s = lane; s < old_slots; s += 64) {
      const uint32_t x = old_table[s];
      if (x != kEmpty32) place32_inline(t, mask, x & t.key_mask, s, safe);
    }
  }
  const int me = (lane + 64 - (int)(first_index % 64u)) % 64;
#pragma unroll 1
  for (int idx = prev_cnt + me; idx < cnt; idx += 64)
    place32_inline(t, mask, (uint32_t)list_load<LIST_IN_LDS>(list, idx), first_index + (uint32_t)(idx - prev_cnt), safe);
}

// One `set(list)` of CPython on the keys list[0 .. n): leaves the final table in t (entries
// (rank in slot order, key)), the keys in slot order in list[], and returns the table's size.
// A phase inserts the previous phase's keys in its slot order, then further keys of the list in
// list order; all that first-come-first-served placement needs of the insertion indices is their
// order, so the previous table's slot number serves as the index of a re-inserted key and no
// compaction is needed between phases.  Only where the next table does not fit the other region
// is the old table first compacted into the list.  The phases of the smallest tables (a few dozen
// keys) are run by the first wave alone, without workgroup barriers.
static constexpr uint32_t kSoloSlots = 128;
// check: see compact_table32; both answers are "no" when the list was rewritten between phases, and
// check.before is then cleared (what it would receive is not the input).
template <int THREADS, bool LIST_IN_LDS>
__device__ __forceinline__ uint32_t rebuild_set32(Table32 &t, const TableRegions &reg, int *list, int &n, OrderCheck &check,
                                                  bool safe) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  uint32_t slots = 8, old_slots = 0;
  uint32_t *cur = nullptr;
  int prev_cnt = 0;
  bool solo_pending = false;  // the first wave ran phases on its own that the others have not waited for yet
  bool list_rewritten = false;  // a compaction between phases already replaced the head of the list
  // the largest table must land in region a: start so that the alternation ends there
  uint32_t phases_to_max = 0;
  for (uint32_t s8 = 8; s8 < reg.cap_a; s8 <<= 2) ++phases_to_max;
  bool next_in_a = (phases_to_max & 1u) == 0u;
  for (;;) {
    const uint32_t thr = resize_threshold(slots);
    const int cnt = min(n, (int)thr);
    const uint32_t mask = slots - 1u;
    uint32_t *nt = next_in_a ? reg.a : reg.b;
    const uint32_t nt_cap = next_in_a ? reg.cap_a : reg.cap_b;
    const bool solo = THREADS > 64 && slots <= kSoloSlots && slots <= nt_cap;
    if (!solo && solo_pending) {
      __syncthreads();
      solo_pending = false;
    }
    if (slots > nt_cap) {
      // the other region is too small: slot order goes to the list and the table is rebuilt in place
      Table32 old = t;
      old.slots = cur;
      prev_cnt = 0;
      list_rewritten = true;
      compact_table32<THREADS, LIST_IN_LDS>(old, old_slots, nt, list, false);
      nt = cur;
      cur = nullptr;
    }
    uint32_t *other = nt == reg.a ? reg.b : reg.a;
    t.slots = nt;
    if (solo) {
      if (wave == 0) {
        for (uint32_t s = lane; s < slots; s += 64) nt[s] = kEmpty32;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");  // the wave's LDS operations execute in order
        __builtin_amdgcn_wave_barrier();
        phase_insert_solo<LIST_IN_LDS>(t, mask, list, cnt, cur, old_slots, prev_cnt, lane, safe);
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
        __builtin_amdgcn_wave_barrier();
      }
      solo_pending = true;
    } else {
      for (uint32_t s = tid; s < slots; s += THREADS) nt[s] = kEmpty32;
      __syncthreads();
      phase_insert<THREADS, LIST_IN_LDS>(t, mask, list, cnt, cur, old_slots, prev_cnt, tid, safe);
      __syncthreads();
    }
    if (n < (int)thr) {
      if (solo_pending) __syncthreads();
      if (list_rewritten || !check.on) check.before = nullptr;
      n = compact_table32<THREADS, LIST_IN_LDS>(t, slots, other, list, true, check.on ? &check : nullptr);
      if (list_rewritten || !check.on) check.same_as_input = check.same_as_before = false;
      return slots;
    }
    cur = nt;
    old_slots = slots;
    prev_cnt = cnt;
    next_in_a = nt != reg.a;
    slots = resized_slots(thr);
  }
}

template <int THREADS, bool LIST_IN_LDS>
__global__ __launch_bounds__(THREADS) void svc_merge_fast_kernel(const SvcArgs a, int cls, int cls_last,
                                                                 uint32_t key_bits, uint32_t max_slots, uint32_t small_slots,
                                                                 int list_cap) {
  extern __shared__ __align__(16) unsigned char smem[];
  // direct mode only: the groups of this launch's classes are listed, and a group's column count is known.
  // A launch takes the classes cls, cls - 1, ..., cls_last (largest groups first).
  const int tid = threadIdx.x;
  int n_groups = 0;
  for (int c = cls; c >= cls_last; --c) n_groups += a.class_counts[c];
  for (int li = blockIdx.x; li < n_groups; li += gridDim.x) {
  int c = cls, at = li;
  while (at >= a.class_counts[c]) at -= a.class_counts[c--];
  const int grp = a.class_lists[(int64_t)c * a.list_stride + at];
  const int r0 = group_first_row(a, grp), r1 = group_first_row(a, grp + 1);
  const int count = a.scanned[grp + 1] - a.scanned[grp];
  const int e0 = a.row_ptr[r0];

  int *scratch = reinterpret_cast<int *>(smem);  // 32 ints
  Table32 t;
  t.slots = reinterpret_cast<uint32_t *>(smem + 128);
  t.key_bits = key_bits;
  t.key_mask = (1u << key_bits) - 1u;
  TableRegions reg;
  reg.a = t.slots;
  reg.cap_a = max_slots;
  reg.b = t.slots + max_slots;
  reg.cap_b = small_slots;
  int *list = LIST_IN_LDS ? reinterpret_cast<int *>(smem + 128 + ((size_t)max_slots + small_slots) * 4) : a.tmp_cols + e0;
  int *const list_before = LIST_IN_LDS ? list + list_cap : nullptr;  // the input of the latest construction
  const int cap = count;

  int n = 0;
  uint32_t slots = 0;
  const RowBounds rows(a, r0, r1);
  // CPython rebuilds the set for every member row, also for one that brings nothing new (an empty row, a row of
  // known columns); the order may still change then, because the keys go in in the previous table's slot order.
  // Two cases need no construction.  period == 1: the latest construction returned its keys in the order it got
  // them, so every further one without new keys does too.  period == 2: it returned the order that went into the
  // construction before it, so further ones alternate between the two orders: they are counted (`owed`, modulo 2)
  // and at most one of them is carried out, when new keys arrive or at the end.
  // The comparisons cost a few per cent of a construction, so they are made where they can pay: when the row
  // brought nothing new itself, or when the row behind it is empty.
  int period = 0, owed = 0, scan_turn = 0;
  bool before_is_input = false;  // list_before holds the input of the construction that produced the list
  // The placements pass over slots without looking for their own key there (place32_inline), which is right as long
  // as no row repeats a column.  A row that does makes the group's keys outnumber its distinct columns sooner or
  // later (`cap`, counted beforehand): the group is then done again with the placements that look.
  bool safe = false;
  OrderCheck check;
  check.wave_words = scratch;
  auto construct = [&](bool without_new_keys, bool compare) {
    const bool had_input = before_is_input;
    check.on = compare;
    check.before = list_before;
    slots = rebuild_set32<THREADS, LIST_IN_LDS>(t, reg, list, n, check, safe);
    period = check.same_as_input ? 1 : (without_new_keys && had_input && check.same_as_before) ? 2 : 0;
    before_is_input = check.before != nullptr;
  };
  for (;;) {
  bool overfull = false;
  n = 0;
  slots = 0;
  period = owed = 0;
  before_is_input = false;
  for (int row = r0; row < r1; ++row) {
    const int b = rows.start(row - r0), e = rows.start(row - r0 + 1);
    // acc + row: append the row's columns that are not in acc yet, in row order
    int appended = 0;
    for (int base = b; base < e; base += THREADS) {
      const int idx = base + tid;
      bool is_new = false;
      uint32_t k = 0;
      if (idx < e) {
        k = (uint32_t)a.col_ind[idx];
        is_new = k < (uint32_t)a.K && ((slots == 0) || find_slot32(t, slots - 1u, k) < 0);
      }
      int total;
      const int rank = block_rank_of_flag<THREADS>(is_new, &total, scratch, scan_turn);
      if (is_new && n + appended + rank < cap) list_store<LIST_IN_LDS>(list, n + appended + rank, (int)k);
      appended += total;
    }
    overfull = appended > cap - n;
    appended = min(appended, cap - n);  // the cap only bites for invalid input (a row that repeats a column)
    __syncthreads();
    if (overfull && !safe) break;
    if (appended == 0 && slots != 0) {
      if (period == 1) continue;
      if (period == 2) {
        owed ^= 1;
        continue;
      }
      construct(true, true);
      continue;
    }
    if (owed) {  // the order the new keys go behind is the other one of the pair (the new keys wait behind list[n])
      construct(true, false);
      owed = 0;
    }
    n += appended;
    construct(false, row + 1 < r1 && rows.start(row - r0 + 1) == rows.start(row - r0 + 2));
  }
  if (!overfull || safe) break;
  safe = true;
  }
  if (owed) construct(true, false);

  write_group_output<THREADS>(a, grp, rows, list, n, [&](uint32_t key) {
    const int sl = find_slot32(t, slots - 1u, key);
    return sl >= 0 ? (int)(t.slots[sl] >> key_bits) : -1;
  });
  __syncthreads();  // the next group reuses the table and the list
  }
}

// Ascending order: a K-bit occupancy bitmap per group plus a per-word running popcount.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void svc_merge_sorted_kernel(const SvcArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int grp = blockIdx.x;
  const int r0 = group_first_row(a, grp), r1 = group_first_row(a, grp + 1);
  const int e0 = a.row_ptr[r0], e1 = a.row_ptr[r1];
  const int words = (a.K + 31) / 32;
  int *scratch = reinterpret_cast<int *>(smem);
  uint32_t *bits = reinterpret_cast<uint32_t *>(smem + 128);
  int *prefix = reinterpret_cast<int *>(smem + 128 + (size_t)words * 4);
  for (int w = threadIdx.x; w < words; w += THREADS) bits[w] = 0;
  __syncthreads();
  for (int idx = e0 + (int)threadIdx.x; idx < e1; idx += THREADS) {
    const uint32_t c = (uint32_t)a.col_ind[idx];
    if (c < (uint32_t)a.K) atomicOr(&bits[c >> 5], 1u << (c & 31u));  // (a column outside [0, K) is ignored)
  }
  __syncthreads();
  const int per = (words + THREADS - 1) / THREADS;
  const int lo = min(words, (int)threadIdx.x * per), hi = min(words, lo + per);
  int mine = 0;
  for (int w = lo; w < hi; ++w) mine += __popc(bits[w]);
  int total;
  int at = block_exclusive_scan<THREADS>(mine, &total, scratch);
  for (int w = lo; w < hi; ++w) {
    prefix[w] = at;
    uint32_t x = bits[w];
    while (x) {
      const int b = __ffs(x) - 1;
      x &= x - 1;
      a.tmp_cols[e0 + at++] = w * 32 + b;
    }
  }
  if (threadIdx.x == 0) a.vec_row_ptr[grp + 1] = total;
  __syncthreads();
  for (int idx = e0 + (int)threadIdx.x; idx < e1; idx += THREADS) {
    const uint32_t c = (uint32_t)a.col_ind[idx];
    a.pos[idx] = c < (uint32_t)a.K ? prefix[c >> 5] + __popc(bits[c >> 5] & ((1u << (c & 31u)) - 1u)) : -1;
  }
}

// Direct mode: the scan above, and every group filed under its size class.  class_lists[c * stride + i] is the
// i-th group of class c (in no particular order), class_counts[c] how many there are.
__global__ __launch_bounds__(1024) void svc_scan_classify_kernel(int m_vec, int32_t *vec_row_ptr, int32_t *class_lists,
                                                                 int32_t *class_counts, int list_stride) {
  __shared__ int scratch[32];
  __shared__ int filed[kClasses];
  if (threadIdx.x < kClasses) filed[threadIdx.x] = 0;
  if (threadIdx.x == 0) vec_row_ptr[0] = 0;
  int carry = 0;
  const int lane = threadIdx.x & 63;
  for (int base = 0; base < m_vec; base += 1024) {
    const int i = base + (int)threadIdx.x;
    const int x = i < m_vec ? vec_row_ptr[i + 1] : 0;
    int total;
    const int ex = block_exclusive_scan<1024>(x, &total, scratch);  // (its barriers also cover filed[]'s set-up)
    if (i < m_vec) vec_row_ptr[i + 1] = carry + ex + x;
    carry += total;
    const int cls = i >= m_vec ? -1 : x <= kSmallKeys ? 0 : x <= kMediumKeys ? 1 : x <= kLargeKeys ? 2 : x <= kXLargeKeys ? 3 : 4;
#pragma unroll
    for (int c = 0; c < kClasses; ++c) {
      const unsigned long long members = __ballot(cls == c);
      if (members == 0) continue;  // uniform over the wave
      int at = 0;
      if (lane == 0) at = atomicAdd(&filed[c], __popcll(members));
      at = __builtin_amdgcn_readfirstlane(at);
      if (cls == c) class_lists[(int64_t)c * list_stride + at + __popcll(members & ((1ull << lane) - 1ull))] = i;
    }
  }
  __syncthreads();
  if (threadIdx.x < kClasses) class_counts[threadIdx.x] = filed[threadIdx.x];
}

// In-place inclusive scan of vec_row_ptr[1..m_vec], vec_row_ptr[0] = 0.  One workgroup walks the
// array in tiles of 1024: m_vec is the row count divided by V, a few thousand to a few hundred
// thousand entries, far too little to be worth a multi-pass scan.
__global__ __launch_bounds__(1024) void svc_scan_kernel(int m_vec, int32_t *vec_row_ptr) {
  __shared__ int scratch[32];
  int carry = 0;
  if (threadIdx.x == 0) vec_row_ptr[0] = 0;
  for (int base = 0; base < m_vec; base += 1024) {
    const int i = base + (int)threadIdx.x;
    const int x = i < m_vec ? vec_row_ptr[i + 1] : 0;
    int total;
    const int ex = block_exclusive_scan<1024>(x, &total, scratch);
    if (i < m_vec) vec_row_ptr[i + 1] = carry + ex + x;
    carry += total;
  }
}

// One workgroup per vector-row group: copy its ordered columns to their final offset, clear its
// value vectors and scatter the group's non-zeros into them.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void svc_fill_kernel(const SvcArgs a, const uint16_t *csr_val,
                                                          const int32_t *vec_row_ptr, int32_t *vec_col,
                                                          uint16_t *vec_val) {
  const int grp = blockIdx.x;
  const int r0 = group_first_row(a, grp), r1 = group_first_row(a, grp + 1);
  const int e0 = a.row_ptr[r0];
  const int v0 = vec_row_ptr[grp], n = vec_row_ptr[grp + 1] - v0;
  if (vec_col)
    for (int p = threadIdx.x; p < n; p += THREADS) vec_col[v0 + p] = a.tmp_cols[e0 + p];
  if (!vec_val) return;
  // A group's value region starts at v0 * V halfs and holds n * V of them: whole 16-byte pieces when V is a
  // multiple of 8 (and vec_val is 16-byte aligned), 4-byte pieces whenever V is even.
  const int64_t halfs = (int64_t)n * a.V;
  uint16_t *out = vec_val + (int64_t)v0 * a.V;
  if ((a.V & 7) == 0 && (reinterpret_cast<uintptr_t>(vec_val) & 15) == 0) {
    uint4 *out128 = reinterpret_cast<uint4 *>(out);
    for (int64_t t = threadIdx.x; t < halfs / 8; t += THREADS) out128[t] = uint4{0u, 0u, 0u, 0u};
  } else if ((a.V & 1) == 0) {
    uint32_t *out32 = reinterpret_cast<uint32_t *>(out);
    for (int64_t t = threadIdx.x; t < halfs / 2; t += THREADS) out32[t] = 0u;
  } else {
    for (int64_t t = threadIdx.x; t < halfs; t += THREADS) out[t] = 0;
  }
  __syncthreads();
  for (int r = r0; r < r1; ++r) {
    const int b = a.row_ptr[r], e = a.row_ptr[r + 1];
    for (int idx = b + (int)threadIdx.x; idx < e; idx += THREADS) {
      const int ps = a.pos[idx];
      if (ps >= 0 && ps < n) out[(int64_t)ps * a.V + (r - r0)] = csr_val[idx];  // (-1: a column outside [0, K))
    }
  }
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Lets a kernel ask for `lds` bytes of dynamic LDS; the runtime is only told when a kernel's need grows
// (`raised`: the limit in force per device, one array per kernel).
static constexpr int kMaxDevices = 16;
static hipError_t raise_lds_limit(const void *kern, size_t lds, int (&raised)[kMaxDevices]) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = -1;
  if (dev >= 0 && raised[dev] >= (int)lds) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e == hipSuccess && dev >= 0) raised[dev] = (int)lds;
  return e;
}

size_t svc_workspace_layout(int64_t nnz, int m_vec, size_t *off_pos, size_t *off_tables, size_t *off_lists) {
  const size_t n = (size_t)(nnz > 0 ? nnz : 1);
  const size_t cols = align256(n * 4);
  const size_t pos = align256(n * 4);
  const size_t tables = align256(n * 64);
  const size_t lists = align256(((size_t)kClasses * (size_t)(m_vec > 0 ? m_vec : 1) + 64) * 4);  // counts, then lists
  if (off_pos) *off_pos = cols;
  if (off_tables) *off_tables = cols + pos;
  if (off_lists) *off_lists = cols + pos + tables;
  return cols + pos + tables + lists;
}

template <int THREADS>
static hipError_t launch_lds_class(const SvcArgs &base, int m_vec, int lo, int hi, int slots, hipStream_t stream) {
  SvcArgs a = base;
  a.lds_table_slots = slots;
  const size_t lds = 128 + (size_t)slots * 8 + (size_t)hi * 4;
  auto kern = svc_merge_cpython_kernel<THREADS, true>;
  if (lds > 64 * 1024) {
    static int raised[kMaxDevices] = {};
    const hipError_t e = raise_lds_limit(reinterpret_cast<const void *>(kern), lds, raised);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3(m_vec), dim3(THREADS), lds, stream, a, lo, hi, hi);
  return hipGetLastError();
}

template <int THREADS, bool LIST_IN_LDS>
static hipError_t launch_fast_class(const SvcArgs &a, int grid, int cls, int cls_last, int hi, uint32_t slots,
                                    uint32_t key_bits, hipStream_t stream, size_t min_lds = 0) {
  // second table region: a quarter of the first (what the phase before the largest needs), less where LDS is short;
  // it also serves as the running-count array of the compaction of a table in the first region (slots / 64 + 1 words)
  uint32_t small_slots = slots / 4u;
  // (a key list in LDS has a second copy behind it: the input of the latest construction)
  const size_t list_bytes = LIST_IN_LDS ? (size_t)hi * 8 : 0;
  // (16 bytes behind everything: a placement reads up to three slots past the end of its table)
  constexpr size_t kTail = 16;
  while (128 + ((size_t)slots + small_slots) * 4 + list_bytes + kTail > 160 * 1024) small_slots /= 4u;
  if (small_slots < slots / 64u + 1u) return hipErrorInvalidValue;
  size_t lds = 128 + ((size_t)slots + small_slots) * 4 + list_bytes + kTail;
  if (lds < min_lds) lds = min_lds;  // asking for more than half of a CU's LDS keeps a workgroup alone on its CU
  auto kern = svc_merge_fast_kernel<THREADS, LIST_IN_LDS>;
  if (lds > 64 * 1024) {
    static int raised[kMaxDevices] = {};
    const hipError_t e = raise_lds_limit(reinterpret_cast<const void *>(kern), lds, raised);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(THREADS), lds, stream, a, cls, cls_last, key_bits, slots, small_slots, hi);
  return hipGetLastError();
}

// The size classes are independent kernels over disjoint groups: they run side by side on three
// helper streams (default priority, created once per device) forked from and joined back into
// the caller's stream with events, so the phase costs what its slowest class costs.
struct SideStreams {
  bool ready = false;
  hipStream_t s[3];
  hipEvent_t fork, join[3];
  // held while a call enqueues its fork .. join sequence: the events are re-recorded by every call, so two host
  // threads must not interleave their sequences on one device
  std::mutex in_use;
};
static SideStreams g_side[16];
static std::mutex g_side_mutex;

static SideStreams *side_streams() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
  std::lock_guard<std::mutex> lock(g_side_mutex);
  SideStreams &ss = g_side[dev];
  if (!ss.ready) {
    for (int i = 0; i < 3; ++i) {
      if (hipStreamCreateWithFlags(&ss.s[i], hipStreamNonBlocking) != hipSuccess) return nullptr;
      if (hipEventCreateWithFlags(&ss.join[i], hipEventDisableTiming) != hipSuccess) return nullptr;
    }
    if (hipEventCreateWithFlags(&ss.fork, hipEventDisableTiming) != hipSuccess) return nullptr;
    ss.ready = true;
  }
  return &ss;
}

// A call that is being recorded into a HIP graph stays on the caller's stream: the helper streams and their
// events are shared by every call on the device, and pulling them into one stream's capture would tie any other
// call that forks before the capture ends to that capture.
static SideStreams *side_streams_for(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();  // (the legacy default stream cannot be asked while another stream captures)
    status = hipStreamCaptureStatusNone;
  }
  return status == hipStreamCaptureStatusNone ? side_streams() : nullptr;
}

static uint32_t bits_of(int K) {
  uint32_t key_bits = 1;
  while (key_bits < 31 && (1u << key_bits) < (uint32_t)K) ++key_bits;
  return key_bits;
}

bool svc_direct(int order, int K) { return order == 0 && bits_of(K) <= 17; }

// Forks the helper streams from `stream`; st[0] is the caller's stream.
static hipError_t fork_streams(SideStreams *ss, hipStream_t stream, hipStream_t (&st)[4], int helpers = 3) {
  for (int i = 0; i < 4; ++i) st[i] = stream;
  if (!ss) return hipSuccess;
  hipError_t e = hipEventRecord(ss->fork, stream);
  if (e != hipSuccess) return e;
  for (int i = 0; i < helpers; ++i) {
    if ((e = hipStreamWaitEvent(ss->s[i], ss->fork, 0)) != hipSuccess) return e;
    st[i + 1] = ss->s[i];
  }
  return hipSuccess;
}

static hipError_t join_streams(SideStreams *ss, hipStream_t stream, int helpers = 3) {
  if (!ss) return hipSuccess;
  for (int i = 0; i < helpers; ++i) {
    hipError_t e = hipEventRecord(ss->join[i], ss->s[i]);
    if (e != hipSuccess) return e;
    if ((e = hipStreamWaitEvent(stream, ss->join[i], 0)) != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_svc_group_rows(int count, int V, int groups, const int32_t *mat_rows, int32_t *group_rows,
                                 int32_t *mat_groups, hipStream_t stream) {
  hipLaunchKernelGGL(svc_group_rows_kernel, dim3(1), dim3(1024), 0, stream, count, V, groups, mat_rows, group_rows, mat_groups);
  return hipGetLastError();
}

hipError_t launch_svc_count(const SvcArgs &a, int order, hipStream_t stream) {
  const int m_vec = a.group_rows ? a.groups : (a.M + a.V - 1) / a.V;
  hipError_t e;
  if (m_vec == 0) {
    // no groups: only the scan runs, which writes vec_row_ptr[0] = 0 (and empty class lists)
  } else if (svc_direct(order, a.K)) {
    const size_t lds = 128 + (size_t)((a.K + 31) / 32) * 4;  // at most 16 KB
    hipLaunchKernelGGL((svc_count_distinct_kernel<256>), dim3(m_vec), dim3(256), lds, stream, a);
    if ((e = hipGetLastError()) != hipSuccess) return e;
  } else if (order == 0) {
    // One pass over the groups per size class, each taking the groups of its class; a group's class
    // is decided from min(non-zeros of the group, K), an upper bound of its distinct columns.
    SideStreams *ss = side_streams_for(stream);
    std::unique_lock<std::mutex> sequence;
    if (ss) sequence = std::unique_lock<std::mutex>(ss->in_use);
    hipStream_t st[4];
    if ((e = fork_streams(ss, stream, st)) != hipSuccess) return e;
    // (from here on the helpers are joined back into the caller's stream whatever happens)
    e = launch_lds_class<64>(a, m_vec, -1, kSmallKeys, 512, st[0]);
    if (e == hipSuccess) e = launch_lds_class<256>(a, m_vec, kSmallKeys, kMediumKeys, 2048, st[1]);
    if (e == hipSuccess) e = launch_lds_class<1024>(a, m_vec, kMediumKeys, kLargeKeys, 8192, st[2]);
    if (e == hipSuccess) {
      hipLaunchKernelGGL((svc_merge_cpython_kernel<1024, false>), dim3(m_vec), dim3(1024), 128, st[3], a, kLargeKeys,
                         0x7fffffff, 0);
      e = hipGetLastError();
    }
    const hipError_t ej = join_streams(ss, stream);
    if (e != hipSuccess) return e;
    if (ej != hipSuccess) return ej;
  } else {
    const int words = (a.K + 31) / 32;
    const size_t lds = 128 + (size_t)words * 8;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    auto kern = svc_merge_sorted_kernel<256>;
    if (lds > 64 * 1024) {
      static int raised[kMaxDevices] = {};
      if ((e = raise_lds_limit(reinterpret_cast<const void *>(kern), lds, raised)) != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kern, dim3(m_vec), dim3(256), lds, stream, a);
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  if (svc_direct(order, a.K))
    hipLaunchKernelGGL(svc_scan_classify_kernel, dim3(1), dim3(1024), 0, stream, m_vec, a.vec_row_ptr, a.class_lists,
                       a.class_counts, a.list_stride);
  else
    hipLaunchKernelGGL(svc_scan_kernel, dim3(1), dim3(1024), 0, stream, m_vec, a.vec_row_ptr);
  return hipGetLastError();
}

hipError_t launch_svc_fill(const SvcArgs &args, int order, const uint16_t *csr_val, const int32_t *vec_row_ptr,
                           int32_t *vec_col, uint16_t *vec_val, hipStream_t stream) {
  const int m_vec = args.group_rows ? args.groups : (args.M + args.V - 1) / args.V;
  if (!svc_direct(order, args.K)) {
    hipLaunchKernelGGL((svc_fill_kernel<512>), dim3(m_vec), dim3(512), 0, stream, args, csr_val, vec_row_ptr, vec_col,
                       csr_val ? vec_val : nullptr);
    return hipGetLastError();
  }
  // Direct mode: the merge itself, one launch per size class over the groups of that class (known exactly from
  // the row pointer), every group writing its own output.  The classes are independent kernels over disjoint
  // groups; the class of the largest groups goes out first, on the caller's stream: a single group of
  // thousands of columns takes longer than all the small groups together.
  SvcArgs a = args;
  a.scanned = vec_row_ptr;
  a.vec_col = vec_col;
  a.vec_val = csr_val ? vec_val : nullptr;
  a.csr_val = csr_val;
  const uint32_t key_bits = bits_of(a.K);
  // A group cannot hold more distinct columns than the matrix has columns or entries: the launches of the classes
  // above that bound are left out (each would cost a launch's latency to find its list empty).
  const long long bound = a.nnz < a.K ? a.nnz : (long long)a.K;
  const bool medium = bound > kSmallKeys, large = bound > kMediumKeys, xlarge = bound > kLargeKeys, beyond = bound > kXLargeKeys;
  const int cus = 256;
  hipError_t e = hipSuccess;
  // Grids: what the chip holds at once for the class's workgroup size and LDS, at most one workgroup per group.
  // The two classes of 1229 .. 4914 and 307 .. 1228 columns share a launch on the caller's stream (1024 threads
  // and 8192-slot tables for both): with one such workgroup per CU resident every group (up to the number of CUs) of either
  // class starts at once, and nothing that could outlast the largest group waits on a helper stream to begin.
  // These workgroups are chains of LDS round trips: each gets a CU to itself (by asking for more than half its LDS).
  auto rare_classes = [&](hipStream_t s) {
    if (e == hipSuccess && xlarge) e = launch_fast_class<1024, false>(a, min(m_vec, cus), 3, 3, kXLargeKeys, 32768, key_bits, s);
    if (e == hipSuccess && beyond) {
      // more columns than a 32768-slot table takes: 64-bit entries in the workspace
      hipLaunchKernelGGL((svc_merge_cpython_kernel<1024, false>), dim3(min(m_vec, cus)), dim3(1024), 128, s, a, 0, 0, 0);
      e = hipGetLastError();
    }
  };
  if (!medium || m_vec <= cus) {
    // Everything on the caller's stream: either no group can be larger than the small class, or the matrix has so
    // few groups that each gets a CU of its own in one launch of the wide workgroups (which then also take the
    // small groups); a fork and a join of a helper stream would cost more than they hide.
    if (!medium)
      e = launch_fast_class<64, true>(a, min(m_vec, 32 * cus), 0, 0, kSmallKeys, 512, key_bits, stream);
    else
      e = launch_fast_class<1024, true>(a, m_vec, large ? 2 : 1, 0, kLargeKeys, 8192, key_bits, stream, 81 * 1024);
    rare_classes(stream);
    return e;
  }
  // The many small groups, and the two classes that are nearly always empty, follow each other on one helper
  // stream: one fork and one join.
  SideStreams *ss = side_streams_for(stream);
  std::unique_lock<std::mutex> sequence;
  if (ss) sequence = std::unique_lock<std::mutex>(ss->in_use);
  hipStream_t st[4];
  if ((e = fork_streams(ss, stream, st, 1)) != hipSuccess) return e;
  // (from here on the helper is joined back into the caller's stream whatever happens)
  e = launch_fast_class<1024, true>(a, min(m_vec, cus), large ? 2 : 1, 1, kLargeKeys, 8192, key_bits, st[0], 81 * 1024);
  if (e == hipSuccess) e = launch_fast_class<64, true>(a, min(m_vec, 32 * cus), 0, 0, kSmallKeys, 512, key_bits, st[1]);
  rare_classes(st[1]);
  const hipError_t ej = join_streams(ss, stream, 1);
  return e != hipSuccess ? e : ej;
}

}  // namespace sspmm
