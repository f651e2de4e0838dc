// Builds the row-panel schedule of the load-balanced SpMM on the device (see schedule.h).
//
// Integer work over the m_vec + 1 row offsets: two reductions and one prefix scan, done by a single
// workgroup of 1024 threads (the offsets of the matrices this format is used on are a few KB to a few
// MB; the work is bound by the latency of a dozen workgroup barriers, not by bytes).
#include "schedule.h"

#include "lane_ops.h"

namespace sspmm {

static constexpr int kBuildThreads = 1024;

__device__ __forceinline__ int steps_of(int len) { return len > 0 ? (len + 31) >> 5 : 1; }
// panels of a row of `steps` steps under `budget` (0: the row stays whole)
__device__ __forceinline__ int pieces_of(int steps, int budget) { return steps > budget ? (steps + budget - 1) / budget : 0; }

// Sum over the workgroup of one 64-bit value per thread.  Contains barriers.
__device__ __forceinline__ unsigned long long block_sum(unsigned long long x, unsigned long long *scratch) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) x += __shfl_xor(x, d, 64);
  __syncthreads();  // scratch may still be read from a previous call
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = x;
  __syncthreads();
  unsigned long long s = 0;
#pragma unroll
  for (int w = 0; w < kBuildThreads / 64; ++w) s += scratch[w];
  return s;
}

__device__ __forceinline__ int block_max(int x, unsigned long long *scratch) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) x = max(x, __shfl_xor(x, d, 64));
  __syncthreads();
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = (unsigned long long)(unsigned)x;
  __syncthreads();
  int s = 0;
#pragma unroll
  for (int w = 0; w < kBuildThreads / 64; ++w) s = max(s, (int)scratch[w]);
  return s;
}

__device__ __forceinline__ void schedule_measure(int m_vec, const int32_t *__restrict__ row_offsets, int budget_in,
                                                 long long slot_cap, int32_t *header, unsigned long long *scratch) {
  unsigned long long steps_sum = 0;
  int steps_max = 0;
  for (int r = threadIdx.x; r < m_vec; r += kBuildThreads) {
    const int s = steps_of(row_offsets[r + 1] - row_offsets[r]);
    steps_sum += (unsigned long long)s;
    steps_max = max(steps_max, s);
  }
  const unsigned long long total = block_sum(steps_sum, scratch);
  const int longest = block_max(steps_max, scratch);
  // Chosen from the pattern: no shorter than twice the mean row, so that only rows well above the rest are cut
  // (a pattern of even rows keeps them whole however long they are).
  long long budget = budget_in;
  if (budget <= 0) {
    const long long by_items = (long long)((total + kScheduleTargetItems - 1) / kScheduleTargetItems);
    const long long by_mean = m_vec > 0 ? (long long)((2 * total + (unsigned long long)m_vec - 1) / (unsigned long long)m_vec) : 0;
    budget = max((long long)kScheduleMinBudget, max(by_items, by_mean));
  }
  unsigned long long slots = 0, split_rows = 0;
  for (;;) {  // (every thread sees the same sums, so the loop is uniform)
    unsigned long long mine = 0;  // panels in the low half, cut rows in the high half
    for (int r = threadIdx.x; r < m_vec; r += kBuildThreads) {
      const int pcs = pieces_of(steps_of(row_offsets[r + 1] - row_offsets[r]), (int)min(budget, (long long)0x7fffffff));
      if (pcs) mine += (unsigned long long)pcs + (1ull << 32);
    }
    const unsigned long long both = block_sum(mine, scratch);
    slots = both & 0xffffffffull;
    split_rows = both >> 32;
    if ((long long)slots <= slot_cap || budget >= longest) break;
    budget *= 2;
  }
  if (threadIdx.x == 0) {
    header[kHdrItems] = (int)(slots + ((unsigned long long)m_vec - split_rows));
    header[kHdrSplitRows] = (int)split_rows;
    header[kHdrSlots] = (int)slots;
    header[kHdrBudget] = (int)min(budget, (long long)0x7fffffff);
    header[kHdrNvec] = m_vec > 0 ? row_offsets[m_vec] : 0;
    header[kHdrMaxSteps] = longest;
    header[kHdrTotalSteps] = (int)min(total, (unsigned long long)0x7fffffff);
    header[7] = 0;
  }
}

__global__ __launch_bounds__(kBuildThreads) void schedule_measure_kernel(int m_vec, const int32_t *__restrict__ row_offsets,
                                                                         int budget_in, long long slot_cap,
                                                                         int32_t *__restrict__ header) {
  __shared__ unsigned long long scratch[kBuildThreads / 64];
  schedule_measure(m_vec, row_offsets, budget_in, slot_cap, header, scratch);
}

// Exclusive prefix sum of one 64-bit value per thread over the workgroup; *total = sum.  Contains barriers.
__device__ __forceinline__ unsigned long long block_exclusive_scan64(unsigned long long x, unsigned long long *total,
                                                                      unsigned long long *scratch) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned long long incl = x;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const unsigned long long y = __shfl_up(incl, d, 64);
    if (lane >= d) incl += y;
  }
  __syncthreads();
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  unsigned long long base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kBuildThreads / 64; ++w) {
    const unsigned long long t = scratch[w];
    if (w < wave) base += t;
    sum += t;
  }
  *total = sum;
  return base + incl - x;
}

__device__ __forceinline__ void schedule_fill(int m_vec, const int32_t *__restrict__ row_offsets, const int32_t *header,
                                              ScheduleItem *__restrict__ items, long long item_cap,
                                              int32_t *__restrict__ counters, long long counters_to_clear,
                                              long long counters_per_cut_row, unsigned long long *scratch,
                                              int32_t *__restrict__ bundles = nullptr, int bundle_steps = 0,
                                              int32_t *header_out = nullptr) {
  if (counters_to_clear < 0) counters_to_clear = (long long)header[kHdrSplitRows] * counters_per_cut_row;
  for (long long i = threadIdx.x; i < counters_to_clear; i += kBuildThreads) counters[i] = 0;
  const int budget = header[kHdrBudget];
  const long long n_slots = header[kHdrSlots], n_items = header[kHdrItems];
  const bool bundling = bundles != nullptr && bundle_steps > 0;
  if (bundling && threadIdx.x == 0) {  // (what a pattern without whole rows leaves: no bundle)
    bundles[0] = (int)n_slots;
    header_out[kHdrBundles] = 0;
  }
  unsigned long long carry_enders = 0;
  // Two scans per 1024 rows: the panels of cut rows together with the number of cut rows (panels in bits 0-39 of
  // the running sum, cut rows from bit 40 on), and the rows that stay whole.
  unsigned long long carry_slots_split = 0, carry_whole = 0;
  for (int base = 0; base < m_vec; base += kBuildThreads) {
    const int r = base + (int)threadIdx.x;
    int beg = 0, end = 0, steps = 0, pcs = 0;
    if (r < m_vec) {
      beg = row_offsets[r];
      end = row_offsets[r + 1];
      steps = steps_of(end - beg);
      pcs = pieces_of(steps, budget);
    }
    unsigned long long t1, t2;
    const unsigned long long ex1 =
        block_exclusive_scan64(r < m_vec && pcs ? (unsigned long long)pcs + (1ull << 40) : 0ull, &t1, scratch);
    // (rows that stay whole: their number in the low half, their steps in the high half)
    const unsigned long long ex2 =
        block_exclusive_scan64(r < m_vec && !pcs ? 1ull + ((unsigned long long)steps << 32) : 0ull, &t2, scratch);
    // Bundles of the rows that stay whole: a row whose steps reach or cross a multiple of bundle_steps in the
    // running sum of steps, or that is the 64th of its bundle (the rows of a bundle are held one per lane), ends
    // its bundle; so does a row of more than half a bundle's steps and the row in front of one (such a row is a
    // bundle of its own: a bundle then never holds more than a bundle and a half).  The number of such rows before
    // a row is the row's bundle.
    unsigned long long ex3 = 0, t3 = 0;
    bool ender = false;
    if (bundling) {  // (uniform)
      const unsigned long long before = (carry_whole + ex2) >> 32, count_before = (carry_whole + ex2) & 0xffffffffull;
      const int next_steps = r + 1 < m_vec ? steps_of(row_offsets[r + 2] - end) : 0;
      ender = r < m_vec && !pcs &&
              ((before + (unsigned long long)steps) / (unsigned)bundle_steps > before / (unsigned)bundle_steps ||
               (count_before & 63ull) == 63ull || 2 * steps > bundle_steps || 2 * next_steps > bundle_steps);
      ex3 = block_exclusive_scan64(ender ? 1ull : 0ull, &t3, scratch);
    }
    if (r < m_vec) {
      if (pcs) {
        const unsigned long long at = carry_slots_split + ex1;
        const long long first_slot = (long long)(at & ((1ull << 40) - 1ull));
        const int split_id = (int)(at >> 40);
        const int per = (steps + pcs - 1) / pcs;  // steps per panel: the panels of a row are even
        for (int pc = 0; pc < pcs; ++pc) {
          if (first_slot + pc >= item_cap) break;
          ScheduleItem it;
          it.row = r;
          it.kbeg = min(end, beg + pc * per * 32);
          it.kend = min(end, it.kbeg + per * 32);
          it.split_id = split_id;
          it.first_slot = (int)first_slot;
          it.pieces = pcs;
          it.piece = pc;
          it.pad = 0;
          items[first_slot + pc] = it;
        }
      } else {
        const long long at = n_slots + (long long)((carry_whole + ex2) & 0xffffffffull);
        if (bundling && at < item_cap) {
          const long long b = (long long)(carry_enders + ex3);
          if (ender) bundles[b + 1] = (int)(at + 1);
          if (at == n_items - 1) {  // the last row that stays whole closes the table
            bundles[b + 1] = (int)n_items;
            header_out[kHdrBundles] = (int)(b + 1);
          }
        }
        if (at < item_cap) {
          ScheduleItem it;
          it.row = r;
          it.kbeg = beg;
          it.kend = end;
          it.split_id = -1;
          it.first_slot = 0;
          it.pieces = 0;
          it.piece = 0;
          it.pad = 0;
          items[at] = it;
        }
      }
    }
    carry_slots_split += t1;
    carry_whole += t2;
    carry_enders += t3;
  }
}

__global__ __launch_bounds__(kBuildThreads) void schedule_fill_kernel(int m_vec, const int32_t *__restrict__ row_offsets,
                                                                      const int32_t *__restrict__ header,
                                                                      ScheduleItem *__restrict__ items, long long item_cap,
                                                                      int32_t *__restrict__ counters, long long counters_to_clear,
                                                                      long long counters_per_cut_row,
                                                                      int32_t *__restrict__ bundles, int bundle_steps,
                                                                      int32_t *__restrict__ header_out) {
  __shared__ unsigned long long scratch[kBuildThreads / 64];
  schedule_fill(m_vec, row_offsets, header, items, item_cap, counters, counters_to_clear, counters_per_cut_row, scratch,
                bundles, bundle_steps, header_out);
}

// Both steps in one launch (the header passes through global memory inside the one workgroup).
__global__ __launch_bounds__(kBuildThreads) void schedule_build_kernel(int m_vec, const int32_t *__restrict__ row_offsets,
                                                                       long long slot_cap, int32_t *header,
                                                                       ScheduleItem *__restrict__ items, long long item_cap,
                                                                       int32_t *__restrict__ counters,
                                                                       long long counters_per_cut_row) {
  __shared__ unsigned long long scratch[kBuildThreads / 64];
  schedule_measure(m_vec, row_offsets, 0, slot_cap, header, scratch);
  __threadfence_block();
  __syncthreads();
  schedule_fill(m_vec, row_offsets, header, items, item_cap, counters, -1, counters_per_cut_row, scratch);
}

// ------------------------------------------------------------------------------------------
// The same schedule for patterns of at most kSmallRows vector-rows, which is what a call that rebuilds
// its schedule every time usually brings.  One workgroup again, arranged for the latency of its one CU:
// every thread keeps its rows' offsets in registers (row offsets are read from memory once instead of
// once per pass); the header reaches the other threads as values every thread computes alike instead
// of through memory; the places of all items come from one scan that carries a value per block of
// 512 rows; a thread's rows are 512 apart, so that the items of rows that stay whole leave the wave
// as contiguous stores; and the panels of cut rows are written one per thread from a list in LDS (a
// loop over a row's panels would make its whole wave wait for the longest row).
// Writes exactly what schedule_measure + schedule_fill write.
static constexpr int kSmallThreads = 512;  // 8 waves: 256 registers per thread (the scans hold many words at once)
static constexpr int kSmallRowsPerThread = 8;
static constexpr int kSmallRows = kSmallRowsPerThread * kSmallThreads;
static constexpr int kSmallCutRows = 2048;  // cut rows whose panels are written one per thread (five words of LDS each)

// What a row adds to the running sums, in one word: its panels in bits 0-31 and 1 in bit 32 if it is cut
// (bits 32-47: cut rows), else 1 in bit 48 (bits 48-63: rows that stay whole; at most kSmallRows = 2^12 rows).
__device__ __forceinline__ unsigned long long row_word(int steps, int pcs) {
  return steps == 0 ? 0ull : pcs ? (unsigned long long)(unsigned)pcs + (1ull << 32) : (1ull << 48);
}

// Sum over the workgroup of a 64-bit value per thread and maximum of an int per thread.  One barrier; `scratch`
// (2 x kSmallThreads / 64 words) must not be in use by an earlier step that some wave may still be reading.
__device__ __forceinline__ unsigned long long small_sum_max(unsigned long long a, int m, int *m_out,
                                                            unsigned long long *scratch) {
  constexpr int W = kSmallThreads / 64;
  a = wave_inclusive_sum(a);
  m = (int)wave_inclusive_max((uint32_t)m);  // (not negative)
  if ((threadIdx.x & 63) == 63) {
    scratch[threadIdx.x >> 6] = a;
    scratch[W + (threadIdx.x >> 6)] = (unsigned long long)(unsigned)m;
  }
  __syncthreads();
  unsigned long long s = 0;
  int mm = 0;
#pragma unroll
  for (int w = 0; w < W; ++w) {
    s += scratch[w];
    mm = max(mm, (int)scratch[W + w]);
  }
  *m_out = mm;
  return s;
}

// R exclusive prefix sums at once, each over the workgroup's threads: x[i] becomes the sum of the x[i] of the
// threads before this one, total[i] the sum over all threads; only for i < n, the others (whose x[i] is 0
// in every thread) get 0.  One barrier; same rule for `scratch` (R x kSmallThreads / 64 words).
template <int R>
__device__ __forceinline__ void small_exclusive_scans(unsigned long long (&x)[R], unsigned long long (&total)[R], int n,
                                                      unsigned long long *scratch) {
  constexpr int W = kSmallThreads / 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned long long incl[R];
#pragma unroll
  for (int i = 0; i < R; ++i) incl[i] = x[i];
#pragma unroll
  for (int i = 0; i < R; ++i)
    if (i < n) incl[i] = wave_inclusive_sum(incl[i]);  // (uniform)
  if (lane == 63) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (i < n) scratch[i * W + wave] = incl[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < R; ++i) {
    unsigned long long base = 0, sum = 0;
    if (i < n) {
#pragma unroll
      for (int w = 0; w < W; ++w) {
        const unsigned long long t = scratch[i * W + w];
        if (w < wave) base += t;
        sum += t;
      }
    }
    total[i] = sum;
    x[i] = base + incl[i] - x[i];
  }
}

__device__ __forceinline__ void store_item(ScheduleItem *__restrict__ at, int row, int kbeg, int kend, int split_id,
                                           int first_slot, int pieces, int piece) {
  ScheduleItem it;
  it.row = row;
  it.kbeg = kbeg;
  it.kend = kend;
  it.split_id = split_id;
  it.first_slot = first_slot;
  it.pieces = pieces;
  it.piece = piece;
  it.pad = 0;
  *at = it;
}

__global__ __launch_bounds__(kSmallThreads) void schedule_build_small_kernel(int m_vec, const int32_t *__restrict__ row_offsets,
                                                                             long long slot_cap, int32_t *__restrict__ header,
                                                                             ScheduleItem *__restrict__ items, long long item_cap,
                                                                             int32_t *__restrict__ counters,
                                                                             long long counters_per_cut_row) {
  constexpr int R = kSmallRowsPerThread, W = kSmallThreads / 64;
  // The sum and the scans of successive budgets each have words of their own: a wave may still be reading the
  // previous step's.  (A wave that writes the words of two steps ago again has passed the barrier in between.)
  __shared__ unsigned long long scratch_sum[2 * W], scratch_scan[2][R * W];
  __shared__ int cut_first[kSmallCutRows], cut_row[kSmallCutRows], cut_beg[kSmallCutRows], cut_end[kSmallCutRows],
      cut_pieces[kSmallCutRows];
  int beg[R], end[R], steps[R];  // of row i * kSmallThreads + threadIdx.x; steps 0: no such row
  unsigned long long steps_sum = 0;
  int steps_max = 0;
  int nvec = 0;  // (thread 0 only; fetched with the rows so that nothing waits for it later)
  if (threadIdx.x == 0) nvec = row_offsets[m_vec];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int r = i * kSmallThreads + (int)threadIdx.x;
    beg[i] = row_offsets[min(r, m_vec)];
    end[i] = row_offsets[min(r + 1, m_vec)];
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    steps[i] = i * kSmallThreads + (int)threadIdx.x < m_vec ? steps_of(end[i] - beg[i]) : 0;
    steps_sum += (unsigned long long)steps[i];
    steps_max = max(steps_max, steps[i]);
  }
  int longest;
  const unsigned long long total = small_sum_max(steps_sum, steps_max, &longest, scratch_sum);
  const long long by_items = (long long)((total + kScheduleTargetItems - 1) / kScheduleTargetItems);
  const long long by_mean = (long long)((2 * total + (unsigned long long)m_vec - 1) / (unsigned long long)m_vec);
  long long budget = max((long long)kScheduleMinBudget, max(by_items, by_mean));
  const int blocks = (m_vec + kSmallThreads - 1) / kSmallThreads;  // blocks of rows that hold rows
  int budget_i, pcs[R];
  unsigned long long before[R], in_block[R];  // row words of the rows before this one in its block; of the whole block
  unsigned long long all = 0;
  for (int turn = 0;; turn ^= 1) {
    budget_i = (int)min(budget, (long long)0x7fffffff);
#pragma unroll
    for (int i = 0; i < R; ++i) {
      pcs[i] = i < blocks ? pieces_of(steps[i], budget_i) : 0;  // (uniform: a wave skips the division)
      before[i] = row_word(steps[i], pcs[i]);
    }
    small_exclusive_scans<R>(before, in_block, blocks, scratch_scan[turn]);
    all = 0;
#pragma unroll
    for (int i = 0; i < R; ++i) all += in_block[i];
    if ((long long)(all & 0xffffffffull) <= slot_cap || budget >= longest) break;
    budget *= 2;
  }
  const long long slots = (long long)(all & 0xffffffffull);
  const int split_rows = (int)((all >> 32) & 0xffffull);
  if (threadIdx.x == 0) {
    header[kHdrItems] = (int)(slots + (long long)(m_vec - split_rows));
    header[kHdrSplitRows] = split_rows;
    header[kHdrSlots] = (int)slots;
    header[kHdrBudget] = budget_i;
    header[kHdrNvec] = nvec;
    header[kHdrMaxSteps] = longest;
    header[kHdrTotalSteps] = (int)min(total, (unsigned long long)0x7fffffff);
    header[7] = 0;
  }
  const long long counters_to_clear = (long long)split_rows * counters_per_cut_row;
  for (long long i = threadIdx.x; i < counters_to_clear; i += kSmallThreads) counters[i] = 0;
  const bool listed = split_rows <= kSmallCutRows;  // (uniform)
  unsigned long long blocks_before = 0;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    if (i >= blocks) break;  // (uniform)
    const unsigned long long at = blocks_before + before[i];
    blocks_before += in_block[i];
    if (!steps[i]) continue;
    const int r = i * kSmallThreads + (int)threadIdx.x;
    if (pcs[i]) {
      const long long first_slot = (long long)(at & 0xffffffffull);
      const int split_id = (int)((at >> 32) & 0xffffull);
      if (listed) {
        cut_first[split_id] = (int)first_slot;
        cut_row[split_id] = r;
        cut_beg[split_id] = beg[i];
        cut_end[split_id] = end[i];
        cut_pieces[split_id] = pcs[i];
      } else {
        const int per = (steps[i] + pcs[i] - 1) / pcs[i];  // steps per panel: the panels of a row are even
        for (int pc = 0; pc < pcs[i] && first_slot + pc < item_cap; ++pc) {
          const int kbeg = min(end[i], beg[i] + pc * per * 32);
          store_item(items + first_slot + pc, r, kbeg, min(end[i], kbeg + per * 32), split_id, (int)first_slot, pcs[i], pc);
        }
      }
    } else {
      const long long whole_at = slots + (long long)(at >> 48);
      if (whole_at < item_cap) store_item(items + whole_at, r, beg[i], end[i], -1, 0, 0, 0);
    }
  }
  if (!listed || slots == 0) return;  // (uniform)
  __syncthreads();
  for (long long slot = threadIdx.x; slot < slots && slot < item_cap; slot += kSmallThreads) {
    int lo = 0, hi = split_rows - 1;  // the last cut row whose first panel is at or before this one
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cut_first[mid] <= (int)slot)
        lo = mid;
      else
        hi = mid - 1;
    }
    const int b = cut_beg[lo], e = cut_end[lo], p = cut_pieces[lo], first_slot = cut_first[lo], pc = (int)slot - first_slot;
    const int per = (steps_of(e - b) + p - 1) / p;  // steps per panel: the panels of a row are even
    const int kbeg = min(e, b + pc * per * 32);
    store_item(items + slot, cut_row[lo], kbeg, min(e, kbeg + per * 32), lo, first_slot, p, pc);
  }
}

hipError_t launch_schedule_measure(int m_vec, const int32_t *row_offsets, int budget, int64_t slot_cap, int32_t *header,
                                   hipStream_t stream) {
  hipLaunchKernelGGL(schedule_measure_kernel, dim3(1), dim3(kBuildThreads), 0, stream, m_vec, row_offsets, budget,
                     (long long)slot_cap, header);
  return hipGetLastError();
}

hipError_t launch_schedule_fill(int m_vec, const int32_t *row_offsets, const ScheduleView &view, int64_t item_cap,
                                int64_t counters_to_clear, int64_t counters_per_cut_row, int bundle_steps,
                                hipStream_t stream) {
  hipLaunchKernelGGL(schedule_fill_kernel, dim3(1), dim3(kBuildThreads), 0, stream, m_vec, row_offsets, view.header,
                     view.items, (long long)item_cap, view.counters, (long long)counters_to_clear,
                     (long long)counters_per_cut_row, view.bundles, bundle_steps, view.header);
  return hipGetLastError();
}

hipError_t launch_schedule_build(int m_vec, const int32_t *row_offsets, int64_t slot_cap, const ScheduleView &view,
                                 int64_t item_cap, int64_t counters_per_cut_row, hipStream_t stream) {
  if (m_vec > 0 && m_vec <= kSmallRows)
    hipLaunchKernelGGL(schedule_build_small_kernel, dim3(1), dim3(kSmallThreads), 0, stream, m_vec, row_offsets,
                       (long long)slot_cap, view.header, view.items, (long long)item_cap, view.counters,
                       (long long)counters_per_cut_row);
  else
    hipLaunchKernelGGL(schedule_build_kernel, dim3(1), dim3(kBuildThreads), 0, stream, m_vec, row_offsets, (long long)slot_cap,
                       view.header, view.items, (long long)item_cap, view.counters, (long long)counters_per_cut_row);
  return hipGetLastError();
}

}  // namespace sspmm
