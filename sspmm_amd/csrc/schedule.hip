// Builds the row-panel schedule of the load-balanced SpMM on the device (see schedule.h).
//
// Integer work over the m_vec + 1 row offsets: two reductions and one prefix scan, done by a single
// workgroup of 1024 threads (the offsets of the matrices this format is used on are a few KB to a few
// MB; the work is bound by the latency of a dozen workgroup barriers, not by bytes).
#include "schedule.h"

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
                                              long long counters_per_cut_row, unsigned long long *scratch) {
  if (counters_to_clear < 0) counters_to_clear = (long long)header[kHdrSplitRows] * counters_per_cut_row;
  for (long long i = threadIdx.x; i < counters_to_clear; i += kBuildThreads) counters[i] = 0;
  const int budget = header[kHdrBudget];
  const long long n_slots = header[kHdrSlots];
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
    const unsigned long long ex2 = block_exclusive_scan64(r < m_vec && !pcs ? 1ull : 0ull, &t2, scratch);
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
        const long long at = n_slots + (long long)(carry_whole + ex2);
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
  }
}

__global__ __launch_bounds__(kBuildThreads) void schedule_fill_kernel(int m_vec, const int32_t *__restrict__ row_offsets,
                                                                      const int32_t *__restrict__ header,
                                                                      ScheduleItem *__restrict__ items, long long item_cap,
                                                                      int32_t *__restrict__ counters, long long counters_to_clear,
                                                                      long long counters_per_cut_row) {
  __shared__ unsigned long long scratch[kBuildThreads / 64];
  schedule_fill(m_vec, row_offsets, header, items, item_cap, counters, counters_to_clear, counters_per_cut_row, scratch);
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

hipError_t launch_schedule_measure(int m_vec, const int32_t *row_offsets, int budget, int64_t slot_cap, int32_t *header,
                                   hipStream_t stream) {
  hipLaunchKernelGGL(schedule_measure_kernel, dim3(1), dim3(kBuildThreads), 0, stream, m_vec, row_offsets, budget,
                     (long long)slot_cap, header);
  return hipGetLastError();
}

hipError_t launch_schedule_fill(int m_vec, const int32_t *row_offsets, const ScheduleView &view, int64_t item_cap,
                                int64_t counters_to_clear, int64_t counters_per_cut_row, hipStream_t stream) {
  hipLaunchKernelGGL(schedule_fill_kernel, dim3(1), dim3(kBuildThreads), 0, stream, m_vec, row_offsets, view.header,
                     view.items, (long long)item_cap, view.counters, (long long)counters_to_clear,
                     (long long)counters_per_cut_row);
  return hipGetLastError();
}

hipError_t launch_schedule_build(int m_vec, const int32_t *row_offsets, int64_t slot_cap, const ScheduleView &view,
                                 int64_t item_cap, int64_t counters_per_cut_row, hipStream_t stream) {
  hipLaunchKernelGGL(schedule_build_kernel, dim3(1), dim3(kBuildThreads), 0, stream, m_vec, row_offsets, (long long)slot_cap,
                     view.header, view.items, (long long)item_cap, view.counters, (long long)counters_per_cut_row);
  return hipGetLastError();
}

}  // namespace sspmm
