// Host side of the SpMM plan (the object behind sspmm_plan_create / sspmm_plan_destroy).
#ifndef SSPMM_AMD_PLAN_H
#define SSPMM_AMD_PLAN_H

#include "schedule.h"
#include "spmm_kernels.h"

namespace sspmm {

struct Plan {
  int device = 0;
  int m_vec = 0, V = 0, K = 0, max_N = 0, max_batch = 0, tiles_max = 0;
  int32_t header[kHdrWords] = {};  // host copy of the schedule's header
  void *memory = nullptr;          // one allocation: header, items, counters, partial tiles
  size_t bytes = 0, counters = 0;
  ScheduleView view = {};
};

// Partial-tile slots that fit into `partial_bytes` for products up to N columns and `batch` elements.
int64_t schedule_slot_cap(size_t partial_bytes, int V, int N, int batch);

// budget: steps per panel, 0 = chosen from the pattern.  Synchronises `stream` (reads the pattern's
// statistics back, allocates, fills the schedule).
hipError_t plan_create(int m_vec, int V, int K, const int32_t *row_offsets, int max_N, int max_batch, int budget,
                       hipStream_t stream, Plan **out);
hipError_t plan_destroy(Plan *plan);

// The SpMM with what the plan knows: the load-balanced kernel when the pattern's rows are uneven, otherwise the
// kernels launch_spmm picks.  Allocates nothing.
hipError_t launch_spmm_planned(const Plan &plan, const SpmmArgs &args, bool out_f16, hipStream_t stream);

// The single product with the load-balanced kernel and no plan: schedule and scratch in a static device array of
// the library, rebuilt by every call.  Only for static_spmm_fits; batch must be 1.  Allocates nothing.
bool static_spmm_fits(int m_vec, int N);
hipError_t launch_spmm_static(const SpmmArgs &args, int V, bool out_f16, hipStream_t stream);

}  // namespace sspmm
#endif
