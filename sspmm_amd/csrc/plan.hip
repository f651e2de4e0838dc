// The plan object of the SpMM: what is worth knowing about a sparsity pattern before its first
// product, computed once (on the device, from the row offsets) and owned by the library.
//
// It holds the pattern's statistics (stored vectors, longest vector-row), which the asynchronous
// entry points without a plan cannot see because the row offsets live in device memory, and the
// row-panel schedule with its scratch memory (schedule.h), so that products with a plan allocate
// nothing.
#include "plan.h"

#include <mutex>
#include <new>

namespace sspmm {

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

// Scratch memory for partial tiles a plan may take; beyond it the budget is doubled until the panels fit.
static constexpr size_t kPlanPartialCap = (size_t)64 << 20;

int64_t schedule_slot_cap(size_t partial_bytes, int V, int N, int batch) {
  const int64_t tiles = ((int64_t)N + 63) / 64;
  const int64_t per_slot = (int64_t)partial_tile_bytes(V) * (tiles > 0 ? tiles : 1) * (batch > 0 ? batch : 1);
  return (int64_t)partial_bytes / per_slot;
}

hipError_t plan_create(int m_vec, int V, int K, const int32_t *row_offsets, int max_N, int max_batch, int budget,
                       hipStream_t stream, Plan **out) {
  *out = nullptr;
  Plan *pl = new (std::nothrow) Plan();
  if (!pl) return hipErrorOutOfMemory;
  hipError_t e = hipGetDevice(&pl->device);
  if (e != hipSuccess) {
    delete pl;
    return e;
  }
  pl->m_vec = m_vec;
  pl->V = V;
  pl->K = K;
  pl->max_N = max_N;
  pl->max_batch = max_batch;
  pl->tiles_max = (max_N + 63) / 64;
  for (int i = 0; i < kHdrWords; ++i) pl->header[i] = 0;
  if (m_vec == 0) {
    *out = pl;
    return hipSuccess;
  }
  int32_t *d_header = nullptr;
  if ((e = hipMalloc(reinterpret_cast<void **>(&d_header), 256)) != hipSuccess) {
    delete pl;
    return e;
  }
  const int64_t slot_cap = schedule_slot_cap(kPlanPartialCap, V, max_N, max_batch);
  e = launch_schedule_measure(m_vec, row_offsets, budget, slot_cap, d_header, stream);
  if (e == hipSuccess) e = hipMemcpyAsync(pl->header, d_header, sizeof(pl->header), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);
  (void)hipFree(d_header);
  if (e != hipSuccess) {
    delete pl;
    return e;
  }
  const size_t n_items = (size_t)pl->header[kHdrItems], n_split = (size_t)pl->header[kHdrSplitRows];
  const size_t n_slots = (size_t)pl->header[kHdrSlots];
  const size_t units = (size_t)(pl->tiles_max > 0 ? pl->tiles_max : 1) * (size_t)(max_batch > 0 ? max_batch : 1);
  const size_t off_bundles = 256;
  const size_t off_items = off_bundles + align256((n_items - n_slots + 2) * sizeof(int32_t));
  const size_t off_counters = off_items + align256(n_items * sizeof(ScheduleItem));
  pl->counters = n_split * units;
  const size_t off_partials = off_counters + align256(pl->counters * 4);
  pl->bytes = off_partials + align256(n_slots * units * partial_tile_bytes(V));
  if ((e = hipMalloc(&pl->memory, pl->bytes)) != hipSuccess) {
    delete pl;
    return e;
  }
  unsigned char *base = static_cast<unsigned char *>(pl->memory);
  pl->view.header = reinterpret_cast<int32_t *>(base);
  pl->view.bundles = reinterpret_cast<int32_t *>(base + off_bundles);
  pl->view.items = reinterpret_cast<ScheduleItem *>(base + off_items);
  pl->view.counters = reinterpret_cast<int32_t *>(base + off_counters);
  pl->view.partials = base + off_partials;
  e = hipMemcpyAsync(pl->view.header, pl->header, sizeof(pl->header), hipMemcpyHostToDevice, stream);
  if (e == hipSuccess)
    e = launch_schedule_fill(m_vec, row_offsets, pl->view, (int64_t)n_items, (int64_t)pl->counters, 0, kScheduleBundleSteps, stream);
  // (the fill leaves the number of bundles in the header)
  if (e == hipSuccess) e = hipMemcpyAsync(pl->header, pl->view.header, sizeof(pl->header), hipMemcpyDeviceToHost, stream);
  if (e == hipSuccess) e = hipStreamSynchronize(stream);  // products with the plan may come on any stream
  if (e != hipSuccess) {
    (void)hipFree(pl->memory);
    delete pl;
    return e;
  }
  *out = pl;
  return hipSuccess;
}

hipError_t plan_destroy(Plan *pl) {
  if (!pl) return hipSuccess;
  hipError_t e = hipSuccess;
  if (pl->memory) e = hipFree(pl->memory);
  delete pl;
  return e;
}

hipError_t launch_spmm_planned(const Plan &pl, const SpmmArgs &a, bool out_f16, hipStream_t stream) {
  const int forced = kernel_override();
  const bool can_balance = balanced_kernel_applies(a, pl.V, out_f16) && a.N <= pl.max_N && a.batch <= pl.max_batch;
  // Rows are cut only when some row is much longer than the rest (the budget is at least twice the mean row):
  // an even pattern keeps the kernels chosen by shape.
  const bool skewed = pl.header[kHdrSplitRows] > 0;
  const bool epilogue = a.bias != nullptr || a.act != 0;  // (the load-balanced kernel does not apply one)
  if (can_balance && !epilogue && (forced == 7 || (forced == 0 && skewed)))
    return launch_spmm_balanced(a, pl.V, out_f16, pl.view,
                                pl.header[kHdrBundles] > 0 ? pl.header[kHdrSlots] + pl.header[kHdrBundles] : pl.header[kHdrItems],
                                false, stream, pl.header[kHdrBundles] > 0 ? pl.header[kHdrSlots] : -1);
  SpmmArgs b = a;
  // (at least 1: an empty pattern is as sparse as it gets, and 0 would say the density is unknown)
  b.mean_row_vectors = pl.m_vec > 0 ? (int)((int64_t)pl.header[kHdrNvec] / pl.m_vec) + 1 : 0;
  return launch_spmm(b, pl.V, out_f16, stream);
}

// ------------------------------------------------------------------------------------------
// The same product for callers that can neither allocate nor keep a plan (a pattern that changes from call to
// call inside a captured graph, a serving loop, a harness that forbids allocation): the schedule, its counters and
// the partial tiles live in one array of device memory that is part of the library's code object, so every GPU the
// library runs on holds it from the first use of the library to the end of the process.  The schedule is built on
// the device by every call (the host never sees the row offsets); the product's grid covers the most items the
// schedule can have, and the workgroups beyond its end return at once.
static constexpr int kStaticMaxRows = 32768;       // vector-rows
static constexpr int kStaticMaxN = 4096;           // columns of B: 64 column tiles
static constexpr int64_t kStaticMaxSlots = 4096;   // panels of cut rows
static constexpr size_t kStaticItemsOff = 256;
static constexpr size_t kStaticCountersOff = kStaticItemsOff + (size_t)(kStaticMaxRows + kStaticMaxSlots) * sizeof(ScheduleItem);
static constexpr size_t kStaticCounters = (size_t)(kStaticMaxSlots / 2) * (kStaticMaxN / 64);  // a cut row has two panels or more
static constexpr size_t kStaticPartialsOff = kStaticCountersOff + kStaticCounters * 4;
static constexpr size_t kStaticPartialBytes = (size_t)8 << 20;
static constexpr size_t kStaticScratchBytes = kStaticPartialsOff + kStaticPartialBytes;  // about 9.7 MB
static_assert(kStaticPartialsOff % 256 == 0, "the partial tiles are read with 16-byte loads");

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// The array's address on each device (the name `scratch` is a host-side stand-in, not a device address), looked up
// once per device with that device current.
static constexpr int kStaticMaxDevices = 64;
static unsigned char *g_scratch_ptr[kStaticMaxDevices] = {};
static std::mutex g_scratch_mutex;

static hipError_t static_scratch(unsigned char **ptr, hipStream_t stream) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kStaticMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    // The look-up is not a call to make while a stream records a graph: the first use on a device has to come
    // before the capture (any call of the entry point outside a capture will do).
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (stream && hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return hipErrorInvalidValue;
    void *p = nullptr;
    if ((e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) != hipSuccess) return e;
    g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
  }
  *ptr = g_scratch_ptr[dev];
  return hipSuccess;
}

bool static_spmm_fits(int m_vec, int N) { return m_vec <= kStaticMaxRows && N <= kStaticMaxN; }

hipError_t launch_spmm_static(const SpmmArgs &a, int V, bool out_f16, hipStream_t stream) {
  if (!balanced_kernel_applies(a, V, out_f16)) return launch_spmm(a, V, out_f16, stream);  // (needs no scratch)
  unsigned char *base = nullptr;
  hipError_t e = static_scratch(&base, stream);
  if (e != hipSuccess) return e;
  ScheduleView view;
  view.header = reinterpret_cast<int32_t *>(base);
  view.bundles = nullptr;
  view.items = reinterpret_cast<ScheduleItem *>(base + kStaticItemsOff);
  view.counters = reinterpret_cast<int32_t *>(base + kStaticCountersOff);
  view.partials = base + kStaticPartialsOff;
  const int64_t tiles = ((int64_t)a.N + 63) / 64;
  int64_t slot_cap = schedule_slot_cap(kStaticPartialBytes, V, a.N, 1);
  if (slot_cap > kStaticMaxSlots) slot_cap = kStaticMaxSlots;
  // Everything the product reads is rewritten first: header, items, and the counters of the rows that are cut
  // (kernels on the caller's stream, which order themselves; no memset node for a capturing caller).
  if ((e = launch_schedule_build(a.m_vec, a.row_offsets, slot_cap, view, (int64_t)kStaticMaxRows + kStaticMaxSlots, tiles,
                                 stream)) != hipSuccess)
    return e;
  // The schedule has at most one item per row that stays whole plus the panels of the cut rows; a row holds at most
  // K vectors (ceil(K / 32) steps) and a panel at least kScheduleMinBudget steps.
  int64_t panels_bound = (int64_t)a.m_vec * ((int64_t)a.K / (32 * kScheduleMinBudget) + 2);
  if (panels_bound > slot_cap) panels_bound = slot_cap;
  return launch_spmm_balanced(a, V, out_f16, view, a.m_vec + (int)panels_bound, true, stream);
}

}  // namespace sspmm
