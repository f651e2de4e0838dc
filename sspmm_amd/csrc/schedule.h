// The row-panel schedule of the load-balanced SpMM: what a plan holds and what the kernels read.
//
// The reference starts one thread block per vector-row whatever its length (reference
// SSpMM/src/sspmm.cu:558-559) and offers SortedRowSwizzle (reference SSpMM/include/bm_test_utils.h:
// 210-225, consumed at end2end/sspmm_e2e/src/cuda/spmm_kernel.cu:48) as its only handle on uneven
// row lengths.  Here a vector-row is cut into panels of at most `budget` steps (a step = 32 stored
// vectors); every panel is one work item of the same size class, the panels of a cut row leave
// partial tiles in scratch memory, and the wave that finishes a row's last outstanding panel adds
// the partial tiles up in panel order, so the result does not depend on which wave that is.
#ifndef SSPMM_AMD_SCHEDULE_H
#define SSPMM_AMD_SCHEDULE_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace sspmm {

// header words
enum {
  kHdrItems = 0,       // work items: panels of cut rows first, then the rows that were left whole
  kHdrSplitRows = 1,   // vector-rows that were cut
  kHdrSlots = 2,       // panels of cut rows = partial tiles per (column tile, batch element)
  kHdrBudget = 3,      // steps per panel at most
  kHdrNvec = 4,        // stored vectors of the pattern
  kHdrMaxSteps = 5,    // steps of the longest vector-row
  kHdrTotalSteps = 6,  // steps of all vector-rows (an empty row counts one: its zeros are written)
  kHdrBundles = 7,     // bundles the rows that were left whole are filed in (0: no bundle table)
  kHdrWords = 8
};

// One work item, 8 ints: vectors [kbeg, kend) of vector-row `row`.  split_id < 0: the whole row, stored to C
// directly.  Otherwise panel `piece` of `pieces` of cut row `split_id`, whose partial tiles are slots
// first_slot .. first_slot + pieces - 1.
struct ScheduleItem {
  int32_t row, kbeg, kend, split_id;
  int32_t first_slot, pieces, piece, pad;
};

static constexpr int kScheduleMinBudget = 8;      // steps: shorter panels are all overhead
static constexpr int kScheduleTargetItems = 512;   // panels of cut rows wanted at most (before the memory cap)
// Steps a bundle of short rows aims at.  Measured on a 16384 x 16384 matrix of power-law rows (2048 vector-rows, 1930
// of them whole, 2.1 steps each on average): 5 and 6 steps 18.2-18.9 us, 8 steps 17.2, 10 17.5, 12 18.3, 16 17.2-20.5,
// against 18.0 with one wave per row.
static constexpr int kScheduleBundleSteps = 8;

// A partial tile: the accumulators of one wave (V rows x 64 columns, fp32) as they lie in its registers,
// 4 x (lanes that hold rows) x 16 bytes.
static constexpr size_t partial_tile_bytes(int V) { return V == 8 ? 4u * 32u * 16u : 4u * 64u * 16u; }

// Bundles: a wave that starts for one short row spends most of its life waiting for two dependent round trips to
// memory (column indices, then the rows of B they name) with nothing else in flight, and a pattern of skewed rows is
// mostly short rows.  The rows that stay whole are therefore filed, in row order, in bundles of about `bundle_steps`
// steps; one wave takes a bundle and runs its rows as one stream of steps, the loads of a row in flight while the
// row before it is contracted.  bundles[b] = first item of bundle b, bundles[header[kHdrBundles]] = item count.
struct ScheduleView {
  int32_t *header;           // kHdrWords ints
  int32_t *bundles;          // header[kHdrBundles] + 1 ints, or null (every row that stays whole is a unit of its own)
  ScheduleItem *items;
  int32_t *counters;         // panels that have delivered, per (batch element, column tile, cut row); zero between launches
  unsigned char *partials;   // partial tiles, per (batch element, column tile, slot)
};

// Measures the pattern and settles the budget: header[kHdrBudget] = `budget` when positive, else the largest of
// kScheduleMinBudget, ceil(total steps / kScheduleTargetItems) and twice the mean steps per row; doubled until the
// cut rows have at most `slot_cap` panels together (slot_cap = 0: no row is cut).  One workgroup.
hipError_t launch_schedule_measure(int m_vec, const int32_t *row_offsets, int budget, int64_t slot_cap, int32_t *header,
                                   hipStream_t stream);
// Writes the items for the budget the header holds (at most item_cap of them: the caller sizes from the header,
// or passes bounds that hold for every pattern), and clears `counters_to_clear` counters, or when that is
// negative the counters_per_cut_row counters of every cut row the header reports.  One workgroup.
// With view.bundles set, also files the rows that stay whole in bundles of about bundle_steps steps (at most 64
// rows each) and leaves their number in header[kHdrBundles].
hipError_t launch_schedule_fill(int m_vec, const int32_t *row_offsets, const ScheduleView &view, int64_t item_cap,
                                int64_t counters_to_clear, int64_t counters_per_cut_row, int bundle_steps,
                                hipStream_t stream);

// launch_schedule_measure (budget chosen from the pattern) and launch_schedule_fill (clearing the counters of the
// cut rows) as one launch; up to 4096 vector-rows by a kernel of its own that writes the same schedule sooner.
hipError_t launch_schedule_build(int m_vec, const int32_t *row_offsets, int64_t slot_cap, const ScheduleView &view,
                                 int64_t item_cap, int64_t counters_per_cut_row, hipStream_t stream);

}  // namespace sspmm
#endif
