// Launchers of the sampler's kernels.  Every kernel family is compiled as a translation unit of its own (k_*.hip):
// the compiler's register allocation for a kernel otherwise depends on which other kernels share its inlined device
// functions (sort_kernel lost 2.4 us per batch to spills when plan_kernel variants with the whole-row path were
// compiled beside it).  Each init function raises the dynamic LDS limit of its family's kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mako_sampler.h"

namespace mako {
struct Scratch;

hipError_t init_scan_kernels();
hipError_t init_finish_kernels();
hipError_t init_plan_alone();
hipError_t init_sort_kernels();
hipError_t init_tail_kernels();

// scan_kernel<vec, kh, above>, grid = (slices, rows), `lds` bytes of dynamic LDS
// (`sc`: the HOST copy of the context's record; the kernels take it by value, so that their first loads need no
// trip to memory for the record itself)
void launch_scan(bool vec, int kh, bool above, dim3 grid, size_t lds, hipStream_t st, const mako_sample_desc& d,
                 const Scratch& sc, uint32_t slice_len, uint32_t cus);
// finish_kernel<vec, kh> on `wgs` workgroups
// (unsorted: the instances for batches of many top_k == 0 rows, whose plans leave shares unsorted; the kernels
// of one batch must agree on it)
void launch_finish(bool vec, int kh, bool unsorted, uint32_t wgs, hipStream_t st, const mako_sample_desc& d, const Scratch& sc,
                   uint32_t slices); // (host copy, by value)
void launch_plan_alone(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices); // (host copy, by value)
// sort_kernel's workgroup i serves entry i of the work list: `grid_rows` * kWorkers workgroups must cover the
// longest list the batch can produce (kWorkers entries per top_k == 0 row); tail_kernel takes one workgroup per possible wide row.  Workgroups beyond the lists leave at once, but each
// of them still has to be dispatched.
void launch_sort(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t grid_rows, bool unsorted); // (host copy)
// (tail_kernel: `tail_cap` workgroups for the possible wide rows, then one per row for what is left of every row)
void launch_tail(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t tail_cap, bool unsorted); // (host copy, by value)
// the three kernels of the rows whose candidates stay in token order (index_rows.h): the weights (before tail_kernel's
// launch, which then leaves such rows alone), the group records, the total and the draw (behind it)
hipError_t init_index_kernels();
void launch_index_weights(bool vec, int kh, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices);
void launch_index_finish(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, bool in_order_rows);
} // namespace mako
