// Launchers of the sampler's kernels.  Every kernel family is compiled as a translation unit of its own (k_*.hip):
// the compiler's register allocation for a kernel otherwise depends on which other kernels share its inlined device
// functions (sort_kernel lost 2.4 us per batch to spills when kernels with the whole-row path were compiled beside
// it).  Each init function raises the dynamic LDS limit of its family's kernels.
// Every kernel takes the context's record (`sc`, the host copy) by value: its first loads then need no trip to
// memory for the record itself, and no launch depends on a copy of it in device memory.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mako_sampler.h"

namespace mako {
struct Scratch;

hipError_t init_scan_kernels();
hipError_t init_second_kernels();
hipError_t init_rows_kernels();
hipError_t init_sort_kernels();
hipError_t init_tail_kernels();

// scan_kernel<vec, kh, above>, grid = (slices, rows), `lds` bytes of dynamic LDS
void launch_scan(bool vec, int kh, bool above, dim3 grid, size_t lds, hipStream_t st, const mako_sample_desc& d,
                 const Scratch& sc, uint32_t slice_len, uint32_t cus);
// second_kernel<vec, kh> on `wgs` workgroups: the second pass's pieces
void launch_second(bool vec, int kh, uint32_t wgs, hipStream_t st, const mako_sample_desc& d, const Scratch& sc,
                   uint32_t slices);
// rows_kernel, one workgroup per row, for a batch without top_k == 0 rows; `any_general`: some row may be without a
// top-p (the whole-row path then has to keep the order of top-k alone)
void launch_rows(bool any_general, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices);
// sort_kernel: `list_cap` workgroups for its work list (room for the longest list the batch can produce; workgroups
// beyond the list leave at once, but each of them still has to be dispatched).  tail_kernel takes one workgroup per
// possible top_k == 0 row (`tail_cap`), then one per row for the rows that need no second pass.
void launch_sort(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t list_cap);
void launch_tail(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t tail_cap);
} // namespace mako
