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
// second_kernel<vec, kh> on `wgs` workgroups: the second pass's pieces, then one workgroup per row
void launch_second(bool vec, int kh, uint32_t wgs, hipStream_t st, const mako_sample_desc& d, const Scratch& sc,
                   uint32_t slices);
// rows_kernel, one workgroup per row, for a batch without top_k == 0 rows: <false> when sort_kernel follows (it has
// the whole-row path), <true> when rows_kernel is the last kernel of the batch
void launch_rows(bool inline_general, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices);
// sort_kernel: kWorkers workgroups per top_k == 0 row (`nucleus_rows` of them at most), then one per row that can
// be on the whole-row list (`list_rows`).  Workgroups beyond the lists leave at once, but each of them still has to
// be dispatched.  tail_kernel takes one workgroup per possible wide row.
void launch_sort(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t nucleus_rows,
                 uint32_t list_rows);
void launch_tail(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t grid_rows);
} // namespace mako
