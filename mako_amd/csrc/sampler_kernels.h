// MI355X (gfx950) token sampler kernels: every family in a header of its own, included here in dependency order.
//
// Pipeline per batch (rows are independent, src/gen/session.cpp:416):
//   scan_kernel       one workgroup per (row, slice): the single coalesced pass over the fp32 logits.  The token
//                     mask and the history penalties are applied in registers; the slice's maximum and its largest
//                     logits (a superset of what top-k can need) go to scratch.
//   finish_kernel     the second, cache-resident pass over top_k == 0 rows: the row's plan from scan_kernel's coarse
//                     counts, exact sums of q = expf((w - m) / T), and the weights the plan keeps handed to the
//                     shares of the 32 workers per row that will sort them.
//   sort_kernel       the wide nuclei: each worker sorts its share; narrow nuclei from the candidate lists.
//   tail_kernel       the wide nuclei cut and drawn from; in the same launch, one workgroup per row, whatever the
//                     earlier kernels left: forced and greedy rows, top-k rows, rows on the whole-row path (exact
//                     for every parameter combination), second looks at cuts too close to call.
//   plan_kernel       instead of the last three, for a batch without top_k == 0 rows: forced, greedy and top-k rows
//                     from the candidate lists, ordered by (q desc, idx asc) and drawn from with the reference's
//                     exact fp32 rounding order.
#pragma once

#include "tuning_stamps.h"
#include "sampler_common.h"
#include "slice_load.h"
#include "work_split.h"
#include "scan_kernel.h"
#include "workgroup_state.h"
#include "row_output.h"
#include "generic_replay.h"
#include "sorted_tail.h"
#include "whole_row.h"
#include "worker_sort.h"
#include "row_records.h"
#include "topk_candidates.h"
#include "second_pass.h"
#include "plan_kernel.h"
#include "sort_kernels.h"
#include "late_rows.h"
#include "tail_kernel.h"
#include "index_rows.h"
