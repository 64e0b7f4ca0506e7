// Instrumentation sites of the kernels.  The shipped library compiles every one of them to nothing.  A tuning build
// names a header of its own on the command line (-DMAKO_TIMING_IMPL='"path"') that defines the same macros.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mako_sampler.h"
#include "block_prims.h"

#ifdef MAKO_TIMING_IMPL
#include MAKO_TIMING_IMPL
#else
#define MAKO_STAMP(i) ((void)0)
#define MAKO_ROW(r) ((void)0)
#define MAKO_COUNT(i, v) ((void)0)
#define MAKO_WG_TIMER ((void)0)
#define MAKO_WG_TAG(v) ((void)0)
#define MAKO_TIC(k) ((void)0)
#define MAKO_TOC(k, i) ((void)0)
#endif
