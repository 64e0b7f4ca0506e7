// Stage timestamps and event counters for tuning builds (-DMAKO_TIMING): never part of the shipped library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mako_sampler.h"
#include "block_prims.h"

namespace mako {

// Optional stage timestamps of row 0 (thread 0), for tuning builds only.
#ifdef MAKO_TIMING
__device__ unsigned long long g_mako_stamp[32];
__shared__ uint32_t s_mako_row; // the row this workgroup serves (set by MAKO_ROW at kernel entry)
#define MAKO_ROW(r)                                                                                                  \
    do {                                                                                                             \
        if (threadIdx.x == 0)                                                                                        \
            s_mako_row = (r);                                                                                        \
    } while (0)
#ifdef MAKO_TIMING_NO_STAMPS // (workgroup timers only: the stamps themselves slow the chains they sit in)
#define MAKO_STAMP(i) ((void)0)
#else
#define MAKO_STAMP(i)                                                                                                \
    do {                                                                                                             \
        if (threadIdx.x == 0 && s_mako_row == 0)                                                                     \
            g_mako_stamp[i] = wall_clock64();                                                                        \
    } while (0)
#endif
__device__ unsigned long long g_mako_wg[2][4096];
struct WgTimer {
    __device__ WgTimer()
    {
        if (threadIdx.x == 0)
            g_mako_wg[0][(blockIdx.y * gridDim.x + blockIdx.x) & 4095] = wall_clock64();
    }
    __device__ ~WgTimer()
    {
        if (threadIdx.x == 0)
            g_mako_wg[1][(blockIdx.y * gridDim.x + blockIdx.x) & 4095] = wall_clock64();
    }
};
#define MAKO_WG_TIMER WgTimer wg_timer_
__device__ uint32_t g_mako_tag[4096]; // what each workgroup worked on, as its kernel describes it
#define MAKO_WG_TAG(v)                                                                                               \
    do {                                                                                                             \
        if (threadIdx.x == 0)                                                                                        \
            g_mako_tag[(blockIdx.y * gridDim.x + blockIdx.x) & 4095] = (v);                                          \
    } while (0)
} // namespace mako
// (readers of the above for the tuning scripts; one translation unit at a time is built with MAKO_TIMING)
extern "C" int mako_sampler_debug_wg(unsigned long long* out8192)
{
    return hipMemcpyFromSymbol(out8192, HIP_SYMBOL(mako::g_mako_wg), 8192 * sizeof(unsigned long long)) == hipSuccess
               ? MAKO_OK : MAKO_ERR_HIP;
}
extern "C" int mako_sampler_debug_tags(uint32_t* out4096)
{
    return hipMemcpyFromSymbol(out4096, HIP_SYMBOL(mako::g_mako_tag), 4096 * sizeof(uint32_t)) == hipSuccess
               ? MAKO_OK : MAKO_ERR_HIP;
}
extern "C" int mako_sampler_debug_stamps(unsigned long long* out32)
{
    return hipMemcpyFromSymbol(out32, HIP_SYMBOL(mako::g_mako_stamp), 32 * sizeof(unsigned long long)) == hipSuccess
               ? MAKO_OK : MAKO_ERR_HIP;
}
namespace mako {
#define MAKO_TIC(k)                                                                                                  \
    __builtin_amdgcn_s_waitcnt(0);                                                                                   \
    const unsigned long long tic_##k = wall_clock64()
#define MAKO_TOC(k, i)                                                                                               \
    do {                                                                                                             \
        __builtin_amdgcn_s_waitcnt(0);                                                                               \
        if (lane_id() == 0 && s_mako_row == 0)                                                                       \
            g_mako_stamp[i] += wall_clock64() - tic_##k;                                                             \
    } while (0)
#ifdef MAKO_TIMING_COUNTS // event counters: each costs a global round trip, so never together with timestamps
#define MAKO_COUNT(i, v)                                                                                             \
    do {                                                                                                             \
        if (lane_id() == 0 && s_mako_row == 0)                                                                       \
            g_mako_stamp[i] += (v);                                                                                  \
    } while (0)
#else
#define MAKO_COUNT(i, v) ((void)0)
#endif
#else
#define MAKO_STAMP(i) ((void)0)
#define MAKO_ROW(r) ((void)0)
#define MAKO_COUNT(i, v) ((void)0)
#define MAKO_WG_TIMER ((void)0)
#define MAKO_WG_TAG(v) ((void)0)
#define MAKO_TIC(k) ((void)0)
#define MAKO_TOC(k, i) ((void)0)
#endif

} // namespace mako
