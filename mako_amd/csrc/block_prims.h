// Workgroup-wide primitives for 1024-thread workgroups of 64-wide wavefronts.
// Every function must be reached by all threads of the workgroup.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "seqfp.h"

// Wavefront reductions and scans of the device library (DPP row shifts and broadcasts: a dozen instructions where
// a shuffle-based butterfly pays six trips through the LDS crossbar).
extern "C" __device__ uint32_t __ockl_wfred_add_u32(uint32_t);
extern "C" __device__ uint32_t __ockl_wfred_min_u32(uint32_t);
extern "C" __device__ uint32_t __ockl_wfred_max_u32(uint32_t);
extern "C" __device__ unsigned long long __ockl_wfred_max_u64(unsigned long long);
extern "C" __device__ double __ockl_wfred_add_f64(double);
extern "C" __device__ uint32_t __ockl_wfscan_add_u32(uint32_t, bool inclusive);
extern "C" __device__ double __ockl_wfscan_add_f64(double, bool inclusive);
extern "C" __device__ float __ockl_wfscan_add_f32(float, bool inclusive);

namespace mako {

constexpr int kThreads = 1024;
constexpr int kWave = 64;
constexpr int kWaves = kThreads / kWave;

__device__ __forceinline__ int lane_id()
{
    return threadIdx.x & (kWave - 1);
}
// (read through a scalar register: the compiler then knows the value is the same in all 64 lanes, and branches
// and loops on it become scalar control flow)
__device__ __forceinline__ int wave_id()
{
    return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
}

// Pointers known to point to device memory, typed so.  A pointer that was itself loaded from memory (the finishing
// kernels keep copies of their argument records in LDS) could point anywhere for all the compiler knows, and accesses
// through it become "flat" instructions: those count as LDS traffic as well, so a barrier that orders LDS only
// (lds_barrier()) would wait for every load from device memory still in flight, and the counters of the two kinds
// of traffic can no longer be waited for one by one.
template <typename T>
using global_ptr = __attribute__((address_space(1))) T*;
template <typename T>
__device__ __forceinline__ global_ptr<T> as_global(T* p)
{
    return (global_ptr<T>)p;
}
typedef uint32_t u32x4 __attribute__((ext_vector_type(4))); // (plain vector types: they load from any address space)
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding
// global load, which would serialise LDS set-up work behind the logits stream it is meant to overlap.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Scratch shared by the primitives; one instance per kernel.
struct BlockScratch {
    unsigned long long u64[kWaves];
    double f64[kWaves];
    seqfp::Step step[kWaves];
    unsigned long long bcast;
};

__device__ __forceinline__ uint32_t block_sum_u32(uint32_t v, BlockScratch& s)
{
    v = __ockl_wfred_add_u32(v);
    if (lane_id() == 0)
        s.u64[wave_id()] = v;
    __syncthreads();
    uint32_t t = 0;
    for (int w = 0; w < kWaves; ++w)
        t += (uint32_t)s.u64[w];
    __syncthreads();
    return t;
}

__device__ __forceinline__ uint32_t block_min_u32(uint32_t v, BlockScratch& s)
{
    v = __ockl_wfred_min_u32(v);
    if (lane_id() == 0)
        s.u64[wave_id()] = v;
    __syncthreads();
    uint32_t t = 0xffffffffu;
    for (int w = 0; w < kWaves; ++w)
        t = min(t, (uint32_t)s.u64[w]);
    __syncthreads();
    return t;
}

// Exclusive prefix sum in thread order; `total` receives the workgroup sum.
__device__ __forceinline__ uint32_t block_excl_scan_u32(uint32_t v, uint32_t& total, BlockScratch& s)
{
    const uint32_t incl = __ockl_wfscan_add_u32(v, true);
    if (lane_id() == kWave - 1)
        s.u64[wave_id()] = incl;
    __syncthreads();
    uint32_t pre = 0, tot = 0;
    for (int w = 0; w < kWaves; ++w) {
        const uint32_t x = (uint32_t)s.u64[w];
        if (w < wave_id())
            pre += x;
        tot += x;
    }
    __syncthreads();
    total = tot;
    return pre + incl - v;
}

// Sum of doubles in a fixed order (the wavefront reduction's, then waves in order):
// the same inputs always give the same bits.
__device__ __forceinline__ double block_sum_f64(double v, BlockScratch& s)
{
    v = __ockl_wfred_add_f64(v);
    if (lane_id() == 0)
        s.f64[wave_id()] = v;
    __syncthreads();
    double t = 0;
    for (int w = 0; w < kWaves; ++w)
        t += s.f64[w];
    __syncthreads();
    return t;
}

// Inclusive prefix sum of doubles in thread order; fixed association.
__device__ __forceinline__ double block_incl_scan_f64(double v, double& total, BlockScratch& s)
{
    v = __ockl_wfscan_add_f64(v, true);
    if (lane_id() == kWave - 1)
        s.f64[wave_id()] = v;
    __syncthreads();
    double pre = 0, tot = 0;
    for (int w = 0; w < kWaves; ++w) {
        const double x = s.f64[w];
        if (w < wave_id())
            pre += x;
        tot += x;
    }
    __syncthreads();
    total = tot;
    return pre + v;
}

// Exclusive scan of two-state maps under composition (earlier thread first);
// `total` receives the composition of all of them.
__device__ __forceinline__ seqfp::Step block_excl_scan_step(seqfp::Step f, seqfp::Step& total, BlockScratch& s)
{
    seqfp::Step incl = f;
    for (int o = 1; o < kWave; o <<= 1) {
        seqfp::Step t;
        t.d0 = __shfl_up(incl.d0, o);
        t.d1 = __shfl_up(incl.d1, o);
        if (lane_id() >= o)
            incl = seqfp::compose(t, incl);
    }
    if (lane_id() == kWave - 1)
        s.step[wave_id()] = incl;
    // exclusive within the wave: the inclusive value of the previous lane
    seqfp::Step excl;
    excl.d0 = __shfl_up(incl.d0, 1);
    excl.d1 = __shfl_up(incl.d1, 1);
    if (lane_id() == 0)
        excl = seqfp::identity();
    __syncthreads();
    seqfp::Step pre = seqfp::identity(), tot = seqfp::identity();
    for (int w = 0; w < kWaves; ++w) {
        const seqfp::Step x = s.step[w];
        if (w < wave_id())
            pre = seqfp::compose(pre, x);
        tot = seqfp::compose(tot, x);
    }
    __syncthreads();
    total = tot;
    return seqfp::compose(pre, excl);
}

} // namespace mako
