// LDS records shared by the finishing kernels: the workgroup's scratch, views into the dynamic LDS block, and
// the kernel arguments staged in LDS.
#pragma once

#include "sampler_common.h"

namespace mako {

struct alignas(16) FinishShared {
    BlockScratch bs;
    uint64_t tab[32];
    uint32_t hist[256];
    uint32_t run[256];
    uint32_t flag;
    uint32_t ticket;
    uint32_t aux;
    uint32_t soff[kMaxSlices + 1]; // first candidate of each slice in the row's flattened candidate list
};

// Views into the first 64 KB of the dynamic LDS block; `cnt` (first pass) overlaps the two others (second pass).
struct FinishLds {
    FinishShared* sm;
    uint32_t* cnt;              // [kSliceMax]
    unsigned long long* sortk;  // [kSortMax]
    uint32_t* wcount;           // [kWaves * 256]
};

// The views as a function that is really called (not inlined) received them by reference, said to the compiler to
// point into LDS: through pointers that could point anywhere every access becomes a "flat" instruction, which takes
// longer than an LDS one and counts as traffic to device memory as well, so that waiting for one kind means waiting
// for both.  Only in sources compiled with calls (MAKO_REAL_CALLS): where everything is inlined the compiler sees
// where the views come from, and the assumption's own loads would only keep the record in memory.
__device__ __forceinline__ void assume_lds(const FinishLds& L)
{
#if defined(MAKO_REAL_CALLS) && defined(__HIP_DEVICE_COMPILE__)
    __builtin_assume(__builtin_amdgcn_is_shared(L.sm));
    __builtin_assume(__builtin_amdgcn_is_shared(L.cnt));
    __builtin_assume(__builtin_amdgcn_is_shared(L.sortk));
    __builtin_assume(__builtin_amdgcn_is_shared(L.wcount));
#else
    (void)L;
#endif
}

__device__ __forceinline__ FinishLds finish_lds_views(FinishShared& sm, unsigned long long* dyn)
{
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(dyn);
    L.sortk = dyn;
    L.wcount = reinterpret_cast<uint32_t*>(dyn + kSortMax);
    return L;
}

// Kernel arguments that are handed on by reference to out-of-line device functions would be spilled to scratch
// memory (a microsecond per access); the two finishing kernels keep their copies in LDS instead.
struct alignas(16) ArgsLds {
    mako_sample_desc d;
    Scratch sc;
    mako_sampling_params P; // the row's parameters
};

// The copy in two halves, so that a kernel can have the loads in flight while it waits for something else: every
// thread asks for its word of each record (from clamped positions: no branch, the loads go out back to back), and
// writes them to LDS later.  The caller's next barrier publishes the copy.
struct ArgWords {
    uint32_t d, sc, p;
};
static_assert(sizeof(mako_sample_desc) % 4 == 0 && sizeof(Scratch) % 4 == 0 && sizeof(mako_sampling_params) % 4 == 0 &&
                  sizeof(mako_sample_desc) / 4 <= kThreads && sizeof(Scratch) / 4 <= kThreads,
              "a word per thread");
__device__ __forceinline__ void fetch_arg_words(const mako_sample_desc& d_arg, const Scratch& sc_arg, ArgWords& r)
{
    const uint32_t tid = threadIdx.x;
    r.d = reinterpret_cast<const uint32_t*>(&d_arg)[min(tid, (uint32_t)(sizeof(mako_sample_desc) / 4 - 1))];
    r.sc = reinterpret_cast<const uint32_t*>(&sc_arg)[min(tid, (uint32_t)(sizeof(Scratch) / 4 - 1))];
}
__device__ __forceinline__ void fetch_param_words(const mako_sample_desc& d_arg, uint32_t row, ArgWords& r)
{
    r.p = reinterpret_cast<const uint32_t*>(d_arg.params + row)[min(threadIdx.x, (uint32_t)(sizeof(mako_sampling_params) / 4 - 1))];
}
__device__ __forceinline__ void place_arg_words(const ArgWords& r, ArgsLds& a)
{
    const uint32_t tid = threadIdx.x;
    if (tid < sizeof(mako_sample_desc) / 4)
        reinterpret_cast<uint32_t*>(&a.d)[tid] = r.d;
    if (tid < sizeof(Scratch) / 4)
        reinterpret_cast<uint32_t*>(&a.sc)[tid] = r.sc;
    if (tid < sizeof(mako_sampling_params) / 4)
        reinterpret_cast<uint32_t*>(&a.P)[tid] = r.p;
}

// The same in two steps for a kernel that learns its row late: the arguments first (no barrier), the row's parameters
// (already in registers, the same in every lane) afterwards; the caller's next barrier publishes both.
__device__ __forceinline__ void stage_args_only(const mako_sample_desc& d_arg, const Scratch& sc_arg, ArgsLds& a)
{
    const uint32_t* src_d = reinterpret_cast<const uint32_t*>(&d_arg);
    const uint32_t* src_s = reinterpret_cast<const uint32_t*>(&sc_arg);
    uint32_t* dst_d = reinterpret_cast<uint32_t*>(&a.d);
    uint32_t* dst_s = reinterpret_cast<uint32_t*>(&a.sc);
    for (uint32_t i = threadIdx.x; i < sizeof(mako_sample_desc) / 4; i += kThreads)
        dst_d[i] = src_d[i];
    for (uint32_t i = threadIdx.x; i < sizeof(Scratch) / 4; i += kThreads)
        dst_s[i] = src_s[i];
}
__device__ __forceinline__ void stage_params(const mako_sampling_params& P, ArgsLds& a)
{
    if (threadIdx.x == 0)
        a.P = P;
}

__device__ __forceinline__ void stage_args(const mako_sample_desc& d_arg, const Scratch& sc_arg, uint32_t row, ArgsLds& a)
{
    ArgWords r;
    fetch_arg_words(d_arg, sc_arg, r);
    fetch_param_words(d_arg, row, r);
    place_arg_words(r, a);
    __syncthreads();
}

} // namespace mako
