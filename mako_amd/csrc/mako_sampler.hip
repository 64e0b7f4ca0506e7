// C ABI of include/mako_sampler.h over the kernels in sampler_kernels.h (launched through launch.h: every kernel
// family is a translation unit of its own).
#include <hip/hip_runtime.h>

#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <new>
#include <string>

#include "../../include/mako_sampler.h"
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
__global__ void debug_expf_kernel(const float* x, float* y, uint32_t n)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        y[i] = expf_glibc(x[i], k_exp2_tab);
}

__global__ void debug_div_kernel(const float* a, const float* b, float* y, uint32_t n)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        y[i] = a[i] / b[i];
}
} // namespace mako

// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------

struct mako_sampler_ctx {
    int device = 0;
    uint32_t max_rows = 0, max_vocab = 0, max_hist = 0;
    mako::Scratch sc{};
    // staging for the host-pointer call
    float* st_logits = nullptr;
    mako_sampling_params* st_params = nullptr;
    float* st_u = nullptr;
    float* st_u2 = nullptr;
    uint32_t* st_mask = nullptr;
    int32_t* st_hist = nullptr;
    uint32_t* st_hcnt = nullptr;
    uint32_t* st_hlen = nullptr;
    int32_t* st_draft = nullptr;
    int32_t* st_tokens = nullptr;
    uint8_t* st_acc = nullptr;
    std::string err = "";
    bool profile = false, profiled = false;
    bool dirty = false; // a launch of the last batch failed: the scratch memory is cleared again before the next one
    uint32_t cus = 256; // compute units: workgroups of the finishing kernels that run at a time
    hipEvent_t ev[MAKO_SAMPLER_KERNELS + 1] = {};
};

namespace {

int fail(mako_sampler_ctx* ctx, int code, const std::string& what)
{
    if (ctx)
        ctx->err = what;
    return code;
}

#define MAKO_HIP(ctx, call)                                                                                        \
    do {                                                                                                           \
        hipError_t e_ = (call);                                                                                    \
        if (e_ != hipSuccess)                                                                                      \
            return fail(ctx, MAKO_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(e_));                     \
    } while (0)

template <typename T>
hipError_t dev_alloc(T** p, size_t count)
{
    return hipMalloc(reinterpret_cast<void**>(p), count * sizeof(T));
}

uint32_t slice_len_for(uint32_t n_vocab, uint32_t slices)
{
    uint32_t len = (n_vocab + slices - 1) / slices;
    return (len + 3u) & ~3u;
}


int run_batch(mako_sampler_ctx* ctx, const mako_sample_desc& d, const mako_sampling_params* params_host, void* stream,
              const mako::Scratch& sc, uint32_t max_rows, uint32_t max_vocab, bool* dirty);

#define MAKO_STR2(x) #x
#define MAKO_STR(x) MAKO_STR2(x)

// The kernels' scratch memory for batches of up to max_rows rows of up to max_vocab logits, every array taken from
// `take` (256-byte aligned blocks).  (The kernels take the record by value.)
template <typename Take>
hipError_t layout_scratch(mako::Scratch& sc, uint32_t max_rows, uint32_t max_vocab, Take take)
{
#define MAKO_TAKE(ptr, count)                                                                                      \
    do {                                                                                                           \
        hipError_t e_ = take(reinterpret_cast<void**>(&(ptr)), (size_t)(count) * sizeof(*(ptr)));                  \
        if (e_ != hipSuccess)                                                                                      \
            return e_;                                                                                             \
    } while (0)
    // (a row's arrays: the vocabulary, room for the slack of the workers' shares in the staging arrays, rounded up)
    sc.vpad = ((uint64_t)max_vocab + max_vocab / 64u + mako::kWorkers * mako::kStageSlack + 1023u) & ~1023ull;
    const size_t rv = (size_t)max_rows * sc.vpad;
    sc.slices_cap = mako_sampler_slices(max_vocab);
    MAKO_TAKE(sc.stats, (size_t)max_rows * mako::kMaxSlices);
    MAKO_TAKE(sc.cand_w, (size_t)max_rows * sc.slices_cap * mako::kCap);
    MAKO_TAKE(sc.cand_i, (size_t)max_rows * sc.slices_cap * mako::kCap);
    MAKO_TAKE(sc.part_sum, (size_t)max_rows * mako::kMaxSlices);
    MAKO_TAKE(sc.plan, (size_t)max_rows);
    MAKO_TAKE(sc.wbuf, rv);
    MAKO_TAKE(sc.cnt, rv);
    MAKO_TAKE(sc.key[0], rv);
    MAKO_TAKE(sc.key[1], rv);
    MAKO_TAKE(sc.idx[0], rv);
    MAKO_TAKE(sc.idx[1], rv);
    sc.g_cap = (uint32_t)(sc.vpad / mako::kGroup) + mako::kWorkers;
    const size_t rg = (size_t)max_rows * sc.g_cap;
    MAKO_TAKE(sc.gt.sum, rg);
    MAKO_TAKE(sc.gt.d0, rg);
    MAKO_TAKE(sc.gt.d1, rg);
    MAKO_TAKE(sc.gt.cmax, rg);
    MAKO_TAKE(sc.gt.start, rg);
    MAKO_TAKE(sc.gt.pack, rg);
    MAKO_TAKE(sc.gt.quarters, rg * 4);
    MAKO_TAKE(sc.gt.walk, rg);
    MAKO_TAKE(sc.log_hist, (size_t)max_rows * sc.slices_cap * mako::kLogBins);
    MAKO_TAKE(sc.work_n, 8);
    MAKO_TAKE(sc.work_sort, (size_t)max_rows * mako::kSortItemsPerRow);
    MAKO_TAKE(sc.work_tail, (size_t)max_rows);
#undef MAKO_TAKE
    return hipSuccess;
}

// What the kernels expect to find zero before a context's first batch (they leave it zero after every batch).
hipError_t zero_scratch(const mako::Scratch& sc, uint32_t max_rows)
{
    hipError_t e = hipMemset(sc.plan, 0, (size_t)max_rows * sizeof(mako::BigPlan));
    if (e == hipSuccess)
        e = hipMemset(sc.cnt, 0, (size_t)max_rows * sc.vpad * sizeof(uint32_t));
    if (e == hipSuccess)
        e = hipMemset(sc.work_n, 0, 8 * sizeof(uint32_t));
    return e;
}

// ---- scratch memory that is part of the library's image: mako_sampler_sample_batch_static() ----
// One array per GPU (the loader places a copy on every device the library runs on, for the life of the process),
// laid out once per device for MAKO_STATIC_MAX_ROWS rows of MAKO_STATIC_MAX_VOCAB logits.  `scratch` itself is only
// a host-side handle: everything below works on the device address hipGetSymbolAddress() returns for the current
// device.
constexpr size_t kStaticBytes = (size_t)MAKO_STATIC_SCRATCH_MIB << 20;
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

constexpr int kStaticDevices = 64;
constexpr uint64_t kGridYMax = 65535; // workgroups in a grid's y dimension
struct StaticScratch {
    bool ready = false;
    hipError_t status = hipSuccess; // of the set-up, kept: a device whose set-up failed refuses every static call
    bool dirty = false;             // as mako_sampler_ctx::dirty, for the device's array (under g_static_mutex)
    mako::Scratch sc{};
};
StaticScratch g_static[kStaticDevices];
std::mutex g_static_mutex;

// Once per device, with that device current (mako_sampler_create() calls it).
hipError_t setup_static_scratch(int device)
{
    if (device < 0 || device >= kStaticDevices)
        return hipSuccess; // (such a device's contexts refuse the static entry point)
    std::lock_guard<std::mutex> lock(g_static_mutex);
    StaticScratch& g = g_static[device];
    if (g.ready)
        return g.status;
    unsigned char* base = nullptr;
    hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&base), HIP_SYMBOL(scratch));
    if (e == hipSuccess && (!base || (reinterpret_cast<uintptr_t>(base) & 255u)))
        e = hipErrorInvalidSymbol;
    size_t used = 0;
    if (e == hipSuccess)
        e = layout_scratch(g.sc, MAKO_STATIC_MAX_ROWS, MAKO_STATIC_MAX_VOCAB, [&](void** p, size_t bytes) {
            if (bytes > kStaticBytes - used)
                return hipErrorOutOfMemory;
            *p = base + used;
            used += (bytes + 255u) & ~(size_t)255u;
            return hipSuccess;
        });
    if (e == hipSuccess)
        e = zero_scratch(g.sc, MAKO_STATIC_MAX_ROWS);
    if (e == hipSuccess)
        e = hipDeviceSynchronize();
    g.status = e;
    g.ready = true;
    return e;
}

} // namespace

extern "C" {

uint32_t mako_sampler_slices(uint32_t n_vocab)
{
    const uint32_t s = (n_vocab + mako::kSliceMax - 1) / mako::kSliceMax;
    return s ? s : 1;
}

int mako_sampler_create(mako_sampler_ctx** out, int device, uint32_t max_rows, uint32_t max_vocab, uint32_t max_hist)
{
    if (!out || max_rows == 0 || max_vocab == 0)
        return MAKO_ERR_INVALID_ARG;
    // (kMaxSlices slices of kSliceMax logits)
    if (mako_sampler_slices(max_vocab) > mako::kMaxSlices)
        return MAKO_ERR_INVALID_ARG;
    // (the largest grid, tail_kernel's, has two workgroups per row in its y dimension)
    if (2ull * max_rows > kGridYMax)
        return MAKO_ERR_INVALID_ARG;
    mako_sampler_ctx* ctx = new (std::nothrow) mako_sampler_ctx;
    if (!ctx)
        return MAKO_ERR_NO_MEMORY;
    *out = ctx;
    ctx->device = device;
    ctx->max_rows = max_rows;
    ctx->max_vocab = max_vocab;
    ctx->max_hist = max_hist;
    MAKO_HIP(ctx, hipSetDevice(device));
    {
        int n = 0;
        MAKO_HIP(ctx, hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device));
        if (n > 0)
            ctx->cus = (uint32_t)n;
    }
    MAKO_HIP(ctx, layout_scratch(ctx->sc, max_rows, max_vocab, [](void** p, size_t bytes) { return hipMalloc(p, bytes); }));
    MAKO_HIP(ctx, zero_scratch(ctx->sc, max_rows));
    // (a device on which the library's own array cannot be set up only refuses mako_sampler_sample_batch_static,
    // which checks the kept status itself)
    (void)setup_static_scratch(device);
    (void)hipGetLastError();
    MAKO_HIP(ctx, hipDeviceSynchronize());
    // the kernels overlay 64 to 128 KB of dynamic LDS (kDynLds, kTailLds, kSortLds) on a few KB of static LDS
    MAKO_HIP(ctx, mako::init_scan_kernels());
    MAKO_HIP(ctx, mako::init_finish_kernels());
    MAKO_HIP(ctx, mako::init_plan_alone());
    MAKO_HIP(ctx, mako::init_sort_kernels());
    MAKO_HIP(ctx, mako::init_tail_kernels());
    MAKO_HIP(ctx, mako::init_index_kernels());
    return MAKO_OK;
}

void mako_sampler_destroy(mako_sampler_ctx* ctx)
{
    if (!ctx)
        return;
    (void)hipSetDevice(ctx->device);
    mako::Scratch& sc = ctx->sc;
    void* ptrs[] = {sc.log_hist, sc.work_n, sc.work_sort, sc.work_tail, sc.gt.sum, sc.gt.d0, sc.gt.d1, sc.gt.cmax, sc.gt.start, sc.gt.pack, sc.gt.quarters, sc.gt.walk,
                    sc.cand_w, sc.cand_i, sc.part_sum, sc.plan,
                    sc.stats,      sc.wbuf,      sc.cnt,        sc.key[0],     sc.key[1],     sc.idx[0],
                    sc.idx[1],     ctx->st_logits, ctx->st_params, ctx->st_u,   ctx->st_u2,    ctx->st_mask,
                    ctx->st_hist,  ctx->st_hcnt, ctx->st_hlen,  ctx->st_draft, ctx->st_tokens, ctx->st_acc};
    for (void* p : ptrs)
        if (p)
            (void)hipFree(p);
    for (hipEvent_t e : ctx->ev)
        if (e)
            (void)hipEventDestroy(e);
    delete ctx;
}

int mako_sampler_set_profile(mako_sampler_ctx* ctx, int enabled)
{
    if (!ctx)
        return MAKO_ERR_INVALID_ARG;
    MAKO_HIP(ctx, hipSetDevice(ctx->device));
    if (enabled)
        for (hipEvent_t& e : ctx->ev)
            if (!e)
                MAKO_HIP(ctx, hipEventCreate(&e));
    ctx->profile = enabled != 0;
    ctx->profiled = false;
    return MAKO_OK;
}

int mako_sampler_kernel_times(mako_sampler_ctx* ctx, float* out_ms)
{
    if (!ctx || !out_ms)
        return MAKO_ERR_INVALID_ARG;
    if (!ctx->profiled)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: no profiled batch to report");
    MAKO_HIP(ctx, hipEventSynchronize(ctx->ev[MAKO_SAMPLER_KERNELS]));
    for (int i = 0; i < MAKO_SAMPLER_KERNELS; ++i)
        MAKO_HIP(ctx, hipEventElapsedTime(&out_ms[i], ctx->ev[i], ctx->ev[i + 1]));
    return MAKO_OK;
}

const char* mako_sampler_last_error(const mako_sampler_ctx* ctx)
{
    return ctx ? ctx->err.c_str() : "null context";
}

int mako_sampler_sample_batch(mako_sampler_ctx* ctx, const mako_sample_desc* desc, void* stream)
{
    return mako_sampler_sample_batch_hinted(ctx, desc, nullptr, stream);
}

int mako_sampler_sample_batch_hinted(mako_sampler_ctx* ctx, const mako_sample_desc* desc,
                                     const mako_sampling_params* params_host, void* stream)
{
    if (!ctx || !desc)
        return MAKO_ERR_INVALID_ARG;
    MAKO_HIP(ctx, hipSetDevice(ctx->device));
    return run_batch(ctx, *desc, params_host, stream, ctx->sc, ctx->max_rows, ctx->max_vocab, &ctx->dirty);
}

int mako_sampler_sample_batch_static(mako_sampler_ctx* ctx, const mako_sample_desc* desc, void* stream)
{
    if (!ctx || !desc)
        return MAKO_ERR_INVALID_ARG;
    if (desc->n_rows > MAKO_STATIC_MAX_ROWS || desc->n_vocab > MAKO_STATIC_MAX_VOCAB)
        return fail(ctx, MAKO_ERR_INVALID_ARG,
                    "sampler: the library's own scratch memory holds batches of up to " MAKO_STR(MAKO_STATIC_MAX_ROWS)
                    " rows of up to " MAKO_STR(MAKO_STATIC_MAX_VOCAB) " logits");
    if (ctx->device < 0 || ctx->device >= kStaticDevices)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: no static scratch memory for this device ordinal");
    StaticScratch& g = g_static[ctx->device]; // (set up by mako_sampler_create(); only `dirty` is written afterwards)
    if (!g.ready || g.status != hipSuccess)
        return fail(ctx, MAKO_ERR_HIP, "sampler: the static scratch memory could not be set up on this device");
    MAKO_HIP(ctx, hipSetDevice(ctx->device));
    return run_batch(ctx, *desc, nullptr, stream, g.sc, MAKO_STATIC_MAX_ROWS, MAKO_STATIC_MAX_VOCAB, &g.dirty);
}

} // extern "C"

namespace {
// One batch through the kernels, on scratch memory laid out for max_rows x max_vocab.  Allocates nothing.
// (`dirty`: of the scratch memory the batch runs on.  The kernels rely on what the last kernels of a batch leave zero
// (BigPlan::flag, the token counts, the work lists' lengths); a batch that stopped at a failed launch may not have
// left it so, and the next batch on that memory clears it again first.)
int run_batch(mako_sampler_ctx* ctx, const mako_sample_desc& d, const mako_sampling_params* params_host, void* stream,
              const mako::Scratch& sc, uint32_t max_rows, uint32_t max_vocab, bool* dirty)
{
    if (d.n_vocab == 0)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: empty vocabulary"); // sampler.cpp:11-12
    if (d.n_rows == 0)
        return MAKO_OK;
    if (!d.logits || !d.params || !d.u || !d.out_tokens)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: logits, params, u and out_tokens are required");
    if (d.n_rows > max_rows || d.n_vocab > max_vocab)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: batch exceeds the context's max_rows/max_vocab");
    if (d.logits_stride < (int64_t)d.n_vocab)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: logits_stride < n_vocab");
    if (d.mask && d.mask_stride < (int64_t)((d.n_vocab + 31) / 32))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: mask_stride < ceil(n_vocab / 32)");
    if (d.hist_tokens && (!d.hist_len || d.hist_stride < 0))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: hist_tokens needs hist_len and a stride");
    if ((d.draft != nullptr) != (d.u2 != nullptr) || (d.draft != nullptr) != (d.out_accepted != nullptr))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: draft, u2 and out_accepted go together");
    if ((d.out_cand_idx != nullptr) != (d.out_cand_q != nullptr))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: out_cand_idx and out_cand_q go together");
    if ((d.force_token || d.close_token) && !d.out_forced)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: force_token / close_token need out_forced");
    if (d.out_above && !d.close_token)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: out_above needs close_token");
    if (d.append_history && (!d.hist_tokens || !d.hist_len || d.hist_counts || d.draft))
        return fail(ctx, MAKO_ERR_INVALID_ARG,
                    "sampler: append_history needs hist_tokens and hist_len, and neither hist_counts nor draft");

    hipStream_t st = static_cast<hipStream_t>(stream);
    if (*dirty) {
        // an earlier batch on this scratch memory stopped at a failed launch: clear what the kernels expect to find
        // zero, which cannot be recorded into a stream capture
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        MAKO_HIP(ctx, hipStreamIsCapturing(st, &capturing));
        if (capturing != hipStreamCaptureStatusNone)
            return fail(ctx, MAKO_ERR_HIP,
                        "sampler: an earlier batch failed at a launch; the next call must come outside stream capture");
        MAKO_HIP(ctx, hipDeviceSynchronize());
        MAKO_HIP(ctx, zero_scratch(sc, max_rows));
        MAKO_HIP(ctx, hipDeviceSynchronize());
        *dirty = false;
    }
    const uint32_t slices = mako_sampler_slices(d.n_vocab);
    // (the largest grid, tail_kernel's, has two workgroups per row in its y dimension)
    if (2ull * d.n_rows > kGridYMax)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: more rows than one launch can index (32767)");
    const uint32_t slice_len = slice_len_for(d.n_vocab, slices);
    const bool vec = d.n_vocab % 4 == 0 && d.logits_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(d.logits) & 15u) == 0;
    const size_t lds = d.hist_tokens ? (size_t)slice_len * sizeof(uint32_t) : 0;
    // (scan_kernel: with histories a row's slices share an XCD)
    const dim3 grid = d.hist_tokens ? dim3((d.n_rows + 7u) & ~7u, slices) : dim3(slices, d.n_rows);
    // The second pass's cut is decided on the device (SecondPassCut): at most one round of workgroups while the rows'
    // pieces fit one, else one workgroup per row or a few; workgroups beyond those with work leave after a look at
    // the cut.
    // histories of up to 2 (8) entries per thread stay in registers; longer ones take the generic route
    const int kh = !d.hist_tokens ? 2 : (d.hist_stride <= 2 * mako::kThreads ? 2 : (d.hist_stride <= 8 * mako::kThreads ? 8 : 0));
    const bool prof = ctx->profile;
#define MAKO_MARK(i)                                                                                               \
    do {                                                                                                           \
        if (prof)                                                                                                  \
            MAKO_HIP(ctx, hipEventRecord(ctx->ev[i], st));                                                         \
    } while (0)
    // which kernels have work: all of them unless the caller's host copy of the parameters says otherwise
    // (any_late: rows that are finished in tail_kernel's launch, after the plan)
    // (any_index: rows cut neither to a top-k nor to a nucleus, whose candidates stay in token order; known only from
    // the caller's copy of the parameters, they get the kernels of index_rows.h instead of a workgroup each on the
    // whole-row path, unless the vocabulary is beyond 262 144)
    bool any_nucleus = true, any_late = true, any_index = false, only_index = false, any_in_order = false;
    uint32_t nucleus_rows = d.n_rows;
    if (params_host) {
        any_nucleus = any_late = false;
        uint32_t n_nucleus = 0, n_index = 0;
        const bool index_served = d.n_vocab <= mako::kIndexMaxVocab;
        for (uint32_t r = 0; r < d.n_rows; ++r) {
            const mako::RowClass c = mako::classify(params_host[r]);
            // (with them every other row of the whole-row class, whose weights the first of those kernels leaves too)
            const bool index_row = index_served && c == mako::kGeneral;
            any_nucleus |= c == mako::kNucleus;
            any_late |= c == mako::kGeneral && !index_row;
            n_index += index_row;
            any_in_order |= index_row && mako::index_order_row(params_host[r]);
            n_nucleus += c == mako::kNucleus;
        }
        nucleus_rows = std::max(n_nucleus, 1u);
        any_index = n_index != 0;
        only_index = n_index == d.n_rows && !d.force_token && !d.close_token; // (a forced row is written by the late rows' launch)
        // (rows of other kinds beside them are finished in tail_kernel's launch, which leaves alone what the index
        // kernels have claimed; plan_kernel would not)
        any_late |= any_index && !only_index;
    }
    const bool launch_sort = any_nucleus || any_late;
    // (finish_kernel's grid: scan_kernel, which cuts the second pass up, is told of it)
    const uint32_t finish_wgs = mako::second_pass_grid(d.n_rows, nucleus_rows, ctx->cus);
    // Batches with many top_k == 0 rows leave the shares of their sorted lists that need no order unsorted
    // (unsorted_shares.h): there sort_kernel is bound by the number of its workgroups, one per CU at a time, and not, as
    // on a small batch, by its slowest worker.  More than four rounds of workers; without the caller's copy of the
    // parameters, from twice as many rows.
    const bool unsorted = params_host ? (uint64_t)nucleus_rows * mako::kWorkers > 4ull * ctx->cus
                                      : (uint64_t)d.n_rows * mako::kWorkers > 8ull * ctx->cus;
    // (a launch that fails stops the batch there: the kernels after it would work on what it did not write)
#define MAKO_LAUNCH(call)                                                                                          \
    do {                                                                                                           \
        call;                                                                                                      \
        const hipError_t e_launch_ = hipGetLastError();                                                            \
        if (e_launch_ != hipSuccess) {                                                                             \
            *dirty = true;                                                                                         \
            return fail(ctx, MAKO_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(e_launch_));             \
        }                                                                                                          \
    } while (0)
    MAKO_MARK(0);
    MAKO_LAUNCH(mako::launch_scan(vec, kh, d.close_token != nullptr, grid, lds, st, d, sc, slice_len, (ctx->cus & 0xffffu) | ((finish_wgs / 8u) << 16)));
    MAKO_MARK(1);
    // top_k == 0 rows: planned and handed out by the second pass, sorted, cut and drawn from; the stages talk through
    // kernel boundaries (device-wide fences inside a kernel cost far more on this chip).  A batch without such rows
    // (and without rows for the whole-row path) ends with plan_kernel instead.
    if (any_index) // (before the launch that finishes late rows: it leaves alone what this one has claimed)
        MAKO_LAUNCH(mako::launch_index_weights(vec, kh, st, d, sc, slices));
    if (any_nucleus)
        MAKO_LAUNCH(mako::launch_finish(vec, kh, unsorted, finish_wgs, st, d, sc, slices));
    if (!launch_sort && !only_index)
        MAKO_LAUNCH(mako::launch_plan_alone(st, d, sc, slices));
    MAKO_MARK(2);
    if (any_nucleus)
        MAKO_LAUNCH(mako::launch_sort(st, d, sc, slices, nucleus_rows, unsorted));
    MAKO_MARK(3);
    if (launch_sort) // (also finishes every row the kernels before it leave: finish_late_row())
        MAKO_LAUNCH(mako::launch_tail(st, d, sc, slices, nucleus_rows, unsorted));
    if (any_index)
        MAKO_LAUNCH(mako::launch_index_finish(st, d, sc, any_in_order));
    MAKO_MARK(4);
#undef MAKO_MARK
#undef MAKO_LAUNCH
    ctx->profiled = prof;
    return MAKO_OK;
}
} // namespace

extern "C" {

int mako_sampler_sample_host(mako_sampler_ctx* ctx, const float* logits, int64_t logits_stride, uint32_t n_rows,
                             uint32_t n_vocab, const mako_sampling_params* params, const float* u,
                             const uint32_t* mask, int64_t mask_stride, const int32_t* hist_tokens,
                             const uint32_t* hist_counts, int64_t hist_stride, const uint32_t* hist_len,
                             const int32_t* draft, const float* u2, uint8_t* out_accepted, int32_t* out_tokens)
{
    if (!ctx)
        return MAKO_ERR_INVALID_ARG;
    if (n_vocab == 0)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: empty vocabulary");
    if (n_rows == 0)
        return MAKO_OK;
    if (!logits || !params || !u || !out_tokens || n_rows > ctx->max_rows || n_vocab > ctx->max_vocab)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: bad host arguments");
    if (hist_tokens && (!hist_len || hist_stride < 0 || (uint64_t)hist_stride > ctx->max_hist))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: history exceeds the context's max_hist");
    if ((draft != nullptr) != (u2 != nullptr) || (draft != nullptr) != (out_accepted != nullptr))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: draft, u2 and out_accepted go together");
    if (logits_stride < (int64_t)n_vocab)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: logits_stride < n_vocab");
    if (mask && mask_stride < (int64_t)(((uint64_t)n_vocab + 31) / 32))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: mask_stride < ceil(n_vocab / 32)");
    if (hist_tokens && hist_stride > 0)
        for (uint32_t r = 0; r < n_rows; ++r) // (columns beyond hist_stride of the staging rows hold older calls' ids)
            if (hist_len[r] > (uint64_t)hist_stride)
                return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: hist_len[r] > hist_stride");
    MAKO_HIP(ctx, hipSetDevice(ctx->device));
    const size_t R = ctx->max_rows;
    const size_t mwords = ((size_t)ctx->max_vocab + 31) / 32;
    // staging buffers are created on first use and kept
    if (!ctx->st_logits) {
        MAKO_HIP(ctx, dev_alloc(&ctx->st_logits, R * ctx->sc.vpad));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_params, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_u, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_u2, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_mask, R * mwords));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_hist, R * (size_t)(ctx->max_hist ? ctx->max_hist : 1)));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_hcnt, R * (size_t)(ctx->max_hist ? ctx->max_hist : 1)));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_hlen, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_draft, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_tokens, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_acc, R));
    }
    const size_t vp = ctx->sc.vpad;
    MAKO_HIP(ctx, hipMemcpy2D(ctx->st_logits, vp * sizeof(float), logits, (size_t)logits_stride * sizeof(float),
                              (size_t)n_vocab * sizeof(float), n_rows, hipMemcpyHostToDevice));
    MAKO_HIP(ctx, hipMemcpy(ctx->st_params, params, n_rows * sizeof(*params), hipMemcpyHostToDevice));
    MAKO_HIP(ctx, hipMemcpy(ctx->st_u, u, n_rows * sizeof(float), hipMemcpyHostToDevice));
    mako_sample_desc d;
    memset(&d, 0, sizeof d);
    d.logits = ctx->st_logits;
    d.logits_stride = (int64_t)vp;
    d.n_rows = n_rows;
    d.n_vocab = n_vocab;
    d.params = ctx->st_params;
    d.u = ctx->st_u;
    if (mask) {
        const size_t w = ((size_t)n_vocab + 31) / 32;
        MAKO_HIP(ctx, hipMemcpy2D(ctx->st_mask, mwords * 4, mask, (size_t)mask_stride * 4, w * 4, n_rows,
                                  hipMemcpyHostToDevice));
        d.mask = ctx->st_mask;
        d.mask_stride = (int64_t)mwords;
    }
    if (hist_tokens && hist_stride > 0) {
        const size_t hs = ctx->max_hist;
        MAKO_HIP(ctx, hipMemcpy2D(ctx->st_hist, hs * 4, hist_tokens, (size_t)hist_stride * 4, (size_t)hist_stride * 4,
                                  n_rows, hipMemcpyHostToDevice));
        if (hist_counts) {
            MAKO_HIP(ctx, hipMemcpy2D(ctx->st_hcnt, hs * 4, hist_counts, (size_t)hist_stride * 4,
                                      (size_t)hist_stride * 4, n_rows, hipMemcpyHostToDevice));
            d.hist_counts = ctx->st_hcnt;
        }
        MAKO_HIP(ctx, hipMemcpy(ctx->st_hlen, hist_len, n_rows * 4, hipMemcpyHostToDevice));
        d.hist_tokens = ctx->st_hist;
        d.hist_stride = (int64_t)hs;
        d.hist_len = ctx->st_hlen;
    }
    if (draft) {
        MAKO_HIP(ctx, hipMemcpy(ctx->st_draft, draft, n_rows * 4, hipMemcpyHostToDevice));
        MAKO_HIP(ctx, hipMemcpy(ctx->st_u2, u2, n_rows * 4, hipMemcpyHostToDevice));
        d.draft = ctx->st_draft;
        d.u2 = ctx->st_u2;
        d.out_accepted = ctx->st_acc;
    }
    d.out_tokens = ctx->st_tokens;
    // (the caller's parameters are in host memory: the call looks at them and leaves out what no row needs)
    const int rc = mako_sampler_sample_batch_hinted(ctx, &d, params, nullptr);
    if (rc != MAKO_OK)
        return rc;
    MAKO_HIP(ctx, hipMemcpy(out_tokens, ctx->st_tokens, n_rows * 4, hipMemcpyDeviceToHost));
    if (draft)
        MAKO_HIP(ctx, hipMemcpy(out_accepted, ctx->st_acc, n_rows, hipMemcpyDeviceToHost));
    return MAKO_OK;
}

int mako_sampler_debug_checks(mako_sampler_ctx* ctx, uint32_t* out_bits)
{
    if (!ctx || !out_bits)
        return MAKO_ERR_INVALID_ARG;
    MAKO_HIP(ctx, hipSetDevice(ctx->device));
    MAKO_HIP(ctx, hipDeviceSynchronize());
    MAKO_HIP(ctx, hipMemcpy(out_bits, ctx->sc.work_n + 2, sizeof(uint32_t), hipMemcpyDeviceToHost));
    MAKO_HIP(ctx, hipMemset(ctx->sc.work_n + 2, 0, sizeof(uint32_t)));
    return MAKO_OK;
}

int mako_sampler_debug_expf(const float* x_dev, float* y_dev, uint32_t n, void* stream)
{
    if (!x_dev || !y_dev)
        return MAKO_ERR_INVALID_ARG;
    if (n)
        hipLaunchKernelGGL(mako::debug_expf_kernel, dim3((n + 255) / 256), dim3(256), 0,
                           static_cast<hipStream_t>(stream), x_dev, y_dev, n);
    return hipGetLastError() == hipSuccess ? MAKO_OK : MAKO_ERR_HIP;
}

int mako_sampler_debug_div(const float* a_dev, const float* b_dev, float* y_dev, uint32_t n, void* stream)
{
    if (!a_dev || !b_dev || !y_dev)
        return MAKO_ERR_INVALID_ARG;
    if (n)
        hipLaunchKernelGGL(mako::debug_div_kernel, dim3((n + 255) / 256), dim3(256), 0,
                           static_cast<hipStream_t>(stream), a_dev, b_dev, y_dev, n);
    return hipGetLastError() == hipSuccess ? MAKO_OK : MAKO_ERR_HIP;
}

} // extern "C"
