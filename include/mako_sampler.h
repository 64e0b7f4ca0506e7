/*
 * mako_sampler.h -- C ABI of the MI355X token sampler.
 *
 * A batched, device-resident replacement for the reference's C++ class
 * mako::gen::Sampler (src/gen/sampler.hpp:22-45): fp32 logits in, the
 * SamplingParams fields, the accept() history, an optional allowed-token
 * bitmask and one caller-supplied uniform per row in, sampled token ids out.
 * Row r of a batch behaves exactly like a fresh reference Sampler with row r's
 * parameters whose accept() was called once per history token and whose
 * sample() (or verify()) is then called on row r's logits, with the uniform
 * draws replaced by the caller's u (and u2).
 *
 * Every pointer inside mako_sample_desc is a DEVICE pointer; the host-pointer
 * convenience call stages through context-owned buffers, which it allocates
 * on its first call.  The library never writes the caller's logits; the
 * mako_sampler_sample_batch* calls allocate nothing (their scratch memory is
 * allocated by mako_sampler_create, or is part of the library's image); and
 * failures are reported as negative status codes (the reference throws
 * std::invalid_argument, src/gen/sampler.cpp:11-12).
 */
#ifndef MAKO_SAMPLER_H
#define MAKO_SAMPLER_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MAKO_OK 0
#define MAKO_ERR_INVALID_ARG (-1) /* null pointer, n_vocab == 0, sizes beyond the context's */
#define MAKO_ERR_HIP (-2)         /* a HIP call failed; see mako_sampler_last_error */
#define MAKO_ERR_NO_MEMORY (-3)

/* Same fields, order, defaults and meaning as SamplingParams,
 * src/gen/sampler.hpp:11-20 (28 bytes).  temperature <= 0 selects greedy. */
typedef struct mako_sampling_params {
    float temperature;
    uint32_t top_k;
    float top_p;
    float min_p;
    float presence_penalty;
    float frequency_penalty;
    float repetition_penalty;
} mako_sampling_params;

/* How a row was resolved (optional diagnostic output). */
#define MAKO_PATH_GREEDY 1u   /* argmax of the (masked) raw logits */
#define MAKO_PATH_FALLBACK 2u /* no candidate survived: most likely token (sampler.cpp:37-38) */
#define MAKO_PATH_TOPK 3u     /* resolved from the per-slice top-k candidates */
#define MAKO_PATH_NUCLEUS 4u  /* top_k == 0: nucleus resolved from the per-slice candidates */
#define MAKO_PATH_GENERAL 5u  /* whole-row sort path */
#define MAKO_PATH_FORCED 6u   /* not sampled: force_token / close_token took the row */
#define MAKO_PATH_SORTED 7u   /* top_k == 0: nucleus cut from the sorted list of the weights the row's plan kept */
#define MAKO_PATH_INDEXED 9u  /* neither top-k nor top-p: total and walk in token order over the whole row, by group maps */
#define MAKO_PATH_SUMMED 8u   /* the same on a batch of many such rows: the parts of the list whose order cannot matter to the
                                 fp32 total and walk were summed, not sorted */

/* out_forced values */
#define MAKO_FORCED_NONE 0u  /* the row was sampled (or verified) */
#define MAKO_FORCED_TOKEN 1u /* force_token was taken */
#define MAKO_FORCED_CLOSE 2u /* close_token was taken: fewer than close_max_above logits above its own */

typedef struct mako_sample_desc {
    /* ---- inputs (device pointers) ---- */
    const float* logits;     /* [n_rows][logits_stride], fp32; read-only (sampler.hpp:27 `const float*`) */
    int64_t logits_stride;   /* elements between rows, >= n_vocab */
    uint32_t n_rows;
    uint32_t n_vocab;        /* > 0 (sampler.cpp:11) */
    const mako_sampling_params* params; /* [n_rows] */
    const float* u;          /* [n_rows] uniforms in [0,1): the draw of sampler.cpp:66, or of :100 when verifying */
    const uint32_t* mask;    /* optional [n_rows][mask_stride]: bit (i & 31) of word i >> 5 set = token i allowed;
                                a cleared bit makes the logit -inf before anything else (no reference counterpart) */
    int64_t mask_stride;     /* 32-bit words between rows, >= ceil(n_vocab / 32) */
    const int32_t* hist_tokens; /* optional [n_rows][hist_stride]: the tokens passed to accept(), sampler.cpp:15-18;
                                   ids outside [0, n_vocab) are ignored */
    const uint32_t* hist_counts; /* optional, same shape: if non-null entry j counts hist_counts[j] occurrences
                                    (pre-aggregated (id, count) pairs, the reference's counts_ map); an entry
                                    that counts 0 occurrences is ignored, like a token accept() never saw */
    int64_t hist_stride;
    const uint32_t* hist_len;   /* [n_rows] valid entries per row (required when hist_tokens is given) */
    /* speculative verification, sampler.cpp:86-107 (optional: all three or none) */
    const int32_t* draft;    /* [n_rows] draft token per row */
    const float* u2;         /* [n_rows] second uniform, consumed by the redraw after a rejection (:106) */
    uint8_t* out_accepted;   /* [n_rows] 1 = draft accepted */
    /* ---- outputs (device pointers) ---- */
    int32_t* out_tokens;     /* [n_rows] sampled token ids */
    /* optional diagnostics for parity checks; any may be null */
    uint32_t* out_n_cand;    /* [n_rows] size of the final candidate list (0 for greedy rows) */
    float* out_total;        /* [n_rows] fp32 total of sampler.cpp:80-82 */
    float* out_q;            /* [n_rows] unnormalised weight of the returned token; probability = q / total */
    uint8_t* out_path;       /* [n_rows] MAKO_PATH_* */
    int32_t* out_cand_idx;   /* [n_rows][cand_cap] first candidates, in candidate order */
    float* out_cand_q;       /* [n_rows][cand_cap] and their weights */
    uint32_t cand_cap;
    /* ---- the decode loop's hooks around the sampler (optional; zero / null = the sampler alone) ----
     * Session::run asks its `forced` callback before every sample() / verify() (src/gen/session.hpp:43-45,
     * src/gen/session.cpp:441-443, 483-485, 524-525): a token >= 0 is taken instead of sampling (a draft is kept
     * only if it equals it), no uniform is consumed, and the token goes through accept() like a sampled one. */
    const int32_t* force_token; /* [n_rows]: >= 0: the callback's answer is already known to the caller */
    /* ReasoningBudget::forced's last stretch (src/server/openai.cpp:589-604): close_token[r] in [0, n_vocab) is
     * taken iff fewer than close_max_above logits of the row are strictly greater than logits[close_token[r]]
     * (the reference stops counting at 3).  The test sees the logits the sampler is given: a token the mask
     * clears counts as -inf, and a cleared close_token is never taken.  force_token[r] >= 0 wins over it. */
    const int32_t* close_token; /* [n_rows], < 0: none */
    uint32_t close_max_above;
    uint8_t* out_forced;        /* [n_rows] MAKO_FORCED_*; required when force_token or close_token is given */
    uint32_t* out_above;        /* optional [n_rows]: logits strictly above logits[close_token[r]] (all of them,
                                   not capped); 0xffffffff where there is no close_token or the mask clears it */
    /* Sampler::accept of the chosen token (src/gen/session.cpp:419-421) without a trip to the host: when nonzero,
     * row r's token is written to hist_tokens[r][hist_len[r]] and hist_len[r] is incremented, provided
     * hist_len[r] < hist_stride (else the history is left as it is).  hist_tokens and hist_len must then be
     * writable device memory, hist_counts null, and draft null (the rows of a verify batch share one history). */
    uint32_t append_history;
} mako_sample_desc;

typedef struct mako_sampler_ctx mako_sampler_ctx;

/* Creates a context on HIP device `device` able to serve batches of up to
 * max_rows x max_vocab with histories of up to max_hist tokens per row; all
 * device scratch is allocated here.  Replaces Sampler::Sampler
 * (src/gen/sampler.cpp:9-13) as the owner of the work buffers. */
int mako_sampler_create(mako_sampler_ctx** out, int device, uint32_t max_rows, uint32_t max_vocab,
                        uint32_t max_hist);
void mako_sampler_destroy(mako_sampler_ctx* ctx);

/* Enqueues one batch on `stream` (a hipStream_t, or null for the default
 * stream) and returns without waiting: Sampler::sample / Sampler::verify
 * (src/gen/sampler.cpp:75-107) for every row.  One batch at a time per context.
 * If a kernel launch fails the call returns MAKO_ERR_HIP at once and the batch's outputs are undefined; the next
 * call on the same context (for the static call: on the same GPU) first waits for the device and clears the
 * kernels' scratch memory again, which it cannot do under stream capture (it then returns MAKO_ERR_HIP). */
int mako_sampler_sample_batch(mako_sampler_ctx* ctx, const mako_sample_desc* desc, void* stream);

/* The same call for a caller that still has the batch's parameters in HOST memory (the SamplingParams originate
 * there, src/gen/session.hpp:19-21): params_host[n_rows] must hold the same values as desc->params.  The call
 * looks at them on the calling thread and leaves out the kernels that no row of the batch needs (a batch without
 * top_k == 0 rows takes two launches instead of four).  Rows that are cut neither to a top-k nor to a nucleus
 * (temperature only: top_k == 0, top_p >= 1), whose candidates stay in token order, get three launches of their own
 * instead of one workgroup each for the whole row (up to 262 144 logits per row), verification and the decode loop's
 * hooks included; the other rows of the whole-row path (a top-k without a top-p, a top-k beyond 128) then get their
 * weights from many workgroups instead of one.  The results never depend on it; null = the call above. */
int mako_sampler_sample_batch_hinted(mako_sampler_ctx* ctx, const mako_sample_desc* desc,
                                     const mako_sampling_params* params_host, void* stream);

/* mako_sampler_sample_batch for callers that must not allocate device memory around the call: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  (The
 * context it is given still holds the scratch memory mako_sampler_create() allocated for it; a context made only for
 * this call can be created with max_rows = 1 and a small max_vocab.)  The kernels' scratch memory (candidate lists, histograms, sort buffers, work lists)
 * is not the context's but an array of MAKO_STATIC_SCRATCH_MIB MiB inside the library's image, of which every GPU
 * that the library runs on holds one copy until the process ends; mako_sampler_create() looks its address up once
 * per device.  Batches of up to MAKO_STATIC_MAX_ROWS rows of up to MAKO_STATIC_MAX_VOCAB logits; anything larger is
 * refused with MAKO_ERR_INVALID_ARG.  No hipMalloc, hipFree or other allocating call is made.  Results are those
 * of mako_sampler_sample_batch, bit for bit.  All contexts of one GPU share that GPU's array: calls that overlap
 * on one GPU (two streams, two threads) race; calls in stream order do not. */
#define MAKO_STATIC_MAX_ROWS 16
#define MAKO_STATIC_MAX_VOCAB 131072
#define MAKO_STATIC_SCRATCH_MIB 52
int mako_sampler_sample_batch_static(mako_sampler_ctx* ctx, const mako_sample_desc* desc, void* stream);

/* Host-pointer convenience call with the reference's calling convention
 * (host logits, src/gen/session.cpp:443): copies the rows to the device,
 * samples, waits and copies the ids back.  Arrays are host arrays here; mask,
 * hist_*, draft/u2/accepted may be null.  PCIe-bound, not the measured path. */
int mako_sampler_sample_host(mako_sampler_ctx* ctx, const float* logits, int64_t logits_stride, uint32_t n_rows,
                             uint32_t n_vocab, const mako_sampling_params* params, const float* u,
                             const uint32_t* mask, int64_t mask_stride, const int32_t* hist_tokens,
                             const uint32_t* hist_counts, int64_t hist_stride, const uint32_t* hist_len,
                             const int32_t* draft, const float* u2, uint8_t* out_accepted, int32_t* out_tokens);

/* Text of the last failure on this context (never null). */
const char* mako_sampler_last_error(const mako_sampler_ctx* ctx);

/* Per-kernel timing for benchmarks (no counterpart in the reference).  While enabled, every
 * mako_sampler_sample_batch records HIP events on its stream around its kernels;
 * mako_sampler_kernel_times waits for the last recorded batch and returns the milliseconds of
 * scan_kernel, finish_kernel (plan_kernel, for a batch that ends with it), sort_kernel and
 * tail_kernel in out_ms[0..3].  Off by default. */
#define MAKO_SAMPLER_KERNELS 4
int mako_sampler_set_profile(mako_sampler_ctx* ctx, int enabled);
int mako_sampler_kernel_times(mako_sampler_ctx* ctx, float* out_ms);

/* Number of slices a row of n_vocab logits is split into by the scan kernel. */
uint32_t mako_sampler_slices(uint32_t n_vocab);

/* Device-side self-check hooks used by the parity tests: evaluate the
 * library's expf (glibc 2.35 bit-exact) and fp32 division on n device values. */
int mako_sampler_debug_expf(const float* x_dev, float* y_dev, uint32_t n, void* stream);
int mako_sampler_debug_div(const float* a_dev, const float* b_dev, float* y_dev, uint32_t n, void* stream);

/* Checked builds of the library (libmako_sampler_checked.so, -DMAKO_CHECKED) compare every index their kernels
 * compute into the context's scratch arrays with the array's bound and record failures instead of trapping: this call
 * waits for the device, returns the failed checks of all batches since the last call as a bit set in *out_bits and
 * clears them.  Bit 31 is set by every batch of a checked build (the checks are there); the other bits name checks that
 * failed.  The shipped library has no checks compiled in and always reports 0. */
int mako_sampler_debug_checks(mako_sampler_ctx* ctx, uint32_t* out_bits);

#ifdef __cplusplus
}
#endif
#endif
