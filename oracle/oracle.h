/*
 * CPU oracle for the token sampler -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference sampler's arithmetic
 * (reference: src/gen/sampler.cpp:9-107, src/gen/sampler.hpp:11-20) taking the
 * uniform draws as explicit arguments.  Nothing the library ships may call
 * into this file; it exists so tests, the smoke check and the bench's CPU
 * baseline leg can check the HIP path.
 *
 * Third-party arithmetic the reference reaches through its toolchain is
 * restated here from the published algorithms and pinned by tests:
 *   - expf: glibc 2.35 sysdeps/ieee754/flt-32/e_expf.c (x86-64 FMA build),
 *     pinned bit-for-bit against libm over every float input.
 *   - std::nth_element: libstdc++ 11.4 bits/stl_algo.h __introselect,
 *     pinned against the compiled reference (candidate order after top-k).
 *   - std::mt19937_64 + std::generate_canonical<float,24>: libstdc++ 11.4
 *     bits/random.tcc, pinned against the compiled reference's draws.
 */
#ifndef MAKO_ORACLE_H
#define MAKO_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Field order and defaults follow SamplingParams, src/gen/sampler.hpp:11-20. */
typedef struct {
    float temperature;
    uint32_t top_k;
    float top_p;
    float min_p;
    float presence_penalty;
    float frequency_penalty;
    float repetition_penalty;
} or_params;

/* Optional per-call trace of the intermediate state. */
typedef struct {
    uint32_t n_cand;      /* candidates left after min_p/top-k/top-p */
    float total;          /* fp32 sequential sum of their q, in candidate order */
    float q_chosen;       /* q of the returned token (0 when greedy) */
    float max_logit;      /* max of the penalised logits */
    uint32_t cap;         /* capacity of the two arrays below (may be 0) */
    int32_t* cand_idx;    /* first min(cap, n_cand) candidate ids, candidate order */
    float* cand_q;        /* and their q */
} or_trace;

/* glibc 2.35 expf restated (FMA variant). */
float or_expf(float x);
void or_expf_array(const float* x, float* y, size_t n);

/* n draws of generate_canonical<float,24>(mt19937_64(seed)). */
void or_uniforms(uint64_t seed, uint32_t n, float* out);

/*
 * One Sampler::sample() call (sampler.cpp:75-84) on a fresh sampler whose
 * accept() history is `hist[0..n_hist)` and whose single uniform is `u`.
 * `mask` (optional): bit i of word i/32 set = token i allowed; a cleared bit
 * turns the logit into -inf before anything else.
 * `order_mode`: 0 = candidate order after top-k is the one libstdc++'s
 * nth_element leaves (what the reference does); 1 = (q desc, idx asc).
 * The two differ only when top_k is active and top_p >= 1.
 */
int32_t or_sample(const float* logits, uint32_t n_vocab, const or_params* p,
                  const int32_t* hist, uint32_t n_hist, const uint32_t* mask,
                  float u, int order_mode, or_trace* trace);

/*
 * One Sampler::verify() call (sampler.cpp:86-107): u1 is consumed by the
 * acceptance test, u2 by the redraw after a rejection.
 */
int32_t or_verify(const float* logits, uint32_t n_vocab, const or_params* p,
                  const int32_t* hist, uint32_t n_hist, const uint32_t* mask,
                  int32_t draft, float u1, float u2, int order_mode,
                  int* accepted, or_trace* trace);

/*
 * The last-stretch test of ReasoningBudget::forced (src/server/openai.cpp:596-604):
 * returns think_end when fewer than max_above (3 in the reference) logits are
 * strictly greater than logits[think_end], else -1; -1 also when think_end is
 * negative or not below n_vocab (:590, :594).  `mask` as in or_sample (a build
 * extension: a cleared bit is -inf, and a cleared think_end is never returned).
 * `above`, if given, receives the full count (the reference stops at 3).
 * Pinned by the known answers of tests/server_test.cpp:142-152.
 */
int32_t or_close_forced(const float* logits, uint32_t n_vocab, const uint32_t* mask, int32_t think_end,
                        uint32_t max_above, uint32_t* above);

/* libstdc++ nth_element restated, exposed for its own pin test:
 * keys are (q, idx) pairs ordered by (q desc, idx asc). */
void or_nth_element(float* q, int32_t* idx, uint32_t n, uint32_t nth);
/* Number of times the restated introselect took its heap-select branch (test hook). */
long or_debug_heap_selects(void);

#ifdef __cplusplus
}
#endif
#endif
