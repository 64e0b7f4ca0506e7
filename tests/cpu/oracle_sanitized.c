/* Drives the plain-C oracle over random rows with every parameter combination, histories, masks and traces, for a
 * build with -fsanitize=address,undefined: the checks are the sanitizers' own, plus range checks on what comes
 * back.  Prints "<n> calls, 0 failures". */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "oracle.h"

static uint64_t s_state = 0x9e3779b97f4a7c15ull;
static uint64_t next_u64(void)
{
    s_state ^= s_state << 13;
    s_state ^= s_state >> 7;
    s_state ^= s_state << 17;
    return s_state;
}
static float unit(void) { return (float)(next_u64() >> 40) / 16777216.0f; }

int main(void)
{
    static const uint32_t vocabs[] = {1, 2, 7, 33, 257, 4096, 50001};
    static const uint32_t top_ks[] = {0, 1, 2, 20, 128, 700, 100000};
    static const float top_ps[] = {1.0f, 0.999f, 0.9f, 0.5f, 0.01f, 0.0f};
    static const float min_ps[] = {0.0f, 0.05f, 0.5f, 1.0f};
    static const float temps[] = {0.0f, 0.05f, 0.7f, 1.0f, 3.0f};
    long calls = 0, failures = 0;
    for (unsigned vi = 0; vi < sizeof vocabs / sizeof *vocabs; ++vi) {
        const uint32_t v = vocabs[vi], words = (v + 31) / 32;
        float* logits = malloc(v * sizeof *logits);
        uint32_t* mask = malloc(words * sizeof *mask);
        int32_t* hist = malloc(300 * sizeof *hist);
        int32_t* cand_idx = malloc(64 * sizeof *cand_idx);
        float* cand_q = malloc(64 * sizeof *cand_q);
        for (int rep = 0; rep < 40; ++rep) {
            for (uint32_t i = 0; i < v; ++i)
                logits[i] = (unit() - 0.5f) * 24.0f;
            if (rep % 7 == 3)
                logits[next_u64() % v] = -INFINITY;
            for (uint32_t i = 0; i < words; ++i)
                mask[i] = (uint32_t)next_u64() | (uint32_t)next_u64();
            mask[0] |= 1u; /* at least one allowed token */
            const uint32_t n_hist = (uint32_t)(next_u64() % 300);
            for (uint32_t i = 0; i < n_hist; ++i)
                hist[i] = (int32_t)(next_u64() % v);
            or_params p;
            p.temperature = temps[next_u64() % 5];
            p.top_k = top_ks[next_u64() % 7];
            p.top_p = top_ps[next_u64() % 6];
            p.min_p = min_ps[next_u64() % 4];
            p.presence_penalty = rep % 2 ? 0.3f : 0.0f;
            p.frequency_penalty = rep % 3 ? 0.2f : 0.0f;
            p.repetition_penalty = rep % 4 ? 1.1f : 1.0f;
            or_trace tr = {0};
            tr.cap = rep % 2 ? 64 : 0;
            tr.cand_idx = cand_idx;
            tr.cand_q = cand_q;
            const uint32_t* m = rep % 3 == 0 ? mask : NULL;
            for (int mode = 0; mode < 2; ++mode) {
                const int32_t t = or_sample(logits, v, &p, hist, n_hist, m, unit(), mode, &tr);
                ++calls;
                if (t < 0 || (uint32_t)t >= v || (p.temperature > 0.0f && (tr.n_cand == 0 || tr.n_cand > v))) {
                    ++failures;
                    fprintf(stderr, "sample v=%u t=%d n_cand=%u T=%g k=%u p=%g minp=%g\n", v, t, tr.n_cand, p.temperature, p.top_k, p.top_p, p.min_p);
                }
                int acc = -1;
                const int32_t t2 = or_verify(logits, v, &p, hist, n_hist, m, (int32_t)(next_u64() % v), unit(), unit(),
                                             mode, &acc, &tr);
                ++calls;
                if (t2 < 0 || (uint32_t)t2 >= v || (acc != 0 && acc != 1)) {
                    ++failures;
                    fprintf(stderr, "verify v=%u t=%d acc=%d\n", v, t2, acc);
                }
            }
            uint32_t above = 0;
            const int32_t te = (int32_t)(next_u64() % v);
            const int32_t f = or_close_forced(logits, v, m, te, 3, &above);
            ++calls;
            if ((f != -1 && f != te) || (above > v && !(f == -1 && above == 0xffffffffu)))
                ++failures;
        }
        free(logits);
        free(mask);
        free(hist);
        free(cand_idx);
        free(cand_q);
    }
    float u[64];
    or_uniforms(12345, 64, u);
    for (int i = 0; i < 64; ++i)
        if (!(u[i] >= 0.0f && u[i] < 1.0f))
            ++failures;
    printf("%ld calls, %ld failures\n", calls, failures);
    return failures != 0;
}
