/*
 * CPU oracle for the token sampler -- TEST INFRASTRUCTURE ONLY (see oracle.h).
 * Build: gcc -O2 -std=c11 -ffp-contract=off -mfma (the explicit fma() calls
 * below must stay single-rounding; nothing else may be contracted).
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ expf */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint64_t d2u(double f) { uint64_t u; memcpy(&u, &f, 8); return u; }
static inline double u2d(uint64_t u) { double f; memcpy(&f, &u, 8); return f; }

/* tab[i] = bits(2^(i/32)) - (i << 47): glibc 2.35 sysdeps/ieee754/flt-32/
 * e_exp2f_data.c; regenerated from 2^(i/32) in exact integer arithmetic. */
static const uint64_t k_exp2_tab[32] = {
    0x3ff0000000000000, 0x3fefd9b0d3158574, 0x3fefb5586cf9890f, 0x3fef9301d0125b51,
    0x3fef72b83c7d517b, 0x3fef54873168b9aa, 0x3fef387a6e756238, 0x3fef1e9df51fdee1,
    0x3fef06fe0a31b715, 0x3feef1a7373aa9cb, 0x3feedea64c123422, 0x3feece086061892d,
    0x3feebfdad5362a27, 0x3feeb42b569d4f82, 0x3feeab07dd485429, 0x3feea47eb03a5585,
    0x3feea09e667f3bcd, 0x3fee9f75e8ec5f74, 0x3feea11473eb0187, 0x3feea589994cce13,
    0x3feeace5422aa0db, 0x3feeb737b0cdc5e5, 0x3feec49182a3f090, 0x3feed503b23e255d,
    0x3feee89f995ad3ad, 0x3feeff76f2fb5e47, 0x3fef199bdd85529c, 0x3fef3720dcef9069,
    0x3fef5818dcfba487, 0x3fef7c97337b9b5f, 0x3fefa4afa2a490da, 0x3fefd0765b6e4540,
};

/* glibc 2.35 sysdeps/ieee754/flt-32/e_expf.c as built for x86-64 with FMA
 * (sysdeps/x86_64/fpu/multiarch/e_expf.c): the products feeding the range
 * reduction and the polynomial are fused.  The reference reaches this through
 * std::exp(float), src/gen/sampler.cpp:33. */
float or_expf(float x)
{
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    const double shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32;
    const double c1 = 0x1.ebfce50fac4f3p-3 / 32 / 32;
    const double c2 = 0x1.62e42ff0c52d6p-1 / 32;
    const uint32_t ix = f2u(x);
    const uint32_t abstop = (ix >> 20) & 0x7ff;
    if (abstop >= (f2u(88.0f) >> 20)) {
        if (ix == f2u(-INFINITY))
            return 0.0f;
        if (abstop >= (f2u(INFINITY) >> 20))
            return x + x;
        if (x > 0x1.62e42ep6f)
            return INFINITY;
        if (x < -0x1.9fe368p6f)
            return 0.0f;
        if (x < -0x1.9d1d9ep6f)
            return 0x1p-149f;
    }
    const double xd = (double)x;
    double kd = fma(inv_ln2_n, xd, shift);
    const uint64_t ki = d2u(kd);
    kd -= shift;
    const double r = fma(inv_ln2_n, xd, -kd);
    const double s = u2d(k_exp2_tab[ki & 31] + (ki << 47));
    const double z = fma(c0, r, c1);
    const double r2 = r * r;
    double y = fma(c2, r, 1.0);
    y = fma(z, r2, y);
    return (float)(y * s);
}

/* or_expf over an array (for tests that compare millions of device results). */
void or_expf_array(const float* x, float* y, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        y[i] = or_expf(x[i]);
}

/* ------------------------------------------------------------- uniforms */

/* std::mt19937_64 (ISO C++ [rand.predef]) followed by libstdc++ 11.4
 * generate_canonical<float,24> (bits/random.tcc:3348-3380): one 64-bit draw,
 * converted to float, divided by 2^64, a result of 1 replaced by the float
 * below 1.  The reference draws through uniform_real_distribution<float>,
 * src/gen/sampler.cpp:66,100. */
void or_uniforms(uint64_t seed, uint32_t n, float* out)
{
    enum { NN = 312, MM = 156 };
    uint64_t mt[NN];
    mt[0] = seed;
    for (int i = 1; i < NN; ++i)
        mt[i] = 6364136223846793005ull * (mt[i - 1] ^ (mt[i - 1] >> 62)) + (uint64_t)i;
    int pos = NN;
    for (uint32_t d = 0; d < n; ++d) {
        if (pos == NN) {
            for (int i = 0; i < NN; ++i) {
                const uint64_t y = (mt[i] & 0xFFFFFFFF80000000ull) | (mt[(i + 1) % NN] & 0x7FFFFFFFull);
                mt[i] = mt[(i + MM) % NN] ^ (y >> 1) ^ ((y & 1) ? 0xB5026F5AA96619E9ull : 0);
            }
            pos = 0;
        }
        uint64_t z = mt[pos++];
        z ^= (z >> 29) & 0x5555555555555555ull;
        z ^= (z << 17) & 0x71D67FFFEDA60000ull;
        z ^= (z << 37) & 0xFFF7EEE000000000ull;
        z ^= z >> 43;
        float r = (float)z / 0x1p64f;
        if (r >= 1.0f)
            r = nextafterf(1.0f, 0.0f);
        out[d] = r;
    }
}

/* ------------------------------------------------- candidate ordering */

typedef struct {
    float q;
    int32_t idx;
} cand_t;

/* The comparator `desc`, src/gen/sampler.cpp:39. */
static inline int before(const cand_t* a, const cand_t* b)
{
    return a->q > b->q || (a->q == b->q && a->idx < b->idx);
}

static int before_qsort(const void* a, const void* b)
{
    const cand_t* x = a;
    const cand_t* y = b;
    return before(x, y) ? -1 : (before(y, x) ? 1 : 0);
}

static inline void swap_c(cand_t* a, cand_t* b)
{
    cand_t t = *a;
    *a = *b;
    *b = t;
}

/* Binary max-heap under `before` (the "largest" element is the one that sorts
 * last), sift-down-to-leaf then sift-up: libstdc++ 11.4 bits/stl_heap.h. */
static void heap_sift(cand_t* h, long hole, long len, cand_t v)
{
    const long top = hole;
    long child = hole;
    while (child < (len - 1) / 2) {
        child = 2 * (child + 1);
        if (before(&h[child], &h[child - 1]))
            --child;
        h[hole] = h[child];
        hole = child;
    }
    if ((len & 1) == 0 && child == (len - 2) / 2) {
        child = 2 * (child + 1);
        h[hole] = h[child - 1];
        hole = child - 1;
    }
    long parent = (hole - 1) / 2;
    while (hole > top && before(&h[parent], &v)) {
        h[hole] = h[parent];
        hole = parent;
        parent = (hole - 1) / 2;
    }
    h[hole] = v;
}

static long g_heap_selects; /* times introselect fell back to heap_select (test hook) */
long or_debug_heap_selects(void) { return g_heap_selects; }

/* libstdc++ 11.4 bits/stl_algo.h __heap_select. */
static void heap_select(cand_t* a, long middle, long last)
{
    ++g_heap_selects;
    if (middle >= 2)
        for (long parent = (middle - 2) / 2;; --parent) {
            heap_sift(a, parent, middle, a[parent]);
            if (parent == 0)
                break;
        }
    for (long i = middle; i < last; ++i)
        if (before(&a[i], &a[0])) {
            cand_t v = a[i];
            a[i] = a[0];
            heap_sift(a, 0, middle, v);
        }
}

/* libstdc++ 11.4 bits/stl_algo.h:1964 __introselect with its median-of-three
 * unguarded Hoare partition and the final insertion sort; reached from
 * std::ranges::nth_element, src/gen/sampler.cpp:41. */
static void introselect(cand_t* a, long first, long nth, long last)
{
    long n = last - first, depth = 0;
    if (n <= 0 || nth == last)
        return;
    while (n > 1) {
        n >>= 1;
        ++depth;
    }
    depth *= 2;
    while (last - first > 3) {
        if (depth == 0) {
            heap_select(a + first, nth + 1 - first, last - first);
            swap_c(&a[first], &a[nth]);
            return;
        }
        --depth;
        /* median of a[first+1], a[mid], a[last-1] goes to a[first] */
        {
            cand_t *r = &a[first], *x = &a[first + 1], *y = &a[first + (last - first) / 2], *z = &a[last - 1];
            if (before(x, y)) {
                if (before(y, z))
                    swap_c(r, y);
                else if (before(x, z))
                    swap_c(r, z);
                else
                    swap_c(r, x);
            } else if (before(x, z))
                swap_c(r, x);
            else if (before(y, z))
                swap_c(r, z);
            else
                swap_c(r, y);
        }
        long lo = first + 1, hi = last;
        for (;;) {
            while (before(&a[lo], &a[first]))
                ++lo;
            --hi;
            while (before(&a[first], &a[hi]))
                --hi;
            if (!(lo < hi))
                break;
            swap_c(&a[lo], &a[hi]);
            ++lo;
        }
        if (lo <= nth)
            first = lo;
        else
            last = lo;
    }
    for (long i = first + 1; i < last; ++i) {
        cand_t v = a[i];
        long j = i;
        if (before(&v, &a[first])) {
            for (; j > first; --j)
                a[j] = a[j - 1];
        } else {
            for (; before(&v, &a[j - 1]); --j)
                a[j] = a[j - 1];
        }
        a[j] = v;
    }
}

void or_nth_element(float* q, int32_t* idx, uint32_t n, uint32_t nth)
{
    cand_t* a = malloc(sizeof(cand_t) * (n ? n : 1));
    for (uint32_t i = 0; i < n; ++i) {
        a[i].q = q[i];
        a[i].idx = idx[i];
    }
    introselect(a, 0, nth, n);
    for (uint32_t i = 0; i < n; ++i) {
        q[i] = a[i].q;
        idx[i] = a[i].idx;
    }
    free(a);
}

/* --------------------------------------------------------- the sampler */

/* std::max_element: first index i such that no later element compares
 * greater under `<` (NaNs never win unless they sit at index 0). */
static uint32_t first_max(const float* v, uint32_t n)
{
    uint32_t best = 0;
    for (uint32_t i = 1; i < n; ++i)
        if (v[best] < v[i])
            best = i;
    return best;
}

typedef struct {
    float* work;
    cand_t* cand;
    uint32_t n;
} dist_t;

/* Masked copy of the logits: the mask is this build's extension and is
 * defined as "-inf before the sampler sees the row". */
static float* masked_copy(const float* logits, uint32_t n_vocab, const uint32_t* mask)
{
    float* w = malloc(sizeof(float) * n_vocab);
    for (uint32_t i = 0; i < n_vocab; ++i)
        w[i] = (!mask || ((mask[i >> 5] >> (i & 31)) & 1u)) ? logits[i] : -INFINITY;
    return w;
}

/* Sampler::distribution, src/gen/sampler.cpp:20-62. */
static dist_t distribution(const float* logits, uint32_t n_vocab, const or_params* p, const int32_t* hist,
                           uint32_t n_hist, const uint32_t* mask, int order_mode)
{
    dist_t d;
    d.work = masked_copy(logits, n_vocab, mask);
    /* accept() history -> per-token counts (sampler.cpp:15-18); each distinct
     * token is penalised once with its count (sampler.cpp:23-28). */
    if (n_hist) {
        uint32_t* counts = calloc(n_vocab, sizeof(uint32_t));
        for (uint32_t h = 0; h < n_hist; ++h)
            if (hist[h] >= 0 && (uint32_t)hist[h] < n_vocab)
                ++counts[hist[h]];
        for (uint32_t h = 0; h < n_hist; ++h) {
            if (hist[h] < 0 || (uint32_t)hist[h] >= n_vocab)
                continue;
            const uint32_t n = counts[hist[h]];
            if (!n)
                continue;
            counts[hist[h]] = 0;
            float l = d.work[hist[h]];
            if (p->repetition_penalty != 1.0f)
                l = l > 0 ? l / p->repetition_penalty : l * p->repetition_penalty;
            const float fr = p->frequency_penalty * (float)n;
            const float dec = p->presence_penalty + fr;
            d.work[hist[h]] = l - dec;
        }
        free(counts);
    }
    const float inv_t = 1.0f / p->temperature;
    const float m = d.work[first_max(d.work, n_vocab)];
    const float floor_q = (1.0f < p->min_p) ? 1.0f : p->min_p; /* std::min(min_p, 1.0f) */
    d.cand = malloc(sizeof(cand_t) * (n_vocab + 1));
    d.n = 0;
    for (uint32_t i = 0; i < n_vocab; ++i) {
        const float diff = d.work[i] - m;
        const float q = or_expf(diff * inv_t);
        if (q >= floor_q && q > 0.0f) {
            d.cand[d.n].q = q;
            d.cand[d.n].idx = (int32_t)i;
            ++d.n;
        }
    }
    if (d.n == 0) {
        d.cand[0].q = 1.0f;
        d.cand[0].idx = (int32_t)first_max(d.work, n_vocab);
        d.n = 1;
    }
    if (p->top_k > 0 && p->top_k < d.n) {
        if (order_mode == 0)
            introselect(d.cand, 0, p->top_k, d.n);
        else
            qsort(d.cand, d.n, sizeof(cand_t), before_qsort);
        d.n = p->top_k;
    }
    if (p->top_p < 1.0f) {
        double total = 0;
        for (uint32_t i = 0; i < d.n; ++i)
            total += d.cand[i].q;
        const double want = p->top_p * total;
        /* The reference sorts a growing prefix (sampler.cpp:50-60); the prefix
         * it keeps is the shortest one of the fully sorted list whose running
         * fp64 sum reaches `want`, the whole list if none does, never empty. */
        qsort(d.cand, d.n, sizeof(cand_t), before_qsort);
        double sum = 0;
        uint32_t n = 0;
        while (n < d.n && sum < want)
            sum += d.cand[n++].q;
        d.n = n > 1 ? n : 1;
    }
    return d;
}

/* Sampler::draw, src/gen/sampler.cpp:64-73, with the uniform made explicit:
 * uniform_real_distribution<float>(0, total) is u * (total - 0) + 0. */
static uint32_t draw(const cand_t* c, uint32_t n, float total, float u)
{
    const float span = total - 0.0f;
    const float prod = u * span;
    float r = prod + 0.0f;
    for (uint32_t i = 0; i < n; ++i) {
        if (r < c[i].q)
            return i;
        r -= c[i].q;
    }
    return n - 1;
}

static void fill_trace(or_trace* t, const dist_t* d, float total, float q_chosen, float m)
{
    if (!t)
        return;
    t->n_cand = d ? d->n : 0;
    t->total = total;
    t->q_chosen = q_chosen;
    t->max_logit = m;
    if (d && t->cap && t->cand_idx && t->cand_q)
        for (uint32_t i = 0; i < d->n && i < t->cap; ++i) {
            t->cand_idx[i] = d->cand[i].idx;
            t->cand_q[i] = d->cand[i].q;
        }
}

static int32_t greedy_pick(const float* logits, uint32_t n_vocab, const uint32_t* mask)
{
    float* w = masked_copy(logits, n_vocab, mask);
    const int32_t t = (int32_t)first_max(w, n_vocab);
    free(w);
    return t;
}

/* Sampler::sample, src/gen/sampler.cpp:75-84. */
int32_t or_sample(const float* logits, uint32_t n_vocab, const or_params* p, const int32_t* hist, uint32_t n_hist,
                  const uint32_t* mask, float u, int order_mode, or_trace* trace)
{
    if (p->temperature <= 0.0f) {
        fill_trace(trace, 0, 0.0f, 0.0f, 0.0f);
        return greedy_pick(logits, n_vocab, mask);
    }
    dist_t d = distribution(logits, n_vocab, p, hist, n_hist, mask, order_mode);
    float total = 0;
    for (uint32_t i = 0; i < d.n; ++i)
        total += d.cand[i].q;
    const uint32_t pick = draw(d.cand, d.n, total, u);
    const int32_t token = d.cand[pick].idx;
    fill_trace(trace, &d, total, d.cand[pick].q, d.work[first_max(d.work, n_vocab)]);
    free(d.work);
    free(d.cand);
    return token;
}

/* Sampler::verify, src/gen/sampler.cpp:86-107. */
int32_t or_verify(const float* logits, uint32_t n_vocab, const or_params* p, const int32_t* hist, uint32_t n_hist,
                  const uint32_t* mask, int32_t draft, float u1, float u2, int order_mode, int* accepted,
                  or_trace* trace)
{
    if (p->temperature <= 0.0f) {
        const int32_t t = greedy_pick(logits, n_vocab, mask);
        *accepted = t == draft;
        fill_trace(trace, 0, 0.0f, 0.0f, 0.0f);
        return t;
    }
    dist_t d = distribution(logits, n_vocab, p, hist, n_hist, mask, order_mode);
    float total = 0, q_draft = 0;
    for (uint32_t i = 0; i < d.n; ++i) {
        total += d.cand[i].q;
        if (d.cand[i].idx == draft)
            q_draft = d.cand[i].q;
    }
    const float m = d.work[first_max(d.work, n_vocab)];
    const float span = total - 0.0f;
    const float prod = u1 * span;
    const float r1 = prod + 0.0f;
    int32_t token = draft;
    float q_out = q_draft;
    *accepted = r1 < q_draft;
    if (!*accepted) {
        uint32_t n = 0;
        for (uint32_t i = 0; i < d.n; ++i)
            if (d.cand[i].idx != draft)
                d.cand[n++] = d.cand[i];
        if (n) {
            d.n = n;
            const uint32_t pick = draw(d.cand, d.n, total - q_draft, u2);
            token = d.cand[pick].idx;
            q_out = d.cand[pick].q;
        }
    }
    fill_trace(trace, &d, total, q_out, m);
    free(d.work);
    free(d.cand);
    return token;
}

/* src/server/openai.cpp:589-604, the part that looks at the logits. */
int32_t or_close_forced(const float* logits, uint32_t n_vocab, const uint32_t* mask, int32_t think_end,
                        uint32_t max_above, uint32_t* above)
{
    if (above)
        *above = 0xffffffffu;
    if (think_end < 0 || (uint32_t)think_end >= n_vocab) /* :590, :594 */
        return -1;
    if (mask && !((mask[(uint32_t)think_end >> 5] >> ((uint32_t)think_end & 31u)) & 1u))
        return -1;
    const float v = logits[think_end]; /* :596 */
    uint32_t n = 0;
    for (uint32_t i = 0; i < n_vocab; ++i) { /* :598-600 */
        const int allowed = !mask || ((mask[i >> 5] >> (i & 31u)) & 1u);
        const float w = allowed ? logits[i] : -INFINITY;
        if (w > v)
            ++n;
    }
    if (above)
        *above = n;
    return n >= max_above ? -1 : think_end; /* :600, :602-603 */
}
