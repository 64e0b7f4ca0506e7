/* Exhaustive pin of the oracle's restated expf: every one of the 2^32 float inputs against this host's libm,
 * and monotonicity over all negative floats (the candidate-coverage certificates of the kernels rely on it). */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

float or_expf(float);

static inline float asfloat(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t asuint(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

typedef struct { uint64_t lo, hi, mism, nonmono; } job_t;

static void* run(void* p)
{
    job_t* j = p;
    float prev = 0;
    int have_prev = 0;
    for (uint64_t u = j->lo; u < j->hi; ++u) {
        const float x = asfloat((uint32_t)u), a = or_expf(x), b = expf(x);
        if (asuint(a) != asuint(b) && !(a != a && b != b))
            ++j->mism;
        /* bit patterns 0x80000000..0xff800000 run from -0 down to -inf */
        if (u >= 0x80000000ull && u <= 0xff800000ull) {
            if (have_prev && a > prev)
                ++j->nonmono;
            prev = a;
            have_prev = 1;
        }
    }
    return 0;
}

int main(void)
{
    enum { NT = 8 };
    pthread_t th[NT];
    job_t jobs[NT];
    const uint64_t per = (1ull << 32) / NT;
    for (int i = 0; i < NT; ++i) {
        /* chunks overlap by one value so the monotonicity check has no seams */
        jobs[i] = (job_t){i ? i * per - 1 : 0, (i + 1) * per, 0, 0};
        pthread_create(&th[i], 0, run, &jobs[i]);
    }
    uint64_t mism = 0, nonmono = 0;
    for (int i = 0; i < NT; ++i) {
        pthread_join(th[i], 0);
        mism += jobs[i].mism;
        nonmono += jobs[i].nonmono;
    }
    printf("mismatches %lu non-monotone %lu\n", (unsigned long)mism, (unsigned long)nonmono);
    return mism || nonmono;
}
