// Device arithmetic that must match the host toolchain bit for bit.
// Compiled with -ffp-contract=off, IEEE fp32 division and subnormals enabled:
// every operator below rounds once, and only the explicit fma() calls fuse.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mako {

// 2^(i/32) table of glibc 2.35 (sysdeps/ieee754/flt-32/e_exp2f_data.c):
// bits(2^(i/32)) - (i << 47).
__device__ const uint64_t k_exp2_tab[32] = {
    0x3ff0000000000000, 0x3fefd9b0d3158574, 0x3fefb5586cf9890f, 0x3fef9301d0125b51,
    0x3fef72b83c7d517b, 0x3fef54873168b9aa, 0x3fef387a6e756238, 0x3fef1e9df51fdee1,
    0x3fef06fe0a31b715, 0x3feef1a7373aa9cb, 0x3feedea64c123422, 0x3feece086061892d,
    0x3feebfdad5362a27, 0x3feeb42b569d4f82, 0x3feeab07dd485429, 0x3feea47eb03a5585,
    0x3feea09e667f3bcd, 0x3fee9f75e8ec5f74, 0x3feea11473eb0187, 0x3feea589994cce13,
    0x3feeace5422aa0db, 0x3feeb737b0cdc5e5, 0x3feec49182a3f090, 0x3feed503b23e255d,
    0x3feee89f995ad3ad, 0x3feeff76f2fb5e47, 0x3fef199bdd85529c, 0x3fef3720dcef9069,
    0x3fef5818dcfba487, 0x3fef7c97337b9b5f, 0x3fefa4afa2a490da, 0x3fefd0765b6e4540,
};

// expf of glibc 2.35 as built for x86-64 with FMA, which is what std::exp(float)
// (src/gen/sampler.cpp:33) resolves to on the host: fp64 range reduction with a
// 32-entry table and a cubic, both multiply-adds of the reduction fused.
// `tab` points at k_exp2_tab or a copy of it in LDS.
__device__ __forceinline__ float expf_glibc(float x, const uint64_t* tab)
{
    const uint32_t ix = __float_as_uint(x);
    const uint32_t abstop = (ix >> 20) & 0x7ffu;
    if (abstop >= 0x42bu) { // |x| >= 88 or non-finite
        if (ix == 0xff800000u)
            return 0.0f;
        if (abstop >= 0x7f8u)
            return x + x;
        if (x > 0x1.62e42ep6f)
            return __uint_as_float(0x7f800000u);
        if (x < -0x1.9fe368p6f)
            return 0.0f;
        if (x < -0x1.9d1d9ep6f)
            return __uint_as_float(1u);
    }
    const double inv_ln2_n = 0x1.71547652b82fep+0 * 32.0;
    const double shift = 0x1.8p+52;
    const double c0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32;
    const double c1 = 0x1.ebfce50fac4f3p-3 / 32 / 32;
    const double c2 = 0x1.62e42ff0c52d6p-1 / 32;
    const double xd = (double)x;
    double kd = fma(inv_ln2_n, xd, shift);
    const uint64_t ki = (uint64_t)__double_as_longlong(kd);
    kd -= shift;
    const double r = fma(inv_ln2_n, xd, -kd);
    const double s = __longlong_as_double((long long)(tab[ki & 31] + (ki << 47)));
    const double z = fma(c0, r, c1);
    const double r2 = r * r;
    double y = fma(c2, r, 1.0);
    y = fma(z, r2, y);
    return (float)(y * s);
}

// The three penalties of src/gen/sampler.cpp:25-27 for a token seen n times.
__device__ __forceinline__ float penalize(float l, uint32_t n, float rep, float presence, float frequency)
{
    if (rep != 1.0f)
        l = l > 0.0f ? l / rep : l * rep;
    const float fr = frequency * (float)n;
    const float dec = presence + fr;
    return l - dec;
}

// q = exp((w - m) * inv_t), src/gen/sampler.cpp:33: subtract, multiply, expf.
__device__ __forceinline__ float weight_of(float w, float m, float inv_t, const uint64_t* tab)
{
    const float diff = w - m;
    const float x = diff * inv_t;
    return expf_glibc(x, tab);
}

} // namespace mako
