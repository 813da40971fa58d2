// Scalar numerics shared by every kernel of the MoE FFN path: a bit-exact float exp, the sigmoid / clamped
// SwiGLU built on it, and the MXFP4 / e4m3 / e8m0 format primitives.  Plain C++ so the same text compiles for
// the device (hipcc) and for a host-side unit test (g++ -ffp-contract=off).
//
// Routing must reproduce the reference's CPU results bit for bit (crates/ferrite-kernel/src/cpu.rs:528-572:
// 1/(1+exp(-l)) with the platform libm's expf, then comparisons on sigmoid+bias).  The reference's libm on
// Linux is glibc, whose expf is the table-plus-cubic algorithm evaluated in double and rounded once to float;
// fe_expf restates that algorithm with every operation an individually rounded IEEE double operation, so the
// device result is the same float.
#pragma once
#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__) || defined(__HIP__)
#define FE_HD __host__ __device__ __forceinline__
#else
#define FE_HD inline
#endif

namespace fe {

FE_HD uint32_t f2u(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
FE_HD float u2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
FE_HD uint64_t d2u(double d) {
    uint64_t u;
    memcpy(&u, &d, 8);
    return u;
}
FE_HD double u2d(uint64_t u) {
    double d;
    memcpy(&d, &u, 8);
    return d;
}

// 2^(i/32) as doubles with i<<47 subtracted from the bit pattern (so adding k<<47 applies the exponent).
#if defined(__HIP_DEVICE_COMPILE__)
__device__ __constant__
#endif
static const uint64_t kExp2Tab[32] = {
    0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
    0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
    0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
    0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
    0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
    0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
    0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
    0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL};

// Individually rounded double ops (no fused multiply-add, whatever the contraction setting).
#if defined(__HIP_DEVICE_COMPILE__)
FE_HD double dmul(double a, double b) { return __dmul_rn(a, b); }
FE_HD double dadd(double a, double b) { return __dadd_rn(a, b); }
FE_HD float fmul(float a, float b) { return __fmul_rn(a, b); }
FE_HD float fadd(float a, float b) { return __fadd_rn(a, b); }
FE_HD float fdiv(float a, float b) { return __fdiv_rn(a, b); }
FE_HD float fsqrt(float a) { return __ocml_sqrt_f32(a); }   // correctly rounded (__fsqrt_rn is the native approximation)
#else
FE_HD double dmul(double a, double b) { volatile double r = a * b; return r; }
FE_HD double dadd(double a, double b) { volatile double r = a + b; return r; }
FE_HD float fmul(float a, float b) { volatile float r = a * b; return r; }
FE_HD float fadd(float a, float b) { volatile float r = a + b; return r; }
FE_HD float fdiv(float a, float b) { volatile float r = a / b; return r; }
FE_HD float fsqrt(float a) { volatile float r = sqrtf(a); return r; }
#endif

// float exp, bit-identical to glibc >= 2.27 expf on x86-64 for finite results.
FE_HD float fe_expf(float x) {
    const double InvLn2N = 0x1.71547652b82fep+0 * 32.0;
    const double Shift = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    uint32_t abstop = (f2u(x) >> 20) & 0x7ff;
    if (abstop >= 0x42b) {  // |x| >= 88 or NaN
        if (f2u(x) == 0xff800000u) return 0.0f;              // -inf
        if (abstop >= 0x7f8) return x + x;                   // +inf, NaN
        if (x > 0x1.62e42ep6f) return u2f(0x7f800000u);      // overflow
        if (x < -0x1.9fe368p6f) return 0.0f;                 // underflow to zero
    }
    double xd = (double)x;
    double z = dmul(InvLn2N, xd);
    double kd = dadd(z, Shift);
    uint64_t ki = d2u(kd);
    kd = dadd(kd, -Shift);
    double r = dadd(z, -kd);
    uint64_t t = kExp2Tab[ki & 31];
    t += ki << (52 - 5);
    double s = u2d(t);
    z = dadd(dmul(C0, r), C1);
    double r2 = dmul(r, r);
    double y = dadd(dmul(C2, r), 1.0);
    y = dadd(dmul(z, r2), y);
    y = dmul(y, s);
    return (float)y;
}

// crates/ferrite-kernel/src/cpu.rs:552: 1.0 / (1.0 + (-l).exp())
FE_HD float sigmoid_ref(float l) { return fdiv(1.0f, fadd(1.0f, fe_expf(-l))); }

// crates/ferrite-kernel/src/cpu.rs:192-201: gate clamped from above only, up clamped both sides
FE_HD float swiglu_ref(float g, float u, float limit) {
    float gi = g > limit ? limit : g;
    float ui = u < -limit ? -limit : (u > limit ? limit : u);
    float silu = fdiv(gi, fadd(1.0f, fe_expf(-gi)));
    return fmul(silu, ui);
}

// ---- formats (crates/ferrite-models/src/dsv41/quant.rs) ----

// quant.rs:22-25 e2m1 value of a 4-bit code: {0,.5,1,1.5,2,3,4,6} with bit 3 the sign (code 8 decodes to 0.0)
FE_HD float e2m1_decode(uint32_t code) {
    uint32_t m = code & 7u;
    // magnitudes as f32 bit patterns: 0, 0.5, 1, 1.5, 2, 3, 4, 6
    uint32_t bits = m == 0 ? 0u : (m == 1 ? 0x3f000000u : (0x3f800000u + ((m - 2u) << 22)));
    float v = u2f(bits);
    return (code & 8u) ? (m == 0 ? 0.0f : -v) : v;
}

// quant.rs:130-136 with the reference's clamp: byte 0 decodes to 0.0, 0xFF to NaN, else 2^(b-127)
FE_HD float ue8m0_decode(uint32_t b) {
    if (b == 0xFFu) return u2f(0x7fc00000u);
    return u2f(b << 23);
}

// quant.rs:84-93
FE_HD float e4m3_decode(uint32_t b) {
    uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
    float mag = e == 0 ? (float)m * (1.0f / 512.0f) : u2f(((e + 120u) << 23) | (m << 20));
    return (b & 0x80u) ? -mag : mag;
}

// quant.rs:155-165,190-198: 2^ceil(log2(amax/448)) floored at the smallest normal; returns the e8m0 byte
FE_HD uint32_t block_scale_e8m0(float amax) {
    float q = fdiv(amax, 448.0f);
    uint32_t bits = f2u(q);
    int ex = (int)((bits >> 23) & 0xFFu);
    int e = ex - 127 + ((bits & 0x7FFFFFu) ? 1 : 0);
    int biased = e + 127;           // fast_pow2 bit pattern (biased << 23); 0 -> 0.0 -> floored to 2^-126
    return (uint32_t)(biased < 1 ? 1 : biased);
}

// quant.rs:98-124, including its subnormal rule: round(a*512) clamped to 7 (so [7.5/512, 8/512) encodes as 7)
FE_HD uint32_t e4m3_encode(float x) {
    uint32_t xb = f2u(x);
    uint32_t sign = (xb >> 24) & 0x80u;
    uint32_t ab = xb & 0x7fffffffu;
    if (ab >= 0x7f800000u) return sign | 0x7Eu;  // non-finite saturates
    if (ab > 0x43e00000u) ab = 0x43e00000u;      // min(|x|, 448)
    if (ab == 0) return sign;
    if (ab < 0x3c800000u) {                      // < 2^-6: subnormal, step 2^-9
        float m = u2f(ab) * 512.0f;              // exact
        // round to nearest even via the 2^23 trick (0 <= m < 8)
        float r = (m + 8388608.0f) - 8388608.0f;
        uint32_t mi = (uint32_t)r;
        return sign | (mi > 7u ? 7u : mi);
    }
    // normal: keep 3 mantissa bits, round to nearest even on the 20 dropped bits
    uint32_t e = ab >> 23;                       // biased f32 exponent, >= 121
    uint32_t man = ab & 0x7fffffu;
    uint32_t keep = man >> 20;
    uint32_t rest = man & 0xfffffu;
    if (rest > 0x80000u || (rest == 0x80000u && (keep & 1u))) ++keep;
    if (keep == 8u) { keep = 0; ++e; }
    if (e > 135u) return sign | 0x7Eu;           // above 2^8 * 1.75: unreachable after the min, kept for safety
    return sign | ((e - 120u) << 3) | keep;
}

}  // namespace fe
