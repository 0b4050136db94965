// TEST INFRASTRUCTURE — not part of the shipped library.
//
// Scalar formats and the two transcendental functions the per-token loop needs,
// restated for the CPU oracle.  Every function is plain IEEE arithmetic with no
// fused multiply-add (compile with -ffp-contract=off), so the HIP kernels can
// run the same sequence of operations and land on the same bits.
//
// Follows /root/reference:
//   src/quant/half.rs:29-63    f16_to_f32, bf16_to_f32
//   src/quant/half.rs:70-114   f32_to_f16 (round to nearest even)
//   src/quant/mod.rs:265       KVALUES_MXFP4
//   src/quant/mod.rs:271-284   ue4m3_to_f32
//
// expf/logf: the reference calls Rust's f32::exp / f32::ln, which forward to the
// platform libm.  That last bit is platform-dependent ("parity unpinned" for the
// final ulp), so the oracle fixes one definition: the table-driven double
// precision algorithm published with glibc >= 2.27 (sysdeps/ieee754/flt-32/
// e_expf.c, e_logf.c; ARM optimized-routines math/expf.c, logf.c), evaluated
// without contraction.  tests/test_oracle_golden.py (test_expf_logf_against_libm_and_float64)
// measures how often it differs from this machine's libm.
#pragma once
#include <stdint.h>
#include <string.h>

static inline uint32_t orc_f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float orc_bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint64_t orc_f64_bits(double f) { uint64_t u; memcpy(&u, &f, 8); return u; }
static inline double orc_bits_f64(uint64_t u) { double f; memcpy(&f, &u, 8); return f; }

// src/quant/half.rs:29-59 — exact widening, subnormals renormalised.
static inline float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    if (exp == 0x1f) return orc_bits_f32(sign | 0x7f800000u | (man << 13));
    if (exp == 0) {
        if (man == 0) return orc_bits_f32(sign);
        // value = man * 2^-24, exact in f32
        float v = (float)man * 5.9604644775390625e-08f;
        return orc_bits_f32(orc_f32_bits(v) | sign);
    }
    return orc_bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline float orc_bf16_to_f32(uint16_t h) { return orc_bits_f32((uint32_t)h << 16); }

// src/quant/half.rs:70-114 — round to nearest even, overflow to infinity.
static inline uint16_t orc_f32_to_f16(float f) {
    uint32_t bits = orc_f32_bits(f);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    int32_t exp = (int32_t)((bits >> 23) & 0xff);
    uint32_t mant = bits & 0x007fffffu;
    if (exp == 0xff) return (uint16_t)(sign | 0x7c00u | (mant != 0 ? 0x0200u : 0u));
    int32_t e = exp - 127 + 15;
    if (e >= 0x1f) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return sign;
        uint32_t m = mant | 0x00800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half & 1u))) half += 1;
        return (uint16_t)(sign | half);
    }
    uint32_t h = ((uint32_t)e << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h += 1;
    return (uint16_t)(sign | h);
}

// src/quant/mod.rs:265 — E2M1 values doubled, sign in bit 3.
static const int8_t ORC_KVALUES_MXFP4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

// src/quant/mod.rs:271-284 — unsigned E4M3, bias 7, halved; 0 and 0x7f read as 0;
// bit 7 is not examined.
static inline float orc_ue4m3_to_f32(uint8_t x) {
    if (x == 0 || x == 0x7f) return 0.0f;
    int exp = (x >> 3) & 0xf;
    float man = (float)(x & 7);
    float raw;
    if (exp == 0) {
        raw = man * 0.001953125f;  // 2^-9
    } else {
        // 2^(exp-7) built from bits: exact
        float p = orc_bits_f32((uint32_t)(exp - 7 + 127) << 23);
        raw = (1.0f + man / 8.0f) * p;
    }
    return raw * 0.5f;
}

// ---------------------------------------------------------------- expf
static const uint64_t ORC_EXP2F_TAB[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

static inline float orc_expf(float x) {
    const double InvLn2N = 0x1.71547652b82fep+0 * 32.0;
    const double Shift = 0x1.8p52;
    const double C0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    uint32_t ux = orc_f32_bits(x);
    uint32_t abstop = (ux >> 20) & 0x7ff;
    if (abstop >= 0x42b) {  // |x| >= 88.0 or not finite
        if (ux == 0xff800000u) return 0.0f;
        if (abstop >= 0x7f8) return x + x;
        if (x > 0x1.62e42ep6f) return orc_bits_f32(0x7f800000u);
        if (x < -0x1.9fe368p6f) return 0.0f;
    }
    double xd = (double)x;
    double z = InvLn2N * xd;
    double kd = z + Shift;
    uint64_t ki = orc_f64_bits(kd);
    kd -= Shift;
    double r = z - kd;
    uint64_t t = ORC_EXP2F_TAB[ki % 32];
    t += ki << (52 - 5);
    double s = orc_bits_f64(t);
    z = C0 * r + C1;
    double r2 = r * r;
    double y = C2 * r + 1.0;
    y = z * r2 + y;
    y = y * s;
    return (float)y;
}

// ---------------------------------------------------------------- logf
static const double ORC_LOGF_TAB[16][2] = {
    {0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2}, {0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2},
    {0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2},  {0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3},
    {0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3}, {0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3},
    {0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4}, {0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4},
    {0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5}, {0x1p+0, 0x0p+0},
    {0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5},  {0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4},
    {0x1.b2036576afce6p-1, 0x1.526e57720db08p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3},
    {0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2},  {0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2},
};

static inline float orc_logf(float x) {
    const double A0 = -0x1.00ea348b88334p-2, A1 = 0x1.5575b0be00b6ap-2, A2 = -0x1.ffffef20a4123p-2;
    const double Ln2 = 0x1.62e42fefa39efp-1;
    uint32_t ix = orc_f32_bits(x);
    if (ix == 0x3f800000u) return 0.0f;
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {
        if (ix * 2 == 0) return orc_bits_f32(0xff800000u);
        if (ix == 0x7f800000u) return x;
        if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return orc_bits_f32(0x7fc00000u);
        ix = orc_f32_bits(x * 0x1p23f);
        ix -= 23u << 23;
    }
    uint32_t tmp = ix - 0x3f330000u;
    int i = (tmp >> (23 - 4)) % 16;
    int32_t k = (int32_t)tmp >> 23;
    uint32_t iz = ix - (tmp & (0x1ffu << 23));
    double invc = ORC_LOGF_TAB[i][0], logc = ORC_LOGF_TAB[i][1];
    double z = (double)orc_bits_f32(iz);
    double r = z * invc - 1.0;
    double y0 = logc + (double)k * Ln2;
    double r2 = r * r;
    double y = A1 * r + A2;
    y = A0 * r2 + y;
    y = y * r2 + (y0 + r);
    return (float)y;
}
