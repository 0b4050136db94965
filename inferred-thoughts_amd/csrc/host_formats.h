// Host-side block formats: what the loader and the synthetic writer need on the CPU
// (embedding-row and small-vector dequantization, Q8_0 quantization of generated
// weights).  Restates /root/reference src/quant/half.rs:29-114 and
// src/quant/mod.rs:96-106, 265-357; the Q8_0 quantizer is ggml's
// quantize_row_q8_0_ref as the reference restates it (src/ops/naive.rs:652-675).
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

namespace ith {

inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

inline float half_to_float(uint16_t h) {
    uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 31, m = h & 1023;
    if (e == 31) return bits_f32(s | 0x7f800000u | (m << 13));
    if (e == 0) {
        float v = std::ldexp((float)m, -24);
        return (h >> 15) ? -v : v;
    }
    return bits_f32(s | ((e + 112) << 23) | (m << 13));
}

inline uint16_t float_to_half(float f) {  // round to nearest even
    uint32_t b = f32_bits(f);
    uint16_t s = (uint16_t)((b >> 16) & 0x8000);
    int32_t ex = (int32_t)((b >> 23) & 255);
    uint32_t man = b & 0x7fffff;
    if (ex == 255) return (uint16_t)(s | 0x7c00 | (man ? 0x200 : 0));
    int32_t e = ex - 112;
    if (e >= 31) return (uint16_t)(s | 0x7c00);
    if (e <= 0) {
        if (e < -10) return s;
        uint32_t m = man | 0x800000, sh = (uint32_t)(14 - e);
        uint32_t q = m >> sh, rem = m & ((1u << sh) - 1), mid = 1u << (sh - 1);
        if (rem > mid || (rem == mid && (q & 1))) q++;
        return (uint16_t)(s | q);
    }
    uint32_t q = ((uint32_t)e << 10) | (man >> 13), rem = man & 0x1fff;
    if (rem > 0x1000 || (rem == 0x1000 && (q & 1))) q++;
    return (uint16_t)(s | q);
}

static const int8_t KVALUES[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

inline float ue4m3_half(uint8_t x) {  // E4M3 magnitude, halved
    if (x == 0 || x == 0x7f) return 0.0f;
    int e = (x >> 3) & 15;
    float m = (float)(x & 7);
    float raw = e == 0 ? std::ldexp(m, -9) : std::ldexp(1.0f + m / 8.0f, e - 7);
    return raw * 0.5f;
}

// nearest UE4M3 code (1..0x7e) to a positive value, ties to the even code
inline uint8_t ue4m3_encode(float v) {
    if (!(v > 0.0f)) return 0;
    uint8_t best = 1;
    double bd = 1e300;
    for (int c = 1; c <= 0x7e; c++) {
        double d = std::fabs(2.0 * (double)ue4m3_half((uint8_t)c) - (double)v);
        if (d < bd || (d == bd && (c & 1) == 0 && (best & 1))) {
            bd = d;
            best = (uint8_t)c;
        }
    }
    return best;
}

inline bool dequantize(uint32_t ty, const uint8_t* data, uint64_t n, float* out) {
    switch (ty) {
        case 0: memcpy(out, data, n * 4); return true;
        case 1:
            for (uint64_t i = 0; i < n; i++) { uint16_t h; memcpy(&h, data + 2 * i, 2); out[i] = half_to_float(h); }
            return true;
        case 30:
            for (uint64_t i = 0; i < n; i++) { uint16_t h; memcpy(&h, data + 2 * i, 2); out[i] = bits_f32((uint32_t)h << 16); }
            return true;
        case 8:
            if (n % 32) return false;
            for (uint64_t b = 0; b < n / 32; b++) {
                uint16_t h; memcpy(&h, data + b * 34, 2);
                float d = half_to_float(h);
                for (int i = 0; i < 32; i++) out[b * 32 + i] = (float)(int8_t)data[b * 34 + 2 + i] * d;
            }
            return true;
        case 40:
            if (n % 64) return false;
            for (uint64_t b = 0; b < n / 64; b++) {
                const uint8_t* blk = data + b * 36;
                for (int s = 0; s < 4; s++) {
                    float d = ue4m3_half(blk[s]);
                    for (int j = 0; j < 8; j++) {
                        uint8_t q = blk[4 + s * 8 + j];
                        out[b * 64 + s * 16 + j] = (float)KVALUES[q & 15] * d;
                        out[b * 64 + s * 16 + j + 8] = (float)KVALUES[q >> 4] * d;
                    }
                }
            }
            return true;
        default: return false;
    }
}

// 32 floats -> one 34-byte Q8_0 block
inline void quantize_block_q8_0(const float* x, uint8_t* out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) amax = std::fmax(amax, std::fabs(x[i]));
    float d = amax / 127.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    uint16_t h = float_to_half(d);
    memcpy(out, &h, 2);
    for (int i = 0; i < 32; i++) {
        float r = std::round(x[i] * id);
        if (r > 127.f) r = 127.f;
        if (r < -128.f) r = -128.f;
        out[2 + i] = (uint8_t)(int8_t)r;
    }
}

}  // namespace ith
