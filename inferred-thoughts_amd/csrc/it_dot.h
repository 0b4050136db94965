// Per-block integer dots shared by the GEMV kernels and the fused decode kernels.
#pragma once
#include "it_device.h"

namespace itk {

// ------------------------------------------------------------------ E2M1 nibbles -> int8
// kvalues (doubled E2M1, /root/reference src/quant/mod.rs:265) through two byte
// permutes: magnitude by the low 3 bits, then the sign bit picks +mag or -mag.
IT_DEV uint32_t fp4x4_to_i8x4(uint32_t v) {  // v: four nibbles, one per byte
    const uint32_t TPlo = 0x03020100u, TPhi = 0x0c080604u;
    const uint32_t TNlo = 0xfdfeff00u, TNhi = 0xf4f8fafcu;
    uint32_t idx = v & 0x07070707u;
    uint32_t mag = __builtin_amdgcn_perm(TPhi, TPlo, idx);
    uint32_t neg = __builtin_amdgcn_perm(TNhi, TNlo, idx);
    uint32_t sel = ((v >> 1) & 0x04040404u) | 0x03020100u;
    return __builtin_amdgcn_perm(neg, mag, sel);
}

IT_DEV int dot4(uint32_t a, uint32_t b, int c) { return __builtin_amdgcn_sdot4((int)a, (int)b, c, false); }

// One 32-element unit of a Q8_0 row against activation block `a` (8 dwords).
IT_DEV float unit_q8_0(const uint4 w0, const uint4 w1, uint16_t dw_bits, const uint4 a0, const uint4 a1,
                       float dx) {
    int s = 0;
    s = dot4(w0.x, a0.x, s); s = dot4(w0.y, a0.y, s); s = dot4(w0.z, a0.z, s); s = dot4(w0.w, a0.w, s);
    s = dot4(w1.x, a1.x, s); s = dot4(w1.y, a1.y, s); s = dot4(w1.z, a1.z, s); s = dot4(w1.w, a1.w, s);
    float dw = it_f16_to_f32(dw_bits);
    return (float)s * (dw * dx);
}

// One 32-element unit (two 16-element sub-blocks) of an NVFP4 row.
IT_DEV void unit_nvfp4(const uint4 w, uint32_t sc2, const uint4 a0, const uint4 a1, float dy, float* tA,
                       float* tB) {
    int sa = 0, sb = 0;
    sa = dot4(fp4x4_to_i8x4(w.x & 0x0f0f0f0fu), a0.x, sa);
    sa = dot4(fp4x4_to_i8x4(w.y & 0x0f0f0f0fu), a0.y, sa);
    sa = dot4(fp4x4_to_i8x4((w.x >> 4) & 0x0f0f0f0fu), a0.z, sa);
    sa = dot4(fp4x4_to_i8x4((w.y >> 4) & 0x0f0f0f0fu), a0.w, sa);
    sb = dot4(fp4x4_to_i8x4(w.z & 0x0f0f0f0fu), a1.x, sb);
    sb = dot4(fp4x4_to_i8x4(w.w & 0x0f0f0f0fu), a1.y, sb);
    sb = dot4(fp4x4_to_i8x4((w.z >> 4) & 0x0f0f0f0fu), a1.z, sb);
    sb = dot4(fp4x4_to_i8x4((w.w >> 4) & 0x0f0f0f0fu), a1.w, sb);
    float dA = it_ue4m3_to_f32(sc2 & 0xffu), dB = it_ue4m3_to_f32((sc2 >> 8) & 0xffu);
    *tA = (dy * dA) * (float)sa;
    *tB = (dy * dB) * (float)sb;
}

// ------------------------------------------------------------------ E2M1 nibbles -> f16
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
// four nibbles (one per byte, 0..15) -> four f16 weights (two dwords), scaled by the sub-block scale
IT_DEV void fp4x4_to_f16x4(uint32_t v, h2 scale, h2* a, h2* b) {
    // f16 high bytes of 128 x the doubled e2m1 magnitudes 0 1 2 3 4 6 8 12 (the low bytes are zero): the 128 pays
    // for the 2^-8 the scale carries (see expand) and the halving that goes with the doubled magnitudes
    const uint32_t mag = __builtin_amdgcn_perm(0x66646260u, 0x5e5c5800u, v & 0x07070707u);
    const uint32_t hb = mag | ((v & 0x08080808u) << 4);
    const uint32_t d0 = __builtin_amdgcn_perm(hb, hb, 0x010c000cu);   // bytes 0, hb.0, 0, hb.1
    const uint32_t d1 = __builtin_amdgcn_perm(hb, hb, 0x030c020cu);   // bytes 0, hb.2, 0, hb.3
    *a = __builtin_bit_cast(h2, d0) * scale;
    *b = __builtin_bit_cast(h2, d1) * scale;
}


// operands of the f16 expert tile kernels (k_gemm_f16.hip, k_gemm_f16s.hip)
struct ExpertsF16P {
    const uint8_t *q, *s, *q2, *s2;
    const uint8_t* const *q_tab, *const *s_tab, *const *q2_tab, *const *s2_tab;  // expert placement tables or null
    int64_t q_stride, s_stride;
    const float *scale2, *scale2_up;
    const uint16_t *xh, *xl;
    const float* rscale;
    float* out;
    int n_in, n_out, x_mode, n_used;
    const int32_t* n_tiles;
    const int4* tiles;
    const int32_t* order;
};

// Serial ascending fold of T per-block terms from a 16-byte aligned LDS row: the loads are
// issued four float4 at a time so the chain of adds never waits on LDS latency.
IT_DEV float fold_terms(const float* tr, int T) {
    float acc = 0.0f;
    int k = 0;
    const float4* t4 = (const float4*)tr;
    for (; k + 16 <= T; k += 16) {
        float4 a = t4[k / 4], b = t4[k / 4 + 1], c = t4[k / 4 + 2], d = t4[k / 4 + 3];
        acc += a.x; acc += a.y; acc += a.z; acc += a.w;
        acc += b.x; acc += b.y; acc += b.z; acc += b.w;
        acc += c.x; acc += c.y; acc += c.z; acc += c.w;
        acc += d.x; acc += d.y; acc += d.z; acc += d.w;
    }
    for (; k < T; k++) acc += tr[k];
    return acc;
}

}  // namespace itk
