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
