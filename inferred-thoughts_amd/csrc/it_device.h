// Device-side scalar helpers shared by every kernel: half/bf16/UE4M3 decodes and
// the two transcendentals in "exact" form.
//
// The exact expf/logf evaluate the same double-precision table algorithm as the
// CPU reference path's libm (glibc >= 2.27 e_expf.c / e_logf.c), as plain IEEE
// operations with contraction off, so a device result is the host result bit for
// bit.  The reference treats device expf as a +-1 ulp class
// (/root/reference src/ops/cuda/ops/mod.rs:18-21); matching it exactly is what
// lets greedy token ids be identical on the small config.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#define IT_DEV __device__ __forceinline__

// the expert cache's device-side read counters: one token's picks on the three tensors of a routed FFN
IT_DEV void it_count_expert_reads(const int32_t* ids, int n_used, uint32_t* cg, uint32_t* cu, uint32_t* cd,
                                  unsigned long long* tally) {
    if (blockIdx.x != 0 || !tally) return;   // a grid row is a token (or, in the order-preserving kernels, never more than one)
    const int t = threadIdx.x;
    if (t < n_used) {
        const int e = ids[t];
        if (cg) atomicAdd(cg + e, 1u);
        if (cu) atomicAdd(cu + e, 1u);
        if (cd) atomicAdd(cd + e, 1u);
    }
    if (t == 0) atomicAdd(tally, (unsigned long long)((cg ? 1 : 0) + (cu ? 1 : 0) + (cd ? 1 : 0)) * n_used);
}

// Expert e's bytes: through the placement table when the pool has one, else at its stride from the tensor's base.  A
// pointer read from the table is device-visible memory (a device slot or mapped pinned host memory), never LDS or
// scratch: saying so keeps the loads through it global loads, whose completion the hardware counts in order (behind a
// generic pointer every load becomes a flat load, and a wait for one of those waits for all of them).
typedef __attribute__((address_space(1))) const uint8_t* it_global_bytes;
IT_DEV const uint8_t* it_expert_at(const uint8_t* base, const uint8_t* const* tab, int64_t e, int64_t stride) {
    // (the table is read as an array of global pointers: a generic -> global -> generic round trip of the loaded
    // value would be folded away again)
    if (tab) return (const uint8_t*)((const it_global_bytes*)tab)[e];
    return base + e * stride;
}

IT_DEV float it_f16_to_f32(uint16_t h) { return __half2float(__ushort_as_half(h)); }
IT_DEV uint16_t it_f32_to_f16(float f) { return __half_as_ushort(__float2half_rn(f)); }
IT_DEV float it_bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// /root/reference src/quant/mod.rs:271-284: unsigned E4M3, bias 7, halved.
IT_DEV float it_ue4m3_to_f32(uint32_t x) {
    x &= 0xffu;
    const uint32_t em = x & 0x7fu;
    // normal: (1 + man/8) * 2^(exp-7) / 2 = exponent field exp + 119 with man in the top mantissa bits;
    // subnormal (exp == 0): man * 2^-9 / 2.  Both are exact in f32, so this is the value the
    // reference's arithmetic gives, without its branches.
    const float normal = __uint_as_float((em << 20) + (119u << 23));
    const float sub = (float)(em & 7u) * 0.0009765625f;
    const float r = (em >> 3) ? normal : sub;
    return x == 0x7fu ? 0.0f : r;
}

__device__ __constant__ const uint64_t IT_EXP2F_TAB[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull,
};

IT_DEV float it_expf(float x) {
    const double InvLn2N = 0x1.71547652b82fep+0 * 32.0;
    const double Shift = 0x1.8p52;
    const double C0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    uint32_t ux = __float_as_uint(x);
    uint32_t abstop = (ux >> 20) & 0x7ff;
    if (abstop >= 0x42b) {
        if (ux == 0xff800000u) return 0.0f;
        if (abstop >= 0x7f8) return x + x;
        if (x > 0x1.62e42ep6f) return __uint_as_float(0x7f800000u);
        if (x < -0x1.9fe368p6f) return 0.0f;
    }
    double xd = (double)x;
    double z = InvLn2N * xd;
    double kd = z + Shift;
    uint64_t ki = (uint64_t)__double_as_longlong(kd);
    kd -= Shift;
    double r = z - kd;
    uint64_t t = IT_EXP2F_TAB[ki % 32];
    t += ki << (52 - 5);
    double s = __longlong_as_double((long long)t);
    z = C0 * r + C1;
    double r2 = r * r;
    double y = C2 * r + 1.0;
    y = z * r2 + y;
    y = y * s;
    return (float)y;
}

__device__ __constant__ const double IT_LOGF_TAB[16][2] = {
    {0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2}, {0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2},
    {0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2},  {0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3},
    {0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3}, {0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3},
    {0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4}, {0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4},
    {0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5}, {0x1p+0, 0x0p+0},
    {0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5},  {0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4},
    {0x1.b2036576afce6p-1, 0x1.526e57720db08p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3},
    {0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2},  {0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2},
};

IT_DEV float it_logf(float x) {
    const double A0 = -0x1.00ea348b88334p-2, A1 = 0x1.5575b0be00b6ap-2, A2 = -0x1.ffffef20a4123p-2;
    const double Ln2 = 0x1.62e42fefa39efp-1;
    uint32_t ix = __float_as_uint(x);
    if (ix == 0x3f800000u) return 0.0f;
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {
        if (ix * 2 == 0) return __uint_as_float(0xff800000u);
        if (ix == 0x7f800000u) return x;
        if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return __uint_as_float(0x7fc00000u);
        ix = __float_as_uint(x * 0x1p23f);
        ix -= 23u << 23;
    }
    uint32_t tmp = ix - 0x3f330000u;
    int i = (tmp >> (23 - 4)) % 16;
    int32_t k = (int32_t)tmp >> 23;
    uint32_t iz = ix - (tmp & (0x1ffu << 23));
    double invc = IT_LOGF_TAB[i][0], logc = IT_LOGF_TAB[i][1];
    double z = (double)__uint_as_float(iz);
    double r = z * invc - 1.0;
    double y0 = logc + (double)k * Ln2;
    double r2 = r * r;
    double y = A1 * r + A2;
    y = A0 * r2 + y;
    y = y * r2 + (y0 + r);
    return (float)y;
}

// silu and sigmoid exactly as the reference writes them
// (/root/reference src/ops/naive.rs:250, :335).
// Fast-mode forms on the transcendental unit (v_exp_f32 / v_log_f32, about 1 ulp on 2^x and log2 x): no table
// fetch and two instructions instead of thirty.  Results differ from the CPU path's libm forms in the last bits,
// so only the kernels that already reorder sums use them.
IT_DEV float fx_expf(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
IT_DEV float fx_logf(float x) { return __builtin_amdgcn_logf(x) * 0.6931471805599453f; }
IT_DEV float fx_sigmoid(float g) { return 1.0f / (1.0f + fx_expf(-g)); }
IT_DEV float fx_silu(float g) { return g / (1.0f + fx_expf(-g)); }
IT_DEV float it_sigmoid(float g) { return 1.0f / (1.0f + it_expf(-g)); }
IT_DEV float it_silu(float g) { return g / (1.0f + it_expf(-g)); }
