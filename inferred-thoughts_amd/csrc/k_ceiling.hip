// This card's MFMA ceilings, measured rather than quoted: back-to-back matrix instructions on eight
// independent accumulators per wave, no memory in the loop, two waves on every SIMD of every CU. The
// prefill kernels' utilisation figures are fractions of these next to the published peaks. The method
// is the one the reference uses for its own card's ceilings (tests/cuda_ops.rs:56-72).
#include "it_device.h"
#include "backend.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int CHAINS = 8;       // independent accumulators per wave
constexpr int CEIL_THREADS = 256;

// KIND: 0 int8 16x16x64, 1 int8 16x16x32, 2 f16 32x32x16, 3 f16 16x16x32, 4 f32 16x16x4
template <int KIND>
__global__ __launch_bounds__(CEIL_THREADS) void mfma_ceiling_k(int iters, float* sink) {
    const int lane = threadIdx.x;
    float total = 0.f;
    if constexpr (KIND == 0) {
        v4i a = {lane, lane + 1, lane + 2, lane + 3}, b = {3 - lane, lane, 7, lane ^ 5};
        v4i c[CHAINS] = {};
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < CHAINS; ++j) c[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < CHAINS; ++j) total += (float)(c[j][0] + c[j][1] + c[j][2] + c[j][3]);
    } else if constexpr (KIND == 1) {
        v2i a = {lane, lane + 1}, b = {3 - lane, lane ^ 5};
        v4i c[CHAINS] = {};
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < CHAINS; ++j) {
                long al, bl;
                __builtin_memcpy(&al, &a, 8);
                __builtin_memcpy(&bl, &b, 8);
                c[j] = __builtin_amdgcn_mfma_i32_16x16x32_i8(al, bl, c[j], 0, 0, 0);
            }
        }
#pragma unroll
        for (int j = 0; j < CHAINS; ++j) total += (float)(c[j][0] + c[j][1] + c[j][2] + c[j][3]);
    } else if constexpr (KIND == 2) {
        v8h a, b;
#pragma unroll
        for (int e = 0; e < 8; ++e) { a[e] = (_Float16)(0.001f * (lane + e)); b[e] = (_Float16)(0.002f * (lane - e)); }
        v16f c[CHAINS] = {};
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < CHAINS; ++j) c[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < CHAINS; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) total += c[j][e];
    } else if constexpr (KIND == 3) {
        v8h a, b;
#pragma unroll
        for (int e = 0; e < 8; ++e) { a[e] = (_Float16)(0.001f * (lane + e)); b[e] = (_Float16)(0.002f * (lane - e)); }
        v4f c[CHAINS] = {};
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < CHAINS; ++j) c[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < CHAINS; ++j) total += c[j][0] + c[j][1] + c[j][2] + c[j][3];
    } else {
        float a = 0.001f * lane, b = 0.002f * (lane - 7);
        v4f c[CHAINS] = {};
        for (int i = 0; i < iters; ++i) {
#pragma unroll
            for (int j = 0; j < CHAINS; ++j) c[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c[j], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < CHAINS; ++j) total += c[j][0] + c[j][1] + c[j][2] + c[j][3];
    }
    // every lane's sums reach memory, so the loop cannot be dropped; the host never reads them
    sink[(size_t)blockIdx.x * CEIL_THREADS + threadIdx.x] = total;
}

// multiply-accumulates of one instruction of each kind
constexpr double KIND_MACS[5] = {16. * 16 * 64, 16. * 16 * 32, 32. * 32 * 16, 16. * 16 * 32, 16. * 16 * 4};

}  // namespace

extern "C" int it_hip_mfma_ceiling(it_hip* be, int kind, int iters, double* ops_per_s) {
    if (!be || kind < 0 || kind > 4 || iters < 1 || !ops_per_s) return 1;
    hipStream_t s = be->stream;
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 2;
    // two blocks of four waves on each CU: two waves per SIMD
    const int blocks = prop.multiProcessorCount * 2;
    float* sink = nullptr;
    if (hipMalloc(&sink, (size_t)blocks * CEIL_THREADS * sizeof(float)) != hipSuccess) return 2;
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    auto launch = [&](int n) {
        switch (kind) {
            case 0: mfma_ceiling_k<0><<<blocks, CEIL_THREADS, 0, s>>>(n, sink); break;
            case 1: mfma_ceiling_k<1><<<blocks, CEIL_THREADS, 0, s>>>(n, sink); break;
            case 2: mfma_ceiling_k<2><<<blocks, CEIL_THREADS, 0, s>>>(n, sink); break;
            case 3: mfma_ceiling_k<3><<<blocks, CEIL_THREADS, 0, s>>>(n, sink); break;
            default: mfma_ceiling_k<4><<<blocks, CEIL_THREADS, 0, s>>>(n, sink); break;
        }
    };
    launch(iters / 8 + 1);  // code object load and clock ramp
    (void)hipEventRecord(e0, s);
    launch(iters);
    (void)hipEventRecord(e1, s);
    int rc = 0;
    float ms = 0.f;
    if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess || ms <= 0.f) rc = 2;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    if (rc) return rc;
    const double insts = (double)blocks * (CEIL_THREADS / 64) * CHAINS * (double)iters;
    *ops_per_s = 2.0 * KIND_MACS[kind] * insts / (ms * 1e-3);
    return 0;
}
