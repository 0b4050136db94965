// it_hip_attend_noalloc: split-K decode attention for callers that cannot allocate.
//
// The backend's it_hip_attend mirrors host buffers on the device and grows its split-K
// scratch (the per-split partial sums, maxima and normalisers) with hipMalloc.  Code
// under HIP graph capture, a tight serving loop or a harness that forbids allocation
// cannot call it.  This entry point runs the same kernels (attend_decode_k or
// attend_split_k, then the merge) on operands that are already device resident and keeps
// the partials in a fixed array inside the code object, so it calls no hipMalloc,
// hipFree or allocating library routine.
//
// The array belongs to the GPU, not to the call: every device the library runs on holds
// its own copy at its own address until the process ends, all calls on a device share
// it, and two calls that overlap on one device (two streams, two threads) race.  Nothing
// in it has to start at zero: every split's slot is written by the split kernel before
// the merge reads it.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <mutex>

#include "../../include/inferred_hip.h"
#include "kernels.h"

namespace {

constexpr size_t SCRATCH_FLOATS = IT_HIP_NOALLOC_SCRATCH_BYTES / sizeof(float);
// the split-K partials: [query row * head][split][head_dim + 2] floats
static __device__ __align__(256) float scratch[SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
std::mutex g_lock;
float* g_scratch_ptr[MAX_DEVICES] = {};  // device address of `scratch` on each device, once looked up

int fail(char* err, size_t err_len, int code, const char* what, const char* detail = nullptr) {
    if (err && err_len) snprintf(err, err_len, "%s%s%s", what, detail ? ": " : "", detail ? detail : "");
    return code;
}

// The device address of this device's copy of `scratch`.  Looked up once per device with that device
// current; host code uses the returned pointer, never the array's name.
hipError_t scratch_of_current_device(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> hold(g_lock);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = (float*)p;
    }
    *out = g_scratch_ptr[dev];
    return hipSuccess;
}

}  // namespace

// called by it_hip_create with the backend's device current, so the first attend pays nothing
extern "C" int it_hip_noalloc_setup(void) {
    float* p = nullptr;
    return scratch_of_current_device(&p) == hipSuccess ? 0 : 1;
}

extern "C" int it_hip_attend_noalloc(const it_attn* a, float* out, uint64_t out_len, void* stream, char* err,
                                     size_t err_len) {
    if (!a || !a->q || !a->k || !a->v || !out) return fail(err, err_len, 1, "attend_noalloc: null argument");
    if (a->head_dim == 0 || a->n_head == 0 || a->n_head_kv == 0 || a->n_head % a->n_head_kv != 0)
        return fail(err, err_len, 1, "attend_noalloc: n_head must be a positive multiple of n_head_kv");
    const uint64_t group = a->n_head / a->n_head_kv;
    if (!(group == 1 || group == 2 || group == 4 || group == 8) || a->head_dim % 8 != 0 || a->head_dim > 256)
        return fail(err, err_len, 1,
                    "attend_noalloc: the split-K kernels take 1, 2, 4 or 8 query heads per kv head and head_dim a "
                    "multiple of 8, at most 256");
    const uint64_t per = a->n_head * a->head_dim;
    if (a->q_len % per != 0 || out_len != a->q_len)
        return fail(err, err_len, 1, "attend_noalloc: q.len() must be rows of n_head*head_dim and equal out.len()");
    const uint64_t n_q = a->q_len / per;
    if (n_q == 0) return 0;
    if (n_q > 16)
        return fail(err, err_len, 1, "attend_noalloc: at most 16 query rows (a decode step or a short verify batch)");
    if (a->kv_dim < a->n_head_kv * a->head_dim || a->kv_dim % 8 != 0)
        return fail(err, err_len, 1, "attend_noalloc: kv_dim too small for n_head_kv*head_dim");
    if (a->n_pos < n_q || a->n_pos > a->kv_len / a->kv_dim || a->n_pos >= (1ull << 31))
        return fail(err, err_len, 1, "attend_noalloc: n_pos outside the slab or smaller than the batch");
    const int n_split = itk::attend_split_count((int)a->n_pos, (int)n_q, (int)a->head_dim, (int)group);
    const uint64_t need = n_q * a->n_head * (uint64_t)n_split * (a->head_dim + 2);
    if (need > SCRATCH_FLOATS) {
        char detail[160];
        snprintf(detail, sizeof detail, "%llu bytes of split-K partials needed, the fixed scratch holds %llu",
                 (unsigned long long)(need * sizeof(float)), (unsigned long long)IT_HIP_NOALLOC_SCRATCH_BYTES);
        return fail(err, err_len, 2, "attend_noalloc: problem too large", detail);
    }
    float* part = nullptr;
    hipError_t e = scratch_of_current_device(&part);
    if (e != hipSuccess) return fail(err, err_len, 3, "attend_noalloc: hipGetSymbolAddress(scratch)", hipGetErrorString(e));
    itk::AttnArgs args{a->q, a->k, a->v, (int)n_q, (int)a->kv_dim, (int)a->n_pos, (int)a->head_dim,
                       (int)a->n_head, (int)a->n_head_kv, a->scale, nullptr};
    if (!itk::attend_split_gated(args, n_split, part, out, nullptr, 0, (hipStream_t)stream))
        return fail(err, err_len, 3, "attend_noalloc: the split-K kernels could not be launched");
    e = hipGetLastError();
    if (e != hipSuccess) return fail(err, err_len, 3, "attend_noalloc: kernel launch", hipGetErrorString(e));
    return 0;
}
