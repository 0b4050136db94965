// The HIP backend: residency, validation and dispatch for every seam op.
//
// Each op validates its operand shapes on the host before anything is launched
// (a kernel never sees a shape its grid does not cover), records the first error
// and keeps going, as the reference's device backend does
// (/root/reference src/ops/cuda/ops/mod.rs:91-110).
#include "backend.h"

#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstring>

using namespace itk;

namespace {
uint64_t type_row_bytes(uint32_t ty, uint64_t n_in) {
    switch (ty) {
        case IT_F32: return n_in * 4;
        case IT_F16: case IT_BF16: return n_in * 2;
        case IT_Q8_0: return n_in % 32 ? 0 : n_in / 32 * 34;
        case IT_NVFP4: return n_in % 64 ? 0 : n_in / 64 * 36;
        default: return 0;
    }
}
uint64_t now_us() {
    return (uint64_t)std::chrono::duration_cast<std::chrono::microseconds>(
               std::chrono::steady_clock::now().time_since_epoch())
        .count();
}
}  // namespace

void it_hip::fail(const std::string& what) {
    if (!has_error) {
        has_error = true;
        error = what;
    }
}
bool it_hip::check(hipError_t e, const char* what) {
    if (e == hipSuccess) return true;
    fail(std::string(what) + ": " + hipGetErrorString(e));
    return false;
}

// ------------------------------------------------------------------ activations
it_hip::Act* it_hip::act_slot(const float* host, size_t len) {
    Act& a = acts[host];
    if (a.cap < len) {
        float* fresh = nullptr;
        size_t cap = len;
        if (!check(hipMalloc((void**)&fresh, cap * sizeof(float)), "hipMalloc(activation mirror)")) return nullptr;
        if (a.dev) {
            if (a.dev_current)
                check(hipMemcpyAsync(fresh, a.dev, a.cap * sizeof(float), hipMemcpyDeviceToDevice, stream),
                      "mirror grow copy");
            check(hipStreamSynchronize(stream), "sync before mirror free");
            mirror_bytes -= a.cap * sizeof(float);
            (void)hipFree(a.dev);
        }
        a.dev = fresh;
        a.cap = cap;
        mirror_bytes += cap * sizeof(float);
    }
    return &a;
}
float* it_hip::act_in(const float* host, size_t len) {
    Act* a = act_slot(host, len);
    if (!a) return nullptr;
    if (!a->dev_current) {
        if (!check(hipMemcpyAsync(a->dev, host, len * sizeof(float), hipMemcpyHostToDevice, stream),
                   "upload activation"))
            return nullptr;
        h2d++;
        h2d_bytes += len * sizeof(float);
        a->dev_current = true;
        a->q_valid = false;
    }
    return a->dev;
}
float* it_hip::act_out(const float* host, size_t len) {
    Act* a = act_slot(host, len);
    if (!a) return nullptr;
    a->dev_current = true;
    a->q_valid = false;
    return a->dev;
}
float* it_hip::act_inout(const float* host, size_t len) {
    float* d = act_in(host, len);
    if (d) acts[host].q_valid = false;
    return d;
}

bool it_hip::act_quantized(const float* host, size_t len, const float** scales, const int8_t** quants,
                           float** dev_x) {
    float* x = act_in(host, len);
    if (!x) return false;
    Act& a = acts[host];
    if (a.q_cap < len) {
        if (a.q_scales) {
            check(hipStreamSynchronize(stream), "sync before quant free");
            quant_bytes -= a.q_cap / 32 * 4 + a.q_cap;
            (void)hipFree(a.q_scales);
            (void)hipFree(a.q_quants);
            a.q_scales = nullptr;
            a.q_quants = nullptr;
        }
        if (!check(hipMalloc((void**)&a.q_scales, (len / 32 + 1) * sizeof(float)), "hipMalloc(q8 scales)") ||
            !check(hipMalloc((void**)&a.q_quants, len + 32), "hipMalloc(q8 quants)"))
            return false;
        a.q_cap = len;
        quant_bytes += len / 32 * 4 + len;
        a.q_valid = false;
    }
    if (!a.q_valid || a.q_len != len) {
        quantize_q8_0(x, a.q_scales, a.q_quants, (int64_t)len, stream);
        launches++;
        a.q_valid = true;
        a.q_len = len;
    }
    *scales = a.q_scales;
    *quants = a.q_quants;
    if (dev_x) *dev_x = x;
    return true;
}

const float* it_hip::const_in(const float* host, size_t len) {
    auto it = consts.find(host);
    if (it != consts.end() && it->second.len >= len) return it->second.dev;
    Const c;
    if (!check(hipMalloc((void**)&c.dev, len * sizeof(float)), "hipMalloc(constant)")) return nullptr;
    if (!check(hipMemcpyAsync(c.dev, host, len * sizeof(float), hipMemcpyHostToDevice, stream), "upload constant"))
        return nullptr;
    c.len = len;
    const_bytes += len * 4;
    if (it != consts.end()) {
        check(hipStreamSynchronize(stream), "sync before constant free");
        (void)hipFree(it->second.dev);
    }
    consts[host] = c;
    return c.dev;
}

// ------------------------------------------------------------------ weights
const it_hip::Resident* it_hip::resident(const uint8_t* data, uint64_t len, uint32_t ty, uint64_t n_in,
                                         uint64_t rows, const char* who) {
    auto it = weights.find(data);
    if (it != weights.end()) {
        if (it->second.fmt == (int)ty && it->second.n_in == n_in && it->second.rows == rows) return &it->second;
        fail(std::string(who) + ": a weight address was seen before with a different shape");
        return nullptr;
    }
    uint64_t row_bytes = type_row_bytes(ty, n_in);
    if (row_bytes == 0) {
        fail(std::string(who) + ": unsupported weight type or row length not a whole number of blocks");
        return nullptr;
    }
    if (len != row_bytes * rows) {
        fail(std::string(who) + ": weight byte length does not match its shape");
        return nullptr;
    }
    uint64_t t0 = now_us();
    Resident r;
    r.fmt = (int)ty;
    r.n_in = n_in;
    r.rows = rows;
    void* raw = nullptr;
    if (!check(hipMalloc(&raw, len), "hipMalloc(weight upload)")) return nullptr;
    if (!check(hipMemcpyAsync(raw, data, len, hipMemcpyHostToDevice, stream), "upload weight")) return nullptr;
    h2d++;
    h2d_bytes += len;
    if (ty == IT_Q8_0) {
        r.q_bytes = rows * n_in;
        r.s_bytes = rows * (n_in / 32) * 2;
        if (!check(hipMalloc(&r.q, r.q_bytes), "hipMalloc(q8_0 quants)") ||
            !check(hipMalloc(&r.scales, r.s_bytes), "hipMalloc(q8_0 scales)"))
            return nullptr;
        repack_q8_0((const uint8_t*)raw, (int8_t*)r.q, (uint16_t*)r.scales, (int64_t)rows, (int)n_in, stream);
        launches++;
        check(hipStreamSynchronize(stream), "repack q8_0");
        (void)hipFree(raw);
    } else if (ty == IT_NVFP4) {
        r.q_bytes = rows * (n_in / 2);
        r.s_bytes = rows * (n_in / 16);
        if (!check(hipMalloc(&r.q, r.q_bytes), "hipMalloc(nvfp4 nibbles)") ||
            !check(hipMalloc(&r.scales, r.s_bytes), "hipMalloc(nvfp4 scales)"))
            return nullptr;
        repack_nvfp4((const uint8_t*)raw, (uint8_t*)r.q, (uint8_t*)r.scales, (int64_t)rows, (int)n_in, stream);
        launches++;
        check(hipStreamSynchronize(stream), "repack nvfp4");
        (void)hipFree(raw);
    } else {
        r.q = raw;
        r.q_bytes = len;
        check(hipStreamSynchronize(stream), "upload weight");
    }
    weight_bytes += r.q_bytes + r.s_bytes;
    setup_us += now_us() - t0;
    auto ins = weights.emplace(data, r);
    return &ins.first->second;
}

bool it_hip::weights_view(const it_weights* w, const char* who, WView* out) {
    if (!w || !w->data) {
        fail(std::string(who) + ": null weights");
        return false;
    }
    if (w->n_in == 0 || w->n_out == 0 || w->n_in > (1u << 24) || w->n_out > (1u << 30)) {
        fail(std::string(who) + ": weight dimensions out of range");
        return false;
    }
    const Resident* r = resident(w->data, w->len, w->ty, w->n_in, w->n_out, who);
    if (!r) return false;
    out->q = r->q;
    out->scales = r->scales;
    out->fmt = r->fmt;
    out->n_in = (int)w->n_in;
    out->n_out = (int)w->n_out;
    return true;
}

bool it_hip::experts_view(const it_experts* w, const char* who, ExpertsView* out) {
    if (!w || !w->data) {
        fail(std::string(who) + ": null experts");
        return false;
    }
    if (w->ty != IT_Q8_0 && w->ty != IT_NVFP4) {
        fail(std::string(who) + ": routed experts must be Q8_0 or NVFP4 on this backend");
        return false;
    }
    if (w->n_in == 0 || w->n_out == 0 || w->n_expert == 0 || w->n_in > (1u << 24) || w->n_out > (1u << 24)) {
        fail(std::string(who) + ": expert dimensions out of range");
        return false;
    }
    if (w->scale && w->scale_len != 0 && w->scale_len != w->n_expert * 4) {
        fail(std::string(who) + ": expert scale length is not n_expert f32");
        return false;
    }
    bool fresh = weights.find(w->data) == weights.end();
    const Resident* r = resident(w->data, w->len, w->ty, w->n_in, w->n_out * w->n_expert, who);
    if (!r) return false;
    if (fresh) {
        // all-resident tier: every expert of the tensor is placed at first sight
        expert_resident += w->n_expert;
        expert_slot_bytes = type_row_bytes(w->ty, w->n_in) * w->n_out;
        if (expert_pool < expert_resident) expert_pool = expert_resident;
    }
    Resident* rw = &weights[w->data];
    if (w->scale && w->scale_len && !rw->scale2) {
        if (!check(hipMalloc((void**)&rw->scale2, w->scale_len), "hipMalloc(expert scales)")) return false;
        if (!check(hipMemcpyAsync(rw->scale2, w->scale, w->scale_len, hipMemcpyHostToDevice, stream),
                   "upload expert scales"))
            return false;
        check(hipStreamSynchronize(stream), "upload expert scales");
    }
    out->q = rw->q;
    out->scales = rw->scales;
    out->fmt = rw->fmt;
    out->n_in = (int)w->n_in;
    out->n_out = (int)w->n_out;
    out->n_expert = (int)w->n_expert;
    if (w->ty == IT_Q8_0) {
        out->q_stride = (int64_t)(w->n_out * w->n_in);
        out->s_stride = (int64_t)(w->n_out * (w->n_in / 32) * 2);
    } else {
        out->q_stride = (int64_t)(w->n_out * (w->n_in / 2));
        out->s_stride = (int64_t)(w->n_out * (w->n_in / 16));
    }
    out->scale2 = (w->scale && w->scale_len) ? rw->scale2 : nullptr;
    return true;
}

// ------------------------------------------------------------------ slabs
void* it_hip::slab_in(const void* host, size_t bytes, bool is_state) {
    Slab& s = slabs[host];
    if (s.dev && s.bytes < bytes) {
        check(hipStreamSynchronize(stream), "sync before slab free");
        (void)hipFree(s.dev);
        kv_bytes -= s.bytes;
        s.dev = nullptr;
        s.dev_owned = false;
    }
    if (!s.dev) {
        if (!check(hipMalloc(&s.dev, bytes), "hipMalloc(slab)")) return nullptr;
        s.bytes = bytes;
        s.is_state = is_state;
        kv_bytes += bytes;
    }
    if (!s.dev_owned) {
        if (!check(hipMemcpyAsync(s.dev, host, bytes, hipMemcpyHostToDevice, stream), "upload slab")) return nullptr;
        h2d++;
        h2d_bytes += bytes;
        s.dev_owned = true;
    }
    return s.dev;
}

// ------------------------------------------------------------------ route storage
bool it_hip::route_reserve(size_t picks) {
    if (route_cap >= picks) return true;
    if (route_ids) {
        check(hipStreamSynchronize(stream), "sync before route free");
        (void)hipFree(route_ids);
        (void)hipFree(route_w);
    }
    size_t cap = picks < 64 ? 64 : picks;
    if (!check(hipMalloc((void**)&route_ids, cap * sizeof(int32_t)), "hipMalloc(route ids)") ||
        !check(hipMalloc((void**)&route_w, cap * sizeof(float)), "hipMalloc(route weights)"))
        return false;
    route_cap = cap;
    return true;
}

bool it_hip::route_stage(const it_route* r, const int32_t** ids, const float** w, uint64_t* n_used,
                         uint64_t* n_tok) {
    if (!r) {
        fail("route: null");
        return false;
    }
    if (r->kind == IT_ROUTE_DEVICE) {
        if (r->n_used != route_n_used || r->n_tok != route_n_tok || !route_ids) {
            fail("route: a device route that this backend did not issue");
            return false;
        }
    } else {
        size_t picks = (size_t)(r->n_used * r->n_tok);
        if (picks == 0 || !r->ids) {
            fail("route: empty host route");
            return false;
        }
        if (!route_reserve(picks)) return false;
        std::vector<int32_t> tmp(picks);
        for (size_t i = 0; i < picks; i++) tmp[i] = (int32_t)r->ids[i];
        if (!check(hipMemcpyAsync(route_ids, tmp.data(), picks * 4, hipMemcpyHostToDevice, stream), "upload ids"))
            return false;
        if (r->weights &&
            !check(hipMemcpyAsync(route_w, r->weights, picks * 4, hipMemcpyHostToDevice, stream), "upload weights"))
            return false;
        check(hipStreamSynchronize(stream), "upload route");
        route_n_used = r->n_used;
        route_n_tok = r->n_tok;
        // remember the ids for bounds checks
    }
    *ids = route_ids;
    *w = route_w;
    *n_used = route_n_used;
    *n_tok = route_n_tok;
    return true;
}

// ------------------------------------------------------------------ rope
const float2* it_hip::rope_table(float theta, uint64_t n_rot, uint64_t need_pos) {
    uint32_t tb;
    memcpy(&tb, &theta, 4);
    uint64_t key = ((uint64_t)tb << 32) | n_rot;
    Rope& r = ropes[key];
    if (r.cap_pos >= need_pos) return r.dev;
    size_t cap = r.cap_pos ? r.cap_pos : 1024;
    while (cap < need_pos) cap *= 2;
    size_t half = n_rot / 2;
    std::vector<float2> tab(cap * half);
    std::vector<double> freq(half);
    for (size_t i = 0; i < half; i++) freq[i] = pow((double)theta, -2.0 * (double)i / (double)n_rot);
    for (size_t p = 0; p < cap; p++)
        for (size_t i = 0; i < half; i++) {
            double th = (double)p * freq[i];
            tab[p * half + i] = make_float2((float)cos(th), (float)sin(th));
        }
    float2* dev = nullptr;
    if (!check(hipMalloc((void**)&dev, tab.size() * sizeof(float2)), "hipMalloc(rope table)")) return nullptr;
    if (!check(hipMemcpyAsync(dev, tab.data(), tab.size() * sizeof(float2), hipMemcpyHostToDevice, stream),
               "upload rope table"))
        return nullptr;
    check(hipStreamSynchronize(stream), "upload rope table");
    if (r.dev) (void)hipFree(r.dev);
    r.dev = dev;
    r.cap_pos = cap;
    return r.dev;
}

float* it_hip::scratch_f32(size_t floats) {
    if (attn_scratch_cap >= floats) return attn_scratch;
    if (attn_scratch) {
        check(hipStreamSynchronize(stream), "sync before scratch free");
        (void)hipFree(attn_scratch);
    }
    attn_scratch = nullptr;
    attn_scratch_cap = 0;
    if (!check(hipMalloc((void**)&attn_scratch, floats * sizeof(float)), "hipMalloc(attention scratch)"))
        return nullptr;
    attn_scratch_cap = floats;
    return attn_scratch;
}

void it_hip::drop_all() {
    if (stream) (void)hipStreamSynchronize(stream);
    for (auto& kv : acts) {
        if (kv.second.dev) (void)hipFree(kv.second.dev);
        if (kv.second.q_scales) (void)hipFree(kv.second.q_scales);
        if (kv.second.q_quants) (void)hipFree(kv.second.q_quants);
    }
    acts.clear();
    for (auto& kv : consts)
        if (kv.second.dev) (void)hipFree(kv.second.dev);
    consts.clear();
    for (auto& kv : weights) {
        if (kv.second.q) (void)hipFree(kv.second.q);
        if (kv.second.scales) (void)hipFree(kv.second.scales);
        if (kv.second.scale2) (void)hipFree(kv.second.scale2);
    }
    weights.clear();
    for (auto& kv : slabs)
        if (kv.second.dev) (void)hipFree(kv.second.dev);
    slabs.clear();
    mirror_bytes = quant_bytes = const_bytes = weight_bytes = kv_bytes = 0;
    expert_resident = 0;
}

it_hip::~it_hip() {
    drop_all();
    for (auto& kv : ropes)
        if (kv.second.dev) (void)hipFree(kv.second.dev);
    if (route_ids) (void)hipFree(route_ids);
    if (route_w) (void)hipFree(route_w);
    if (attn_scratch) (void)hipFree(attn_scratch);
    if (argmax_idx) (void)hipFree(argmax_idx);
    if (argmax_val) (void)hipFree(argmax_val);
    if (argmax_out) (void)hipFree(argmax_out);
    if (argmax_host) (void)hipHostFree(argmax_host);
    if (dyn_dev) (void)hipFree(dyn_dev);
    if (dyn_host) (void)hipHostFree(dyn_host);
    if (graph.exec) (void)hipGraphExecDestroy(graph.exec);
    if (graph.graph) (void)hipGraphDestroy(graph.graph);
    if (stream) (void)hipStreamDestroy(stream);
}

// =================================================================== C ABI
extern "C" {

it_hip* it_hip_create(uint32_t flags, int device, char* err, size_t err_len) {
    auto bad = [&](const std::string& m) -> it_hip* {
        if (err && err_len) snprintf(err, err_len, "%s", m.c_str());
        return nullptr;
    };
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) return bad(std::string("no HIP device: ") + hipGetErrorString(e));
    if (device < 0 || device >= n) return bad("device index out of range");
    if ((e = hipSetDevice(device)) != hipSuccess) return bad(std::string("hipSetDevice: ") + hipGetErrorString(e));
    hipDeviceProp_t prop;
    if ((e = hipGetDeviceProperties(&prop, device)) != hipSuccess)
        return bad(std::string("hipGetDeviceProperties: ") + hipGetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return bad(std::string("this library is built for gfx950 only; device is ") + prop.gcnArchName);
    it_hip* be = new it_hip();
    be->device = device;
    be->exact = (flags & IT_HIP_EXACT) != 0;
    be->allow_graph = (flags & IT_HIP_NO_GRAPH) == 0;
    if ((e = hipStreamCreate(&be->stream)) != hipSuccess) {
        delete be;
        return bad(std::string("hipStreamCreate: ") + hipGetErrorString(e));
    }
    return be;
}

void it_hip_destroy(it_hip* be) { delete be; }

int it_hip_take_error(it_hip* be, char* msg, size_t msg_len) {
    if (!be->has_error) {
        // surface asynchronous faults too
        hipError_t e = hipStreamSynchronize(be->stream);
        if (e != hipSuccess) be->fail(std::string("device: ") + hipGetErrorString(e));
    }
    if (!be->has_error) return 0;
    if (msg && msg_len) snprintf(msg, msg_len, "%s", be->error.c_str());
    be->has_error = false;
    be->error.clear();
    return 1;
}

int it_hip_check_expert_types(uint32_t gate, uint32_t up, uint32_t down, char* msg, size_t msg_len) {
    auto ok1 = [](uint32_t t) { return t == IT_Q8_0 || t == IT_NVFP4; };
    if (ok1(gate) && gate == up && ok1(down)) return 0;
    if (msg && msg_len)
        snprintf(msg, msg_len,
                 "type %u (gate) / %u (up) / %u (down): --backend hip runs Q8_0 or NVFP4 experts, gate and up of "
                 "the same type",
                 gate, up, down);
    return 1;
}

#define BE_STREAM be->stream
#define REQUIRE(cond, msg)   \
    do {                     \
        if (!(cond)) {       \
            be->fail(msg);   \
            return;          \
        }                    \
    } while (0)

void it_hip_rms_norm(it_hip* be, const float* x, uint64_t x_len, const float* w, uint64_t w_len, float eps,
                     float* out, uint64_t out_len) {
    REQUIRE(w_len > 0 && x_len % w_len == 0 && x_len == out_len, "rms_norm: x.len() must be a multiple of weight.len() and equal out.len()");
    REQUIRE(w_len <= 12288, "rms_norm: row longer than the kernel's LDS tile");
    if (x_len == 0) return;
    const float* dw = be->const_in(w, w_len);
    float* dx = be->act_in(x, x_len);
    float* dout = (out == x) ? dx : be->act_out(out, out_len);
    if (!dw || !dx || !dout) return;
    if (out == x) be->acts[x].q_valid = false;
    rms_norm(dx, dw, eps, dout, (int64_t)(x_len / w_len), (int)w_len, be->exact, BE_STREAM);
    be->launches++;
}

void it_hip_rms_norm_heads(it_hip* be, float* x, uint64_t x_len, const float* w, uint64_t w_len,
                           uint64_t head_dim, float eps) {
    REQUIRE(head_dim > 0 && w_len == head_dim && x_len % head_dim == 0, "rms_norm_heads: weight.len() must equal head_dim and divide x.len()");
    REQUIRE(head_dim <= 12288, "rms_norm_heads: head longer than the kernel's LDS tile");
    if (x_len == 0) return;
    const float* dw = be->const_in(w, w_len);
    float* dx = be->act_inout(x, x_len);
    if (!dw || !dx) return;
    rms_norm_heads(dx, dw, (int)head_dim, eps, (int64_t)(x_len / head_dim), be->exact, BE_STREAM);
    be->launches++;
}

static void matmul_impl(it_hip* be, const it_weights* w, const float* x, uint64_t x_len, float* out,
                        uint64_t out_len, const char* who) {
    WView v;
    if (!be->weights_view(w, who, &v)) return;
    if (x_len % w->n_in != 0 || out_len != x_len / w->n_in * w->n_out) {
        be->fail(std::string(who) + ": x.len() must be a multiple of n_in and out.len() == n * n_out");
        return;
    }
    uint64_t n = x_len / w->n_in;
    if (n == 0) return;
    if (n > 65535) {
        be->fail(std::string(who) + ": more than 65535 tokens in one call");
        return;
    }
    const float* as = nullptr;
    const int8_t* aq = nullptr;
    float* dx = nullptr;
    if (v.fmt == W_Q8_0 || v.fmt == W_NVFP4) {
        if (!be->act_quantized(x, x_len, &as, &aq, &dx)) return;
    } else {
        dx = be->act_in(x, x_len);
        if (!dx) return;
    }
    float* dout = be->act_out(out, out_len);
    if (!dout) return;
    matmul(v, dx, as, aq, (int)n, dout, 1.0f, BE_STREAM);
    be->launches++;
}

void it_hip_matmul(it_hip* be, const it_weights* w, const float* x, uint64_t x_len, float* out,
                   uint64_t out_len) {
    matmul_impl(be, w, x, x_len, out, out_len, "matmul");
}

void it_hip_matmul_pair(it_hip* be, const it_weights* a, const it_weights* b, const float* x, uint64_t x_len,
                        float* out_a, uint64_t out_a_len, float* out_b, uint64_t out_b_len) {
    matmul_impl(be, a, x, x_len, out_a, out_a_len, "matmul_pair(a)");
    matmul_impl(be, b, x, x_len, out_b, out_b_len, "matmul_pair(b)");
}

void it_hip_rope_neox(it_hip* be, float* x, uint64_t x_len, uint64_t pos, uint64_t head_dim, uint64_t n_rot,
                      uint64_t n_heads, float theta) {
    uint64_t per_row = head_dim * n_heads;
    REQUIRE(per_row > 0 && x_len % per_row == 0, "rope_neox: x.len() must be a multiple of head_dim * n_heads");
    REQUIRE(n_rot % 2 == 0 && n_rot <= head_dim, "rope_neox: n_rot must be even and at most head_dim");
    if (x_len == 0 || n_rot == 0) return;
    uint64_t n = x_len / per_row;
    REQUIRE(pos + n < (1ull << 31), "rope_neox: position out of range");
    const float2* tab = be->rope_table(theta, n_rot, pos + n);
    float* dx = be->act_inout(x, x_len);
    if (!tab || !dx) return;
    rope_neox(dx, tab, (int)(n_rot / 2), (int64_t)n, (int)pos, nullptr, (int)head_dim, (int)n_rot, (int)n_heads,
              BE_STREAM);
    be->launches++;
}

void it_hip_softmax(it_hip* be, float* x, uint64_t x_len, uint64_t row) {
    if (row == 0 || x_len == 0) return;
    REQUIRE(x_len % row == 0, "softmax: x.len() must be a multiple of row");
    REQUIRE(row <= 12288, "softmax: row longer than the kernel's LDS tile");
    float* dx = be->act_inout(x, x_len);
    if (!dx) return;
    softmax_rows(dx, (int64_t)(x_len / row), (int)row, be->exact, BE_STREAM);
    be->launches++;
}

void it_hip_attend(it_hip* be, const it_attn* a, float* out, uint64_t out_len) {
    REQUIRE(a && a->q && a->k && a->v, "attend: null argument");
    REQUIRE(a->head_dim > 0 && a->n_head > 0 && a->n_head_kv > 0 && a->n_head % a->n_head_kv == 0,
            "attend: n_head must be a positive multiple of n_head_kv");
    REQUIRE(a->head_dim % 8 == 0 && a->head_dim <= 1024, "attend: head_dim must be a multiple of 8, at most 1024");
    uint64_t per = a->n_head * a->head_dim;
    REQUIRE(a->q_len % per == 0 && out_len == a->q_len, "attend: q.len() must be rows of n_head*head_dim and equal out.len()");
    uint64_t n_q = a->q_len / per;
    if (n_q == 0) return;
    REQUIRE(a->kv_dim >= a->n_head_kv * a->head_dim && a->kv_dim % 8 == 0, "attend: kv_dim too small for n_head_kv*head_dim");
    REQUIRE(a->n_pos >= n_q && a->n_pos * a->kv_dim <= a->kv_len, "attend: n_pos outside the slab or smaller than the batch");
    REQUIRE(a->n_pos < (1ull << 31) && n_q * a->n_head < (1ull << 31), "attend: sizes out of range");
    float* dq = be->act_in(a->q, a->q_len);
    uint16_t* dk = (uint16_t*)be->slab_in(a->k, a->kv_len * 2, false);
    uint16_t* dv = (uint16_t*)be->slab_in(a->v, a->kv_len * 2, false);
    float* dout = be->act_out(out, out_len);
    if (!dq || !dk || !dv || !dout) return;
    AttnArgs args{dq, dk, dv, (int)n_q, (int)a->kv_dim, (int)a->n_pos, (int)a->head_dim,
                  (int)a->n_head, (int)a->n_head_kv, a->scale, nullptr};
    uint64_t group = a->n_head / a->n_head_kv;
    bool split_ok = (group == 1 || group == 2 || group == 4 || group == 8) && a->head_dim <= 256;
    if (be->exact || !split_ok) {
        float* sc = be->scratch_f32((size_t)(n_q * a->n_head * a->n_pos));
        if (!sc) return;
        attend_exact(args, sc, dout, BE_STREAM);
        be->launches++;
    } else {
        int n_split = attend_split_count((int)a->n_pos);
        float* sc = be->scratch_f32((size_t)(n_q * a->n_head) * n_split * (a->head_dim + 2));
        if (!sc) return;
        attend_split(args, n_split, sc, dout, BE_STREAM);
        be->launches += 2;
    }
}

static void ew2(it_hip* be, float* a, uint64_t a_len, const float* b, uint64_t b_len, const char* who, int op,
                float v) {
    if (a_len != b_len) {
        be->fail(std::string(who) + ": the two buffers differ in length");
        return;
    }
    if (a_len == 0) return;
    float* da = be->act_inout(a, a_len);
    float* db = be->act_in(b, b_len);
    if (!da || !db) return;
    switch (op) {
        case 0: silu_mul(da, db, (int64_t)a_len, be->stream); break;
        case 1: sigmoid_mul(da, db, (int64_t)a_len, be->stream); break;
        case 2: add_assign(da, db, (int64_t)a_len, be->stream); break;
        case 3: add_scaled(da, db, v, (int64_t)a_len, be->stream); break;
    }
    be->launches++;
}

void it_hip_silu_mul(it_hip* be, float* gate, uint64_t gate_len, const float* up, uint64_t up_len) {
    ew2(be, gate, gate_len, up, up_len, "silu_mul", 0, 0.f);
}
void it_hip_sigmoid_mul(it_hip* be, float* x, uint64_t x_len, const float* g, uint64_t g_len) {
    ew2(be, x, x_len, g, g_len, "sigmoid_mul", 1, 0.f);
}
void it_hip_add_assign(it_hip* be, float* a, uint64_t a_len, const float* b, uint64_t b_len) {
    ew2(be, a, a_len, b, b_len, "add_assign", 2, 0.f);
}
void it_hip_add_scaled(it_hip* be, float* a, uint64_t a_len, const float* b, uint64_t b_len, float scale_v) {
    ew2(be, a, a_len, b, b_len, "add_scaled", 3, scale_v);
}

void it_hip_scale(it_hip* be, float* buf, uint64_t len, float s) {
    if (len == 0) return;
    float* d = be->act_inout(buf, len);
    if (!d) return;
    scale(d, s, (int64_t)len, BE_STREAM);
    be->launches++;
}

void it_hip_l2_norm_heads(it_hip* be, float* x, uint64_t x_len, uint64_t head_dim, float eps) {
    REQUIRE(head_dim > 0 && x_len % head_dim == 0, "l2_norm_heads: head_dim must divide x.len()");
    REQUIRE(head_dim <= 12288, "l2_norm_heads: head longer than the kernel's LDS tile");
    if (x_len == 0) return;
    float* dx = be->act_inout(x, x_len);
    if (!dx) return;
    l2_norm_heads(dx, (int)head_dim, eps, (int64_t)(x_len / head_dim), be->exact, BE_STREAM);
    be->launches++;
}

void it_hip_ssm_conv(it_hip* be, float* state, uint64_t state_len, const float* x, uint64_t x_len,
                     const float* weight, uint64_t w_len, uint64_t kernel, float* out, uint64_t out_len) {
    REQUIRE(kernel >= 2 && kernel <= 5, "ssm_conv: kernel size must be 2..5");
    REQUIRE(w_len % kernel == 0 && w_len > 0, "ssm_conv: weight.len() must be a multiple of kernel");
    uint64_t nc = w_len / kernel;
    REQUIRE(state_len == nc * (kernel - 1), "ssm_conv: state.len() must be channels * (kernel - 1)");
    REQUIRE(x_len == out_len && x_len % nc == 0, "ssm_conv: x and out must be whole rows of the channel count");
    if (x_len == 0) return;
    REQUIRE(nc < (1ull << 31) && x_len / nc < (1ull << 31), "ssm_conv: sizes out of range");
    const float* dw = be->const_in(weight, w_len);
    float* dstate = (float*)be->slab_in(state, state_len * 4, true);
    float* dx = be->act_in(x, x_len);
    float* dout = be->act_out(out, out_len);
    if (!dw || !dstate || !dx || !dout) return;
    ssm_conv(dstate, dx, dw, (int)kernel, (int)nc, (int)(x_len / nc), dout, BE_STREAM);
    be->launches++;
}

void it_hip_gather_chunks(it_hip* be, const float* src, uint64_t src_len, uint64_t chunk, uint64_t stride,
                          uint64_t offset, float* out, uint64_t out_len) {
    REQUIRE(chunk > 0 && out_len % chunk == 0, "gather_chunks: chunk must divide out.len()");
    if (out_len == 0) return;
    uint64_t n = out_len / chunk;
    REQUIRE((n - 1) * stride + offset + chunk <= src_len, "gather_chunks: reads past the end of src");
    float* ds = be->act_in(src, src_len);
    float* dout = be->act_out(out, out_len);
    if (!ds || !dout) return;
    gather_chunks(ds, (int64_t)chunk, (int64_t)stride, (int64_t)offset, dout, (int64_t)out_len, BE_STREAM);
    be->launches++;
}

void it_hip_scatter_chunks(it_hip* be, const float* src, uint64_t src_len, uint64_t chunk, uint64_t stride,
                           uint64_t offset, float* dst, uint64_t dst_len) {
    REQUIRE(chunk > 0 && src_len % chunk == 0, "scatter_chunks: chunk must divide src.len()");
    if (src_len == 0) return;
    uint64_t n = src_len / chunk;
    REQUIRE((n - 1) * stride + offset + chunk <= dst_len, "scatter_chunks: writes past the end of dst");
    float* ds = be->act_in(src, src_len);
    float* dd = be->act_inout(dst, dst_len);
    if (!ds || !dd) return;
    scatter_chunks(ds, (int64_t)src_len, (int64_t)chunk, (int64_t)stride, (int64_t)offset, dd, BE_STREAM);
    be->launches++;
}

void it_hip_delta_rule(it_hip* be, const it_delta* d, float* state, uint64_t state_len, float* out,
                       uint64_t out_len) {
    REQUIRE(d && d->q && d->k && d->v && d->alpha && d->beta && d->ssm_a && d->dt_bias, "delta_rule: null argument");
    REQUIRE(d->head_k_dim == 32 || d->head_k_dim == 64 || d->head_k_dim == 128, "delta_rule: head_k_dim must be 32, 64 or 128");
    REQUIRE(d->head_v_dim > 0 && d->n_k_heads > 0 && d->n_v_heads > 0, "delta_rule: zero dimension");
    uint64_t kper = d->n_k_heads * d->head_k_dim, vper = d->n_v_heads * d->head_v_dim;
    REQUIRE(state_len == d->n_v_heads * d->head_k_dim * d->head_v_dim, "delta_rule: state.len() must be n_v_heads * head_k_dim * head_v_dim");
    REQUIRE(out_len == d->n_tokens * vper, "delta_rule: out.len() must be n_tokens * n_v_heads * head_v_dim");
    if (d->n_tokens == 0) return;
    REQUIRE(d->n_tokens < (1ull << 31), "delta_rule: too many tokens");
    uint64_t n = d->n_tokens;
    float* dq = be->act_in(d->q, n * kper);
    float* dk = be->act_in(d->k, n * kper);
    float* dv = be->act_in(d->v, n * vper);
    float* da = be->act_in(d->alpha, n * d->n_v_heads);
    float* db = be->act_in(d->beta, n * d->n_v_heads);
    const float* dssm = be->const_in(d->ssm_a, d->n_v_heads);
    const float* ddt = be->const_in(d->dt_bias, d->n_v_heads);
    float* dstate = (float*)be->slab_in(state, state_len * 4, true);
    float* dout = be->act_out(out, out_len);
    if (!dq || !dk || !dv || !da || !db || !dssm || !ddt || !dstate || !dout) return;
    DeltaArgs args{dq, dk, dv, da, db, dssm, ddt, (int)n, (int)d->head_k_dim, (int)d->head_v_dim,
                   (int)d->n_k_heads, (int)d->n_v_heads};
    delta_rule(args, dstate, dout, be->exact, BE_STREAM);
    be->launches++;
}

void it_hip_route(it_hip* be, float* probs, uint64_t probs_len, uint64_t n_expert, uint64_t n_used,
                  it_route* out) {
    if (out) *out = it_route{IT_ROUTE_DEVICE, 0, nullptr, nullptr, n_used, 0};
    REQUIRE(out, "route: null output");
    REQUIRE(n_expert > 0 && n_used > 0 && n_used <= n_expert && n_used <= 64, "route: need 0 < n_used <= min(n_expert, 64)");
    REQUIRE(n_expert <= 12288, "route: more experts than the kernel's LDS tile");
    REQUIRE(probs_len % n_expert == 0, "route: probs.len() must be a multiple of n_expert");
    uint64_t n_tok = probs_len / n_expert;
    out->n_tok = n_tok;
    if (n_tok == 0) return;
    REQUIRE(n_tok < (1ull << 24), "route: too many tokens");
    float* dp = be->act_in(probs, probs_len);
    if (!dp || !be->route_reserve((size_t)(n_tok * n_used))) return;
    route_topk(dp, (int)n_tok, (int)n_expert, (int)n_used, be->route_ids, be->route_w, BE_STREAM);
    be->launches++;
    be->route_n_used = n_used;
    be->route_n_tok = n_tok;
}

static int x_mode_of(uint64_t rows, uint64_t picks) { return rows == picks ? 0 : (rows > 1 ? 1 : 2); }

static bool host_ids_in_range(it_hip* be, const it_route* r, uint64_t n_expert, const char* who) {
    if (r->kind != IT_ROUTE_HOST) return true;  // device ids come from route_topk over n_expert columns
    for (uint64_t i = 0; i < r->n_used * r->n_tok; i++)
        if (r->ids[i] >= n_expert) {
            be->fail(std::string(who) + ": expert id out of range");
            return false;
        }
    return true;
}

void it_hip_matmul_experts(it_hip* be, const it_experts* w, const it_route* route, const float* x,
                           uint64_t x_len, float* out, uint64_t out_len) {
    ExpertsView v;
    if (!be->experts_view(w, "matmul_experts", &v)) return;
    REQUIRE(route && (route->kind == IT_ROUTE_DEVICE || route->ids), "matmul_experts: null route");
    if (!host_ids_in_range(be, route, w->n_expert, "matmul_experts")) return;
    const int32_t* ids;
    const float* rw;
    uint64_t n_used, n_tok;
    if (!be->route_stage(route, &ids, &rw, &n_used, &n_tok)) return;
    uint64_t picks = n_used * n_tok;
    REQUIRE(x_len % w->n_in == 0, "matmul_experts: x.len() must be a multiple of n_in");
    uint64_t rows = x_len / w->n_in;
    REQUIRE(rows == picks || rows == n_tok || rows == 1, "matmul_experts: x must hold one row per pick, per token, or one row");
    REQUIRE(out_len == picks * w->n_out, "matmul_experts: out.len() must be picks * n_out");
    if (picks == 0) return;
    REQUIRE(picks <= 65535, "matmul_experts: more than 65535 picks in one call");
    const float* as;
    const int8_t* aq;
    if (!be->act_quantized(x, x_len, &as, &aq, nullptr)) return;
    float* dout = be->act_out(out, out_len);
    if (!dout) return;
    matmul_experts(v, ids, (int)picks, (int)n_used, x_mode_of(rows, picks), as, aq, dout, BE_STREAM);
    be->launches++;
    be->expert_lookups += picks;
}

void it_hip_moe_glu(it_hip* be, const it_experts* gate, const it_experts* up, const it_route* route,
                    const float* x, uint64_t x_len, float* out, uint64_t out_len, float* scratch,
                    uint64_t scratch_len) {
    (void)scratch;
    (void)scratch_len;
    ExpertsView g, u;
    if (!be->experts_view(gate, "moe_glu(gate)", &g) || !be->experts_view(up, "moe_glu(up)", &u)) return;
    REQUIRE(gate->ty == up->ty && gate->n_in == up->n_in && gate->n_out == up->n_out && gate->n_expert == up->n_expert,
            "moe_glu: gate and up must have the same type and shape");
    REQUIRE(route && (route->kind == IT_ROUTE_DEVICE || route->ids), "moe_glu: null route");
    if (!host_ids_in_range(be, route, gate->n_expert, "moe_glu")) return;
    const int32_t* ids;
    const float* rw;
    uint64_t n_used, n_tok;
    if (!be->route_stage(route, &ids, &rw, &n_used, &n_tok)) return;
    uint64_t picks = n_used * n_tok;
    REQUIRE(x_len % gate->n_in == 0, "moe_glu: x.len() must be a multiple of n_in");
    uint64_t rows = x_len / gate->n_in;
    REQUIRE(rows == picks || rows == n_tok || rows == 1, "moe_glu: x must hold one row per pick, per token, or one row");
    REQUIRE(out_len == picks * gate->n_out, "moe_glu: out.len() must be picks * n_out");
    if (picks == 0) return;
    REQUIRE(picks <= 65535, "moe_glu: more than 65535 picks in one call");
    const float* as;
    const int8_t* aq;
    if (!be->act_quantized(x, x_len, &as, &aq, nullptr)) return;
    float* dout = be->act_out(out, out_len);
    if (!dout) return;
    moe_glu(g, u, ids, (int)picks, (int)n_used, x_mode_of(rows, picks), as, aq, dout, BE_STREAM);
    be->launches++;
    be->expert_lookups += 2 * picks;
}

void it_hip_moe_finish(it_hip* be, float* out, uint64_t out_len, uint64_t at, uint64_t n, const float* rows,
                       uint64_t rows_len, const it_route* route, const float* shared, uint64_t shared_len,
                       const float* logit, uint64_t logit_len, uint64_t logit_at) {
    REQUIRE(route && (route->kind == IT_ROUTE_DEVICE || route->weights), "moe_finish: null route");
    const int32_t* ids;
    const float* rw;
    uint64_t n_used, n_tok;
    if (route->kind == IT_ROUTE_HOST) {
        // weights only: stage them without needing ids
        uint64_t picks = route->n_used * route->n_tok;
        REQUIRE(picks > 0, "moe_finish: empty route");
        if (!be->route_reserve((size_t)picks)) return;
        if (!be->check(hipMemcpyAsync(be->route_w, route->weights, picks * 4, hipMemcpyHostToDevice, be->stream), "upload weights")) return;
        be->check(hipStreamSynchronize(be->stream), "upload weights");
        be->route_n_used = route->n_used;
        be->route_n_tok = route->n_tok;
        rw = be->route_w;
        n_used = route->n_used;
        n_tok = route->n_tok;
    } else if (!be->route_stage(route, &ids, &rw, &n_used, &n_tok)) {
        return;
    }
    REQUIRE(n > 0 && rows_len == n_tok * n_used * n, "moe_finish: rows.len() must be n_tok * n_used * n");
    REQUIRE(shared_len >= n_tok * n, "moe_finish: shared is shorter than n_tok * n");
    REQUIRE(logit_at + n_tok <= logit_len, "moe_finish: logit index out of range");
    REQUIRE(at + n_tok * n <= out_len, "moe_finish: writes past the end of out");
    REQUIRE(n < (1ull << 31) && n_tok < (1ull << 31), "moe_finish: sizes out of range");
    float* dr = be->act_in(rows, rows_len);
    float* ds = be->act_in(shared, shared_len);
    float* dl = be->act_in(logit, logit_len);
    // rows outside [at, at + n_tok*n) keep their contents, so a stale mirror must be current first
    bool covers_all = (at == 0 && n_tok * n == out_len);
    float* dout = covers_all ? be->act_out(out, out_len) : be->act_inout(out, out_len);
    if (!dr || !ds || !dl || !dout) return;
    moe_finish(dout, (int64_t)at, (int)n, dr, rw, (int)n_tok, (int)n_used, ds, dl, (int64_t)logit_at, BE_STREAM);
    be->launches++;
}

void it_hip_add_scaled_rows(it_hip* be, float* acc, uint64_t acc_len, const float* rows, uint64_t rows_len,
                            const float* scales, uint64_t scales_len) {
    REQUIRE(rows_len == scales_len * acc_len, "add_scaled_rows: rows.len() must be scales.len() * acc.len()");
    if (acc_len == 0) return;
    REQUIRE(scales_len < (1ull << 31), "add_scaled_rows: too many rows");
    float* dr = be->act_in(rows, rows_len);
    float* dsc = be->act_in(scales, scales_len);
    float* da = be->act_out(acc, acc_len);
    if (!dr || !dsc || !da) return;
    add_scaled_rows(da, (int64_t)acc_len, dr, dsc, (int)scales_len, BE_STREAM);
    be->launches++;
}

void it_hip_add_scaled_sigmoid(it_hip* be, float* acc, uint64_t acc_len, const float* b, uint64_t b_len,
                               const float* logit, uint64_t logit_len) {
    REQUIRE(acc_len == b_len && logit_len >= 1, "add_scaled_sigmoid: acc and b must match and logit be non-empty");
    if (acc_len == 0) return;
    float* da = be->act_inout(acc, acc_len);
    float* db = be->act_in(b, b_len);
    float* dl = be->act_in(logit, logit_len);
    if (!da || !db || !dl) return;
    add_scaled_sigmoid(da, db, (int64_t)acc_len, dl, BE_STREAM);
    be->launches++;
}

void it_hip_kv_write(it_hip* be, uint16_t* slab, uint64_t slab_len, uint64_t offset, const float* src,
                     uint64_t src_len) {
    REQUIRE(offset + src_len <= slab_len, "kv_write: writes past the end of the slab");
    if (src_len == 0) return;
    float* ds = be->act_in(src, src_len);
    uint16_t* dslab = (uint16_t*)be->slab_in(slab, slab_len * 2, false);
    if (!ds || !dslab) return;
    kv_write(dslab, (int64_t)offset, nullptr, 0, ds, (int64_t)src_len, BE_STREAM);
    be->launches++;
}

// ------------------------------------------------------------------ residency
void it_hip_host_wrote(it_hip* be, const float* buf, uint64_t len) {
    (void)len;
    auto it = be->acts.find(buf);
    if (it != be->acts.end()) {
        it->second.dev_current = false;
        it->second.q_valid = false;
    }
}

void it_hip_host_needs(it_hip* be, float* buf, uint64_t len) {
    auto it = be->acts.find(buf);
    if (it == be->acts.end() || !it->second.dev_current) return;
    if (be->in_pass) be->mid_pass_read = true;
    size_t n = len < it->second.cap ? len : it->second.cap;
    if (!be->check(hipMemcpyAsync(buf, it->second.dev, n * sizeof(float), hipMemcpyDeviceToHost, be->stream), "download activation")) return;
    be->check(hipStreamSynchronize(be->stream), "download activation");
    be->d2h++;
    be->d2h_bytes += n * 4;
}

void it_hip_begin_pass(it_hip* be, uint64_t n_tokens) {
    be->in_pass = true;
    be->pass_tokens = n_tokens;
    for (auto& kv : be->acts) {
        kv.second.dev_current = false;
        kv.second.q_valid = false;
    }
}

void it_hip_end_pass(it_hip* be) { be->in_pass = false; }

void it_hip_forget_state(it_hip* be) {
    for (auto& kv : be->slabs)
        if (kv.second.is_state) kv.second.dev_owned = false;
}

void it_hip_read_state(it_hip* be, float* host, uint64_t len) {
    auto it = be->slabs.find(host);
    if (it == be->slabs.end() || !it->second.dev_owned) return;
    size_t bytes = len * 4 < it->second.bytes ? len * 4 : it->second.bytes;
    if (!be->check(hipMemcpyAsync(host, it->second.dev, bytes, hipMemcpyDeviceToHost, be->stream), "download state")) return;
    be->check(hipStreamSynchronize(be->stream), "download state");
    be->d2h++;
    be->d2h_bytes += bytes;
}

void it_hip_read_kv(it_hip* be, uint16_t* slab, uint64_t len) {
    auto it = be->slabs.find(slab);
    if (it == be->slabs.end() || !it->second.dev_owned) return;
    size_t bytes = len * 2 < it->second.bytes ? len * 2 : it->second.bytes;
    if (!be->check(hipMemcpyAsync(slab, it->second.dev, bytes, hipMemcpyDeviceToHost, be->stream), "download kv")) return;
    be->check(hipStreamSynchronize(be->stream), "download kv");
    be->d2h++;
    be->d2h_bytes += bytes;
}

// ------------------------------------------------------------------ reports
void it_hip_device_report(it_hip* be) {
    fprintf(stderr, "[hip] launches %llu  h2d %llu (%.1f MiB)  d2h %llu (%.1f MiB)  weights %.1f MiB  kv+state %.1f MiB\n",
            (unsigned long long)be->launches, (unsigned long long)be->h2d, be->h2d_bytes / 1048576.0,
            (unsigned long long)be->d2h, be->d2h_bytes / 1048576.0, be->weight_bytes / 1048576.0,
            be->kv_bytes / 1048576.0);
}
void it_hip_reserve_activations(it_hip* be, uint64_t bytes) { (void)be; (void)bytes; }

int it_hip_tier_counters(it_hip* be, it_tier_counters* out) {
    if (!out) return 0;
    memset(out, 0, sizeof *out);
    size_t fr = 0, tot = 0;
    (void)hipMemGetInfo(&fr, &tot);
    out->vram_free = fr;
    out->vram_total = tot;
    out->lookups = be->expert_lookups;
    out->slot_bytes = be->expert_slot_bytes;
    out->slots = be->expert_resident;
    out->mirrors = be->acts.size();
    out->mirror_bytes = be->mirror_bytes;
    out->weight_bytes = be->weight_bytes;
    out->kv_bytes = be->kv_bytes;
    out->quant_bytes = be->quant_bytes;
    out->pool_bytes = be->attn_scratch_cap * 4;
    out->resident_bytes = be->weight_bytes + be->kv_bytes + be->quant_bytes + be->mirror_bytes +
                          be->const_bytes + out->pool_bytes;
    out->oversubscribed = 0;
    return 1;
}

size_t it_hip_config_report(it_hip* be, char* buf, size_t buf_len) {
    int n = snprintf(buf, buf_len,
                     "backend=hip gfx950\nreductions=%s\ndecode graph=%s\nattention=%s\nexpert tier=all-resident\n",
                     be->exact ? "serial (CPU order)" : "tree / split-K", be->allow_graph ? "on" : "off",
                     be->exact ? "exact" : "split-K flash decoding (128-position chunks)");
    return n < 0 ? 0 : (size_t)n;
}

uint64_t it_hip_setup_cost(it_hip* be, char* label, size_t label_len) {
    if (label && label_len) snprintf(label, label_len, "weight upload and repack");
    return be->setup_us;
}
void it_hip_prefetch_hint(it_hip* be, const it_weights* w, const float* x, uint64_t x_len, uint64_t k) {
    (void)be; (void)w; (void)x; (void)x_len; (void)k;  // every expert is resident: nothing to fetch
}

void it_hip_set_expert_budget(it_hip* be, uint64_t bytes) { be->expert_budget = bytes; }
void it_hip_set_expert_host_budget(it_hip* be, uint64_t bytes) { be->expert_host_budget = bytes; }
void it_hip_set_expert_slots(it_hip* be, uint64_t n) { be->expert_slots_req = n; }
void it_hip_set_expert_pool(it_hip* be, uint64_t n) { be->expert_pool = n; }
void it_hip_expert_stats(it_hip* be, it_expert_stats* out) {
    if (!out) return;
    memset(out, 0, sizeof *out);
    out->slots = be->expert_resident;
    out->slot_bytes = be->expert_slot_bytes;
    out->resident = be->expert_resident;
    out->pool = be->expert_pool;
    out->lookups = be->expert_lookups;
    out->hits = be->expert_lookups;
}

// GCLOCK (src/ops/cuda/experts.rs:2215-2233): sweep from the hand, skipping leased
// slots; a slot with heat left loses one and is passed over; the first with none is
// the victim.  Two full sweeps bound the walk (heat is at most HEAT_MAX = 3 ... the
// caller's counters decide; the bound below is n * 256 steps).
int64_t it_hip_clock_pick(uint8_t* heat, const uint8_t* leased, uint64_t n, uint64_t* hand) {
    if (n == 0) return -1;
    bool any_free = false;
    for (uint64_t i = 0; i < n; i++) any_free |= !leased[i];
    if (!any_free) return -1;
    for (uint64_t step = 0; step < n * 256 + 1; step++) {
        uint64_t i = *hand % n;
        *hand = (i + 1) % n;
        if (leased[i]) continue;
        if (heat[i] == 0) return (int64_t)i;
        heat[i]--;
    }
    return -1;
}

// ------------------------------------------------------------------ extensions
uint32_t it_hip_argmax(it_hip* be, const float* buf, uint64_t len) {
    if (len == 0) return 0;
    float* d = be->act_in(buf, len);
    if (!d) return 0;
    if (!be->argmax_idx) {
        if (!be->check(hipMalloc((void**)&be->argmax_idx, 64 * 4), "hipMalloc(argmax)") ||
            !be->check(hipMalloc((void**)&be->argmax_val, 64 * 4), "hipMalloc(argmax)") ||
            !be->check(hipMalloc((void**)&be->argmax_out, 4), "hipMalloc(argmax)") ||
            !be->check(hipHostMalloc((void**)&be->argmax_host, 4, hipHostMallocDefault), "hipHostMalloc(argmax)"))
            return 0;
    }
    argmax(d, (int64_t)len, be->argmax_out, be->argmax_idx, be->argmax_val, be->stream);
    be->launches += 2;
    if (!be->check(hipMemcpyAsync(be->argmax_host, be->argmax_out, 4, hipMemcpyDeviceToHost, be->stream), "download argmax")) return 0;
    be->check(hipStreamSynchronize(be->stream), "download argmax");
    be->d2h++;
    be->d2h_bytes += 4;
    return (uint32_t)*be->argmax_host;
}

void it_hip_sync(it_hip* be) { be->check(hipStreamSynchronize(be->stream), "sync"); }
void it_hip_drop_mirrors(it_hip* be) { be->drop_all(); }
uint64_t it_hip_launch_count(it_hip* be) { return be->launches; }

}  // extern "C"
