// The HIP backend: residency, validation and dispatch for every seam op.
//
// Each op validates its operand shapes on the host before anything is launched
// (a kernel never sees a shape its grid does not cover), records the first error
// and keeps going, as the reference's device backend does
// (/root/reference src/ops/cuda/ops/mod.rs:91-110).
#include "backend.h"

#include <mutex>

#include <chrono>
#include <cmath>
#include <cstdio>
#include <algorithm>
#include <cstdlib>
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
// A cheap identity of a host weight: its length and 48 sampled bytes.  Resident copies are keyed on the host address,
// and a second model file mapped where the first one was has the same addresses, types and shapes.
uint64_t weight_ident(const uint8_t* data, uint64_t len) {
    uint64_t h = 0xcbf29ce484222325ull ^ len;
    auto mix = [&](const uint8_t* p, uint64_t n) {
        for (uint64_t i = 0; i < n; i++) h = (h ^ p[i]) * 0x100000001b3ull;
    };
    const uint64_t n = len < 16 ? len : 16;
    mix(data, n);
    mix(data + (len - n) / 2, n);
    mix(data + len - n, n);
    return h;
}
uint64_t now_us() {
    return (uint64_t)std::chrono::duration_cast<std::chrono::microseconds>(
               std::chrono::steady_clock::now().time_since_epoch())
        .count();
}
}  // namespace

// FNV-1a over the raw bytes of each argument
template <class... A>
static uint64_t sig_of(const A&... a) {
    uint64_t h = 0xcbf29ce484222325ull;
    auto mix = [&](const void* p, size_t n) {
        const uint8_t* b = (const uint8_t*)p;
        for (size_t i = 0; i < n; i++) h = (h ^ b[i]) * 0x100000001b3ull;
    };
    (mix(&a, sizeof(a)), ...);
    return h;
}

const int* it_hip::dyn_slot(int value) {
    if (mode == Mode::Eager) return nullptr;
    if (dyn_count >= DYN_CAP) {
        need_eager("too many position-dependent launches in one pass");
        return nullptr;
    }
    dyn_host[dyn_count] = value;
    return dyn_dev + dyn_count++;
}

void it_hip::dyn_rotate() {
    dyn_cur ^= 1;
    if (dyn_evt_used[dyn_cur]) check(hipEventSynchronize(dyn_evt[dyn_cur]), "wait for the position staging buffer");
    dyn_evt_used[dyn_cur] = false;
    dyn_host = dyn_hosts[dyn_cur];
    dyn_count = 0;
}
void it_hip::dyn_upload() {
    if (!dyn_count) return;
    // a token's pass has a few dozen: they go with a small kernel's arguments (between two replayed passes a
    // host-to-device copy is a transfer the stream waits for); a long pass's thousands are copied
    if (itk::poke_ints(dyn_dev, dyn_host, (int)dyn_count, stream)) return;
    check(hipMemcpyAsync(dyn_dev, dyn_host, dyn_count * sizeof(int), hipMemcpyHostToDevice, stream), "upload positions");
    if (hipEventRecord(dyn_evt[dyn_cur], stream) == hipSuccess) dyn_evt_used[dyn_cur] = true;
}

void it_hip::drop_graph() {
    if (graph.exec) (void)hipGraphExecDestroy(graph.exec);
    if (graph.graph) (void)hipGraphDestroy(graph.graph);
    graph.exec = nullptr;
    graph.graph = nullptr;
    graph.valid = false;
    graph.signature.clear();
    graph.attn_slots.clear();
    stable_passes = 0;
}

// what a deferred pass has recorded so far goes to the stream, fused; the pass stays deferred
void it_hip::flush_deferred() {
    if (chain_enabled && fuse_enabled && !exact && !expert_cold_entries && (!itk::layer_chain_fits() || !chain_acquire())) chain_enabled = false;
    for (auto& c : precopies) check(hipMemcpyAsync(c.dev, c.host, c.bytes, hipMemcpyHostToDevice, stream), "upload activation");
    precopies.clear();
    dyn_upload();
    if (pending.empty()) return;
    auto todo = std::move(pending);
    pending.clear();
    run_fused(todo);
    check(hipGetLastError(), "kernel launch");
    mark_elided(fused_elided);
    if (chain_launches) chain_ran = true;
}

void it_hip::need_eager(const char* why) {
    if (!held.empty()) release_held();   // whatever follows (a copy, a free, a wait) must find the stream complete
    if (mode == Mode::Eager) return;
    (void)why;
    if (mode == Mode::Deferred) {
        flush_deferred();
        return;
    }
    drop_graph();
    graph_aborts++;
    mode = Mode::Eager;
    for (auto& c : precopies) check(hipMemcpyAsync(c.dev, c.host, c.bytes, hipMemcpyHostToDevice, stream), "upload activation");
    precopies.clear();
    dyn_upload();
    auto todo = std::move(pending);
    pending.clear();
    for (auto& op : todo) op.run(stream);
    check(hipGetLastError(), "kernel launch");
}

void it_hip::finish_pass() {
    if (!held.empty()) release_held();
    if (mode == Mode::Deferred) {
        flush_deferred();
        mode = Mode::Eager;
        stable_passes = 0;
        return;
    }
    if (mode == Mode::Eager) {
        if (pass_tokens == 1 && allow_graph && !mid_pass_read && !prof_on) {
            stable_passes = (pass_signature == prev_signature && !pass_signature.empty()) ? stable_passes + 1 : 0;
            prev_signature = pass_signature;
        } else {
            stable_passes = 0;
        }
        return;
    }
    if (mode == Mode::Capture) {
        // inputs first (they are not part of the graph), then record the fused pass
        for (auto& c : precopies) check(hipMemcpyAsync(c.dev, c.host, c.bytes, hipMemcpyHostToDevice, stream), "upload activation");
        precopies.clear();
        hipGraph_t g = nullptr;
        // a chain's hand-off space is allocated and cleared here: neither is allowed while the stream is capturing
        if (chain_enabled && fuse_enabled && !exact && (!itk::layer_chain_fits() || !chain_acquire())) chain_enabled = false;
        hipError_t e = hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed);
        if (e == hipSuccess) {
            run_fused(pending);
            hipError_t le = hipGetLastError();
            e = hipStreamEndCapture(stream, &g);
            if (le != hipSuccess) e = le;
        }
        mode = Mode::Eager;
        if (e == hipSuccess && g) {
            hipGraphExec_t ex = nullptr;
            e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
            if (e == hipSuccess && ex) {
                drop_graph();
                graph.graph = g;
                graph.exec = ex;
                graph.signature = pass_signature;
                graph.attn_slots = fused_attn_slots;
                graph.elided = fused_elided;
                graph.has_chain = chain_launches > 0;
                graph.valid = true;
                graph_captures++;
                stable_passes = 1;
            } else if (g) {
                (void)hipGraphDestroy(g);
            }
        }
        (void)hipGetLastError();
        if (!graph.valid) {  // could not build a graph: run the pass eagerly
            mode = Mode::Replay;  // reuse the fallback path
            need_eager("graph instantiation failed");
            allow_graph = false;
            return;
        }
    } else {  // Replay
        mode = Mode::Eager;
        if (replay_cursor != graph.signature.size()) {
            mode = Mode::Replay;
            need_eager("the pass ended early");
            return;
        }
        if (!attn_positions_agree(graph.attn_slots)) {
            mode = Mode::Replay;
            need_eager("a fused attention block's rope, cache-write and context positions do not agree");
            return;
        }
    }
    for (auto& c : precopies) check(hipMemcpyAsync(c.dev, c.host, c.bytes, hipMemcpyHostToDevice, stream), "upload activation");
    precopies.clear();
    dyn_upload();
    if (profile_pass) {
        run_fused(pending);  // the launches the graph holds, each between two events
        check(hipGetLastError(), "kernel launch");
    } else {
        check(hipGraphLaunch(graph.exec, stream), "hipGraphLaunch");
        graph_launches++;
    }
    mark_elided(graph.elided);
    if (graph.has_chain) chain_ran = true;
    pending.clear();
}

bool it_hip::attn_positions_agree(const std::vector<std::array<int, 4>>& slots) const {
    for (const auto& t : slots) {
        for (int i : t)
            if (i < 0 || (size_t)i >= dyn_count) return false;
        const int pos = dyn_host[t[0]];
        if (dyn_host[t[1]] != pos || dyn_host[t[2]] != pos || dyn_host[t[3]] != pos + 1) return false;
    }
    return true;
}

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
        need_eager("an activation mirror has to grow");
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
    if (a->dev_current && a->elided) {
        fail("an op reads a buffer whose producer was folded into a fused kernel that does not write it");
        return nullptr;
    }
    if (!a->dev_current) {
        if (mode != Mode::Eager) {
            precopies.push_back(PreCopy{a->dev, host, len * sizeof(float)});
        } else {
            // ops held back run later than this copy: if one of them touches the buffer, it has to run first
            if (!held.empty() && held_touches(a->dev, a->cap * sizeof(float))) release_held();
            if (!check(hipMemcpyAsync(a->dev, host, len * sizeof(float), hipMemcpyHostToDevice, stream), "upload activation"))
                return nullptr;
        }
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
    a->elided = false;
    a->q_valid = false;
    return a->dev;
}
bool it_hip::held_touches(const void* dev, size_t bytes) const {
    const char* lo = (const char*)dev;
    for (const OpRec& op : held)
        for (const void* q : op.p)
            if (q && (const char*)q >= lo && (const char*)q < lo + bytes) return true;
    return false;
}
it_hip::Act* it_hip::act_by_dev(const void* dev) {
    for (auto& kv : acts) {
        const char* base = (const char*)kv.second.dev;
        if (base && (const char*)dev >= base && (const char*)dev < base + kv.second.cap * sizeof(float)) return &kv.second;
    }
    return nullptr;
}
void it_hip::mark_elided(const std::vector<const void*>& devs) {
    for (const void* d : devs)
        if (Act* a = act_by_dev(d)) a->elided = true;
}
float* it_hip::act_inout(const float* host, size_t len) {
    float* d = act_in(host, len);
    if (d) acts[host].q_valid = false;
    return d;
}

bool it_hip::act_q_reserve(Act& a, size_t len) {
    if (a.q_cap >= len) return true;
    need_eager("a quantized-activation buffer has to grow");
    if (a.q_scales) {
        check(hipStreamSynchronize(stream), "sync before quant free");
        quant_bytes -= a.q_cap / 32 * 4 + a.q_cap;
        (void)hipFree(a.q_scales);
        (void)hipFree(a.q_quants);
        a.q_scales = nullptr;
        a.q_quants = nullptr;
        a.q_cap = 0;
    }
    if (!check(hipMalloc((void**)&a.q_scales, (len / 32 + 1) * sizeof(float)), "hipMalloc(q8 scales)") ||
        !check(hipMalloc((void**)&a.q_quants, len + 32), "hipMalloc(q8 quants)"))
        return false;
    a.q_cap = len;
    quant_bytes += len / 32 * 4 + len;
    a.q_valid = false;
    return true;
}

bool it_hip::act_quantized(const float* host, size_t len, const float** scales, const int8_t** quants,
                           float** dev_x) {
    float* x = act_in(host, len);
    if (!x) return false;
    Act& a = acts[host];
    if (!act_q_reserve(a, len)) return false;
    if (!a.q_valid || a.q_len != len) {
        float* qs = a.q_scales;
        int8_t* qq = a.q_quants;
        OpRec rec;
        rec.id = 101;  // OP_QUANT
        rec.p[0] = x; rec.p[1] = qs; rec.p[2] = qq; rec.i[0] = (int64_t)len;
        submit(FAM_OTHER, len * 5, sig_of(101, x, qs, qq, len), rec,
               [=](hipStream_t s) { quantize_q8_0(x, qs, qq, (int64_t)len, s); });
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
    const uint64_t ident = weight_ident((const uint8_t*)host, len * sizeof(float));
    if (it != consts.end() && it->second.len == len && it->second.ident == ident) return it->second.dev;
    need_eager("a constant is uploaded for the first time");
    if (it != consts.end()) drop_graph();  // a captured graph holds the copy that is about to go
    Const c;
    c.ident = ident;
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
    uint64_t row_bytes = type_row_bytes(ty, n_in);
    if (row_bytes == 0) {
        fail(std::string(who) + ": unsupported weight type or row length not a whole number of blocks");
        return nullptr;
    }
    if (len != row_bytes * rows) {
        fail(std::string(who) + ": weight byte length does not match its shape");
        return nullptr;
    }
    auto it = weights.find(data);
    if (it != weights.end()) {
        const bool same_shape = it->second.fmt == (int)ty && it->second.n_in == n_in && it->second.rows == rows;
        if (same_shape && it->second.ident == weight_ident(data, len)) return &it->second;
        if (same_shape && it->second.counter_base < 0) {
            // the same address, type and shape but other bytes: another file was mapped where the last one was.
            // The stale copy goes and the weight is uploaded again.  (An expert tensor keeps its slots and counters
            // for the life of the pool: that case is refused below.)
            need_eager("a resident weight no longer matches its host bytes");
            drop_graph();
            check(hipStreamSynchronize(stream), "sync before a stale weight is freed");
            weight_bytes -= it->second.q_bytes + it->second.s_bytes;
            if (it->second.q) (void)hipFree(it->second.q);
            if (it->second.scales) (void)hipFree(it->second.scales);
            if (it->second.scale2) (void)hipFree(it->second.scale2);
            weights.erase(it);
        } else {
            fail(std::string(who) + (same_shape ? ": a pooled expert tensor changed under its address; call drop_mirrors when a model file is unmapped"
                                                : ": a weight address was seen before with a different shape"));
            return nullptr;
        }
    }
    need_eager("a weight is uploaded for the first time");
    uint64_t t0 = now_us();
    Resident r;
    r.fmt = (int)ty;
    r.n_in = n_in;
    r.rows = rows;
    r.ident = weight_ident(data, len);
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
        check(hipStreamSynchronize(stream), "repack q8_0");
        (void)hipFree(raw);
    } else if (ty == IT_NVFP4) {
        r.q_bytes = rows * (n_in / 2);
        r.s_bytes = rows * (n_in / 16);
        if (!check(hipMalloc(&r.q, r.q_bytes), "hipMalloc(nvfp4 nibbles)") ||
            !check(hipMalloc(&r.scales, r.s_bytes), "hipMalloc(nvfp4 scales)"))
            return nullptr;
        repack_nvfp4((const uint8_t*)raw, (uint8_t*)r.q, (uint8_t*)r.scales, (int64_t)rows, (int)n_in, stream);
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
    if (fresh) {
        // the slab's slot is one expert matrix of the first pooled tensor; a tensor of another size does not fit
        // the arena (src/ops/cuda/experts.rs:890-901, 1621-1630)
        const uint64_t one = type_row_bytes(w->ty, w->n_in) * w->n_out;
        if (one == 0 || w->len != one * w->n_expert) {
            fail(std::string(who) + ": expert tensor length is not n_expert matrices of its shape");
            return false;
        }
        if (expert_slot_bytes && expert_slot_bytes != one) {
            fail(std::string(who) + ": expert matrix is " + std::to_string(one) + " bytes but the slab's slot is " +
                 std::to_string(expert_slot_bytes) + "; the pool is not uniform, which this arena assumes");
            return false;
        }
        if (!expert_slot_bytes) {
            // sized at the first pooled tensor, from what is free then (placement.rs:294-312, 423-453)
            expert_slot_bytes = one;
            size_t fr = 0, tot = 0;
            (void)hipMemGetInfo(&fr, &tot);
            const uint64_t by_budget = expert_budget ? expert_budget : (fr > expert_reserve ? fr - expert_reserve : 0);
            expert_slots_cap = expert_slots_req ? expert_slots_req : by_budget / one;
        }
        if (!expert_counters_reserve(expert_counted + w->n_expert)) return false;
    }
    if (fresh && expert_resident + w->n_expert > expert_slots_cap) {
        // The pool outgrows the device tier: the experts that still fit take device slots, the rest go to pinned host
        // memory, and from here on every pooled tensor is read through its placement table.
        const uint64_t free_slots = expert_slots_cap > expert_resident ? expert_slots_cap - expert_resident : 0;
        if (!place_two_tier(w, std::min<uint64_t>(free_slots, w->n_expert), who)) return false;
    } else {
        const Resident* r = resident(w->data, w->len, w->ty, w->n_in, w->n_out * w->n_expert, who);
        if (!r) return false;
        if (fresh) {
            expert_resident += w->n_expert;
            Resident& nr = weights[w->data];
            nr.n_expert = w->n_expert;
            nr.q_stride = nr.q_bytes / w->n_expert;
            nr.s_stride = nr.s_bytes / w->n_expert;
            if (pool_tabled && !table_for(nr)) return false;
        }
    }
    if (fresh) {
        const uint64_t placed = expert_resident + expert_host_entries + expert_cold_entries;
        if (expert_pool < placed) expert_pool = placed;
        weights[w->data].counter_base = (int64_t)expert_counted;
        expert_counted += w->n_expert;
        cold_ring_changed();
    }
    Resident* rw = &weights[w->data];
    if (w->scale && w->scale_len && !rw->scale2) {
        need_eager("expert scales are uploaded for the first time");
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
    out->counts = rw->counter_base >= 0 ? expert_counts + rw->counter_base : nullptr;
    out->q_tab = rw->q_tab;
    out->s_tab = rw->s_tab;
    out->tier = rw->tier;
    return true;
}

// ------------------------------------------------------------------ two-tier placement
// src/ops/cuda/experts.rs:34-62: an expert lives in a device slot or in a page-locked host block that the device
// addresses directly, so a kernel dereferences it either way and a miss is slow, never blocking.  Placement is first
// touch wins device memory; replace_by_counts() later exchanges busy host experts with idle device ones.
static constexpr uint64_t DEFAULT_EXPERT_HOST_BUDGET = 64ull << 30;

bool it_hip::table_upload(Resident& r) {
    const size_t n = r.n_expert;
    if (!r.q_tab) {
        if (!check(hipMalloc((void**)&r.q_tab, n * sizeof(void*)), "hipMalloc(expert table)") ||
            !check(hipMalloc((void**)&r.s_tab, n * sizeof(void*)), "hipMalloc(expert table)") ||
            !check(hipMalloc((void**)&r.tier, n), "hipMalloc(expert tiers)"))
            return false;
    }
    return check(hipMemcpy(r.q_tab, r.h_q.data(), n * sizeof(void*), hipMemcpyHostToDevice), "upload expert table") &&
           check(hipMemcpy(r.s_tab, r.h_s.data(), n * sizeof(void*), hipMemcpyHostToDevice), "upload expert table") &&
           check(hipMemcpy(r.tier, r.h_tier.data(), n, hipMemcpyHostToDevice), "upload expert tiers");
}

bool it_hip::table_for(Resident& r) {
    if (r.q_tab || !r.n_expert) return true;
    need_eager("an expert tensor gets a placement table");
    drop_graph();   // a captured graph reads this tensor at its stride
    check(hipStreamSynchronize(stream), "sync before an expert table is made");
    r.h_q.resize(r.n_expert);
    r.h_s.resize(r.n_expert);
    r.h_tier.assign(r.n_expert, 0);
    for (uint64_t e = 0; e < r.n_expert; e++) {
        r.h_q[e] = (const uint8_t*)r.q + e * r.q_stride;
        r.h_s[e] = (const uint8_t*)r.scales + e * r.s_stride;
    }
    return table_upload(r);
}

bool it_hip::place_two_tier(const it_experts* w, uint64_t n_dev, const char* who) {
    const uint64_t n = w->n_expert;
    const uint64_t raw_one = type_row_bytes(w->ty, w->n_in) * w->n_out;
    const bool q8 = w->ty == IT_Q8_0;
    const uint64_t q_stride = q8 ? w->n_out * w->n_in : w->n_out * (w->n_in / 2);
    const uint64_t s_stride = q8 ? w->n_out * (w->n_in / 32) * 2 : w->n_out * (w->n_in / 16);
    const uint64_t budget = expert_host_budget ? expert_host_budget : DEFAULT_EXPERT_HOST_BUDGET;
    // what the pinned tier still takes; the rest of the tensor is cold: no copy is made, the entries point at the
    // sentinel, and a pick is fetched from the file when a layer asks for it (experts.rs:969-980)
    const uint64_t room = budget > expert_host_bytes ? (budget - expert_host_bytes) / (q_stride + s_stride) : 0;
    const uint64_t n_host = std::min<uint64_t>(n - n_dev, room), n_cold = n - n_dev - n_host, n_placed = n_dev + n_host;
    need_eager("an expert tensor is placed in two tiers");
    drop_graph();
    check(hipStreamSynchronize(stream), "sync before two-tier placement");
    uint64_t t0 = now_us();
    // every tensor placed so far is read through a table from now on
    if (!pool_tabled) {
        pool_tabled = true;
        for (auto& kv : weights)
            if (kv.second.counter_base >= 0 && !table_for(kv.second)) return false;
    }
    const uint8_t *cold_q = nullptr, *cold_s = nullptr;
    if (n_cold && !cold_sentinel(&cold_q, &cold_s, q_stride, s_stride)) return false;
    Resident r;
    r.fmt = (int)w->ty;
    r.n_in = w->n_in;
    r.rows = w->n_out * n;
    r.ident = weight_ident(w->data, w->len);
    r.n_expert = n;
    r.q_stride = q_stride;
    r.s_stride = s_stride;
    r.q_bytes = n_dev * q_stride;
    r.s_bytes = n_dev * s_stride;
    void *raw = nullptr, *tq = nullptr, *ts = nullptr;
    auto give_up = [&]() {   // a failed placement leaves nothing behind
        for (void* d : {r.q, r.scales, raw, tq, ts, (void*)r.q_tab, (void*)r.s_tab, (void*)r.tier})
            if (d) (void)hipFree(d);
        if (r.host_q) (void)hipHostFree(r.host_q);
        if (r.host_s) (void)hipHostFree(r.host_s);
        return false;
    };
    if (n_dev && (!check(hipMalloc(&r.q, r.q_bytes), "hipMalloc(expert quants)") ||
                  !check(hipMalloc(&r.scales, r.s_bytes), "hipMalloc(expert scales)")))
        return give_up();
    uint8_t *dq_host = nullptr, *ds_host = nullptr;   // the pinned blocks as the device addresses them
    if (n_host) {
        if (!check(hipHostMalloc(&r.host_q, n_host * q_stride, hipHostMallocMapped | hipHostMallocPortable), "hipHostMalloc(expert host tier)") ||
            !check(hipHostMalloc(&r.host_s, n_host * s_stride, hipHostMallocMapped | hipHostMallocPortable), "hipHostMalloc(expert host tier)") ||
            !check(hipHostGetDevicePointer((void**)&dq_host, r.host_q, 0), "hipHostGetDevicePointer") ||
            !check(hipHostGetDevicePointer((void**)&ds_host, r.host_s, 0), "hipHostGetDevicePointer"))
            return give_up();
    }
    // upload and repack a few experts at a time through device staging, then move each to its place; the bytes of a
    // cold expert are not touched
    bool ok = true;
    if (n_placed) {
        const uint64_t chunk = std::min<uint64_t>(8, n_placed);
        if (!check(hipMalloc(&raw, chunk * raw_one), "hipMalloc(expert staging)") ||
            !check(hipMalloc(&tq, chunk * q_stride), "hipMalloc(expert staging)") ||
            !check(hipMalloc(&ts, chunk * s_stride), "hipMalloc(expert staging)"))
            return give_up();
        for (uint64_t e0 = 0; e0 < n_placed && ok; e0 += chunk) {
            const uint64_t m = std::min(chunk, n_placed - e0);
            ok = ok && check(hipMemcpyAsync(raw, w->data + e0 * raw_one, m * raw_one, hipMemcpyHostToDevice, stream), "upload experts");
            if (q8) repack_q8_0((const uint8_t*)raw, (int8_t*)tq, (uint16_t*)ts, (int64_t)(m * w->n_out), (int)w->n_in, stream);
            else repack_nvfp4((const uint8_t*)raw, (uint8_t*)tq, (uint8_t*)ts, (int64_t)(m * w->n_out), (int)w->n_in, stream);
            for (uint64_t k = 0; k < m && ok; k++) {
                const uint64_t e = e0 + k;
                const uint8_t* fq = (const uint8_t*)tq + k * q_stride;
                const uint8_t* fs = (const uint8_t*)ts + k * s_stride;
                if (e < n_dev) {
                    ok = check(hipMemcpyAsync((uint8_t*)r.q + e * q_stride, fq, q_stride, hipMemcpyDeviceToDevice, stream), "place expert") &&
                         check(hipMemcpyAsync((uint8_t*)r.scales + e * s_stride, fs, s_stride, hipMemcpyDeviceToDevice, stream), "place expert");
                } else {
                    ok = check(hipMemcpyAsync((uint8_t*)r.host_q + (e - n_dev) * q_stride, fq, q_stride, hipMemcpyDeviceToHost, stream), "place expert in the host tier") &&
                         check(hipMemcpyAsync((uint8_t*)r.host_s + (e - n_dev) * s_stride, fs, s_stride, hipMemcpyDeviceToHost, stream), "place expert in the host tier");
                }
            }
            ok = ok && check(hipStreamSynchronize(stream), "place experts");
        }
    }
    if (!ok) return give_up();
    (void)hipFree(raw);
    (void)hipFree(tq);
    (void)hipFree(ts);
    raw = tq = ts = nullptr;
    h2d++;
    h2d_bytes += n_placed * raw_one;
    r.h_q.resize(n);
    r.h_s.resize(n);
    r.h_tier.resize(n);
    for (uint64_t e = 0; e < n; e++) {
        const bool dev = e < n_dev, pinned = !dev && e < n_placed;
        r.h_q[e] = dev ? (const uint8_t*)r.q + e * q_stride : pinned ? dq_host + (e - n_dev) * q_stride : cold_q;
        r.h_s[e] = dev ? (const uint8_t*)r.scales + e * s_stride : pinned ? ds_host + (e - n_dev) * s_stride : cold_s;
        r.h_tier[e] = dev ? 0 : pinned ? 1 : 2;
    }
    if (!table_upload(r)) return give_up();
    weight_bytes += r.q_bytes + r.s_bytes;
    expert_resident += n_dev;
    expert_host_entries += n_host;
    expert_host_bytes += n_host * (q_stride + s_stride);
    expert_cold_entries += n_cold;
    expert_cold_at_load += n_cold;
    setup_us += now_us() - t0;
    weights.emplace(w->data, std::move(r));
    (void)who;
    return true;
}

// Exchange busy host-tier experts with idle device-tier ones until every device expert has been read at least as often
// as every host one (replace_experts_by_counts, placement.rs:113-128; the counts are kept).  Returns the exchanges.
// Between passes, never inside one (placement.rs:21-80): every 64 tokens of evidence the busiest host-tier experts
// change places with the idlest device-tier ones, 200 exchanges per 64 tokens and 2,000 per boundary at most, so that a
// boundary cannot turn into a visible stall.  The tables are ordinary device memory: a recorded graph reads the new
// addresses at its next replay, with no re-record.  Stops by itself once no host expert is busier than a device one.
void it_hip::migrate_at_boundary(uint64_t n_tokens) {
    if (!pool_tabled || !expert_host_entries || expert_cold_entries) return;
    tokens_since_migration += n_tokens;
    if (tokens_since_migration < 64) return;
    const uint64_t budget = std::min<uint64_t>(200 * (tokens_since_migration / 64), 2000);
    tokens_since_migration = 0;
    (void)replace_by_counts(budget);
}

int64_t it_hip::replace_by_counts(uint64_t budget) {
    std::vector<uint32_t> counts;
    uint64_t tally[2];
    if (!expert_counters_read(&counts, tally)) return -1;
    // with cold experts every slot change is the fetch path's (leases, heat): migration is paused (experts.rs:1857-1870)
    if (!pool_tabled || !expert_host_entries || expert_cold_entries) return 0;
    struct Entry { Resident* r; uint32_t e; uint32_t count; };
    std::vector<Entry> dev, host;
    for (auto& kv : weights) {
        Resident& r = kv.second;
        if (r.counter_base < 0 || !r.q_tab) continue;
        for (uint64_t e = 0; e < r.n_expert; e++) {
            Entry en{&r, (uint32_t)e, counts[(size_t)r.counter_base + e]};
            (r.h_tier[e] ? host : dev).push_back(en);
        }
    }
    // idle device experts first, busy host experts first; ties by placement order so that the outcome is repeatable
    std::stable_sort(dev.begin(), dev.end(), [](const Entry& a, const Entry& b) {
        return a.count != b.count ? a.count < b.count : (a.r->counter_base + a.e) < (b.r->counter_base + b.e);
    });
    std::stable_sort(host.begin(), host.end(), [](const Entry& a, const Entry& b) {
        return a.count != b.count ? a.count > b.count : (a.r->counter_base + a.e) < (b.r->counter_base + b.e);
    });
    size_t pairs = 0;
    while (pairs < dev.size() && pairs < host.size() && pairs < budget && host[pairs].count > dev[pairs].count) pairs++;
    if (!pairs) return 0;
    need_eager("experts move between tiers");
    if (!check(hipStreamSynchronize(stream), "sync before experts move")) return -1;
    const uint64_t qs = dev[0].r->q_stride, ss = dev[0].r->s_stride;
    void *tq = nullptr, *ts = nullptr;
    if (!check(hipMalloc(&tq, qs), "hipMalloc(expert exchange)") || !check(hipMalloc(&ts, ss), "hipMalloc(expert exchange)")) return -1;
    bool ok = true;
    std::vector<Resident*> touched;
    for (size_t k = 0; k < pairs && ok; k++) {
        Entry &d = dev[k], &h = host[k];
        uint8_t* slot_q = const_cast<uint8_t*>(d.r->h_q[d.e]);
        uint8_t* slot_s = const_cast<uint8_t*>(d.r->h_s[d.e]);
        uint8_t* blk_q = const_cast<uint8_t*>(h.r->h_q[h.e]);   // device-visible addresses of the pinned block
        uint8_t* blk_s = const_cast<uint8_t*>(h.r->h_s[h.e]);
        ok = check(hipMemcpyAsync(tq, slot_q, qs, hipMemcpyDeviceToDevice, stream), "exchange experts") &&
             check(hipMemcpyAsync(ts, slot_s, ss, hipMemcpyDeviceToDevice, stream), "exchange experts") &&
             check(hipMemcpyAsync(slot_q, blk_q, qs, hipMemcpyDefault, stream), "exchange experts") &&
             check(hipMemcpyAsync(slot_s, blk_s, ss, hipMemcpyDefault, stream), "exchange experts") &&
             check(hipMemcpyAsync(blk_q, tq, qs, hipMemcpyDefault, stream), "exchange experts") &&
             check(hipMemcpyAsync(blk_s, ts, ss, hipMemcpyDefault, stream), "exchange experts");
        d.r->h_q[d.e] = blk_q; d.r->h_s[d.e] = blk_s; d.r->h_tier[d.e] = 1;
        h.r->h_q[h.e] = slot_q; h.r->h_s[h.e] = slot_s; h.r->h_tier[h.e] = 0;
        touched.push_back(d.r);
        touched.push_back(h.r);
    }
    ok = ok && check(hipStreamSynchronize(stream), "exchange experts");
    (void)hipFree(tq);
    (void)hipFree(ts);
    std::sort(touched.begin(), touched.end());
    touched.erase(std::unique(touched.begin(), touched.end()), touched.end());
    for (Resident* r : touched) ok = ok && table_upload(*r);
    if (!ok) return -1;
    expert_swaps += pairs;
    return (int64_t)pairs;
}

// the device read counters hold at least `entries` (tensor, expert) entries; existing counts survive a growth
bool it_hip::expert_counters_reserve(size_t entries) {
    if (!expert_tally) {
        if (!check(hipMalloc((void**)&expert_tally, 2 * sizeof(unsigned long long)), "hipMalloc(expert tally)") ||
            !check(hipMemset(expert_tally, 0, 2 * sizeof(unsigned long long)), "hipMemset(expert tally)"))
            return false;
    }
    if (entries <= expert_counts_cap) return true;
    need_eager("the expert read counters have to grow");
    drop_graph();  // a captured graph holds the old array
    size_t cap = std::max<size_t>({entries, 2 * expert_counts_cap, (size_t)expert_pool, (size_t)4096});
    uint32_t* fresh = nullptr;
    if (!check(hipMalloc((void**)&fresh, cap * sizeof(uint32_t)), "hipMalloc(expert read counters)") ||
        !check(hipMemset(fresh, 0, cap * sizeof(uint32_t)), "hipMemset(expert read counters)"))
        return false;
    if (expert_counts) {
        check(hipStreamSynchronize(stream), "sync before the counters move");
        check(hipMemcpy(fresh, expert_counts, expert_counts_cap * sizeof(uint32_t), hipMemcpyDeviceToDevice), "copy expert read counters");
        (void)hipFree(expert_counts);
    }
    expert_counts = fresh;
    expert_counts_cap = cap;
    return true;
}

// Bring the device-side read counters home (absorb_expert_counters, placement.rs:130-152); costs a synchronize
bool it_hip::expert_counters_read(std::vector<uint32_t>* counts, uint64_t tally[2]) {
    tally[0] = tally[1] = 0;
    if (counts) counts->assign(expert_counted, 0);
    if (!expert_tally || !expert_counted) return true;
    if (!held.empty()) release_held();
    if (in_pass) finish_pass();
    if (!check(hipStreamSynchronize(stream), "sync before reading the expert counters")) return false;
    unsigned long long t[2] = {0, 0};
    if (!check(hipMemcpy(t, expert_tally, sizeof t, hipMemcpyDeviceToHost), "download expert tally")) return false;
    tally[0] = t[0];
    tally[1] = t[1];
    if (counts && !check(hipMemcpy(counts->data(), expert_counts, expert_counted * sizeof(uint32_t), hipMemcpyDeviceToHost),
                         "download expert read counters"))
        return false;
    return true;
}

// ------------------------------------------------------------------ slabs
void* it_hip::slab_in(const void* host, size_t bytes, bool is_state) {
    Slab& s = slabs[host];
    if (!s.dev || s.bytes < bytes || !s.dev_owned) need_eager("a slab is uploaded");
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
    need_eager("route storage has to grow");
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
        need_eager("a host route is staged");
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
        route_gen++;
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
    need_eager("the rope table has to grow");
    size_t cap = r.cap_pos ? r.cap_pos : 8192;
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

void* it_hip::moe_f16_for(size_t bytes) {
    if (moe_f16_bytes < bytes) {
        need_eager("expert activation scratch has to grow");
        if (moe_f16) {
            check(hipStreamSynchronize(stream), "sync before scratch free");
            (void)hipFree(moe_f16);
            moe_f16 = nullptr;
            moe_f16_bytes = 0;
        }
        const size_t want = bytes + bytes / 4;
        if (!check(hipMalloc(&moe_f16, want), "hipMalloc(expert activation scratch)")) return nullptr;
        moe_f16_bytes = want;
    }
    return moe_f16;
}

const int32_t* it_hip::zero_ids_for(size_t n) {
    if (zero_ids_n < n) {
        need_eager("the one-expert id list has to grow");
        if (zero_ids) {
            check(hipStreamSynchronize(stream), "sync before scratch free");
            (void)hipFree(zero_ids);
            zero_ids = nullptr;
            zero_ids_n = 0;
        }
        const size_t want = n + n / 2;
        if (!check(hipMalloc((void**)&zero_ids, want * sizeof(int32_t)), "hipMalloc(one-expert id list)")) return nullptr;
        if (!check(hipMemset(zero_ids, 0, want * sizeof(int32_t)), "hipMemset(one-expert id list)")) return nullptr;
        zero_ids_n = want;
    }
    return zero_ids;
}

float* it_hip::gdn_work_for(size_t floats) {
    if (gdn_work_floats < floats) {
        need_eager("delta rule chunk scratch has to grow");
        if (gdn_work) {
            check(hipStreamSynchronize(stream), "sync before scratch free");
            (void)hipFree(gdn_work);
            gdn_work = nullptr;
            gdn_work_floats = 0;
        }
        if (!check(hipMalloc((void**)&gdn_work, floats * sizeof(float)), "hipMalloc(delta rule chunk scratch)")) return nullptr;
        gdn_work_floats = floats;
    }
    return gdn_work;
}

// true when moe_work already holds this grouping (the gate/up and down products of one MoE layer share it);
// records the grouping as held otherwise.  Eager passes only: a recorded launch may run later.
bool it_hip::group_cached(int picks, int n_expert, int tile) {
    if (mode != Mode::Eager) {
        group_gen = ~0ull;
        return false;
    }
    const bool hit = group_gen == route_gen && group_picks == picks && group_experts == n_expert && group_tile == tile;
    group_gen = route_gen;
    group_picks = picks;
    group_experts = n_expert;
    group_tile = tile;
    return hit;
}

int32_t* it_hip::moe_work_for(size_t picks, size_t n_expert, size_t* ints) {
    *ints = 0;
    if (picks < 32) return nullptr;
    const size_t need = itk::experts_group_work_ints((int)picks, (int)n_expert);
    if (moe_work_ints < need) {
        need_eager("expert grouping scratch has to grow");
        if (moe_work) {
            check(hipStreamSynchronize(stream), "sync before scratch free");
            (void)hipFree(moe_work);
            moe_work = nullptr;
            moe_work_ints = 0;
        }
        const size_t want = need + need / 2;
        group_gen = ~0ull;
        if (!check(hipMalloc((void**)&moe_work, want * sizeof(int32_t)), "hipMalloc(expert grouping scratch)")) return nullptr;
        moe_work_ints = want;
    }
    *ints = moe_work_ints;
    return moe_work;
}

float* it_hip::scratch_f32(size_t floats) {
    if (attn_scratch_cap >= floats) return attn_scratch;
    need_eager("attention scratch has to grow");
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

// ------------------------------------------------------------------ event timing
hipEvent_t it_hip::prof_event() {
    if (prof_pool_next < prof_pool.size()) return prof_pool[prof_pool_next++];
    hipEvent_t e = nullptr;
    if (prof_pool.size() >= 32768 || hipEventCreate(&e) != hipSuccess) return nullptr;
    prof_pool.push_back(e);
    prof_pool_next++;
    return e;
}
it_hip::Span::Span(it_hip* b, int fam, uint64_t bytes) : be(b), live(false) {
    if (!b->prof_on) return;
    s.a = b->prof_event();
    s.b = b->prof_event();
    if (!s.a || !s.b) return;
    s.fam = fam;
    s.bytes = bytes;
    live = hipEventRecord(s.a, b->stream) == hipSuccess;
}
it_hip::Span::~Span() {
    if (!live) return;
    if (hipEventRecord(s.b, be->stream) == hipSuccess) be->prof_spans.push_back(s);
}

void it_hip::drop_all() {
    need_eager("mirrors are dropped");
    drop_graph();
    cold_drop();
    prev_signature.clear();
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
        if (kv.second.q_tab) (void)hipFree((void*)kv.second.q_tab);
        if (kv.second.s_tab) (void)hipFree((void*)kv.second.s_tab);
        if (kv.second.tier) (void)hipFree(kv.second.tier);
        if (kv.second.host_q) (void)hipHostFree(kv.second.host_q);
        if (kv.second.host_s) (void)hipHostFree(kv.second.host_s);
    }
    weights.clear();
    for (auto& kv : slabs)
        if (kv.second.dev) (void)hipFree(kv.second.dev);
    slabs.clear();
    mirror_bytes = quant_bytes = const_bytes = weight_bytes = kv_bytes = 0;
    // the pool is gone with the weights: the next pooled tensor sizes a new slab; counters start over
    expert_resident = 0;
    expert_slot_bytes = 0;
    expert_slots_cap = 0;
    expert_counted = 0;
    expert_host_entries = expert_host_bytes = expert_swaps = tokens_since_migration = 0;
    expert_cold_entries = expert_cold_at_load = expert_fetched = expert_fetch_bytes = expert_cold_evictions = 0;
    fetch_read_us = fetch_upload_us = fetch_writes_us = picks_wait_us = picks_copy_us = 0;
    prefetch_reads = prefetch_used = prefetch_wasted = 0;
    pool_tabled = false;
    if (expert_counts) (void)hipMemset(expert_counts, 0, expert_counts_cap * sizeof(uint32_t));
    if (expert_tally) (void)hipMemset(expert_tally, 0, 2 * sizeof(unsigned long long));
}

it_hip::~it_hip() {
    drop_all();
    for (auto& kv : ropes)
        if (kv.second.dev) (void)hipFree(kv.second.dev);
    if (route_ids) (void)hipFree(route_ids);
    if (route_w) (void)hipFree(route_w);
    if (attn_scratch) (void)hipFree(attn_scratch);
    if (gdn_work) (void)hipFree(gdn_work);
    if (moe_f16) (void)hipFree(moe_f16);
    if (zero_ids) (void)hipFree(zero_ids);
    if (moe_work) (void)hipFree(moe_work);
    if (argmax_idx) (void)hipFree(argmax_idx);
    if (argmax_val) (void)hipFree(argmax_val);
    if (argmax_out) (void)hipFree(argmax_out);
    if (argmax_host) (void)hipHostFree(argmax_host);
    for (auto e : prof_pool) (void)hipEventDestroy(e);
    if (dyn_dev) (void)hipFree(dyn_dev);
    if (route_counter) (void)hipFree(route_counter);
    if (expert_counts) (void)hipFree(expert_counts);
    if (expert_tally) (void)hipFree(expert_tally);
    for (int i = 0; i < 2; i++) {
        if (dyn_hosts[i]) (void)hipHostFree(dyn_hosts[i]);
        if (dyn_evt[i]) (void)hipEventDestroy(dyn_evt[i]);
    }
    drop_graph();
    chain_release();
    if (stream) (void)hipStreamDestroy(stream);
}

// ------------------------------------------------------------------ layer-chain resources
namespace {
std::mutex chain_pool_mu;
std::vector<it_hip::ChainRes> chain_pool;   // handed back by backends that are gone; never freed
}  // namespace

bool it_hip::chain_acquire() {
    if (chain.ll) return true;
    {
        std::lock_guard<std::mutex> g(chain_pool_mu);
        for (size_t i = 0; i < chain_pool.size(); i++) {
            if (chain_pool[i].device == device) {
                chain = chain_pool[i];
                chain_pool.erase(chain_pool.begin() + (long)i);
                break;
            }
        }
    }
    if (!chain.ll) {
        ChainRes r;
        r.device = device;
        if (hipExtMallocWithFlags((void**)&r.ll, itk::CHAIN_LL_WORDS * 8, hipDeviceMallocUncached) != hipSuccess ||
            hipExtMallocWithFlags((void**)&r.abort_flag, 256, hipDeviceMallocUncached) != hipSuccess ||
            hipMalloc((void**)&r.epoch, 256) != hipSuccess) {
            (void)hipGetLastError();
            return false;   // (what was allocated stays allocated: a handful of kilobytes, once)
        }
        if (hipMemset(r.ll, 0, itk::CHAIN_LL_WORDS * 8) != hipSuccess || hipMemset(r.abort_flag, 0, 256) != hipSuccess ||
            hipMemset(r.epoch, 0, 256) != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        chain = r;
    }
    return true;
}

void it_hip::chain_release() {
    if (!chain.ll) return;
    if (stream) (void)hipStreamSynchronize(stream);
    (void)hipMemset(chain.abort_flag, 0, 4);
    std::lock_guard<std::mutex> g(chain_pool_mu);
    chain_pool.push_back(chain);
    chain = ChainRes{};
}

void it_hip::chain_check() {
    if (!chain_ran || !chain.abort_flag) return;
    chain_ran = false;
    unsigned flag = 0;
    if (hipMemcpy(&flag, chain.abort_flag, 4, hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    if (!flag) return;
    // a wait inside a chain ran out of tries: what the pass computed is void.  The chains are switched off for this
    // backend, the graph that holds them is dropped and the hand-off space starts from zero again.
    chain_enabled = false;
    drop_graph();
    stable_passes = 0;
    (void)hipMemset(chain.abort_flag, 0, 4);
    (void)hipMemset(chain.ll, 0, itk::CHAIN_LL_WORDS * 8);
    fail("layer chain: a hand-off wait inside the persistent decode kernel gave up (the grid was not resident at once, or a "
         "block stalled); the pass's results are void and the chains are switched off for this backend");
}

// =================================================================== C ABI
extern "C" int it_hip_noalloc_setup(void);  // k_noalloc.hip

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
    be->fuse_enabled = (flags & IT_HIP_NO_FUSE) == 0 && getenv("INFERRED_HIP_NO_FUSE") == nullptr;
    be->chain_enabled = (flags & IT_HIP_NO_CHAIN) == 0 && getenv("INFERRED_HIP_NO_CHAIN") == nullptr;
    be->eager_fused = getenv("INFERRED_HIP_EAGER_FUSED") != nullptr;
    be->count_reads_in_fused = getenv("INFERRED_HIP_NO_READ_COUNTERS") == nullptr;
    be->small_ffn_enabled = getenv("INFERRED_HIP_NO_SMALL_FFN") == nullptr;
    be->chain_attn_enabled = getenv("INFERRED_HIP_NO_CHAIN_ATTN") == nullptr;
    be->chain_max_layers = itk::CHAIN_MAX_LAYERS;
    if (const char* cl = getenv("INFERRED_HIP_CHAIN_LAYERS")) {
        const int v = atoi(cl);
        if (v >= 1 && v <= itk::CHAIN_MAX_LAYERS) be->chain_max_layers = v;
    }
    if (getenv("INFERRED_HIP_NO_GRAPH")) be->allow_graph = false;
    if (const char* sl = getenv("INFERRED_HIP_CHAIN_SPINS")) {
        const long v = atol(sl);
        if (v > 0 && v < (1l << 30)) be->chain_spin_limit = (int)v;
    }
    if ((e = hipStreamCreate(&be->stream)) != hipSuccess) {
        delete be;
        return bad(std::string("hipStreamCreate: ") + hipGetErrorString(e));
    }
    if (hipMalloc((void**)&be->dyn_dev, it_hip::DYN_CAP * sizeof(int)) != hipSuccess ||
        hipHostMalloc((void**)&be->dyn_hosts[0], it_hip::DYN_CAP * sizeof(int), hipHostMallocDefault) != hipSuccess ||
        hipHostMalloc((void**)&be->dyn_hosts[1], it_hip::DYN_CAP * sizeof(int), hipHostMallocDefault) != hipSuccess ||
        hipEventCreateWithFlags(&be->dyn_evt[0], hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&be->dyn_evt[1], hipEventDisableTiming) != hipSuccess) {
        delete be;
        return bad("cannot allocate the position staging buffers");
    }
    be->dyn_host = be->dyn_hosts[0];
    // the allocation-free attention entry point looks up its fixed scratch once per device, here
    if (it_hip_noalloc_setup() != 0) {
        delete be;
        return bad("cannot resolve the fixed attention scratch on this device");
    }
    if (hipMalloc((void**)&be->route_counter, sizeof(unsigned)) != hipSuccess ||
        hipMemset(be->route_counter, 0, sizeof(unsigned)) != hipSuccess) {
        delete be;
        return bad("cannot allocate the router counter");
    }
    return be;
}

void it_hip_destroy(it_hip* be) { delete be; }

int it_hip_take_error(it_hip* be, char* msg, size_t msg_len) {
    if (!be->has_error) {
        // surface asynchronous faults too
        hipError_t e = hipStreamSynchronize(be->stream);
        if (e != hipSuccess) be->fail(std::string("device: ") + hipGetErrorString(e));
        else be->chain_check();
    }
    if (!be->has_error) return 0;
    if (msg && msg_len) snprintf(msg, msg_len, "%s", be->error.c_str());
    be->has_error = false;
    be->error.clear();
    return 1;
}

int it_hip_has_error(it_hip* be) { return be->has_error ? 1 : 0; }

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
    int64_t rows = (int64_t)(x_len / w_len);
    int nd = (int)w_len, exact = be->exact;
    // A batch's normed rows go to products with quantized weights next (qwen35.rs:1006-1093): their Q8_0 form is
    // written by the same launch.  Single-token passes keep the two ops apart for the pass fuser.
    float* qs = nullptr;
    int8_t* qq = nullptr;
    if (rows > 1 && be->mode == it_hip::Mode::Eager && rms_norm_writes_q8(dx, dw, dout, nd)) {
        it_hip::Act& a = be->acts[out];
        if (be->act_q_reserve(a, out_len)) {
            qs = a.q_scales;
            qq = a.q_quants;
            a.q_valid = true;
            a.q_len = out_len;
        }
    }
    it_hip::OpRec rec;
    rec.id = OP_RMS; rec.p[0] = dx; rec.p[1] = dw; rec.p[2] = dout; rec.i[0] = rows; rec.i[1] = nd; rec.f[0] = eps;
    be->submit(it_hip::FAM_NORM, x_len * 8, sig_of(OP_RMS, dx, dw, eps, dout, rows, nd), rec,
               [=](hipStream_t s) { rms_norm(dx, dw, eps, dout, rows, nd, exact, s, qs, qq); });
}

void it_hip_rms_norm_heads(it_hip* be, float* x, uint64_t x_len, const float* w, uint64_t w_len,
                           uint64_t head_dim, float eps) {
    REQUIRE(head_dim > 0 && w_len == head_dim && x_len % head_dim == 0, "rms_norm_heads: weight.len() must equal head_dim and divide x.len()");
    REQUIRE(head_dim <= 12288, "rms_norm_heads: head longer than the kernel's LDS tile");
    if (x_len == 0) return;
    const float* dw = be->const_in(w, w_len);
    float* dx = be->act_inout(x, x_len);
    if (!dw || !dx) return;
    int hd = (int)head_dim, exact = be->exact;
    int64_t heads = (int64_t)(x_len / head_dim);
    it_hip::OpRec rec;
    rec.id = OP_RMS_HEADS; rec.p[0] = dx; rec.p[1] = dw; rec.i[0] = hd; rec.i[1] = heads; rec.f[0] = eps;
    be->submit(it_hip::FAM_NORM, x_len * 8, sig_of(OP_RMS_HEADS, dx, dw, hd, eps, heads), rec,
               [=](hipStream_t s) { rms_norm_heads(dx, dw, hd, eps, heads, exact, s); });
}

void it_hip_l2_norm_heads(it_hip* be, float* x, uint64_t x_len, uint64_t head_dim, float eps) {
    REQUIRE(head_dim > 0 && x_len % head_dim == 0, "l2_norm_heads: head_dim must divide x.len()");
    REQUIRE(head_dim <= 12288, "l2_norm_heads: head longer than the kernel's LDS tile");
    if (x_len == 0) return;
    float* dx = be->act_inout(x, x_len);
    if (!dx) return;
    int hd = (int)head_dim, exact = be->exact;
    int64_t heads = (int64_t)(x_len / head_dim);
    it_hip::OpRec rec;
    rec.id = OP_L2; rec.p[0] = dx; rec.i[0] = hd; rec.i[1] = heads; rec.f[0] = eps;
    be->submit(it_hip::FAM_NORM, x_len * 8, sig_of(OP_L2, dx, hd, eps, heads), rec,
               [=](hipStream_t s) { l2_norm_heads(dx, hd, eps, heads, exact, s); });
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
    int nt = (int)n;
    const int exact = be->exact;
    // A dense NVFP4 matrix over a batch (the shared expert of an NVFP4 file during prefill) has no int8 tile kernel
    // of its own; in fast mode it runs as a batch of one expert on the f16 tile kernel instead of one GEMV per token.
    ExpertsView ev{};
    const int32_t* zids = nullptr;
    int32_t* work = nullptr;
    void* fwork = nullptr;
    size_t work_ints = 0, fwork_bytes = 0;
    bool one_expert = false, grouped = false;
    // (from 513 tokens on: a call costs 55-80 us for the grouping, the f16 split and a latency-bound handful of
    // tiles, which the GEMVs reach at about 512 tokens)
    // A dense NVFP4 matrix over 128 .. 512 tokens whose shape the 16-pair tiles do not take: eight or sixteen tokens per
    // pass over the rows (k_moe_rows.hip) instead of one GEMV per token (32 against 70 us for 2048 x 512 at 512 tokens;
    // below 128 tokens the GEMVs, which fill the chip with one block row per token, are as fast).
    ExpertsView rv{};
    rv.q = v.q; rv.scales = v.scales; rv.q_stride = 0; rv.s_stride = 0; rv.fmt = v.fmt; rv.n_in = v.n_in; rv.n_out = v.n_out;
    rv.n_expert = 1; rv.scale2 = nullptr; rv.counts = nullptr;
    // 128 .. 1,024 tokens: as a batch of ONE expert on the 16-pair tiles (2048 x 512 over 1,024 tokens: 34 against 68 us
    // on the 128-pair tiles, whose handful of blocks is latency-bound there; 16 against 19 us of GEMVs at 128 tokens)
    bool skinny_dense = false;
    if (!exact && v.fmt == W_NVFP4 && n >= 128 && n <= 1024) {
        ev.q = v.q; ev.scales = v.scales; ev.q_stride = 0; ev.s_stride = 0;
        ev.fmt = v.fmt; ev.n_in = v.n_in; ev.n_out = v.n_out; ev.n_expert = 1; ev.scale2 = nullptr; ev.counts = nullptr;
        zids = be->zero_ids_for(n);
        work = be->moe_work_for(n, 1, &work_ints);
        fwork_bytes = itk::experts_f16_work_bytes(nt, v.n_in);
        fwork = be->moe_f16_for(fwork_bytes);
        skinny_dense = zids && work && fwork && itk::experts_f16s_takes(ev, nullptr, nt, aq, dout);
        if (skinny_dense) grouped = be->group_cached(nt, 1, 16);
    }
    const bool rows_dense = !skinny_dense && !exact && v.fmt == W_NVFP4 && n >= 128 && n <= 512 && itk::expert_rows_takes(rv, nullptr, aq);
    if (!skinny_dense && !exact && v.fmt == W_NVFP4 && n > 512) {   // the 128-pair tiles (82 against 736 us at 5,700 tokens)
        ev.q = v.q; ev.scales = v.scales; ev.q_stride = 0; ev.s_stride = 0;
        ev.fmt = v.fmt; ev.n_in = v.n_in; ev.n_out = v.n_out; ev.n_expert = 1; ev.scale2 = nullptr; ev.counts = nullptr;
        zids = be->zero_ids_for(n);
        work = be->moe_work_for(n, 1, &work_ints);
        fwork_bytes = itk::experts_f16_work_bytes(nt, v.n_in);
        fwork = be->moe_f16_for(fwork_bytes);
        one_expert = zids && work && fwork && itk::experts_f16_takes(ev, nullptr, nt, aq, dout);
        if (one_expert) grouped = be->group_cached(nt, 1, 128);
    }
    it_hip::OpRec rec;
    rec.id = OP_MATMUL; rec.p[0] = v.q; rec.p[1] = v.scales; rec.p[2] = dx; rec.p[3] = as; rec.p[4] = aq; rec.p[5] = dout;
    rec.i[0] = v.fmt; rec.i[1] = v.n_in; rec.i[2] = v.n_out; rec.i[3] = nt;
    be->submit(it_hip::FAM_MATMUL, w->len + n * w->n_in + n * w->n_out * 4,
               sig_of(OP_MATMUL, v.q, v.scales, v.fmt, v.n_in, v.n_out, dx, as, aq, nt, dout), rec,
               [=](hipStream_t s) {
                   if (skinny_dense && experts_gemm_f16s(ev, nullptr, zids, nt, 1, 0, as, aq, dout, work, work_ints, fwork, fwork_bytes, grouped, s))
                       return;
                   if (rows_dense && expert_rows(rv, nullptr, nullptr, nt, 1, 0, as, aq, dout, 1.0f, nullptr, 0, false, s)) return;
                   if (one_expert && experts_gemm_f16(ev, nullptr, zids, nt, 1, 0, as, aq, dout, work, work_ints, fwork,
                                                      fwork_bytes, grouped, s))
                       return;
                   matmul(v, dx, as, aq, nt, dout, 1.0f, exact, s);
               });
}

void it_hip_matmul(it_hip* be, const it_weights* w, const float* x, uint64_t x_len, float* out,
                   uint64_t out_len) {
    matmul_impl(be, w, x, x_len, out, out_len, "matmul");
}

void it_hip_matmul_pair(it_hip* be, const it_weights* a, const it_weights* b, const float* x, uint64_t x_len,
                        float* out_a, uint64_t out_a_len, float* out_b, uint64_t out_b_len) {
    // A batch against two unquantized matrices (the F32 router with the shared-gate logit, ssm alpha with beta, of a
    // real file): one launch reads the activations once for both.  Single-token passes keep two ops for the fuser.
    const bool floats = a && b && a->data && b->data && (a->ty == IT_F32 || a->ty == IT_F16 || a->ty == IT_BF16) && a->ty == b->ty;
    if (!be->exact && floats && a->n_in == b->n_in && a->n_in && x_len % a->n_in == 0 && x_len / a->n_in > 16 &&
        x_len / a->n_in <= 65535 && out_a_len == x_len / a->n_in * a->n_out && out_b_len == x_len / a->n_in * b->n_out) {
        WView va, vb;
        if (!be->weights_view(a, "matmul_pair(a)", &va) || !be->weights_view(b, "matmul_pair(b)", &vb)) return;
        const float* dx = be->act_in(x, x_len);
        float* da = be->act_out(out_a, out_a_len);
        float* db = be->act_out(out_b, out_b_len);
        if (!dx || !da || !db) return;
        const int nt = (int)(x_len / a->n_in);
        if ((reinterpret_cast<uintptr_t>(va.q) & 15) == 0 && (reinterpret_cast<uintptr_t>(vb.q) & 15) == 0 && va.n_in % 16 == 0) {
            it_hip::OpRec rec;
            rec.id = OP_MATMUL;
            be->submit(it_hip::FAM_MATMUL, a->len + b->len + x_len * 4 + (out_a_len + out_b_len) * 4,
                       sig_of(OP_MATMUL, va.q, vb.q, va.fmt, va.n_in, va.n_out, vb.n_out, dx, nt, da, db), rec,
                       [=](hipStream_t s) { float_matmul_pair(va, vb, dx, nt, da, db, s); });
            return;
        }
    }
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
    const int* dyn = be->dyn_slot((int)pos);
    int pv = dyn ? 0 : (int)pos, half = (int)(n_rot / 2), hd = (int)head_dim, nr = (int)n_rot, nh = (int)n_heads;
    int64_t nt = (int64_t)n;
    it_hip::OpRec rec;
    rec.id = OP_ROPE; rec.p[0] = dx; rec.p[1] = tab; rec.p[2] = dyn;
    rec.i[0] = half; rec.i[1] = nt; rec.i[2] = hd; rec.i[3] = nr; rec.i[4] = nh; rec.i[5] = pv;
    be->submit(it_hip::FAM_OTHER, x_len * 8, sig_of(OP_ROPE, dx, tab, half, nt, dyn, hd, nr, nh), rec,
               [=](hipStream_t s) { rope_neox(dx, tab, half, nt, pv, dyn, hd, nr, nh, s); });
}

void it_hip_softmax(it_hip* be, float* x, uint64_t x_len, uint64_t row) {
    if (row == 0 || x_len == 0) return;
    REQUIRE(x_len % row == 0, "softmax: x.len() must be a multiple of row");
    REQUIRE(row <= 12288, "softmax: row longer than the kernel's LDS tile");
    float* dx = be->act_inout(x, x_len);
    if (!dx) return;
    int64_t rows = (int64_t)(x_len / row);
    int r = (int)row, exact = be->exact;
    it_hip::OpRec rec;
    rec.id = OP_SOFTMAX; rec.p[0] = dx; rec.i[0] = rows; rec.i[1] = r;
    be->submit(it_hip::FAM_ROUTER, x_len * 8, sig_of(OP_SOFTMAX, dx, rows, r), rec,
               [=](hipStream_t s) { softmax_rows(dx, rows, r, exact, s); });
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
    uint64_t group = a->n_head / a->n_head_kv;
    bool split_ok = (group == 1 || group == 2 || group == 4 || group == 8) && a->head_dim <= 256;
    bool graphed = be->mode != it_hip::Mode::Eager;
    // a graphed pass keeps one launch shape while the context grows: size for the whole slab
    uint64_t n_pos_cap = graphed ? a->kv_len / a->kv_dim : a->n_pos;
    uint64_t bytes = a->n_pos * a->n_head_kv * a->head_dim * 4 + a->q_len * 8;
    if (be->exact || !split_ok) {
        float* sc = be->scratch_f32((size_t)(n_q * a->n_head * n_pos_cap));
        if (!sc) return;
        const int* dyn = be->dyn_slot((int)a->n_pos);
        AttnArgs args{dq, dk, dv, (int)n_q, (int)a->kv_dim, dyn ? (int)n_pos_cap : (int)a->n_pos, (int)a->head_dim,
                      (int)a->n_head, (int)a->n_head_kv, a->scale, dyn};
        AttnArgs sg = args;
        it_hip::OpRec rec;
        rec.id = OP_ATTEND; rec.p[0] = dq; rec.p[1] = dk; rec.p[2] = dv; rec.p[3] = dyn; rec.p[4] = sc; rec.p[5] = dout;
        rec.i[0] = args.n_q; rec.i[1] = args.kv_dim; rec.i[2] = args.head_dim; rec.i[3] = args.n_head;
        rec.i[4] = args.n_head_kv; rec.i[6] = 1; rec.i[8] = (int64_t)a->n_pos; rec.f[0] = args.scale;  // exact form: launched as is
        be->submit(it_hip::FAM_ATTEND, bytes,
                   sig_of(OP_ATTEND, 0, sg.q, sg.k, sg.v, sg.n_q, sg.kv_dim, dyn ? sg.n_pos : 0, sg.head_dim, sg.n_head,
                          sg.n_head_kv, sg.scale, dyn, sc, dout), rec,
                   [=](hipStream_t s) { attend_exact(args, sc, dout, s); });
    } else {
        int n_split = attend_split_count((int)n_pos_cap, (int)n_q, (int)a->head_dim, (int)group);
        // the one-pass kernel of a large batch (never a graphed pass) keeps no partial results: what is reserved is
        // what the single-token passes that follow will ask for (the whole slab's splits), so that they do not grow it
        AttnArgs probe{dq, dk, dv, (int)n_q, (int)a->kv_dim, (int)a->n_pos, (int)a->head_dim, (int)a->n_head, (int)a->n_head_kv,
                       a->scale, nullptr};
        const bool one_pass = !graphed && attend_prefill_takes(probe, dout);
        const size_t decode_floats = (size_t)a->n_head * attend_split_count((int)(a->kv_len / a->kv_dim), 1, (int)a->head_dim, (int)group) *
                                     (a->head_dim + 2);
        // a few-query call reserves the decode size too, so that the first graphed pass after it (whose split count is
        // the whole slab's) does not have to grow the scratch in the middle of a capture
        const size_t call_floats = (size_t)(n_q * a->n_head) * n_split * (a->head_dim + 2);
        float* sc = be->scratch_f32(one_pass ? decode_floats : std::max(call_floats, decode_floats));
        if (!sc) return;
        const int* dyn = be->dyn_slot((int)a->n_pos);
        AttnArgs args{dq, dk, dv, (int)n_q, (int)a->kv_dim, dyn ? 0 : (int)a->n_pos, (int)a->head_dim,
                      (int)a->n_head, (int)a->n_head_kv, a->scale, dyn};
        it_hip::OpRec rec;
        rec.id = OP_ATTEND; rec.p[0] = dq; rec.p[1] = dk; rec.p[2] = dv; rec.p[3] = dyn; rec.p[4] = sc; rec.p[5] = dout;
        rec.i[0] = args.n_q; rec.i[1] = args.kv_dim; rec.i[2] = args.head_dim; rec.i[3] = args.n_head;
        rec.i[4] = args.n_head_kv; rec.i[5] = n_split; rec.i[6] = 0; rec.i[7] = args.n_pos; rec.i[8] = (int64_t)a->n_pos;
        rec.f[0] = args.scale;
        be->submit(it_hip::FAM_ATTEND, bytes,
                   sig_of(OP_ATTEND, 1, dq, dk, dv, args.n_q, args.kv_dim, args.head_dim, args.n_head, args.n_head_kv,
                          args.scale, dyn, dyn ? n_split : 0, sc, dout), rec,
                   [=](hipStream_t s) {
                       // a one-pass prefill reserved the decode passes' scratch only: it must not fall into the split
                       // kernels, whose partials for the whole batch would not fit there
                       if (one_pass) {
                           if (!attend_prefill(args, dout, s)) be->fail("attend: the one-pass prefill kernel could not be launched");
                       } else if (!attend_split_gated(args, n_split, sc, dout, nullptr, 0, s)) {
                           be->fail("attend: the split-K kernels could not be launched");
                       }
                   });
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
    int64_t n = (int64_t)a_len;
    it_hip::OpRec rec;
    rec.id = OP_EW; rec.p[0] = da; rec.p[1] = db; rec.i[0] = op; rec.i[1] = n; rec.f[0] = v;
    const int exact = be->exact;
    be->submit(it_hip::FAM_OTHER, a_len * 12, sig_of(OP_EW, op, da, db, n, v), rec, [=](hipStream_t s) {
        switch (op) {
            case 0: silu_mul(da, db, n, exact, s); break;
            case 1: sigmoid_mul(da, db, n, exact, s); break;
            case 2: add_assign(da, db, n, s); break;
            case 3: add_scaled(da, db, v, n, s); break;
        }
    });
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

void it_hip_scale(it_hip* be, float* buf, uint64_t len, float sv) {
    if (len == 0) return;
    float* d = be->act_inout(buf, len);
    if (!d) return;
    int64_t n = (int64_t)len;
    it_hip::OpRec rec;
    rec.id = OP_SCALE; rec.p[0] = d; rec.i[0] = n; rec.f[0] = sv;
    be->submit(it_hip::FAM_OTHER, len * 8, sig_of(OP_SCALE, d, sv, n), rec, [=](hipStream_t s) { scale(d, sv, n, s); });
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
    int k = (int)kernel, c = (int)nc, nt = (int)(x_len / nc);
    it_hip::OpRec rec;
    rec.id = OP_CONV; rec.p[0] = dstate; rec.p[1] = dx; rec.p[2] = dw; rec.p[3] = dout; rec.i[0] = k; rec.i[1] = c; rec.i[2] = nt;
    be->submit(it_hip::FAM_OTHER, x_len * 8 + state_len * 8, sig_of(OP_CONV, dstate, dx, dw, k, c, nt, dout), rec,
               [=, exact = (int)be->exact](hipStream_t s) { ssm_conv(dstate, dx, dw, k, c, nt, dout, exact, s); });
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
    int64_t c = (int64_t)chunk, st = (int64_t)stride, off = (int64_t)offset, ol = (int64_t)out_len;
    it_hip::OpRec rec;
    rec.id = OP_GATHER; rec.p[0] = ds; rec.p[1] = dout; rec.i[0] = c; rec.i[1] = st; rec.i[2] = off; rec.i[3] = ol;
    be->submit(it_hip::FAM_OTHER, out_len * 8, sig_of(OP_GATHER, ds, c, st, off, dout, ol), rec,
               [=](hipStream_t s) { gather_chunks(ds, c, st, off, dout, ol, s); });
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
    int64_t sl = (int64_t)src_len, c = (int64_t)chunk, st = (int64_t)stride, off = (int64_t)offset;
    it_hip::OpRec rec;
    rec.id = OP_SCATTER;
    be->submit(it_hip::FAM_OTHER, src_len * 8, sig_of(OP_SCATTER, ds, sl, c, st, off, dd), rec,
               [=](hipStream_t s) { scatter_chunks(ds, sl, c, st, off, dd, s); });
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
    int exact = be->exact;
    float* work = nullptr;
    size_t work_floats = 0;
    if (!exact && n >= 64 && (d->head_k_dim == 64 || d->head_k_dim == 128) && d->head_v_dim % 16 == 0) {
        work_floats = itk::gdn_chunk_work_floats((int)n, (int)d->n_v_heads);
        work = be->gdn_work_for(work_floats);
        if (!work) return;
    }
    it_hip::OpRec rec;
    rec.id = OP_DELTA; rec.p[0] = dq; rec.p[1] = dk; rec.p[2] = dv; rec.p[3] = da; rec.p[4] = db; rec.p[5] = dssm;
    rec.p[6] = ddt; rec.p[7] = dstate; rec.p[8] = dout;
    rec.i[0] = args.n_tokens; rec.i[1] = args.head_k_dim; rec.i[2] = args.head_v_dim; rec.i[3] = args.n_k_heads; rec.i[4] = args.n_v_heads;
    be->submit(it_hip::FAM_DELTA, state_len * 8 + n * (2 * kper + 2 * vper) * 4,
               sig_of(OP_DELTA, dq, dk, dv, da, db, dssm, ddt, args.n_tokens, args.head_k_dim, args.head_v_dim,
                      args.n_k_heads, args.n_v_heads, dstate, dout), rec,
               [=](hipStream_t s) { delta_rule(args, dstate, dout, exact, work, work_floats, s); });
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
    int32_t* ids = be->route_ids;
    float* rw = be->route_w;
    int nt = (int)n_tok, ne = (int)n_expert, nu = (int)n_used;
    it_hip::OpRec rec;
    rec.id = OP_ROUTE; rec.p[0] = dp; rec.p[1] = ids; rec.p[2] = rw; rec.i[0] = nt; rec.i[1] = ne; rec.i[2] = nu;
    be->submit(it_hip::FAM_ROUTER, probs_len * 4, sig_of(OP_ROUTE, dp, nt, ne, nu, ids, rw), rec,
               [=](hipStream_t s) { route_topk(dp, nt, ne, nu, ids, rw, s); });
    be->route_n_used = n_used;
    be->route_n_tok = n_tok;
    be->route_gen++;
    be->cold_clear_lease();   // a new routing decision: the last one's experts may be evicted again
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

// Expert-sorted tiles read an expert's rows once for all of its pairs; the per-pair kernels read them once per
// pair but stream them at several times the rate.  Measured on the 512-expert shape (pairs per expert 0.08 .. 5):
// the tiles win from about 3.5 pairs per expert on (a batch of 128 tokens at top-10 still takes 653 us per pair
// against 772 us tiled; at 256 tokens it is 1,180 against 848).
static bool expert_tiles_pay(uint64_t picks, uint64_t n_expert) { return picks >= 32 && 2 * picks >= 7 * n_expert; }
// Fast mode between the per-pair GEMVs and the wide matrix-core tiles, measured on the 512-expert top-10 FFN (hidden
// 2048, inter 512): from 1.25 pairs per expert on, grouping the pairs by expert beats one GEMV per pair; NVFP4 then
// runs 16-pair tiles on the f16 matrix cores (k_gemm_f16s.hip) up to 48 pairs per expert (2,048 tokens: 961 against
// 1,017 us for the whole FFN; 4,096 tokens: 1,571 against 1,447), where the 128-pair tiles take over; what that kernel does not take (Q8_0, odd shapes) streams each expert's rows once for all its pairs
// (k_moe_rows.hip) until the int8 tiles pay.
static bool expert_grouping_pays(const it_hip* be, uint64_t picks, uint64_t n_expert) {
    return !be->exact && picks >= 32 && 4 * picks >= 5 * n_expert;
}
static bool expert_skinny_pay(const it_hip* be, uint64_t picks, uint64_t n_expert) {
    return expert_grouping_pays(be, picks, n_expert) && picks < 48 * n_expert;
}
static bool expert_rows_pay(const it_hip* be, uint64_t picks, uint64_t n_expert) {
    return expert_grouping_pays(be, picks, n_expert) && !expert_tiles_pay(picks, n_expert);
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
    if (be->expert_cold_entries) {
        const uint8_t* keys[1] = {w->data};
        if (!be->cold_resolve(keys, 1, route, false)) return;
    }
    const float* as;
    const int8_t* aq;
    if (!be->act_quantized(x, x_len, &as, &aq, nullptr)) return;
    float* dout = be->act_out(out, out_len);
    if (!dout) return;
    int np = (int)picks, nu = (int)n_used, xm = x_mode_of(rows, picks);
    size_t work_ints = 0;
    const bool skinny_pay = expert_skinny_pay(be, picks, w->n_expert) && v.fmt == itk::W_NVFP4;
    const bool rows_pay = !skinny_pay && expert_rows_pay(be, picks, w->n_expert);
    int32_t* work = skinny_pay || rows_pay || expert_tiles_pay(picks, w->n_expert) ? be->moe_work_for(picks, w->n_expert, &work_ints) : nullptr;
    const bool rows_shape = rows_pay && work && itk::expert_rows_takes(v, nullptr, aq);
    void* fwork = nullptr;
    size_t fwork_bytes = 0;
    if (!be->exact && work && !rows_shape && v.fmt == itk::W_NVFP4) {
        fwork_bytes = itk::experts_f16_work_bytes((int)rows, (int)w->n_in);
        fwork = be->moe_f16_for(fwork_bytes);
    }
    const bool skinny_shape = skinny_pay && fwork && itk::experts_f16s_takes(v, nullptr, np, aq, dout);
    // the tile size the launch below will group for: 8 or 16 pairs for the row kernel, 128 for the wide f16 kernel,
    // 16 for the skinny f16 kernel and the int8 one
    const bool f16_shape = !skinny_shape && fwork && itk::experts_f16_takes(v, nullptr, np, aq, dout);
    const bool grouped = work && be->group_cached(np, (int)w->n_expert, rows_shape ? itk::expert_rows_tile(np, (int)w->n_expert, v.n_in) : f16_shape ? 128 : 16);
    it_hip::OpRec rec;
    rec.id = OP_EXPERTS; rec.p[0] = v.q; rec.p[1] = v.scales; rec.p[2] = v.scale2; rec.p[3] = ids; rec.p[4] = as; rec.p[5] = aq;
    rec.p[6] = dout; rec.i[0] = v.fmt; rec.i[1] = v.n_in; rec.i[2] = v.n_out; rec.i[3] = np; rec.i[4] = nu; rec.i[5] = xm;
    rec.i[6] = v.q_stride; rec.i[7] = v.s_stride; rec.p[7] = v.counts; rec.i[8] = v.q_tab ? 1 : 0;
    unsigned long long* tally = be->expert_tally;
    uint32_t* counts = v.counts;
    be->submit(it_hip::FAM_MOE_DOWN, picks * (w->len / w->n_expert) + x_len + out_len * 4,
               sig_of(OP_EXPERTS, v.q, v.scales, (const void*)v.q_tab, v.fmt, v.n_in, v.n_out, v.scale2, ids, np, nu, xm, as, aq, dout), rec,
               [=](hipStream_t s) {
                   expert_count(ids, np, v.n_expert, counts, nullptr, tally, s, v.tier, nullptr);
                   if (skinny_shape && experts_gemm_f16s(v, nullptr, ids, np, nu, xm, as, aq, dout, work, work_ints, fwork, fwork_bytes, grouped, s))
                       return;
                   if (rows_shape && expert_rows(v, nullptr, ids, np, nu, xm, as, aq, dout, 1.0f, work, work_ints, grouped, s)) return;
                   if (f16_shape && experts_gemm_f16(v, nullptr, ids, np, nu, xm, as, aq, dout, work, work_ints, fwork, fwork_bytes, grouped, s))
                       return;
                   if (!experts_gemm(v, nullptr, ids, np, nu, xm, as, aq, dout, work, work_ints, grouped && !f16_shape, s))
                       matmul_experts(v, ids, np, nu, xm, as, aq, dout, s);
               });
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
    if (be->expert_cold_entries) {
        const uint8_t* keys[2] = {gate->data, up->data};
        if (!be->cold_resolve(keys, 2, route, true)) return;
    }
    const float* as;
    const int8_t* aq;
    if (!be->act_quantized(x, x_len, &as, &aq, nullptr)) return;
    float* dout = be->act_out(out, out_len);
    if (!dout) return;
    int np = (int)picks, nu = (int)n_used, xm = x_mode_of(rows, picks);
    size_t work_ints = 0;
    const bool skinny_pay = expert_skinny_pay(be, picks, gate->n_expert) && g.fmt == itk::W_NVFP4;
    const bool rows_pay = !skinny_pay && expert_rows_pay(be, picks, gate->n_expert);
    int32_t* work = skinny_pay || rows_pay || expert_tiles_pay(picks, gate->n_expert) ? be->moe_work_for(picks, gate->n_expert, &work_ints) : nullptr;
    const bool rows_shape = rows_pay && work && itk::expert_rows_takes(g, &u, aq);
    void* fwork = nullptr;
    size_t fwork_bytes = 0;
    if (!be->exact && work && !rows_shape && g.fmt == itk::W_NVFP4) {
        fwork_bytes = itk::experts_f16_work_bytes((int)rows, (int)gate->n_in);
        fwork = be->moe_f16_for(fwork_bytes);
    }
    const bool skinny_shape = skinny_pay && fwork && itk::experts_f16s_takes(g, &u, np, aq, dout);
    const bool f16_shape = !skinny_shape && fwork && itk::experts_f16_takes(g, &u, np, aq, dout);
    const bool grouped = work && be->group_cached(np, (int)gate->n_expert, rows_shape ? itk::expert_rows_tile(np, (int)gate->n_expert, g.n_in) : f16_shape ? 128 : 16);
    it_hip::OpRec rec;
    rec.id = OP_GLU; rec.p[0] = g.q; rec.p[1] = g.scales; rec.p[2] = u.q; rec.p[3] = u.scales; rec.p[4] = g.scale2;
    rec.p[5] = u.scale2; rec.p[6] = ids; rec.p[7] = as; rec.p[8] = aq; rec.p[9] = dout;
    rec.i[0] = g.fmt; rec.i[1] = g.n_in; rec.i[2] = g.n_out; rec.i[3] = np; rec.i[4] = nu; rec.i[5] = xm;
    rec.i[6] = g.q_stride; rec.i[7] = g.s_stride; rec.p[10] = g.counts; rec.p[11] = u.counts; rec.i[8] = (g.q_tab || u.q_tab) ? 1 : 0;
    unsigned long long* tally = be->expert_tally;
    uint32_t *cg = g.counts, *cu = u.counts;
    be->submit(it_hip::FAM_MOE_GLU, 2 * picks * (gate->len / gate->n_expert) + x_len + out_len * 4,
               sig_of(OP_GLU, g.q, g.scales, u.q, u.scales, (const void*)g.q_tab, (const void*)u.q_tab, g.fmt, g.n_in, g.n_out, g.scale2, u.scale2, ids, np, nu, xm,
                      as, aq, dout), rec,
               [=](hipStream_t s) {
                   expert_count(ids, np, g.n_expert, cg, cu, tally, s, g.tier, u.tier);
                   if (skinny_shape && experts_gemm_f16s(g, &u, ids, np, nu, xm, as, aq, dout, work, work_ints, fwork, fwork_bytes, grouped, s))
                       return;
                   if (rows_shape && expert_rows(g, &u, ids, np, nu, xm, as, aq, dout, 1.0f, work, work_ints, grouped, s)) return;
                   if (f16_shape && experts_gemm_f16(g, &u, ids, np, nu, xm, as, aq, dout, work, work_ints, fwork, fwork_bytes, grouped, s))
                       return;
                   if (!experts_gemm(g, &u, ids, np, nu, xm, as, aq, dout, work, work_ints, grouped && !f16_shape, s))
                       moe_glu(g, u, ids, np, nu, xm, as, aq, dout, s);
               });
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
        be->need_eager("a host route is staged");
        if (!be->route_reserve((size_t)picks)) return;
        if (!be->check(hipMemcpyAsync(be->route_w, route->weights, picks * 4, hipMemcpyHostToDevice, be->stream), "upload weights")) return;
        be->check(hipStreamSynchronize(be->stream), "upload weights");
        be->route_n_used = route->n_used;
        be->route_n_tok = route->n_tok;
        be->route_gen++;
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
    int64_t a64 = (int64_t)at, la = (int64_t)logit_at;
    int ni = (int)n, nt = (int)n_tok, nu = (int)n_used;
    it_hip::OpRec rec;
    rec.id = OP_FINISH; rec.p[0] = dout; rec.p[1] = dr; rec.p[2] = rw; rec.p[3] = ds; rec.p[4] = dl;
    rec.i[0] = a64; rec.i[1] = ni; rec.i[2] = nt; rec.i[3] = nu; rec.i[4] = la;
    be->submit(it_hip::FAM_OTHER, rows_len * 4 + n_tok * n * 8, sig_of(OP_FINISH, dout, a64, ni, dr, rw, nt, nu, ds, dl, la), rec,
               [=, exact = (int)be->exact](hipStream_t s) { moe_finish(dout, a64, ni, dr, rw, nt, nu, ds, dl, la, exact, s); });
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
    int64_t n = (int64_t)acc_len;
    int ns = (int)scales_len;
    it_hip::OpRec rec;
    rec.id = OP_ROWS;
    be->submit(it_hip::FAM_OTHER, rows_len * 4, sig_of(OP_ROWS, da, n, dr, dsc, ns), rec,
               [=](hipStream_t s) { add_scaled_rows(da, n, dr, dsc, ns, s); });
}

void it_hip_add_scaled_sigmoid(it_hip* be, float* acc, uint64_t acc_len, const float* b, uint64_t b_len,
                               const float* logit, uint64_t logit_len) {
    REQUIRE(acc_len == b_len && logit_len >= 1, "add_scaled_sigmoid: acc and b must match and logit be non-empty");
    if (acc_len == 0) return;
    float* da = be->act_inout(acc, acc_len);
    float* db = be->act_in(b, b_len);
    float* dl = be->act_in(logit, logit_len);
    if (!da || !db || !dl) return;
    int64_t n = (int64_t)acc_len;
    it_hip::OpRec rec;
    rec.id = OP_SIGADD;
    be->submit(it_hip::FAM_OTHER, acc_len * 12, sig_of(OP_SIGADD, da, db, n, dl), rec,
               [=](hipStream_t s) { add_scaled_sigmoid(da, db, n, dl, s); });
}

void it_hip_kv_write(it_hip* be, uint16_t* slab, uint64_t slab_len, uint64_t offset, const float* src,
                     uint64_t src_len) {
    REQUIRE(offset + src_len <= slab_len, "kv_write: writes past the end of the slab");
    if (src_len == 0) return;
    float* ds = be->act_in(src, src_len);
    uint16_t* dslab = (uint16_t*)be->slab_in(slab, slab_len * 2, false);
    if (!ds || !dslab) return;
    // a graphed decode pass writes row `pos` of the slab: offset = pos * src_len
    const int* dyn = nullptr;
    int64_t mul = 0, off = (int64_t)offset, n = (int64_t)src_len;
    if (be->mode != it_hip::Mode::Eager && offset % src_len == 0 && offset / src_len < (1ull << 31)) {
        dyn = be->dyn_slot((int)(offset / src_len));
        if (dyn) {
            mul = n;
            off = 0;
        }
    } else {
        be->need_eager("a kv_write offset is not a whole row");
    }
    it_hip::OpRec rec;
    rec.id = OP_KVWRITE; rec.p[0] = dslab; rec.p[1] = dyn; rec.p[2] = ds; rec.i[0] = mul; rec.i[1] = off; rec.i[2] = n;
    be->submit(it_hip::FAM_OTHER, src_len * 6, sig_of(OP_KVWRITE, dslab, dyn, mul, ds, n), rec,
               [=](hipStream_t s) { kv_write(dslab, off, dyn, mul, ds, n, s); });
}


// ------------------------------------------------------------------ qwen4exp-only methods (mod.rs:705-966)
// Outside this backend's path: nothing is launched, the first such call leaves its name in the sticky error.
#define IT_UNSUPPORTED(name) be->fail(name ": qwen4exp-only op, not implemented by the hip backend")
void it_hip_mean_streams(it_hip* be, const float*, uint64_t, uint64_t, uint64_t, float, float*, uint64_t) { IT_UNSUPPORTED("mean_streams"); }
void it_hip_mul_rows(it_hip* be, float*, uint64_t, const float*, uint64_t) { IT_UNSUPPORTED("mul_rows"); }
void it_hip_silu(it_hip* be, float*, uint64_t) { IT_UNSUPPORTED("silu"); }
void it_hip_sigmoid(it_hip* be, float*, uint64_t) { IT_UNSUPPORTED("sigmoid"); }
void it_hip_mul_streams(it_hip* be, float*, uint64_t, const float*, uint64_t, const float*, uint64_t, uint64_t) { IT_UNSUPPORTED("mul_streams"); }
void it_hip_row_dot(it_hip* be, const float*, uint64_t, const float*, uint64_t, uint64_t, float*, uint64_t) { IT_UNSUPPORTED("row_dot"); }
void it_hip_signed_sqrt_sigmoid(it_hip* be, float*, uint64_t) { IT_UNSUPPORTED("signed_sqrt_sigmoid"); }
void it_hip_dilated_conv(it_hip* be, float*, uint64_t, const float*, uint64_t, const float*, uint64_t, uint64_t, uint64_t, float*,
                         uint64_t) { IT_UNSUPPORTED("dilated_conv"); }
void it_hip_qsa_pool(it_hip* be, const uint16_t*, uint64_t, float*, uint64_t, const it_qsa_pool*) { IT_UNSUPPORTED("qsa_pool"); }
void it_hip_qsa_select(it_hip* be, const float*, uint64_t, const float*, uint64_t, const it_qsa_select*, float*, uint64_t, uint32_t*,
                       uint64_t) { IT_UNSUPPORTED("qsa_select"); }
void it_hip_attend_sparse(it_hip* be, const it_attn*, const uint32_t*, uint64_t, const it_qsa_select*, float*, uint64_t) { IT_UNSUPPORTED("attend_sparse"); }
#undef IT_UNSUPPORTED

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
    if (!be->held.empty()) be->release_held();
    if (it->second.elided) {
        be->fail("host_needs: the op that writes this buffer was folded into a fused kernel that does not write it");
        return;
    }
    if (be->in_pass) {
        // a read inside a pass cannot be served from a graph that has not run yet:
        // graphs are latched off for this backend (src/ops/cuda/ops/mod.rs:565-582)
        be->mid_pass_read = true;
        be->need_eager("the host read a device buffer inside a pass");
    }
    size_t n = len < it->second.cap ? len : it->second.cap;
    if (!be->check(hipMemcpyAsync(buf, it->second.dev, n * sizeof(float), hipMemcpyDeviceToHost, be->stream), "download activation")) return;
    be->check(hipStreamSynchronize(be->stream), "download activation");
    be->chain_check();
    be->d2h++;
    be->d2h_bytes += n * 4;
}

void it_hip_begin_pass(it_hip* be, uint64_t n_tokens) {
    if (be->in_pass) {
        be->finish_pass();
        be->in_pass = false;
    }
    be->mode = it_hip::Mode::Eager;
    be->migrate_at_boundary(n_tokens);
    be->in_pass = true;
    be->pass_tokens = n_tokens;
    be->pass_signature.clear();
    be->pending.clear();
    be->precopies.clear();
    be->dyn_rotate();
    be->replay_cursor = 0;
    be->mode = it_hip::Mode::Eager;
    be->profile_pass = false;
    // cold experts are resolved from the picks inside the pass, which a graph cannot replay (experts.rs:91-93)
    if (n_tokens == 1 && be->allow_graph && !be->mid_pass_read && !be->has_error && !be->expert_cold_entries) {
        if (be->graph.valid) {
            // while profiling, the pass is recorded like a replay and its fused launches are
            // then issued one by one between timing events instead of as the graph
            be->mode = it_hip::Mode::Replay;
            be->profile_pass = be->prof_on;
        } else if (be->stable_passes >= 1 && !be->prof_on) {
            be->mode = it_hip::Mode::Capture;
        }
    } else if (n_tokens == 1 && be->expert_cold_entries && be->fuse_enabled && !be->has_error) {
        be->mode = it_hip::Mode::Deferred;   // picks are read back inside the pass: fused launches, no graph
    } else if (n_tokens == 1 && be->eager_fused && !be->allow_graph && be->fuse_enabled && !be->has_error && !be->prof_on) {
        // the fused launches queued on the stream pass after pass, with no graph around them (a measurement switch)
        be->mode = it_hip::Mode::Deferred;
    }
    for (auto& kv : be->acts) {
        kv.second.dev_current = false;
        kv.second.elided = false;
        kv.second.q_valid = false;
    }
}

void it_hip_end_pass(it_hip* be) {
    if (!be->in_pass) return;
    be->finish_pass();
    be->in_pass = false;
}

void it_hip_forget_state(it_hip* be) {
    for (auto& kv : be->slabs)
        if (kv.second.is_state) kv.second.dev_owned = false;
}

void it_hip_zero_state(it_hip* be) {
    // the host copies were just zeroed: zero the device copies in place instead of uploading zeros at the next use
    for (auto& kv : be->slabs) {
        if (!kv.second.is_state) continue;
        if (kv.second.dev) {
            fill_zero(kv.second.dev, (int64_t)kv.second.bytes, be->stream);
            kv.second.dev_owned = true;
        } else {
            kv.second.dev_owned = false;
        }
    }
}

void it_hip_read_state(it_hip* be, float* host, uint64_t len) {
    be->need_eager("a state slab is read");
    auto it = be->slabs.find(host);
    if (it == be->slabs.end() || !it->second.dev_owned) return;
    size_t bytes = len * 4 < it->second.bytes ? len * 4 : it->second.bytes;
    if (!be->check(hipMemcpyAsync(host, it->second.dev, bytes, hipMemcpyDeviceToHost, be->stream), "download state")) return;
    be->check(hipStreamSynchronize(be->stream), "download state");
    be->d2h++;
    be->d2h_bytes += bytes;
}

void it_hip_read_kv(it_hip* be, uint16_t* slab, uint64_t len) {
    be->need_eager("a kv slab is read");
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
    uint64_t tally[2];
    be->expert_counters_read(nullptr, tally);
    out->lookups = tally[0] + tally[1];
    out->host_reads = tally[1];
    out->slot_bytes = be->expert_slot_bytes;
    out->slots = be->expert_slots_cap;
    out->mirrors = be->acts.size();
    out->mirror_bytes = be->mirror_bytes;
    out->weight_bytes = be->weight_bytes;
    out->kv_bytes = be->kv_bytes;
    out->quant_bytes = be->quant_bytes;
    out->pool_bytes = be->attn_scratch_cap * 4;
    out->resident_bytes = be->weight_bytes + be->kv_bytes + be->quant_bytes + be->mirror_bytes +
                          be->const_bytes + out->pool_bytes;
    out->oversubscribed = be->expert_cold_entries ? 1 : 0;
    out->fetched = be->expert_fetched;
    out->fetch_bytes = be->expert_fetch_bytes;
    out->read_us = be->fetch_read_us;
    out->upload_us = be->fetch_upload_us;
    out->writes_us = be->fetch_writes_us;
    out->picks_wait_us = be->picks_wait_us;
    out->picks_copy_us = be->picks_copy_us;
    out->prefetch_reads = be->prefetch_reads;
    out->prefetch_used = be->prefetch_used;
    return 1;
}

size_t it_hip_config_report(it_hip* be, char* buf, size_t buf_len) {
    int n = snprintf(buf, buf_len,
                     "backend=hip gfx950\nreductions=%s\ndecode graph=%s\nattention=%s\nexpert tier=%s\n"
                     "expert slots=%llu of %llu bytes (%s)\nexpert host tier=%llu experts, %llu bytes of a budget of %llu\n"
                     "expert cold tier=%llu experts (fetched on demand from %s)\n"
                     "expert prefetch=%s (acts on cold experts only: a host-tier expert is read in place)\n"
                     "model path=%s\n",
                     be->exact ? "serial (CPU order)" : "tree / split-K", be->allow_graph ? "on" : "off",
                     be->exact ? "exact" : "split-K flash decoding (128-position chunks)",
                     be->expert_cold_entries ? "device memory + pinned host + cold (fetched on demand), read through placement tables"
                     : be->pool_tabled     ? "device memory + pinned host, read through placement tables"
                                           : "all-resident",
                     (unsigned long long)be->expert_slots_cap, (unsigned long long)be->expert_slot_bytes,
                     be->expert_slots_req ? "fixed" : be->expert_budget ? "by budget" : "by free device memory",
                     (unsigned long long)be->expert_host_entries, (unsigned long long)be->expert_host_bytes,
                     (unsigned long long)(be->expert_host_budget ? be->expert_host_budget : DEFAULT_EXPERT_HOST_BUDGET),
                     (unsigned long long)be->expert_cold_entries,
                     !be->model_path.empty() && be->map_base ? "the model file" : "the tensors' mapping",
                     be->expert_prefetch ? "on" : "off",
                     be->model_path.empty() ? "(not set)" : be->model_path.c_str());
    return n < 0 ? 0 : (size_t)n;
}

uint64_t it_hip_setup_cost(it_hip* be, char* label, size_t label_len) {
    if (label && label_len) snprintf(label, label_len, "weight upload and repack");
    return be->setup_us;
}
// src/ops/mod.rs:915-924: acts only while some expert is cold; with every expert addressable there is nothing to read ahead
void it_hip_prefetch_hint(it_hip* be, const it_weights* w, const float* x, uint64_t x_len, uint64_t k) {
    be->cold_hint(w, x, x_len, k);
}

// Cap the expert slab, in bytes; 0 restores sizing from free device memory (placement.rs:178-189).  Like the
// reference's, read once: when the first pooled tensor sizes the slab.
void it_hip_set_expert_budget(it_hip* be, uint64_t bytes) { be->expert_budget = bytes; }
// The pinned-host tier behind the slab (placement.rs:322-326): experts that do not fit the device tier go to page-locked
// host memory up to this many bytes (0 = the default of 64 GiB); a pool that outgrows both is refused.
void it_hip_set_expert_host_budget(it_hip* be, uint64_t bytes) { be->expert_host_budget = bytes; }
// Fix the slab at n slots whatever the budget says; 0 restores sizing by budget (placement.rs:157-159)
void it_hip_set_expert_slots(it_hip* be, uint64_t n) { be->expert_slots_req = n; }
// How many expert matrices the model has: sizes the device read counters up front (placement.rs, experts.rs:424-438)
void it_hip_set_expert_pool(it_hip* be, uint64_t n) {
    be->expert_pool = n;
    if (n) be->expert_counters_reserve((size_t)n);
}
// Leave room for the permanent weights / the KV cache when the slab is sized automatically (placement.rs:203-209,
// 341-343): weights raise the reserve to at least dense + 1 GiB, KV adds to it.  No effect on an explicit budget.
void it_hip_reserve_for_weights(it_hip* be, uint64_t dense_bytes) {
    if (be->expert_budget) return;
    be->expert_reserve = std::max<uint64_t>(be->expert_reserve, dense_bytes + (1ull << 30));
}
void it_hip_reserve_for_kv(it_hip* be, uint64_t bytes) { be->expert_reserve += bytes; }
// Lookahead prefetch of the next layer's experts (placement.rs:164-168): nothing to fetch when every expert is
// resident; the switch is kept and reported.
void it_hip_set_prefetch(it_hip* be, int on) { be->expert_prefetch = on != 0; }
void it_hip_set_model_path(it_hip* be, const char* path) { be->model_path = path ? path : ""; }
void it_hip_set_map_base(it_hip* be, uint64_t base) { be->map_base = base; }

void it_hip_expert_stats(it_hip* be, it_expert_stats* out) {
    if (!out) return;
    memset(out, 0, sizeof *out);
    uint64_t tally[2];
    be->expert_counters_read(nullptr, tally);
    out->slots = be->expert_slots_cap;
    out->slot_bytes = be->expert_slot_bytes;
    out->resident = be->expert_resident;
    out->pool = be->expert_pool;
    out->lookups = tally[0] + tally[1];
    out->hits = tally[0];
    out->host_slots = be->expert_host_entries;
    out->evictions = be->expert_swaps + be->expert_cold_evictions;
    out->fetched = be->expert_fetched;
    out->oversubscribed = be->expert_cold_entries ? 1 : 0;
}

// What fraction of all expert reads the busiest slab-many matrices took, and the reads counted
// (ExpertCache::coverage, experts.rs:861-873).  0 = ok, 1 = no pooled tensor seen yet.
int it_hip_expert_coverage(it_hip* be, double* fraction, uint64_t* total_reads) {
    std::vector<uint32_t> counts;
    uint64_t tally[2];
    if (!be->expert_counted || !be->expert_counters_read(&counts, tally)) return 1;
    std::sort(counts.begin(), counts.end(), [](uint32_t a, uint32_t b) { return a > b; });
    uint64_t total = 0, top = 0;
    for (size_t i = 0; i < counts.size(); i++) {
        total += counts[i];
        if (i < be->expert_slots_cap) top += counts[i];
    }
    if (fraction) *fraction = total ? (double)top / (double)total : 0.0;
    if (total_reads) *total_reads = total;
    return 0;
}

// Re-place the pool by the reads counted so far (placement.rs:113-128): busy experts of the pinned host tier change
// places with idle ones of the device tier; with every expert in device memory nothing moves.  Returns the experts
// moved into device memory, or -1 on a device error.
int64_t it_hip_replace_experts_by_counts(it_hip* be) { return be->replace_by_counts(); }

// per-expert read counts of one tensor, in expert order (the rows of `counts` the gather wrote for it); returns the
// number of entries written, 0 when the tensor has not been seen
uint64_t it_hip_expert_counts(it_hip* be, const uint8_t* tensor_data, uint32_t* out, uint64_t cap) {
    auto it = be->weights.find(tensor_data);
    if (it == be->weights.end() || it->second.counter_base < 0) return 0;
    std::vector<uint32_t> counts;
    uint64_t tally[2];
    if (!be->expert_counters_read(&counts, tally)) return 0;
    // the tensor's entries run to the next tensor's base (or the end)
    size_t lo = (size_t)it->second.counter_base, hi = counts.size();
    for (auto& kv : be->weights)
        if (kv.second.counter_base > (int64_t)lo && (size_t)kv.second.counter_base < hi) hi = (size_t)kv.second.counter_base;
    uint64_t n = std::min<uint64_t>(hi - lo, cap);
    for (uint64_t i = 0; i < n; i++) out[i] = counts[lo + i];
    return n;
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
}  // extern "C"

bool it_hip::argmax_ready() {
    if (argmax_idx) return true;
    need_eager("argmax scratch is allocated");
    return check(hipMalloc((void**)&argmax_idx, 64 * 4), "hipMalloc(argmax)") &&
           check(hipMalloc((void**)&argmax_val, 64 * 4), "hipMalloc(argmax)") &&
           check(hipMalloc((void**)&argmax_out, 4), "hipMalloc(argmax)") &&
           check(hipMalloc((void**)&tok_ring, TOK_RING_CAP * 4), "hipMalloc(token ring)") &&
           check(hipHostMalloc((void**)&argmax_host, 4, hipHostMallocDefault), "hipHostMalloc(argmax)");
}

extern "C" {

uint32_t it_hip_argmax(it_hip* be, const float* buf, uint64_t len) {
    if (len == 0) return 0;
    float* d = be->act_in(buf, len);
    if (!d) return 0;
    if (!be->argmax_ready()) return 0;
    be->need_eager("argmax");
    argmax(d, (int64_t)len, be->argmax_out, be->argmax_idx, be->argmax_val, be->stream);
    be->launches += 2;
    if (!be->check(hipMemcpyAsync(be->argmax_host, be->argmax_out, 4, hipMemcpyDeviceToHost, be->stream), "download argmax")) return 0;
    be->check(hipStreamSynchronize(be->stream), "download argmax");
    be->d2h++;
    be->d2h_bytes += 4;
    return (uint32_t)*be->argmax_host;
}

int it_hip_embed_argmax(it_hip* be, const it_weights* table, const float* logits, uint64_t logits_len, float* x,
                        uint64_t x_len, uint64_t ring_index) {
    if (!table || !logits || !x || table->n_out != logits_len || table->n_in != x_len || logits_len == 0 ||
        logits_len >= (1ull << 31))
        return 0;
    if (table->ty != IT_Q8_0 && table->ty != IT_F16 && table->ty != IT_BF16 && table->ty != IT_F32) return 0;
    if (be->has_error) return 0;
    itk::WView w;
    if (!be->weights_view(table, "embed_argmax", &w)) return 0;
    // the logits are read where the previous pass left them: the device mirror, which begin_pass
    // has already marked stale with respect to the host copy
    auto lm = be->acts.find(logits);
    if (lm == be->acts.end() || !lm->second.dev || lm->second.cap < logits_len) return 0;
    float* dl = lm->second.dev;
    float* dx = be->act_out(x, x_len);
    if (!dx || !be->argmax_ready()) return 0;
    const int slot = (int)(ring_index % it_hip::TOK_RING_CAP);
    const int* dyn = be->dyn_slot(slot);
    int32_t *out = be->argmax_out, *idx = be->argmax_idx, *ring = be->tok_ring;
    float* val = be->argmax_val;
    int64_t n = (int64_t)logits_len;
    it_hip::OpRec rec;
    rec.id = OP_EMBED; rec.p[0] = dl; rec.p[1] = dx; rec.p[2] = w.q; rec.i[0] = n; rec.i[1] = w.n_in;
    be->launches += 1;
    be->submit(it_hip::FAM_OTHER, logits_len * 4 + x_len * 6, sig_of(OP_EMBED, dl, dx, w.q, w.scales, w.fmt, n, w.n_in, dyn ? 1 : 0),
               rec, [=](hipStream_t s) {
                   argmax_embed(dl, n, out, idx, val, w, dx, ring, slot, dyn, s);
               });
    return 1;
}

void it_hip_read_tokens(it_hip* be, uint64_t first_index, uint64_t n, uint32_t* out) {
    if (!n || !out) return;
    if (be->in_pass) be->finish_pass();
    if (!be->tok_ring || n > it_hip::TOK_RING_CAP) {
        be->fail("read_tokens: no tokens were picked on the device, or more than the ring holds");
        return;
    }
    be->check(hipStreamSynchronize(be->stream), "sync before reading token ids");
    be->chain_check();
    for (uint64_t i = 0; i < n;) {
        const uint64_t at = (first_index + i) % it_hip::TOK_RING_CAP;
        const uint64_t take = std::min<uint64_t>(n - i, it_hip::TOK_RING_CAP - at);
        be->check(hipMemcpy(out + i, be->tok_ring + at, take * 4, hipMemcpyDeviceToHost), "download token ids");
        i += take;
    }
    be->d2h++;
    be->d2h_bytes += n * 4;
}

void it_hip_release(it_hip* be, const void* host) {
    be->need_eager("a buffer is released");
    be->drop_graph();  // a captured graph may hold the pointers being freed
    auto a = be->acts.find(host);
    auto s = be->slabs.find(host);
    auto c = be->consts.find(host);
    if (a == be->acts.end() && s == be->slabs.end() && c == be->consts.end()) return;
    be->check(hipStreamSynchronize(be->stream), "sync before release");
    if (a != be->acts.end()) {
        be->mirror_bytes -= a->second.cap * sizeof(float);
        if (a->second.q_scales) be->quant_bytes -= a->second.q_cap / 32 * 4 + a->second.q_cap;
        if (a->second.dev) (void)hipFree(a->second.dev);
        if (a->second.q_scales) (void)hipFree(a->second.q_scales);
        if (a->second.q_quants) (void)hipFree(a->second.q_quants);
        be->acts.erase(a);
    }
    if (s != be->slabs.end()) {
        be->kv_bytes -= s->second.bytes;
        if (s->second.dev) (void)hipFree(s->second.dev);
        be->slabs.erase(s);
    }
    if (c != be->consts.end()) {
        be->const_bytes -= c->second.len * 4;
        if (c->second.dev) (void)hipFree(c->second.dev);
        be->consts.erase(c);
    }
}

void it_hip_graph_stats(it_hip* be, uint64_t out[4]) {
    out[0] = be->graph_captures;
    out[1] = be->graph_launches;
    out[2] = be->graph_aborts;
    out[3] = be->fused_launches;
}

void it_hip_chain_stats(it_hip* be, uint64_t out[4]) {
    out[0] = be->chain_launches;   // persistent-kernel launches in the last fused pass
    out[1] = be->chain_layers;     // layers they cover
    out[2] = be->chain_enabled ? 1 : 0;
    out[3] = (uint64_t)be->chain_spin_limit;
}

void it_hip_profile_begin(it_hip* be) {
    be->need_eager("profiling");
    be->check(hipStreamSynchronize(be->stream), "sync");
    be->prof_spans.clear();
    be->prof_pool_next = 0;
    be->prof_on = true;
}

int it_hip_profile_end(it_hip* be, it_profile_row* rows, int max_rows) {
    static const char* names[it_hip::FAM_COUNT] = {"matmul (dense GEMV/GEMM)", "moe_glu (expert gate+up)",
                                                   "matmul_experts (expert down)", "delta_rule", "attend",
                                                   "norms", "router (softmax + top-k)", "other",
                                                   "fused_gemv (norm + quantize + dense GEMVs)", "lm_head (norm + GEMV)",
                                                   "gdn_rows (l2 norm + delta rule)", "attn_prep (norm + rope + kv write)",
                                                   "layer_chain (a run of layers, persistent)"};
    be->prof_on = false;
    be->check(hipStreamSynchronize(be->stream), "sync");
    it_profile_row acc[it_hip::FAM_COUNT];
    memset(acc, 0, sizeof acc);
    for (auto& sp : be->prof_spans) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, sp.a, sp.b) != hipSuccess) continue;
        acc[sp.fam].launches++;
        acc[sp.fam].ms_total += ms;
        acc[sp.fam].bytes_total += sp.bytes;
    }
    int n = 0;
    for (int f = 0; f < it_hip::FAM_COUNT && n < max_rows; f++) {
        if (!acc[f].launches) continue;
        snprintf(acc[f].name, sizeof acc[f].name, "%s", names[f]);
        rows[n++] = acc[f];
    }
    be->prof_spans.clear();
    return n;
}

void it_hip_sync(it_hip* be) {
    if (!be->held.empty()) be->release_held();
    be->check(hipStreamSynchronize(be->stream), "sync");
    be->chain_check();
}
void it_hip_drop_mirrors(it_hip* be) { be->drop_all(); }
uint64_t it_hip_launch_count(it_hip* be) { return be->launches; }

}  // extern "C"
