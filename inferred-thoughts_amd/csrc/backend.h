// The HIP backend behind the C ABI: device mirrors keyed on host addresses,
// resident (repacked) weights, device-owned KV and recurrent-state slabs, a sticky
// error, and one stream on which every kernel is issued in call order.
//
// Mirrors the behaviour of the reference's device backend
// (/root/reference src/ops/cuda/ops/mod.rs:150-633, residency.rs) without its
// structure: there is no driver-API module loader and no hand-built graph; kernels
// are ordinary HIP launches and decode passes are captured with stream capture.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/inferred_hip.h"
#include "kernels.h"

struct it_hip {
    // ---- configuration
    bool exact = false;
    bool allow_graph = true;
    int device = 0;
    hipStream_t stream = nullptr;

    // ---- sticky error (src/ops/cuda/ops/mod.rs:91-110)
    std::string error;
    bool has_error = false;
    void fail(const std::string& what);
    bool check(hipError_t e, const char* what);

    // ---- activation mirrors (keyed on host address)
    struct Act {
        float* dev = nullptr;
        size_t cap = 0;  // floats
        bool dev_current = false;
        // cached Q8_0 form of the first q_len floats
        float* q_scales = nullptr;
        int8_t* q_quants = nullptr;
        size_t q_cap = 0;  // floats covered
        size_t q_len = 0;
        bool q_valid = false;
    };
    std::unordered_map<const void*, Act> acts;
    Act* act_slot(const float* host, size_t len);
    float* act_in(const float* host, size_t len);     // device copy current for reading
    float* act_out(const float* host, size_t len);    // device copy about to be overwritten
    float* act_inout(const float* host, size_t len);  // read then written in place
    bool act_quantized(const float* host, size_t len, const float** scales, const int8_t** quants,
                       float** dev_x);

    // ---- constants (f32 vectors uploaded once: norm weights, conv taps, ssm_a, dt_bias)
    struct Const {
        float* dev = nullptr;
        size_t len = 0;
    };
    std::unordered_map<const void*, Const> consts;
    const float* const_in(const float* host, size_t len);

    // ---- resident weights (keyed on the mmap address, repacked at upload)
    struct Resident {
        void* q = nullptr;
        void* scales = nullptr;
        size_t q_bytes = 0, s_bytes = 0;
        int fmt = 0;
        uint64_t n_in = 0, rows = 0;
        float* scale2 = nullptr;  // experts' per-expert second scale
    };
    std::unordered_map<const void*, Resident> weights;
    const Resident* resident(const uint8_t* data, uint64_t len, uint32_t ty, uint64_t n_in, uint64_t rows,
                             const char* who);
    bool weights_view(const it_weights* w, const char* who, itk::WView* out);
    bool experts_view(const it_experts* w, const char* who, itk::ExpertsView* out);

    // ---- device-owned slabs (KV as u16, recurrent state as f32)
    struct Slab {
        void* dev = nullptr;
        size_t bytes = 0;
        bool dev_owned = false;
        bool is_state = false;
    };
    std::unordered_map<const void*, Slab> slabs;
    void* slab_in(const void* host, size_t bytes, bool is_state);

    // ---- device route storage (Route::Device)
    int32_t* route_ids = nullptr;
    float* route_w = nullptr;
    size_t route_cap = 0;  // picks
    uint64_t route_n_used = 0, route_n_tok = 0;
    bool route_reserve(size_t picks);
    bool route_stage(const it_route* r, const int32_t** ids, const float** w, uint64_t* n_used, uint64_t* n_tok);

    // ---- RoPE tables, built on the host in f64 (naive.rs:205-208)
    struct Rope {
        float2* dev = nullptr;
        size_t cap_pos = 0;
    };
    std::unordered_map<uint64_t, Rope> ropes;
    const float2* rope_table(float theta, uint64_t n_rot, uint64_t need_pos);

    // ---- scratch
    float* attn_scratch = nullptr;
    size_t attn_scratch_cap = 0;  // floats
    float* scratch_f32(size_t floats);
    int32_t* argmax_idx = nullptr;
    float* argmax_val = nullptr;
    int32_t* argmax_out = nullptr;
    int32_t* argmax_host = nullptr;  // pinned

    // ---- pass / graph state
    bool in_pass = false;
    uint64_t pass_tokens = 0;
    // decode graph (captured stream work of one n == 1 pass)
    struct Graph {
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        std::vector<uint64_t> signature;  // hash of each seam call's static arguments
        bool valid = false;
    };
    Graph graph;
    enum class Mode { Eager, Capture, Replay } mode = Mode::Eager;
    uint64_t decode_passes = 0;
    std::vector<uint64_t> pass_signature;
    size_t replay_cursor = 0;
    bool replay_broken = false;
    int* dyn_dev = nullptr;    // device ints read by position-dependent kernels
    int* dyn_host = nullptr;   // pinned staging
    size_t dyn_count = 0, dyn_cap = 0;
    bool graph_note(uint64_t sig);  // returns true when the kernel must actually be launched
    const int* dyn_slot(int value);
    bool mid_pass_read = false;

    // ---- counters
    uint64_t launches = 0, h2d = 0, d2h = 0, h2d_bytes = 0, d2h_bytes = 0;
    uint64_t weight_bytes = 0, kv_bytes = 0, quant_bytes = 0, mirror_bytes = 0, const_bytes = 0;
    uint64_t setup_us = 0;
    uint64_t expert_lookups = 0, expert_resident = 0, expert_slot_bytes = 0, expert_pool = 0;
    uint64_t expert_budget = 0, expert_host_budget = 0, expert_slots_req = 0;

    void drop_all();
    ~it_hip();
};
