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

#include <array>
#include <cstdint>
#include <cstring>
#include <functional>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/inferred_hip.h"
#include "kernels.h"
#include "kernels_fused.h"

// Seam ops as recorded for the fuser.  Pointer/int slots per op:
//   RMS        p: x, w, out                 i: rows, nd                       f: eps
//   RMS_HEADS  p: x, w                      i: head_dim, heads                f: eps
//   L2         p: x                         i: head_dim, heads                f: eps
//   QUANT      p: x, scales, quants         i: len
//   MATMUL     p: wq, ws, x, act_scales, act_quants, out   i: fmt, n_in, n_out, n_tok
//   CONV       p: state, x, w, out          i: kernel, channels, n_tok
//   GATHER     p: src, out                  i: chunk, stride, offset, out_len
//   DELTA      p: q, k, v, alpha, beta, ssm_a, dt_bias, state, out   i: n_tok, dk, dv, n_k, n_v
//   EW         p: a, b                      i: op (0 silu_mul, 1 sigmoid_mul, 2 add_assign, 3 add_scaled), n
//   SOFTMAX    p: x                         i: rows, row
//   ROUTE      p: probs, ids, weights       i: n_tok, n_expert, n_used
//   GLU        p: gq, gs, uq, us, gscale2, uscale2, ids, act_scales, act_quants, out
//              i: fmt, n_in, n_out, picks, n_used, x_mode, q_stride, s_stride
//   EXPERTS    p: q, s, scale2, ids, act_scales, act_quants, out     i: as GLU
//   FINISH     p: out, rows, weights, shared, logit   i: at, n, n_tok, n_used, logit_at
//   ROPE       p: x, table, dyn             i: half, n_tok, head_dim, n_rot, n_heads, pos
//   KVWRITE    p: slab, dyn, src            i: mul, offset, n
//   ATTEND     p: q, k, v, dyn, scratch, out   i: n_q, kv_dim, head_dim, n_head, n_head_kv, n_split, exact, n_pos  f: scale
enum OpId : int {
    OP_RMS = 1, OP_RMS_HEADS, OP_L2, OP_MATMUL, OP_ROPE, OP_SOFTMAX, OP_ATTEND, OP_EW, OP_SCALE, OP_CONV, OP_GATHER,
    OP_SCATTER, OP_DELTA, OP_ROUTE, OP_EXPERTS, OP_GLU, OP_FINISH, OP_ROWS, OP_SIGADD, OP_KVWRITE, OP_EMBED,
    OP_QUANT = 101
};

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
        bool elided = false;   // the op that writes this buffer was folded into a kernel that does not: the device copy is not its value
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
    bool act_q_reserve(Act& a, size_t len);  // room for the Q8_0 form of `len` floats
    Act* act_by_dev(const void* dev);        // the mirror whose device buffer holds `dev`, or null
    bool held_touches(const void* dev, size_t bytes) const;   // an op held back reads or writes inside [dev, dev + bytes)
    // marks the mirrors at these device addresses as not holding their ops' values (a fused kernel skipped the writes):
    // a host read of one raises the sticky error instead of returning what the buffer happens to hold
    void mark_elided(const std::vector<const void*>& devs);

    // ---- constants (f32 vectors uploaded once: norm weights, conv taps, ssm_a, dt_bias)
    struct Const {
        float* dev = nullptr;
        size_t len = 0;
        uint64_t ident = 0;  // as for weights: the vectors of another model may sit at the same host address
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
        int64_t counter_base = -1;  // first of this tensor's entries in expert_counts (expert tensors only)
        uint64_t ident = 0;         // length and a sample of the host bytes: another file mapped at the same address differs
        // Two-tier placement of an expert tensor (src/ops/cuda/experts.rs:34-52): once the pool outgrows its device tier
        // every pooled tensor is read through a table of per-expert addresses, each a device slot or a block of pinned
        // host memory mapped into the device's address space.  Host copies of the tables beside the device arrays.
        uint64_t n_expert = 0, q_stride = 0, s_stride = 0;
        const uint8_t** q_tab = nullptr;
        const uint8_t** s_tab = nullptr;
        uint8_t* tier = nullptr;                 // device: 0 = device memory, 1 = pinned host, 2 = cold (no copy held)
        std::vector<const uint8_t*> h_q, h_s;
        std::vector<uint8_t> h_tier;
        void* host_q = nullptr;                  // pinned blocks of the experts first placed in the host tier
        void* host_s = nullptr;
        std::vector<int32_t> slot_at;            // per expert: its slot in the cold tier's ring of device slots, or -1
    };
    bool place_two_tier(const it_experts* w, uint64_t n_dev, const char* who);
    bool table_for(Resident& r);                 // an identity table for a tensor that sits in device memory whole
    bool table_upload(Resident& r);
    int64_t replace_by_counts(uint64_t budget = ~0ull);
    void migrate_at_boundary(uint64_t n_tokens);   // bounded exchange every 64 tokens of evidence (placement.rs:33-80)
    uint64_t expert_host_entries = 0, expert_host_bytes = 0, expert_swaps = 0, tokens_since_migration = 0;
    bool pool_tabled = false;                    // some pooled tensor did not fit the device tier
    // The third tier (src/ops/cuda/experts.rs:67-93): experts that found room in neither tier are cold.  A cold
    // expert's table entry points at a zeroed sentinel; before an expert kernel runs, the picks are read back, every
    // cold pick is fetched from the model file (or its mapping) into a device slot taken from an expert the layer did
    // not pick (GCLOCK with leases), and the tables are patched.  State and code in expert_cold.cpp.
    struct ColdTier;
    ColdTier* cold = nullptr;
    uint64_t expert_cold_entries = 0, expert_cold_at_load = 0, expert_fetched = 0, expert_fetch_bytes = 0;
    uint64_t expert_cold_evictions = 0, fetch_read_us = 0, fetch_upload_us = 0, fetch_writes_us = 0;
    uint64_t picks_wait_us = 0, picks_copy_us = 0, prefetch_reads = 0, prefetch_used = 0, prefetch_wasted = 0;
    bool cold_sentinel(const uint8_t** q, const uint8_t** s, uint64_t q_stride, uint64_t s_stride);
    // make every expert that `route` picks from these tensors readable (fetching the cold ones) and lease them
    bool cold_resolve(const uint8_t* const* tensor_keys, int n_tensors, const it_route* route, bool opens_layer);
    void cold_clear_lease();
    void cold_ring_changed();                    // a pooled tensor was placed: the ring of device slots is rebuilt
    void cold_hint(const it_weights* next_router, const float* x, uint64_t x_len, uint64_t k);
    void cold_drop();
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
    uint64_t route_gen = 0;   // bumped whenever the device route ids are rewritten
    // the expert grouping that moe_work holds: valid for one route generation, pick count, expert count and tile size
    uint64_t group_gen = ~0ull;
    int group_picks = 0, group_experts = 0, group_tile = 0;
    bool group_cached(int picks, int n_expert, int tile);
    bool route_reserve(size_t picks);
    // scratch of the grouped expert matmuls (expert-sorted pair lists and their tiles)
    int32_t* moe_work = nullptr;
    size_t moe_work_ints = 0;
    int32_t* moe_work_for(size_t picks, size_t n_expert, size_t* ints);
    void* moe_f16 = nullptr;     // f16 hi / lo copies of the expert GEMM's activations
    int32_t* zero_ids = nullptr;  // expert id 0 for every token: a dense NVFP4 matrix run as a one-expert batch
    size_t zero_ids_n = 0;
    const int32_t* zero_ids_for(size_t n);
    size_t moe_f16_bytes = 0;
    void* moe_f16_for(size_t bytes);
    float* gdn_work = nullptr;   // T and P matrices of the chunked delta rule
    size_t gdn_work_floats = 0;
    float* gdn_work_for(size_t floats);
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
    bool argmax_ready();
    // ids picked on the device by embed_argmax, in call order (a ring)
    int32_t* tok_ring = nullptr;
    static constexpr size_t TOK_RING_CAP = 1 << 16;

    // ---- pass / graph state
    bool in_pass = false;
    uint64_t pass_tokens = 0;
    // decode graph (captured stream work of one n == 1 pass)
    struct Graph {
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        std::vector<uint64_t> signature;  // hash of each seam call's static arguments
        bool valid = false;
        // position slots of every fused attention block: {rope, key write, value write, attend}.  The fused kernel
        // takes ONE position for all four, so a replay is only valid while write row == rope position and the
        // context length == position + 1 (the seam does not tie them together; the model loop does)
        std::vector<std::array<int, 4>> attn_slots;
        std::vector<const void*> elided;   // device buffers whose ops the graph's fused kernels skip
        bool has_chain = false;
    };
    Graph graph;
    // Deferred: a single-token pass whose ops are recorded like a captured pass's and issued as fused launches whenever
    // something needs them on the stream (a cold expert's resolve reads the picks back, a host read, the pass's end):
    // the fusion of the decode path without its graph, for passes a graph cannot hold.
    enum class Mode { Eager, Capture, Replay, Deferred } mode = Mode::Eager;
    void flush_deferred();
    std::vector<uint64_t> pass_signature, prev_signature;
    int stable_passes = 0;      // consecutive eager decode passes with the same op sequence
    size_t replay_cursor = 0;
    uint64_t graph_launches = 0, graph_captures = 0, graph_aborts = 0;
    // work of the pass being captured or replayed, kept so it can run eagerly if the graph path breaks
    // One seam op as the fuser sees it: an id, its device pointers and integer
    // arguments (meaning per op, see the OpId table in backend.cpp), and the launch.
    struct OpRec {
        int id = 0;
        int fam = 0;          // timing family and algorithmic bytes of the launch (kept for ops that are held back)
        uint64_t bytes = 0;
        const void* p[12] = {};
        int64_t i[10] = {};
        float f[2] = {};
        std::function<void(hipStream_t)> run;
    };
    std::vector<OpRec> pending;
    bool fuse_enabled = true;
    unsigned* route_counter = nullptr;  // device word used by the fused router (zero between launches)
    uint64_t fused_launches = 0;  // launches in the captured graph after fusion
    void run_fused(std::vector<OpRec>& ops);
    std::vector<std::array<int, 4>> fused_attn_slots;  // filled by run_fused for the pass being captured
    // ---- layer chains (k_chain.hip): runs of decode layers as one persistent kernel each
    // hand-off words in uncached device memory, the epoch counter and the abort word; taken from a per-process pool
    // at the first chain and handed back when the backend goes (uncached memory is never freed once a kernel read it)
    struct ChainRes {
        unsigned long long* ll = nullptr;
        unsigned* epoch = nullptr;
        unsigned* abort_flag = nullptr;
        int device = -1;
    };
    ChainRes chain;
    bool chain_enabled = true;
    int chain_max_layers = 56;               // layers a chain may hold (CHAIN_MAX_LAYERS); INFERRED_HIP_CHAIN_LAYERS=n cuts a token into shorter chains (a measurement switch: hardware counters read short over a dispatch of a millisecond)
    bool chain_attn_enabled = true;          // attention mixers inside the chains; INFERRED_HIP_NO_CHAIN_ATTN=1 keeps their kernels between two chains (a measurement switch)
    bool count_reads_in_fused = true;  // the fused decode kernels add the picks to the expert read counters (off: a measurement switch)
    bool eager_fused = false;          // single-token passes without a graph still go through the fuser (measurement switch)
    bool chain_ran = false;            // a chain has been issued since the abort word was last looked at
    int chain_spin_limit = 1 << 21;
    uint64_t chain_launches = 0, chain_layers = 0;   // per fused pass, for the statistics
    bool chain_acquire();
    void chain_release();
    void chain_check();                // after a stream synchronisation: raises the sticky error if a chain gave up
    std::vector<const void*> fused_elided;   // device buffers the pass being fused no longer writes (filled by run_fused)
    bool attn_positions_agree(const std::vector<std::array<int, 4>>& slots) const;
    struct PreCopy {
        void* dev;
        const void* host;
        size_t bytes;
    };
    // ops of a batch pass held back because they begin a run that has a one-kernel form (fuser.cpp)
    std::vector<OpRec> held;
    int hold_step(const OpRec& rec) const;   // 0: not part of a run, 1: continues it, 2: completes it
    void release_held();                     // the run broke off: issue what is held op by op, in order
    void finish_held();                      // the run is complete: one kernel (or op by op when its shape is not taken)
    bool small_ffn(const std::vector<OpRec>& run);   // the routed FFN of a short batch as two launches
    bool small_ffn_enabled = true;           // INFERRED_HIP_NO_SMALL_FFN=1 issues it op by op (a measurement switch)
    std::vector<PreCopy> precopies;  // host -> device inputs of a graphed pass, issued before the graph
    int* dyn_dev = nullptr;    // device ints read by position-dependent kernels
    // pinned staging, double-buffered: a pass may fill one while the previous pass's async
    // copy of the other has not run yet
    int* dyn_hosts[2] = {nullptr, nullptr};
    hipEvent_t dyn_evt[2] = {nullptr, nullptr};
    bool dyn_evt_used[2] = {false, false};
    int dyn_cur = 0;
    int* dyn_host = nullptr;   // = dyn_hosts[dyn_cur]
    void dyn_rotate();
    void dyn_upload();
    size_t dyn_count = 0;
    static constexpr size_t DYN_CAP = 4096;
    const int* dyn_slot(int value);   // null in eager mode: the kernel takes the scalar by value
    void need_eager(const char* why); // leave capture/replay: run what the pass queued so far eagerly
    void finish_pass();
    bool mid_pass_read = false;
    bool profile_pass = false;  // a replay-shaped pass whose fused launches run one by one between timing events

    // Every kernel launch goes through here.  `sig` hashes the launch's static arguments
    // (pointers, shapes); position-dependent scalars never enter it.
    template <class F>
    void submit(int fam, uint64_t bytes, uint64_t sig, OpRec rec, F&& f) {
        launches++;
        if (mode == Mode::Eager) {
            if (in_pass && pass_tokens == 1) pass_signature.push_back(sig);
            if (in_pass && pass_tokens > 1 && !exact && fuse_enabled) {
                // a batch pass in fast mode holds back the ops of two known elementwise runs and issues each run as
                // one kernel once it is complete (hold_step, fuser.cpp); anything else releases what is held first
                int st = hold_step(rec);
                if (!st && !held.empty()) {
                    release_held();
                    st = hold_step(rec);
                }
                if (st) {
                    rec.run = f;
                    rec.fam = fam;
                    rec.bytes = bytes;
                    held.push_back(std::move(rec));
                    if (st == 2) finish_held();
                    return;
                }
            } else if (!held.empty()) {
                release_held();
            }
            Span sp(this, fam, bytes);
            f(stream);
            check(hipGetLastError(), "kernel launch");
            return;
        }
        rec.run = f;
        pending.push_back(std::move(rec));
        pass_signature.push_back(sig);
        if (mode == Mode::Deferred) return;
        if (mode == Mode::Capture) {
            // queued: the whole pass is fused and captured at end_pass
        } else if (replay_cursor >= graph.signature.size() || graph.signature[replay_cursor] != sig) {
            need_eager("the op sequence changed");
        } else {
            replay_cursor++;
        }
    }

    // ---- per-kernel-family timing with HIP events on the launch stream
    enum Family { FAM_MATMUL = 0, FAM_MOE_GLU, FAM_MOE_DOWN, FAM_DELTA, FAM_ATTEND, FAM_NORM, FAM_ROUTER, FAM_OTHER,
                  FAM_FUSED_GEMV, FAM_LM_HEAD, FAM_GDN_ROWS, FAM_ATTN_PREP, FAM_CHAIN, FAM_COUNT };
    struct ProfSpan {
        hipEvent_t a, b;
        int fam;
        uint64_t bytes;
    };
    bool prof_on = false;
    std::vector<ProfSpan> prof_spans;
    std::vector<hipEvent_t> prof_pool;
    size_t prof_pool_next = 0;
    hipEvent_t prof_event();
    // RAII span: records an event before and after the launches issued inside its scope
    struct Span {
        it_hip* be;
        ProfSpan s;
        bool live;
        Span(it_hip* b, int fam, uint64_t bytes);
        ~Span();
    };

    // ---- counters
    uint64_t launches = 0, h2d = 0, d2h = 0, h2d_bytes = 0, d2h_bytes = 0;
    uint64_t weight_bytes = 0, kv_bytes = 0, quant_bytes = 0, mirror_bytes = 0, const_bytes = 0;
    uint64_t setup_us = 0;
    // ---- expert cache (src/ops/cuda/ops/placement.rs, experts.rs)
    // Every expert matrix of a pooled tensor is placed at first sight of the tensor: in device memory while slots are
    // left, else in pinned host memory (place_two_tier).  The slab has one uniform slot size (the bytes of one expert
    // matrix in the file); its capacity in slots comes from set_expert_slots, else set_expert_budget, else free
    // device memory minus the reserves.  Reads are counted on the device.
    uint64_t expert_resident = 0, expert_slot_bytes = 0, expert_pool = 0, expert_slots_cap = 0;
    uint64_t expert_budget = 0, expert_host_budget = 0, expert_slots_req = 0, expert_reserve = 1ull << 30;
    bool expert_prefetch = true;
    std::string model_path;
    uint64_t map_base = 0;
    uint32_t* expert_counts = nullptr;            // device: reads per (tensor, expert), in placement order
    size_t expert_counts_cap = 0, expert_counted = 0;
    unsigned long long* expert_tally = nullptr;   // device: [0] reads served from device memory, [1] from a host tier
    bool expert_counters_reserve(size_t entries);
    bool expert_counters_read(std::vector<uint32_t>* counts, uint64_t tally[2]);

    void drop_all();
    void drop_graph();
    ~it_hip();
};
