// The third tier of the expert pool: experts that found room neither in device memory nor in pinned host memory.
//
// Behaviour follows the reference's cold tier (src/ops/cuda/experts.rs:67-93, resolve :1047-1190, fetch_batch and
// make_resident :1418-1540, start_prefetch :1196-1280, evict_unleased and clock_pick :2112-2233; the caller's side in
// src/ops/cuda/ops/moe.rs:820-1060).  A cold expert has no copy anywhere but the model file; its table entry points at
// a zeroed sentinel.  Before an expert kernel of an oversubscribed pool is launched the picks are read back (a host
// decision inside the pass, so such passes never run from a graph), every pick is leased, and each cold pick
// is fetched into a device slot taken from an expert the layer did not pick: GCLOCK over a ring of all device slots,
// heat 0..3, an arrival entering at 1.  The victim's entry is pointed at the sentinel, the fetched expert's at the
// slot.  All of it is ordered on the launch stream: the copies into a slot, the repack and the table patches are
// queued behind every kernel that may still read the victim, and ahead of the kernel that reads the arrival.
//
// The bytes come from the model file through a pool of reader threads (pread at the tensor's offset when the file and
// the mapping's base are known, else a copy out of the mapping) into pinned staging, cross the bus in one copy per
// chunk of experts, and are repacked on the device straight into the slot.  Tensors that were read under the same
// routing decision before (up and down after gate) are fetched with the opener's resolve, as one batch.  With a hint
// (the next layer's router on this layer's input) the likely picks of the next layer are read into pinned staging
// while the device computes this layer; the next resolve publishes what finished.
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <deque>
#include <mutex>
#include <thread>

#include "backend.h"

using namespace itk;

namespace {

constexpr uint8_t HEAT_MAX = 3;      // experts.rs:2136
constexpr uint8_t HEAT_NEW = 1;      // experts.rs:2164
constexpr size_t FETCH_CHUNK = 16;   // experts read, uploaded and repacked as one batch
constexpr size_t PREFETCH_SLOTS = 48;

uint64_t clock_us() {
    return (uint64_t)std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// Threads that bring expert bytes into pinned staging.  A job is done when its state word is 1 (read) or 2 (failed).
class ReadPool {
  public:
    struct Job {
        uint8_t* dst;
        const uint8_t* src;   // the expert's bytes in the mapping
        size_t len;
        int* state;           // written under the pool's lock
    };
    explicit ReadPool(int n) {
        for (int i = 0; i < n; i++) threads_.emplace_back([this] { work(); });
    }
    ~ReadPool() {
        {
            std::lock_guard<std::mutex> g(m_);
            stop_ = true;
        }
        cv_.notify_all();
        for (auto& t : threads_) t.join();
        if (fd_ >= 0) close(fd_);
        if (dfd_ >= 0) close(dfd_);
    }
    // reads that went through the unbuffered descriptor, and reads in all
    void counts(uint64_t* direct, uint64_t* all) {
        std::lock_guard<std::mutex> g(m_);
        *direct = n_direct_;
        *all = n_reads_;
    }
    // read from `path` at (address - base) instead of copying out of the mapping; an empty path goes back to the mapping
    void source(const std::string& path, uint64_t base) {
        std::lock_guard<std::mutex> g(m_);
        if (path == path_ && base == base_) return;
        if (fd_ >= 0) close(fd_);
        if (dfd_ >= 0) close(dfd_);
        fd_ = dfd_ = -1;
        file_size_ = 0;
        path_ = path;
        base_ = base;
        if (path.empty() || !base) return;
        int fd = open(path.c_str(), O_RDONLY | O_CLOEXEC);
        struct stat st;
        if (fd >= 0 && fstat(fd, &st) == 0) {
            fd_ = fd;
            file_size_ = (uint64_t)st.st_size;
        } else if (fd >= 0) {
            close(fd);
        }
        // Unbuffered reads (platform.rs:60-96, 200-215; fetch.rs:71-73): the fetches of a token stay out of the page
        // cache, which the mapping of the same file would otherwise share with them.  On by default, as in the
        // reference on Linux; INFERRED_FETCH_DIRECT=0 / =1 overrides; a file system that refuses the flag (tmpfs) or a
        // read that fails with it falls back to the buffered descriptor.
        const char* e = getenv("INFERRED_FETCH_DIRECT");
        const bool want = e ? strcmp(e, "0") != 0 : true;
        if (want && fd_ >= 0) dfd_ = open(path.c_str(), O_RDONLY | O_CLOEXEC | O_DIRECT);
    }
    void submit(const Job& j) {
        {
            std::lock_guard<std::mutex> g(m_);
            *j.state = 0;
            jobs_.push_back(j);
        }
        cv_.notify_one();
    }
    // blocks until the job that owns `state` has finished; true when it read its bytes
    bool wait(int* state) {
        std::unique_lock<std::mutex> g(m_);
        done_.wait(g, [&] { return *state != 0; });
        return *state == 1;
    }

  private:
    static constexpr size_t DIRECT_ALIGN = 4096;   // platform.rs:78
    void work() {
        uint8_t* bounce = nullptr;
        size_t bounce_len = 0;
        for (;;) {
            Job j;
            int fd, dfd;
            uint64_t base, size;
            {
                std::unique_lock<std::mutex> g(m_);
                cv_.wait(g, [&] { return stop_ || !jobs_.empty(); });
                if (jobs_.empty()) {
                    free(bounce);
                    return;
                }
                j = jobs_.front();
                jobs_.pop_front();
                fd = fd_;
                dfd = dfd_;
                base = base_;
                size = file_size_;
            }
            bool ok = true, direct = false;
            const uint64_t addr = (uint64_t)(uintptr_t)j.src;
            if (fd >= 0 && addr >= base && addr - base + j.len <= size) {
                const uint64_t off = addr - base;
                if (dfd >= 0) {
                    // the aligned range around the expert's bytes into this thread's aligned buffer (offset, address and
                    // length in whole DIRECT_ALIGN units; the range of the file's last expert may run past its end and
                    // comes back short), then the bytes themselves to where the job wants them
                    const uint64_t lo = off & ~(uint64_t)(DIRECT_ALIGN - 1);
                    const size_t span = (size_t)(((off + j.len + DIRECT_ALIGN - 1) & ~(uint64_t)(DIRECT_ALIGN - 1)) - lo);
                    if (span > bounce_len) {
                        free(bounce);
                        bounce = nullptr;
                        bounce_len = 0;
                        void* mem = nullptr;
                        if (posix_memalign(&mem, DIRECT_ALIGN, span) == 0) {
                            bounce = (uint8_t*)mem;
                            bounce_len = span;
                        }
                    }
                    if (bounce) {
                        const size_t need = (size_t)(off - lo) + j.len;
                        size_t got = 0;
                        direct = true;
                        while (got < need) {
                            // a short read leaves an unaligned remainder: what is still missing is then read from the last
                            // whole unit on
                            const size_t at = got & ~(size_t)(DIRECT_ALIGN - 1);
                            ssize_t r = pread(dfd, bounce + at, span - at, (off_t)(lo + at));
                            if (r <= 0) {
                                direct = false;
                                break;
                            }
                            got = at + (size_t)r;
                        }
                        if (direct) memcpy(j.dst, bounce + (off - lo), j.len);
                    }
                }
                if (!direct) {
                    size_t got = 0;
                    while (got < j.len) {
                        ssize_t r = pread(fd, j.dst + got, j.len - got, (off_t)(off + got));
                        if (r <= 0) {
                            ok = false;
                            break;
                        }
                        got += (size_t)r;
                    }
                }
            } else {
                memcpy(j.dst, j.src, j.len);
            }
            {
                std::lock_guard<std::mutex> g(m_);
                *j.state = ok ? 1 : 2;
                n_reads_++;
                if (direct) n_direct_++;
            }
            done_.notify_all();
        }
    }
    std::vector<std::thread> threads_;
    std::mutex m_;
    std::condition_variable cv_, done_;
    std::deque<Job> jobs_;
    bool stop_ = false;
    int fd_ = -1, dfd_ = -1;
    uint64_t base_ = 0, file_size_ = 0, n_direct_ = 0, n_reads_ = 0;
    std::string path_;
};

// it_hip_clock_pick's walk (experts.rs:2215-2233) without its scan for an unleased slot before the walk: heat is at
// most HEAT_MAX, so a ring with an unleased slot yields it within HEAT_MAX + 1 sweeps, and one sweep more finds none.
int64_t clock_walk(uint8_t* heat, const uint8_t* leased, uint64_t n, uint64_t* hand) {
    for (uint64_t step = 0; step < (uint64_t)(HEAT_MAX + 2) * n; step++) {
        const uint64_t i = *hand % n;
        *hand = (i + 1) % n;
        if (leased[i]) continue;
        if (heat[i] == 0) return (int64_t)i;
        heat[i]--;
    }
    return -1;
}

int fetch_threads() {
    const char* e = getenv("INFERRED_FETCH_THREADS");   // the reference's switch (experts.rs:556-560)
    int n = e ? atoi(e) : 8;
    return n < 1 ? 1 : n > 64 ? 64 : n;
}

}  // namespace

struct it_hip::ColdTier {
    struct Slot {
        uint8_t* q;
        uint8_t* s;
        Resident* owner;
        uint32_t e;
    };
    // every device slot of the pool, in placement order; heat and lease flags beside it
    std::vector<Slot> ring;
    std::vector<uint8_t> heat, leased;
    uint64_t hand = 0;
    bool ring_valid = false;
    uint64_t q_stride = 0, s_stride = 0;
    // the current lease: the (tensor, expert) entries of the routing decision being computed; `leased` flags the ring
    // slots they hold and is kept in step entry by entry (a sweep over the ring per resolve would cost more than the
    // fetches of a large pool)
    std::vector<std::pair<Resident*, uint32_t>> lease;
    std::vector<uint32_t> lease_picks;
    void lease_add(Resident* r, uint32_t e) {
        lease.emplace_back(r, e);
        if (ring_valid && r->slot_at.size() > e && r->slot_at[e] >= 0) leased[(size_t)r->slot_at[e]] = 1;
    }
    void lease_clear() {
        if (ring_valid)
            for (auto& le : lease)
                if (le.first->slot_at.size() > le.second && le.first->slot_at[le.second] >= 0) leased[(size_t)le.first->slot_at[le.second]] = 0;
        lease.clear();
        lease_picks.clear();
    }
    // the picks of a device route, read back once per decision
    std::vector<int32_t> picks;
    uint64_t picks_gen = ~0ull;
    uint8_t *sentinel_q = nullptr, *sentinel_s = nullptr;
    // fetch staging, double-buffered: pinned host bytes as in the file, the same on the device, an event per half
    uint8_t* pin[2] = {nullptr, nullptr};
    uint8_t* raw[2] = {nullptr, nullptr};
    hipEvent_t evt[2] = {nullptr, nullptr};
    bool evt_used[2] = {false, false};
    int cur = 0;
    uint64_t raw_one = 0;
    int read_state[FETCH_CHUNK] = {};
    // table patches of one resolve, read by the patch kernel from pinned memory
    ExpertPatch* patches = nullptr;
    size_t patch_cap = 0, n_patch = 0;
    hipEvent_t patch_evt = nullptr;
    bool patch_evt_used = false;
    ReadPool* pool = nullptr;
    // which tensors are read under one routing decision (opener = the first, i.e. gate), and which opener follows which
    std::unordered_map<const uint8_t*, std::vector<const uint8_t*>> group;
    std::unordered_map<const uint8_t*, const uint8_t*> next_opener;
    const uint8_t* cur_opener = nullptr;
    std::vector<uint32_t> opener_picks;
    // lookahead: the next router's logits on this layer's input, and reads started from its top-k
    std::vector<float> hint_logits;
    size_t hint_n = 0, hint_k = 0;
    bool hint_pending = false;
    uint64_t hint_gen = 0;
    std::vector<uint32_t> hint_ids;
    uint8_t* pre_pin = nullptr;
    int pre_state[PREFETCH_SLOTS] = {};
    std::vector<int> pre_free;
    std::unordered_map<uint64_t, int> pre_entries;   // counter index -> staging slot
    hipEvent_t pre_evt = nullptr;                    // the uploads queued out of the lookahead staging
    bool pre_evt_used = false;
};

void it_hip::cold_ring_changed() {
    if (cold) cold->ring_valid = false;
}

void it_hip::cold_clear_lease() {
    if (!cold) return;
    cold->lease_clear();
}

void it_hip::cold_drop() {
    if (!cold) return;
    ColdTier& c = *cold;
    delete c.pool;   // joins the readers: nothing writes the staging after this
    if (stream) (void)hipStreamSynchronize(stream);
    if (!c.hint_logits.empty()) it_hip_release(this, c.hint_logits.data());
    for (int i = 0; i < 2; i++) {
        if (c.pin[i]) (void)hipHostFree(c.pin[i]);
        if (c.raw[i]) (void)hipFree(c.raw[i]);
        if (c.evt[i]) (void)hipEventDestroy(c.evt[i]);
    }
    if (c.patches) (void)hipHostFree(c.patches);
    if (c.patch_evt) (void)hipEventDestroy(c.patch_evt);
    if (c.pre_pin) (void)hipHostFree(c.pre_pin);
    if (c.pre_evt) (void)hipEventDestroy(c.pre_evt);
    if (c.sentinel_q) (void)hipFree(c.sentinel_q);
    if (c.sentinel_s) (void)hipFree(c.sentinel_s);
    delete cold;
    cold = nullptr;
}

// The zeroed slot every cold entry points at (experts.rs:1579-1600).  A correct pass never reads it.
bool it_hip::cold_sentinel(const uint8_t** q, const uint8_t** s, uint64_t q_stride, uint64_t s_stride) {
    if (!cold) cold = new ColdTier();
    ColdTier& c = *cold;
    if (!c.sentinel_q) {
        if (!check(hipMalloc((void**)&c.sentinel_q, q_stride), "hipMalloc(cold sentinel)") ||
            !check(hipMalloc((void**)&c.sentinel_s, s_stride), "hipMalloc(cold sentinel)") ||
            !check(hipMemset(c.sentinel_q, 0, q_stride), "hipMemset(cold sentinel)") ||
            !check(hipMemset(c.sentinel_s, 0, s_stride), "hipMemset(cold sentinel)"))
            return false;
        c.q_stride = q_stride;
        c.s_stride = s_stride;
    }
    if (q_stride != c.q_stride || s_stride != c.s_stride) {
        fail("expert pool: an oversubscribed pool needs one repacked expert size, and this tensor's differs");
        return false;
    }
    *q = c.sentinel_q;
    *s = c.sentinel_s;
    return true;
}

namespace {

// a cold pick: its tensor (the placement record and the host address of its bytes) and the expert
struct Want {
    it_hip::Resident* r;
    const uint8_t* key;
    uint32_t e;
};

}  // namespace

// Lookahead (Ops::prefetch_hint, src/ops/mod.rs:915-924; moe.rs:820-845): the next router on this layer's input, queued
// before this layer's resolve so that its one readback brings the logits home too.  Changes no value the model computes.
void it_hip::cold_hint(const it_weights* w, const float* x, uint64_t x_len, uint64_t k) {
    if (!expert_cold_entries || !expert_prefetch || !w || !x || !k || w->n_out == 0 || x_len != w->n_in) return;
    if (!cold) cold = new ColdTier();
    ColdTier& c = *cold;
    if (c.hint_logits.size() < w->n_out) {
        if (!c.hint_logits.empty()) it_hip_release(this, c.hint_logits.data());
        c.hint_logits.assign(std::max<size_t>(w->n_out, 1024), 0.0f);
    }
    it_hip_matmul(this, w, x, x_len, c.hint_logits.data(), w->n_out);
    c.hint_n = w->n_out;
    c.hint_k = std::min<uint64_t>(k, w->n_out);
    c.hint_gen = route_gen;
    c.hint_pending = !has_error;
}

bool it_hip::cold_resolve(const uint8_t* const* keys, int n_keys, const it_route* route, bool opens_layer) {
    if (!expert_cold_entries) return true;
    if (!cold) cold = new ColdTier();
    ColdTier& c = *cold;
    Resident* first = &weights[keys[0]];
    const uint64_t n_expert = first->n_expert;

    // ---- 1. the picks, on the host
    std::vector<uint32_t> uniq;
    if (route->kind == IT_ROUTE_HOST) {
        const uint64_t n = route->n_used * route->n_tok;
        uniq.reserve(n);
        for (uint64_t i = 0; i < n; i++)
            if (route->ids[i] < n_expert) uniq.push_back((uint32_t)route->ids[i]);
    } else {
        const size_t n = (size_t)(route_n_used * route_n_tok);
        if (c.picks_gen != route_gen || c.picks.size() != n) {
            need_eager("the picks are read back");   // the route kernel itself may still be waiting in a recorded pass
            uint64_t t0 = clock_us();
            if (!check(hipStreamSynchronize(stream), "sync before the picks are read back")) return false;
            uint64_t t1 = clock_us();
            c.picks.resize(n);
            if (!check(hipMemcpy(c.picks.data(), route_ids, n * sizeof(int32_t), hipMemcpyDeviceToHost), "download picks")) return false;
            c.picks_gen = route_gen;
            picks_wait_us += t1 - t0;
            picks_copy_us += clock_us() - t1;
            d2h++;
            d2h_bytes += n * 4;
        }
        uniq.reserve(n);
        for (int32_t id : c.picks)
            if (id >= 0 && (uint64_t)id < n_expert) uniq.push_back((uint32_t)id);
    }
    std::sort(uniq.begin(), uniq.end());
    uniq.erase(std::unique(uniq.begin(), uniq.end()), uniq.end());
    if (uniq.empty()) return true;

    // the hint's logits come home with the picks; the top-k is taken here (512 logits are 2 KB: moe.rs:823-827)
    c.hint_ids.clear();
    if (c.hint_pending && opens_layer) {
        c.hint_pending = false;
        need_eager("the hint's logits are read back");
        auto a = acts.find(c.hint_logits.data());
        if (c.hint_gen == route_gen && a != acts.end() && a->second.dev && a->second.dev_current) {
            std::vector<float> host(c.hint_n);
            if (check(hipStreamSynchronize(stream), "sync before the hint is read back") &&
                check(hipMemcpy(host.data(), a->second.dev, c.hint_n * sizeof(float), hipMemcpyDeviceToHost), "download hint logits")) {
                std::vector<uint32_t> order(c.hint_n);
                for (size_t i = 0; i < c.hint_n; i++) order[i] = (uint32_t)i;
                std::partial_sort(order.begin(), order.begin() + c.hint_k, order.end(), [&](uint32_t x, uint32_t y) {
                    return host[x] != host[y] ? host[x] > host[y] : x < y;
                });
                c.hint_ids.assign(order.begin(), order.begin() + c.hint_k);
                std::sort(c.hint_ids.begin(), c.hint_ids.end());
            }
        }
    }

    // ---- 2. a new routing decision ends the lease of the last one (moe.rs:847-853)
    if (uniq != c.lease_picks) {
        c.lease_clear();
        c.lease_picks = uniq;
    }

    // ---- 3. which tensors this decision reads: the call's own and, for the opener, those that followed it before
    std::vector<const uint8_t*> tensors(keys, keys + n_keys);
    if (opens_layer) {
        if (c.cur_opener && c.cur_opener != keys[0]) c.next_opener[c.cur_opener] = keys[0];
        c.cur_opener = keys[0];
        c.opener_picks = uniq;
        auto g = c.group.find(keys[0]);
        if (g != c.group.end())
            for (const uint8_t* t : g->second)
                if (std::find(tensors.begin(), tensors.end(), t) == tensors.end()) tensors.push_back(t);
    } else if (c.cur_opener && uniq == c.opener_picks) {
        auto& g = c.group[c.cur_opener];
        for (int i = 0; i < n_keys; i++)
            if (keys[i] != c.cur_opener && std::find(g.begin(), g.end(), keys[i]) == g.end()) g.push_back(keys[i]);
    }

    // ---- 4. the ring of device slots
    if (!c.ring_valid) {
        std::vector<Resident*> all;
        for (auto& kv : weights)
            if (kv.second.counter_base >= 0 && kv.second.q_tab) all.push_back(&kv.second);
        std::sort(all.begin(), all.end(), [](Resident* a, Resident* b) { return a->counter_base < b->counter_base; });
        c.ring.clear();
        for (Resident* r : all) {
            if (r->q_stride != c.q_stride || r->s_stride != c.s_stride) {
                fail("expert pool: an oversubscribed pool needs one repacked expert size");
                return false;
            }
            r->slot_at.assign(r->n_expert, -1);
            for (uint64_t e = 0; e < r->n_expert; e++)
                if (r->h_tier[e] == 0) {
                    r->slot_at[e] = (int32_t)c.ring.size();
                    c.ring.push_back({const_cast<uint8_t*>(r->h_q[e]), const_cast<uint8_t*>(r->h_s[e]), r, (uint32_t)e});
                }
        }
        c.heat.assign(c.ring.size(), 0);
        c.leased.assign(c.ring.size(), 0);
        c.hand = 0;
        c.ring_valid = true;
        auto held_lease = std::move(c.lease);   // the flags of a lease taken before the ring was (re)built
        c.lease.clear();
        for (auto& le : held_lease) c.lease_add(le.first, le.second);
    }
    if (c.ring.empty()) {
        fail("expert pool: cold experts were picked but the device tier has no slot to fetch them into");
        return false;
    }

    // ---- 5. lease every pick of every tensor before anything is fetched, so that resolving one cannot evict another
    std::vector<Want> want;
    for (const uint8_t* t : tensors) {
        auto it = weights.find(t);
        if (it == weights.end() || it->second.counter_base < 0 || it->second.n_expert != n_expert || !it->second.q_tab) continue;
        Resident* r = &it->second;
        for (uint32_t e : uniq) {
            c.lease_add(r, e);
            if (r->h_tier[e] == 2) want.push_back({r, t, e});
            else if (r->h_tier[e] == 0 && r->slot_at[e] >= 0) {
                uint8_t& h = c.heat[(size_t)r->slot_at[e]];
                h = (uint8_t)std::min<int>(h + 1, HEAT_MAX);
            }
        }
    }
    if (want.empty() && c.hint_ids.empty()) return true;
    // slots change hands on the stream: everything recorded so far must be ahead of that
    need_eager("cold experts are fetched");

    // ---- 6. staging
    const uint64_t raw_one = expert_slot_bytes;
    if (!c.pin[0] || c.raw_one != raw_one) {
        if (c.pin[0]) {
            fail("expert pool: the slot size changed under the cold tier");
            return false;
        }
        for (int i = 0; i < 2; i++)
            if (!check(hipHostMalloc((void**)&c.pin[i], FETCH_CHUNK * raw_one, hipHostMallocDefault), "hipHostMalloc(fetch staging)") ||
                !check(hipMalloc((void**)&c.raw[i], FETCH_CHUNK * raw_one), "hipMalloc(fetch staging)") ||
                !check(hipEventCreateWithFlags(&c.evt[i], hipEventDisableTiming), "hipEventCreate"))
                return false;
        if (!check(hipEventCreateWithFlags(&c.patch_evt, hipEventDisableTiming), "hipEventCreate") ||
            !check(hipEventCreateWithFlags(&c.pre_evt, hipEventDisableTiming), "hipEventCreate"))
            return false;
        c.raw_one = raw_one;
    }
    if (!c.pool) c.pool = new ReadPool(fetch_threads());
    c.pool->source(model_path, map_base);
    const size_t need_patches = 2 * want.size() + 8;
    if (c.patch_cap < need_patches) {
        if (c.patch_evt_used) check(hipEventSynchronize(c.patch_evt), "wait for the last table patches");
        c.patch_evt_used = false;
        if (c.patches) (void)hipHostFree(c.patches);
        c.patch_cap = std::max<size_t>(need_patches, 256);
        if (!check(hipHostMalloc((void**)&c.patches, c.patch_cap * sizeof(ExpertPatch), hipHostMallocMapped), "hipHostMalloc(table patches)")) {
            c.patches = nullptr;
            c.patch_cap = 0;
            return false;
        }
    }
    if (c.patch_evt_used) {
        check(hipEventSynchronize(c.patch_evt), "wait for the last table patches");
        c.patch_evt_used = false;
    }
    c.n_patch = 0;

    // one expert's bytes (in staging on the device at `src`) into a slot taken from an unleased expert
    auto place = [&](const Want& w, const uint8_t* dev_raw) -> bool {
        const int64_t at = clock_walk(c.heat.data(), c.leased.data(), c.ring.size(), &c.hand);
        if (at < 0) {
            fail("expert pool: every one of the " + std::to_string(c.ring.size()) +
                 " device slots holds an expert the layer being resolved picked; the device tier is smaller than one layer's picks");
            return false;
        }
        ColdTier::Slot& sl = c.ring[(size_t)at];
        uint64_t t0 = clock_us();
        if (sl.owner) {   // the victim goes cold: its entry is pointed at the sentinel (experts.rs:1527-1540)
            Resident* v = sl.owner;
            v->h_q[sl.e] = c.sentinel_q;
            v->h_s[sl.e] = c.sentinel_s;
            v->h_tier[sl.e] = 2;
            v->slot_at[sl.e] = -1;
            c.patches[c.n_patch++] = {v->q_tab + sl.e, v->s_tab + sl.e, v->tier + sl.e, c.sentinel_q, c.sentinel_s, 2u, 0u};
            expert_cold_evictions++;
        }
        const int64_t rows = (int64_t)(w.r->rows / w.r->n_expert);
        if (w.r->fmt == (int)IT_Q8_0) repack_q8_0(dev_raw, (int8_t*)sl.q, (uint16_t*)sl.s, rows, (int)w.r->n_in, stream);
        else repack_nvfp4(dev_raw, sl.q, sl.s, rows, (int)w.r->n_in, stream);
        sl.owner = w.r;
        sl.e = w.e;
        c.heat[(size_t)at] = HEAT_NEW;   // an arrival survives one pass of the hand and no more unless picked again
        c.leased[(size_t)at] = 1;
        w.r->h_q[w.e] = sl.q;
        w.r->h_s[w.e] = sl.s;
        w.r->h_tier[w.e] = 0;
        w.r->slot_at[w.e] = (int32_t)at;
        c.patches[c.n_patch++] = {w.r->q_tab + w.e, w.r->s_tab + w.e, w.r->tier + w.e, sl.q, sl.s, 0u, 0u};
        fetch_writes_us += clock_us() - t0;
        expert_fetched++;
        expert_fetch_bytes += raw_one;
        return true;
    };

    // ---- 7. what the lookahead already read is published from its staging; the rest is read now, a chunk at a time
    bool ok = true;
    std::vector<Want> rest;
    bool published = false;
    for (const Want& w : want) {
        auto pe = c.pre_entries.find((uint64_t)w.r->counter_base + w.e);
        if (pe == c.pre_entries.end()) {
            rest.push_back(w);
            continue;
        }
        const int slot = pe->second;
        c.pre_entries.erase(pe);
        uint64_t t0 = clock_us();
        const bool got = c.pool->wait(&c.pre_state[slot]);
        fetch_read_us += clock_us() - t0;
        if (!got) {
            c.pre_free.push_back(slot);
            rest.push_back(w);
            continue;
        }
        // through the device staging like any other fetch, one expert at a time
        const int b = c.cur;
        uint64_t t1 = clock_us();
        ok = ok && check(hipMemcpyAsync(c.raw[b], c.pre_pin + (size_t)slot * raw_one, raw_one, hipMemcpyHostToDevice, stream), "upload a prefetched expert");
        fetch_upload_us += clock_us() - t1;
        ok = ok && place(w, c.raw[b]);
        c.pre_free.push_back(slot);
        prefetch_used++;
        published = true;
        if (!ok) break;
    }
    if (published && hipEventRecord(c.pre_evt, stream) == hipSuccess) c.pre_evt_used = true;
    for (size_t c0 = 0; c0 < rest.size() && ok; c0 += FETCH_CHUNK) {
        const size_t m = std::min(FETCH_CHUNK, rest.size() - c0);
        const int b = c.cur;
        c.cur ^= 1;
        if (c.evt_used[b]) {   // the copy out of this half of the pinned staging must have run
            ok = check(hipEventSynchronize(c.evt[b]), "wait for the fetch staging");
            c.evt_used[b] = false;
        }
        uint64_t t0 = clock_us();
        for (size_t k = 0; k < m; k++) {
            const Want& w = rest[c0 + k];
            c.pool->submit({c.pin[b] + k * raw_one, w.key + (uint64_t)w.e * raw_one, (size_t)raw_one, &c.read_state[k]});
        }
        for (size_t k = 0; k < m; k++)
            if (!c.pool->wait(&c.read_state[k]) && ok) {
                fail("expert pool: reading a cold expert from the model file failed");
                ok = false;
            }
        fetch_read_us += clock_us() - t0;
        if (!ok) break;
        uint64_t t1 = clock_us();
        ok = check(hipMemcpyAsync(c.raw[b], c.pin[b], m * raw_one, hipMemcpyHostToDevice, stream), "upload cold experts");
        if (ok && hipEventRecord(c.evt[b], stream) == hipSuccess) c.evt_used[b] = true;
        fetch_upload_us += clock_us() - t1;
        h2d++;
        h2d_bytes += m * raw_one;
        for (size_t k = 0; k < m && ok; k++) ok = place(rest[c0 + k], c.raw[b] + k * raw_one);
    }
    // ---- 8. the tables, in one launch (also after a failure, so that they never disagree with the host's copy)
    if (c.n_patch) {
        ExpertPatch* dev_patches = nullptr;
        if (check(hipHostGetDevicePointer((void**)&dev_patches, c.patches, 0), "hipHostGetDevicePointer(table patches)")) {
            expert_patch(dev_patches, (int)c.n_patch, stream);
            check(hipGetLastError(), "patch expert tables");
            if (hipEventRecord(c.patch_evt, stream) == hipSuccess) c.patch_evt_used = true;
        }
    }
    if (!ok) return false;

    // ---- 9. start reading the next layer's likely experts while the device computes this one
    if (opens_layer && !c.hint_ids.empty() && expert_prefetch) {
        // slots freed by this resolve's publishes are read into again below: their queued uploads must have run
        if (c.pre_evt_used) {
            check(hipEventSynchronize(c.pre_evt), "wait for the lookahead staging");
            c.pre_evt_used = false;
        }
        // guesses left from the last decision are dropped
        for (auto& kv : c.pre_entries) {
            (void)c.pool->wait(&c.pre_state[kv.second]);
            c.pre_free.push_back(kv.second);
            prefetch_wasted++;
        }
        c.pre_entries.clear();
        auto nx = c.next_opener.find(c.cur_opener);
        if (nx != c.next_opener.end()) {
            if (!c.pre_pin) {
                if (!check(hipHostMalloc((void**)&c.pre_pin, PREFETCH_SLOTS * raw_one, hipHostMallocDefault), "hipHostMalloc(lookahead staging)")) return false;
                for (int i = (int)PREFETCH_SLOTS - 1; i >= 0; i--) c.pre_free.push_back(i);
            }
            std::vector<const uint8_t*> next{nx->second};
            auto g = c.group.find(nx->second);
            if (g != c.group.end()) next.insert(next.end(), g->second.begin(), g->second.end());
            for (const uint8_t* t : next) {
                auto it = weights.find(t);
                if (it == weights.end() || it->second.counter_base < 0 || !it->second.q_tab) continue;
                Resident* r = &it->second;
                for (uint32_t e : c.hint_ids) {
                    if (e >= r->n_expert || r->h_tier[e] != 2 || c.pre_free.empty()) continue;
                    const uint64_t id = (uint64_t)r->counter_base + e;
                    if (c.pre_entries.count(id)) continue;
                    const int slot = c.pre_free.back();
                    c.pre_free.pop_back();
                    c.pool->submit({c.pre_pin + (size_t)slot * raw_one, t + (uint64_t)e * raw_one, (size_t)raw_one, &c.pre_state[slot]});
                    c.pre_entries[id] = slot;
                    prefetch_reads++;
                }
            }
        }
    }
    return true;
}

void it_hip_fetch_read_counts(it_hip* be, uint64_t out[2]) {
    out[0] = out[1] = 0;
    if (be && be->cold && be->cold->pool) be->cold->pool->counts(&out[0], &out[1]);
}
