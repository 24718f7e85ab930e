// C-ABI of the decode path, device half: kernel context (device tables, partial buffers,
// launches).  The host-only half (table builder, prefix-tree manager) is in c_api_host.cpp.
// Declarations and their reference counterparts are in include/chunk_attn_hip.h.
#include "chunk_attn_hip.h"

#include <dlfcn.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <exception>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>
#include <vector>

#include "c_api_common.h"
#include "kernels.h"
#include "tables.h"

namespace {

using ca::abi::fail;
using ca::abi::guarded;

int fail_hip(hipError_t e, const char* what) {
    return fail(CA_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

#define CA_HIP(call)                                        \
    do {                                                    \
        hipError_t e_ = (call);                             \
        if (e_ != hipSuccess) return fail_hip(e_, #call);   \
    } while (0)

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Named ranges in a profiler's marker trace (the reference brackets the same places with NVTX
// ranges, kernel_cuda.cu:1334-1433).  The marker library is looked up at run time, only when
// ca_set_markers asks for it: the shared library does not depend on it.
// Process-wide: `on` is read by every entry point of every thread, the function pointers are
// written once (under the mutex) before `on` is first set.
struct Markers {
    std::mutex load;  // serialises the lookup of the marker library
    int (*push)(const char*) = nullptr;
    int (*pop)() = nullptr;
    std::atomic<bool> on{ false };
};
Markers g_markers;

struct Range {
    bool open;
    explicit Range(const char* name) : open(g_markers.on.load(std::memory_order_acquire)) {
        if (open) g_markers.push(name);
    }
    ~Range() {
        if (open) g_markers.pop();
    }
    Range(const Range&) = delete;
    Range& operator=(const Range&) = delete;
};

}  // namespace

int ca_set_markers(int enable) {
    if (!enable) {
        g_markers.on.store(false, std::memory_order_release);
        return CA_OK;
    }
    std::lock_guard<std::mutex> lock(g_markers.load);
    if (!g_markers.push) {
        void* lib = nullptr;
        for (const char* name : { "librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4", "libroctx64.so" }) {
            lib = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
            if (lib) break;
        }
        if (!lib) return fail(CA_ERR_STATE, "no marker library (roctx) could be loaded");
        auto push = reinterpret_cast<int (*)(const char*)>(dlsym(lib, "roctxRangePushA"));
        auto pop = reinterpret_cast<int (*)()>(dlsym(lib, "roctxRangePop"));
        if (!push || !pop) return fail(CA_ERR_STATE, "the marker library lacks roctxRangePushA / roctxRangePop");
        g_markers.push = push;
        g_markers.pop = pop;
    }
    g_markers.on.store(true, std::memory_order_release);
    return CA_OK;
}

// ---- kernel context ------------------------------------------------------------------------

struct ca_ctx {
    int H = 0, d = 0, C = 0;
    void* k_pool = nullptr;
    void* v_pool = nullptr;
    int max_chunks = 0;
    int tpp_threshold = 1;
    int device = 0;
    int n_cus = 256;
    int seg_chunks = 0, stream_chunks = 0;

    bool valid = false;
    int delta_tokens = 0;
    int partition = 0;  // partition the current plan was built for

    // rows of the last refresh (to rebuild for another partition, and for the reference-form
    // tables).  Tail roll-overs patched into the plan since then are only logged: rows() replays
    // the log when somebody asks for the rows.
    mutable std::vector<ca::ChunkRow> rows;
    struct Roll {
        int delta_tokens;
        std::vector<int32_t> seqs, slots;
    };
    mutable std::vector<Roll> pending_rolls;
    int n_seqs = 0;
    mutable ca::RefTables ref;  // reference-form tables of `rows`: use ref_tables(), never directly
    mutable bool ref_valid = false;
    ca::Plan plan;

    // device tables: one blob, uploaded from a ring of pinned staging buffers (the host may run
    // kStaging refreshes ahead of the device before it has to wait for a buffer)
    static constexpr int kStaging = 4;
    char* dev_blob = nullptr;
    size_t dev_blob_cap = 0;
    char* host_blob[kStaging] = {};
    size_t host_blob_cap[kStaging] = {};
    hipEvent_t host_blob_free[kStaging] = {};
    int next_host = 0;
    // offsets into dev_blob
    size_t off_shared = 0, off_stream = 0, off_slots = 0, off_seq_len = 0, off_part_ptr = 0,
           off_tail_slot = 0, off_tail_fill = 0;
    int schedule = 0;  // 0: partial-producing launch + merge launch; 1: one launch, last finisher merges
    int plan_schedule = 0;  // schedule the current plan was built for
    int stream_hint = 0;    // non-temporal loads of private chunks: 0 by working-set size, 1 always, 2 never
    int replan_percent = 25;  // patched tables are rebuilt once the attended tokens drifted this far; 0: never
    int64_t full_builds = 0, patches = 0;  // how the tables came about so far (ca_ctx_table_stats)

    float* part = nullptr;
    size_t part_cap = 0;  // bytes
    int32_t* counters = nullptr;  // [n_seqs * H] partials finished per (sequence, head)
    size_t counters_cap = 0;      // bytes
    // Device buffers that were outgrown.  Launches already queued may still read them, and
    // hipFree waits for the whole device, so they are kept until the context is destroyed
    // (capacities double: together they never hold more than the live buffer does).
    std::vector<void*> retired;
    std::vector<void*> retired_host;  // pinned staging buffers that were outgrown

    // optional timing: events recorded on the caller's stream around the launches.
    // 1: the forward as it runs; 2: forward run as three timed launches (chunk-first, sequence-first, merge)
    int timing = 0;
    hipEvent_t ev[4] = { nullptr, nullptr, nullptr, nullptr };
    bool ev_pending = false;
    double phase_ms[3] = { 0, 0, 0 };
    int64_t phase_calls = 0;
};

namespace {

// Makes *p hold at least `need` bytes.  A new buffer is twice what is asked for (tables and
// partial rows grow step by step while sequences grow, and an allocation in the middle of a
// decode loop costs the host hundreds of microseconds); the old one is retired instead of freed:
// nothing on the decode step's path waits for the device.
int ensure_dev(ca_ctx* c, char** p, size_t* cap, size_t need) {
    if (need <= *cap) return CA_OK;
    const size_t want = align_up(std::max(2 * need, 2 * *cap), 4096);
    void* fresh = nullptr;
    CA_HIP(hipMalloc(&fresh, want));
    if (*p) c->retired.push_back(*p);
    *p = static_cast<char*>(fresh);
    *cap = want;
    return CA_OK;
}

ca::LaunchArgs launch_args(const ca_ctx* c, const void* q, void* out) {
    ca::LaunchArgs a;
    a.q = q;
    a.out = out;
    a.kpool = c->k_pool;
    a.vpool = c->v_pool;
    a.part = c->part;
    a.shared_items = reinterpret_cast<const ca::WorkItem*>(c->dev_blob + c->off_shared);
    a.stream_items = reinterpret_cast<const ca::WorkItem*>(c->dev_blob + c->off_stream);
    a.slots = reinterpret_cast<const int32_t*>(c->dev_blob + c->off_slots);
    a.part_ptr = reinterpret_cast<const int32_t*>(c->dev_blob + c->off_part_ptr);
    a.counters = c->counters;
    a.delta_tokens = c->delta_tokens;
    a.H = c->H;
    a.C = c->C;
    a.d = c->d;
    a.scale_log2 = 1.4426950408889634f / std::sqrt(static_cast<float>(c->d));
    a.stream_per_wave = c->plan.stream_per_wave;
    a.shared_narrow = c->plan.shared_narrow;
    // 256 MiB of Infinity Cache on this part.  A forward that attends more than that cannot find
    // its K/V there again on the next step, and plain loads top out near 6.3 TB/s against
    // 7.2 TB/s for loads with the non-temporal hint (measured with a bare read kernel): stream
    // the private chunks around the cache then.  Smaller working sets keep plain loads.
    // The caller may know better (ca_ctx_set_stream_hint): the layers of a model each have a cache
    // of their own and together never fit.
    a.stream_nt = c->stream_hint == 1 ||
                  (c->stream_hint == 0 &&
                   (int64_t(c->plan.stream_tokens) + c->plan.shared_tokens) * 4 * c->H * c->d > (int64_t(256) << 20));
    return a;
}

int launch_rc(int rc, const char* what) {
    if (rc == 0) return CA_OK;
    if (rc < 0) return fail(CA_ERR_INVALID, std::string(what) + ": unsupported shape");
    return fail_hip(static_cast<hipError_t>(rc), what);
}

// Brings c->rows up to date with the roll-overs patched into the plan since the last refresh:
// every sequence's last chunk gains the appended tokens, rolled sequences get their new empty
// chunk as a row right after the old last one (where a pre-order walk of the tree puts it).
const std::vector<ca::ChunkRow>& current_rows(const ca_ctx* c) {
    for (const ca_ctx::Roll& roll : c->pending_rolls) {
        std::vector<int> tail_row(c->n_seqs, -1);
        for (size_t i = 0; i < c->rows.size(); i++) {
            if (c->rows[i].seq_end - c->rows[i].seq_begin == 1) tail_row[c->rows[i].seq_begin] = static_cast<int>(i);
        }
        std::vector<int32_t> new_slot(c->n_seqs, -1);
        for (size_t k = 0; k < roll.seqs.size(); k++) new_slot[roll.seqs[k]] = roll.slots[k];
        std::vector<ca::ChunkRow> next;
        next.reserve(c->rows.size() + roll.seqs.size());
        for (size_t i = 0; i < c->rows.size(); i++) {
            ca::ChunkRow r = c->rows[i];
            const bool is_tail = r.seq_end - r.seq_begin == 1 && tail_row[r.seq_begin] == static_cast<int>(i);
            if (is_tail) r.n_tokens += roll.delta_tokens;
            next.push_back(r);
            if (is_tail && new_slot[r.seq_begin] >= 0) next.push_back({ new_slot[r.seq_begin], 0, r.seq_begin, r.seq_end });
        }
        c->rows.swap(next);
    }
    c->pending_rolls.clear();
    return c->rows;
}

ca::PlanParams plan_params(const ca_ctx* c, int partition) {
    ca::PlanParams pp;
    pp.tpp_threshold = c->tpp_threshold;
    pp.partition = partition;
    pp.shared_seg_chunks = c->seg_chunks;
    pp.stream_chunks = c->stream_chunks;
    pp.n_heads = c->H;
    pp.n_cus = c->n_cus;
    pp.allow_per_wave = c->schedule == 0;  // the single-launch schedule synchronises workgroups
    return pp;
}

// Copies c->plan into a pinned staging buffer and queues its upload on `st`; sizes the
// partial-row buffer for it.
int upload_plan(ca_ctx* c, hipStream_t st) {
    ca::Plan& p = c->plan;
    size_t off = 0;
    auto place = [&](size_t bytes) {
        const size_t at = off;
        off = align_up(off + bytes, 64);
        return at;
    };
    c->off_shared = place(p.shared_items.size() * sizeof(ca::WorkItem));
    c->off_stream = place(p.stream_items.size() * sizeof(ca::WorkItem));
    c->off_slots = place(p.slots.size() * 4);
    c->off_seq_len = place(p.seq_len.size() * 4);
    c->off_part_ptr = place(p.part_ptr.size() * 4);
    c->off_tail_slot = place(p.tail_slot.size() * 4);
    c->off_tail_fill = place(p.tail_fill.size() * 4);
    const size_t total = std::max<size_t>(off, 64);  // a multiple of 64

    if (int rc = ensure_dev(c, &c->dev_blob, &c->dev_blob_cap, total)) return rc;
    const int hb = c->next_host;
    c->next_host = (c->next_host + 1) % ca_ctx::kStaging;
    if (total > c->host_blob_cap[hb]) {
        // the whole ring grows at once, with headroom: pinned allocations cost the host a hundred
        // microseconds each and must not recur on the following decode steps
        const size_t want = align_up(std::max(2 * total, 2 * c->host_blob_cap[hb]), 4096);
        for (int b = 0; b < ca_ctx::kStaging; b++) {
            if (c->host_blob_cap[b] >= want) continue;
            void* fresh = nullptr;
            CA_HIP(hipHostMalloc(&fresh, want, hipHostMallocDefault));
            // the old buffer may still be the source of a queued upload: freed with the context
            if (c->host_blob[b]) c->retired_host.push_back(c->host_blob[b]);
            c->host_blob[b] = static_cast<char*>(fresh);
            c->host_blob_cap[b] = want;
        }
    }
    // the staging buffer may still be the source of an earlier asynchronous upload
    CA_HIP(hipEventSynchronize(c->host_blob_free[hb]));
    char* hbuf = c->host_blob[hb];
    auto put = [&](size_t at, const void* src, size_t bytes) {
        if (bytes) std::memcpy(hbuf + at, src, bytes);
    };
    put(c->off_shared, p.shared_items.data(), p.shared_items.size() * sizeof(ca::WorkItem));
    put(c->off_stream, p.stream_items.data(), p.stream_items.size() * sizeof(ca::WorkItem));
    put(c->off_slots, p.slots.data(), p.slots.size() * 4);
    put(c->off_seq_len, p.seq_len.data(), p.seq_len.size() * 4);
    put(c->off_part_ptr, p.part_ptr.data(), p.part_ptr.size() * 4);
    put(c->off_tail_slot, p.tail_slot.data(), p.tail_slot.size() * 4);
    put(c->off_tail_fill, p.tail_fill.data(), p.tail_fill.size() * 4);
    // a copy kernel, not hipMemcpyAsync: the copy engine's hand-over stalls the stream for
    // several microseconds in the middle of a decode step
    if (int rc = launch_rc(ca::launch_upload(c->dev_blob, hbuf, total, st), "table upload")) return rc;
    CA_HIP(hipEventRecord(c->host_blob_free[hb], st));

    const size_t part_bytes = std::max<size_t>(size_t(p.n_part_rows) * c->H * ca::PART_STRIDE * 4, 256);
    return ensure_dev(c, reinterpret_cast<char**>(&c->part), &c->part_cap, part_bytes);
}

// Builds the plan for `partition` from the context's rows and uploads it.
int build_and_upload(ca_ctx* c, int partition, hipStream_t st) {
    const std::vector<ca::ChunkRow>& rows = current_rows(c);
    const ca::PlanParams pp = plan_params(c, partition);
    ca::build_plan(rows.data(), static_cast<int>(rows.size()), c->n_seqs, c->C, pp, &c->plan);
    if (int rc = upload_plan(c, st)) return rc;
    // completion counters (single-launch schedule only; a change of schedule rebuilds the plan and
    // comes through here): they start at zero, and each forward leaves them at zero again
    if (c->schedule != 0) {
        const int n_counters = std::max(c->n_seqs * c->H, 1);
        if (int rc = ensure_dev(c, reinterpret_cast<char**>(&c->counters), &c->counters_cap, size_t(n_counters) * 4)) return rc;
        if (int rc = launch_rc(ca::launch_fill(c->counters, n_counters, 0, st), "counter reset")) return rc;
    }
    c->partition = partition;
    c->plan_schedule = c->schedule;
    c->full_builds++;
    return CA_OK;
}

// Reference-form tables of the rows the context holds, built on first use after a refresh.
const ca::RefTables& ref_tables(const ca_ctx* c) {
    if (!c->ref_valid) {
        const std::vector<ca::ChunkRow>& rows = current_rows(c);
        ca::build_ref_tables(rows.data(), static_cast<int>(rows.size()), c->n_seqs, c->C, c->tpp_threshold, &c->ref);
        c->ref_valid = true;
    }
    return c->ref;
}

int check_ready(ca_ctx* c, const void* q, int n_seqs) {
    if (!c) return fail(CA_ERR_INVALID, "null context");
    if (!c->valid) return fail(CA_ERR_STATE, "kernel context is not valid: call ca_refresh_kernel_context first");
    if (n_seqs != c->n_seqs) {
        return fail(CA_ERR_STATE, "n_seqs (" + std::to_string(n_seqs) + ") does not match the tables (" +
                                    std::to_string(c->n_seqs) + ")");
    }
    if (n_seqs > 0 && !q) return fail(CA_ERR_INVALID, "null device pointer");
    return CA_OK;
}

// The attention kernels exist for the shapes the reference's GPU kernels take
// (kernel_cuda.cu:1199, 1256-1265 there); like there, other shapes fail when attention is asked for.
int check_attention_shape(const ca_ctx* c) {
    if (c->d != 128) return fail(CA_ERR_INVALID, "unsupported head dim " + std::to_string(c->d));
    if (c->C != 32 && c->C != 64 && c->C != 128) {
        return fail(CA_ERR_INVALID, "unsupported chunk_size " + std::to_string(c->C));
    }
    return CA_OK;
}

// Adds the elapsed times of the last timed ca_attention call to the accumulators.
int collect_timing(ca_ctx* c) {
    if (!c->ev_pending) return CA_OK;
    CA_HIP(hipEventSynchronize(c->ev[3]));
    for (int i = 0; i < 3; i++) {
        float ms = 0.f;
        CA_HIP(hipEventElapsedTime(&ms, c->ev[i], c->ev[i + 1]));
        c->phase_ms[i] += ms;
    }
    c->phase_calls++;
    c->ev_pending = false;
    return CA_OK;
}

int run_shared(ca_ctx* c, const void* q, hipStream_t st) {
    const ca::LaunchArgs a = launch_args(c, q, nullptr);
    return launch_rc(ca::launch_decode(a, static_cast<int>(c->plan.shared_items.size()), 0, false, st),
                     "chunk-first launch");
}

int run_stream(ca_ctx* c, const void* q, void* out, hipStream_t st) {
    const ca::LaunchArgs a = launch_args(c, q, out);
    return launch_rc(ca::launch_decode(a, 0, static_cast<int>(c->plan.stream_items.size()), false, st),
                     "sequence-first launch");
}

int run_merge(ca_ctx* c, void* out, hipStream_t st) {
    if (c->plan.n_part_rows == 0) return CA_OK;
    const ca::LaunchArgs a = launch_args(c, nullptr, out);
    return launch_rc(ca::launch_merge(a, c->n_seqs, true, st), "merge launch");
}

int run_fused(ca_ctx* c, const void* q, void* out, hipStream_t st) {
    const ca::LaunchArgs a = launch_args(c, q, out);
    if (c->schedule == 0) {
        // both phases in one launch (shared and stream workgroups overlap), then the merge
        if (int rc = launch_rc(ca::launch_decode(a, static_cast<int>(c->plan.shared_items.size()),
                                                 static_cast<int>(c->plan.stream_items.size()), false, st), "decode launch")) return rc;
        return run_merge(c, out, st);
    }
    return launch_rc(ca::launch_decode(a, static_cast<int>(c->plan.shared_items.size()),
                                       static_cast<int>(c->plan.stream_items.size()), true, st),
                     "decode launch");
}

}  // namespace

extern "C" {

int ca_ctx_create(ca_ctx** out, int n_heads, int d_head, int chunk_size, void* k_pool,
                  void* v_pool, int max_chunks, int tpp_threshold) {
    if (!out) return fail(CA_ERR_INVALID, "null output pointer");
    *out = nullptr;
    if (n_heads <= 0 || d_head <= 0 || chunk_size <= 0 || max_chunks < 0 || tpp_threshold < 0) {
        return fail(CA_ERR_INVALID, "bad shape argument");
    }
    if (max_chunks > 0 && (!k_pool || !v_pool)) return fail(CA_ERR_INVALID, "null KV pool");
    int n_dev = 0;
    hipError_t e = hipGetDeviceCount(&n_dev);
    if (e != hipSuccess || n_dev <= 0) {
        return fail(CA_ERR_HIP, "no HIP device available: the decode path has no CPU fallback");
    }
    return guarded([&]() -> int {
        ca_ctx* c = new ca_ctx();
        c->H = n_heads;
        c->d = d_head;
        c->C = chunk_size;
        c->k_pool = k_pool;
        c->v_pool = v_pool;
        c->max_chunks = max_chunks;
        c->tpp_threshold = tpp_threshold;
        hipError_t err = hipGetDevice(&c->device);
        hipDeviceProp_t prop;
        if (err == hipSuccess) err = hipGetDeviceProperties(&prop, c->device);
        if (err == hipSuccess) c->n_cus = prop.multiProcessorCount;
        for (int i = 0; i < ca_ctx::kStaging && err == hipSuccess; i++) {
            err = hipEventCreateWithFlags(&c->host_blob_free[i], hipEventDisableTiming);
        }
        // address of this device's static scratch (for ca_attention_noalloc), once per device
        if (err == hipSuccess) err = static_cast<hipError_t>(ca::scratch_setup(c->device));
        if (err != hipSuccess) {
            ca_ctx_destroy(c);
            return fail_hip(err, "context setup");
        }
        *out = c;
        return CA_OK;
    });
}

void ca_ctx_destroy(ca_ctx* c) {
    if (!c) return;
    if (c->dev_blob) (void)hipFree(c->dev_blob);
    if (c->part) (void)hipFree(c->part);
    if (c->counters) (void)hipFree(c->counters);
    for (void* p : c->retired) (void)hipFree(p);
    for (void* p : c->retired_host) (void)hipHostFree(p);
    for (int i = 0; i < ca_ctx::kStaging; i++) {
        if (c->host_blob_free[i]) {
            (void)hipEventSynchronize(c->host_blob_free[i]);
            (void)hipEventDestroy(c->host_blob_free[i]);
        }
        if (c->host_blob[i]) (void)hipHostFree(c->host_blob[i]);
    }
    for (int i = 0; i < 4; i++) {
        if (c->ev[i]) (void)hipEventDestroy(c->ev[i]);
    }
    delete c;
}

int ca_refresh_kernel_context(ca_ctx* c, const ca_chunk_row* rows, int n_rows, int n_seqs,
                              void* stream) {
    if (!c || n_rows < 0 || n_seqs < 0 || (n_rows > 0 && !rows)) return fail(CA_ERR_INVALID, "bad argument");
    Range range("ca_refresh_kernel_context");
    return guarded([&]() -> int {
        static_assert(sizeof(ca_chunk_row) == sizeof(ca::ChunkRow), "row layouts must agree");
        for (int i = 0; i < n_rows; i++) {
            if (rows[i].slot < 0 || rows[i].slot >= c->max_chunks || rows[i].n_tokens < 0 ||
                rows[i].n_tokens > c->C) {
                return fail(CA_ERR_INVALID, "chunk row " + std::to_string(i) + " is outside the pool or over-full");
            }
        }
        c->valid = false;
        c->pending_rolls.clear();
        c->rows.resize(n_rows);
        if (n_rows) std::memcpy(c->rows.data(), rows, sizeof(ca_chunk_row) * n_rows);
        c->n_seqs = n_seqs;
        c->ref_valid = false;  // reference-form tables are for inspection: built when asked for
        if (int rc = build_and_upload(c, 0, static_cast<hipStream_t>(stream))) return rc;
        c->delta_tokens = 0;
        c->valid = true;
        return CA_OK;
    });
}

int ca_ctx_roll_tails(ca_ctx* c, const int32_t* seq_idx, const int32_t* new_slots, int n, void* stream) {
    if (!c || n < 0 || (n > 0 && (!seq_idx || !new_slots))) return fail(CA_ERR_INVALID, "bad argument");
    if (!c->valid) return fail(CA_ERR_STATE, "kernel context is not valid: call ca_refresh_kernel_context first");
    if (c->schedule != c->plan_schedule) return fail(CA_ERR_STATE, "the tables were built for another schedule");
    for (int i = 0; i < n; i++) {
        if (new_slots[i] < 0 || new_slots[i] >= c->max_chunks) return fail(CA_ERR_INVALID, "slot outside the pool");
    }
    Range range("ca_ctx_roll_tails");
    return guarded([&]() -> int {
        try {
            ca::roll_tails(&c->plan, c->C, plan_params(c, c->partition), c->delta_tokens, seq_idx, new_slots, n);
        } catch (const std::invalid_argument& e) {
            return fail(CA_ERR_STATE, e.what());  // plan untouched: the caller refreshes in full instead
        }
        ca_ctx::Roll roll;
        roll.delta_tokens = c->delta_tokens;
        roll.seqs.assign(seq_idx, seq_idx + n);
        roll.slots.assign(new_slots, new_slots + n);
        c->pending_rolls.push_back(std::move(roll));
        // the log is replayed into the rows only when somebody asks for them: keep it short
        if (c->pending_rolls.size() > 16) (void)current_rows(c);
        c->ref_valid = false;
        c->valid = false;
        if (ca::plan_is_stale(c->plan, c->replan_percent)) {
            // the work-item sizes were derived for a step of another size (ca_ctx_set_replan):
            // derive them again from the rows as they are now
            if (int rc = build_and_upload(c, c->partition, static_cast<hipStream_t>(stream))) return rc;
        } else {
            if (int rc = upload_plan(c, static_cast<hipStream_t>(stream))) return rc;
            c->patches++;
        }
        c->delta_tokens = 0;
        c->valid = true;
        return CA_OK;
    });
}

int ca_ctx_valid(const ca_ctx* c) { return c && c->valid; }
void ca_ctx_invalidate(ca_ctx* c) {
    if (c) c->valid = false;
}
int ca_ctx_delta_tokens(const ca_ctx* c) { return c ? c->delta_tokens : 0; }
int ca_ctx_set_delta_tokens(ca_ctx* c, int delta_tokens) {
    if (!c) return fail(CA_ERR_INVALID, "null context");
    // a negative value would put the next appended row in front of its chunk
    if (delta_tokens < 0) return fail(CA_ERR_INVALID, "delta_tokens must not be negative");
    c->delta_tokens = delta_tokens;
    return CA_OK;
}

int ca_attention(ca_ctx* c, const void* q, void* out, int n_seqs, int partition, void* stream) {
    if (partition < 0 || partition > 2) return fail(CA_ERR_INVALID, "Unsupported partition type");
    if (int rc = check_ready(c, q, n_seqs)) return rc;
    if (int rc = check_attention_shape(c)) return rc;
    if (n_seqs > 0 && !out) return fail(CA_ERR_INVALID, "null device pointer");
    if (n_seqs == 0) return CA_OK;
    Range range("ca_attention");
    return guarded([&]() -> int {
        hipStream_t st = static_cast<hipStream_t>(stream);
        if (partition != c->partition || c->schedule != c->plan_schedule) {
            if (int rc = build_and_upload(c, partition, st)) return rc;
        }
        if (!c->timing) return run_fused(c, q, out, st);
        if (int rc = collect_timing(c)) return rc;
        CA_HIP(hipEventRecord(c->ev[0], st));
        if (c->timing == 1 && c->schedule == 0) {
            // the forward as it normally runs: decode launch, then merge launch
            const ca::LaunchArgs a = launch_args(c, q, out);
            if (int rc = launch_rc(ca::launch_decode(a, static_cast<int>(c->plan.shared_items.size()),
                                                     static_cast<int>(c->plan.stream_items.size()), false, st), "decode launch")) return rc;
            CA_HIP(hipEventRecord(c->ev[1], st));
            CA_HIP(hipEventRecord(c->ev[2], st));
            if (int rc = run_merge(c, out, st)) return rc;
        } else if (c->timing == 1) {
            if (int rc = run_fused(c, q, out, st)) return rc;
            CA_HIP(hipEventRecord(c->ev[1], st));
            CA_HIP(hipEventRecord(c->ev[2], st));
        } else {
            if (int rc = run_shared(c, q, st)) return rc;
            CA_HIP(hipEventRecord(c->ev[1], st));
            if (int rc = run_stream(c, q, out, st)) return rc;
            CA_HIP(hipEventRecord(c->ev[2], st));
            if (int rc = run_merge(c, out, st)) return rc;
        }
        CA_HIP(hipEventRecord(c->ev[3], st));
        c->ev_pending = true;
        return CA_OK;
    });
}

int ca_attention_noalloc(ca_ctx* c, const void* q, void* out, int n_seqs, void* stream) {
    if (int rc = check_ready(c, q, n_seqs)) return rc;
    if (int rc = check_attention_shape(c)) return rc;
    if (n_seqs > 0 && !out) return fail(CA_ERR_INVALID, "null device pointer");
    if (n_seqs == 0) return CA_OK;
    // nothing here may build or upload tables: they must already be those of the default forward
    if (c->partition != 0 || c->schedule != 0 || c->plan_schedule != 0) {
        return fail(CA_ERR_STATE, "the tables were built for another partition or schedule: "
                                  "ca_attention_noalloc runs partition 0 in the two-launch schedule only");
    }
    float* scratch = ca::scratch_ptr(c->device);
    if (!scratch) return fail(CA_ERR_STATE, "the static scratch of this device was not set up");
    const size_t need = size_t(c->plan.n_part_rows) * c->H * ca::PART_STRIDE * 4;
    if (need > ca::kScratchBytes) {
        return fail(CA_ERR_INVALID, "this forward needs " + std::to_string(need) + " bytes of partial rows, the static "
                                    "scratch holds " + std::to_string(ca::kScratchBytes) + ": use ca_attention");
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    ca::LaunchArgs a = launch_args(c, q, out);
    a.part = scratch;  // every row that the merge reads is written by the decode launch first
    if (int rc = launch_rc(ca::launch_decode(a, static_cast<int>(c->plan.shared_items.size()),
                                             static_cast<int>(c->plan.stream_items.size()), false, st), "decode launch")) return rc;
    if (c->plan.n_part_rows == 0) return CA_OK;
    return launch_rc(ca::launch_merge(a, c->n_seqs, true, st), "merge launch");
}

static_assert(CA_NOALLOC_SCRATCH_BYTES == ca::kScratchBytes, "the header's scratch size and the kernels' must agree");

namespace {
// The fused decode step: append and attention in the decode launch plus the merge launch.
int decode_step(ca_ctx* c, const void* q, const void* k, const void* v, void* out, int n_seqs, hipStream_t st) {
    if (c->partition != 0 || c->schedule != c->plan_schedule) {
        if (int rc = build_and_upload(c, 0, st)) return rc;
    }
    if (c->schedule == 0 && c->plan.tails_streamed) {
        // no append launch: the workgroup that streams a sequence's last chunk takes the new row
        // from k / v, and the merge launch writes the rows into the pool
        c->delta_tokens += 1;
        ca::LaunchArgs a = launch_args(c, q, out);
        a.k_new = k;
        a.v_new = v;
        a.tail_slot = reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_slot);
        a.tail_fill = reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_fill);
        int rc = launch_rc(ca::launch_decode(a, static_cast<int>(c->plan.shared_items.size()),
                                             static_cast<int>(c->plan.stream_items.size()), false, st), "decode launch");
        // the merge launch also puts the new rows into the pool (after every read of this step)
        if (rc == CA_OK) rc = launch_rc(ca::launch_merge(a, c->n_seqs, c->plan.n_part_rows > 0, st), "merge launch");
        if (rc != CA_OK) c->delta_tokens -= 1;
        return rc;
    }
    // last chunks attended chunk-first, or the single-launch schedule: append, then attend
    const ca::LaunchArgs a = launch_args(c, nullptr, nullptr);
    if (int rc = launch_rc(ca::launch_append(a, k, v, reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_slot),
                                             reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_fill),
                                             n_seqs, st), "append launch")) return rc;
    c->delta_tokens += 1;
    return run_fused(c, q, out, st);
}

int check_decode_step(ca_ctx* c, const void* q, const void* k, const void* v, void* out, int n_seqs) {
    if (int rc = check_ready(c, q, n_seqs)) return rc;
    if (int rc = check_attention_shape(c)) return rc;
    if (n_seqs > 0 && (!out || !k || !v)) return fail(CA_ERR_INVALID, "null device pointer");
    for (int s = 0; s < n_seqs; s++) {
        if (c->plan.tail_fill[s] + c->delta_tokens >= c->C) {
            return fail(CA_ERR_STATE, "sequence " + std::to_string(s) + " has no free row in its last chunk: reserve and refresh first");
        }
    }
    return CA_OK;
}
}  // namespace

int ca_decode_step(ca_ctx* c, const void* q, const void* k, const void* v, void* out, int n_seqs, void* stream) {
    if (int rc = check_decode_step(c, q, k, v, out, n_seqs)) return rc;
    if (n_seqs == 0) return CA_OK;
    Range range("ca_decode_step");
    return guarded([&]() -> int { return decode_step(c, q, k, v, out, n_seqs, static_cast<hipStream_t>(stream)); });
}

int ca_ctx_set_timing(ca_ctx* c, int enable) {
    if (!c) return fail(CA_ERR_INVALID, "null context");
    if (enable < 0 || enable > 2) return fail(CA_ERR_INVALID, "timing mode must be 0, 1 or 2");
    if (enable && !c->ev[0]) {
        for (int i = 0; i < 4; i++) CA_HIP(hipEventCreate(&c->ev[i]));
    }
    if (int rc = collect_timing(c)) return rc;
    c->timing = enable;
    return CA_OK;
}

int ca_ctx_read_timing(ca_ctx* c, double* shared_ms, double* stream_ms, double* merge_ms,
                       int64_t* calls, int reset) {
    if (!c) return fail(CA_ERR_INVALID, "null context");
    if (int rc = collect_timing(c)) return rc;
    if (shared_ms) *shared_ms = c->phase_ms[0];
    if (stream_ms) *stream_ms = c->phase_ms[1];
    if (merge_ms) *merge_ms = c->phase_ms[2];
    if (calls) *calls = c->phase_calls;
    if (reset) {
        c->phase_ms[0] = c->phase_ms[1] = c->phase_ms[2] = 0;
        c->phase_calls = 0;
    }
    return CA_OK;
}

int ca_attn_chunks_first(ca_ctx* c, const void* q, int n_seqs, void* stream) {
    if (int rc = check_ready(c, q, n_seqs)) return rc;
    if (int rc = check_attention_shape(c)) return rc;
    return guarded([&]() -> int { return run_shared(c, q, static_cast<hipStream_t>(stream)); });
}

int ca_attn_seqs_first(ca_ctx* c, const void* q, void* out, int n_seqs, void* stream) {
    if (int rc = check_ready(c, q, n_seqs)) return rc;
    if (int rc = check_attention_shape(c)) return rc;
    if (n_seqs > 0 && !out) return fail(CA_ERR_INVALID, "null device pointer");
    return guarded([&]() -> int {
        if (int rc = run_stream(c, q, out, static_cast<hipStream_t>(stream))) return rc;
        return run_merge(c, out, static_cast<hipStream_t>(stream));
    });
}

int ca_append_kv(ca_ctx* c, const void* k, const void* v, int n_seqs, void* stream) {
    if (int rc = check_ready(c, k, n_seqs)) return rc;
    if (n_seqs > 0 && !v) return fail(CA_ERR_INVALID, "null device pointer");
    if (c->delta_tokens < 0) return fail(CA_ERR_STATE, "delta_tokens is negative");
    for (int s = 0; s < n_seqs; s++) {
        if (c->plan.tail_fill[s] + c->delta_tokens >= c->C) {
            return fail(CA_ERR_STATE, "sequence " + std::to_string(s) + " has no free row in its last chunk: reserve and refresh first");
        }
    }
    Range range("ca_append_kv");
    const ca::LaunchArgs a = launch_args(c, nullptr, nullptr);
    return launch_rc(ca::launch_append(a, k, v, reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_slot),
                                       reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_fill),
                                       n_seqs, static_cast<hipStream_t>(stream)), "append launch");
}

int ca_rotary_embedding(const int64_t* positions, void* query, void* key, const void* cos_sin_cache,
                        int64_t n_tokens, int n_heads, int n_kv_heads, int head_size, int rot_dim,
                        int max_position, int64_t query_stride, int64_t key_stride, int is_neox,
                        void* stream) {
    if (n_tokens < 0 || n_heads < 0 || n_kv_heads < 0 || head_size <= 0 || max_position <= 0) {
        return fail(CA_ERR_INVALID, "bad argument");
    }
    if (rot_dim <= 0 || rot_dim % 2 != 0 || rot_dim > head_size) {
        return fail(CA_ERR_INVALID, "rot_dim must be even and within [2, head_size]");
    }
    if (n_tokens == 0 || n_heads + n_kv_heads == 0) return CA_OK;
    if (!positions || !cos_sin_cache || (n_heads > 0 && !query) || (n_kv_heads > 0 && !key)) {
        return fail(CA_ERR_INVALID, "null device pointer");
    }
    if (query_stride < int64_t(n_heads) * head_size || key_stride < int64_t(n_kv_heads) * head_size) {
        return fail(CA_ERR_INVALID, "token stride smaller than a token's row");
    }
    ca::RotaryArgs r;
    r.positions = positions;
    r.query = query;
    r.key = key;
    r.cos_sin_cache = cos_sin_cache;
    r.n_tokens = n_tokens;
    r.n_heads = n_heads;
    r.n_kv_heads = n_kv_heads;
    r.head_size = head_size;
    r.rot_dim = rot_dim;
    r.max_position = max_position;
    r.query_stride = query_stride;
    r.key_stride = key_stride;
    r.is_neox = is_neox != 0;
    return launch_rc(ca::launch_rotary(r, static_cast<hipStream_t>(stream)), "rotary launch");
}

namespace {
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
}  // namespace

int ca_rms_norm(void* out, const void* input, const void* weight, float epsilon, int64_t n_tokens,
                int hidden_size, void* stream) {
    if (n_tokens < 0 || hidden_size <= 0 || !(epsilon >= 0.f)) return fail(CA_ERR_INVALID, "bad argument");
    if (n_tokens == 0) return CA_OK;
    if (!out || !input || !weight) return fail(CA_ERR_INVALID, "null device pointer");
    const bool vec8 = hidden_size % 8 == 0 && aligned16(out) && aligned16(input) && aligned16(weight);
    return launch_rc(ca::launch_rms_norm(out, const_cast<void*>(input), nullptr, weight, epsilon, n_tokens,
                                         hidden_size, vec8, static_cast<hipStream_t>(stream)), "rms_norm launch");
}

int ca_fused_add_rms_norm(void* input, void* residual, const void* weight, float epsilon, int64_t n_tokens,
                          int hidden_size, void* stream) {
    if (n_tokens < 0 || hidden_size <= 0 || !(epsilon >= 0.f)) return fail(CA_ERR_INVALID, "bad argument");
    if (n_tokens == 0) return CA_OK;
    if (!input || !residual || !weight) return fail(CA_ERR_INVALID, "null device pointer");
    if (input == residual) return fail(CA_ERR_INVALID, "input and residual must be different buffers");
    const bool vec8 = hidden_size % 8 == 0 && aligned16(input) && aligned16(residual) && aligned16(weight);
    return launch_rc(ca::launch_rms_norm(nullptr, input, residual, weight, epsilon, n_tokens, hidden_size, vec8,
                                         static_cast<hipStream_t>(stream)), "fused_add_rms_norm launch");
}

int ca_rope_append_kv(ca_ctx* c, const int64_t* positions, void* q, const void* k, const void* v,
                      const void* cos_sin_cache, int max_position, int rot_dim, int is_neox,
                      int n_seqs, void* stream) {
    if (int rc = check_ready(c, k, n_seqs)) return rc;
    if (n_seqs > 0 && (!v || !q || !cos_sin_cache)) return fail(CA_ERR_INVALID, "null device pointer");
    if (max_position <= 0 || rot_dim <= 0 || rot_dim > c->d || rot_dim % (is_neox ? 16 : 8) != 0) {
        return fail(CA_ERR_INVALID, "rot_dim must be a multiple of 16 (NeoX) or 8 (GPT-J) within d_head, max_position positive");
    }
    if (c->d % 8 != 0 || 64 % (c->d / 8) != 0) {
        return fail(CA_ERR_INVALID, "fused rotary append needs d_head in {8, 16, 32, 64, 128, 256, 512}");
    }
    if (c->delta_tokens < 0) return fail(CA_ERR_STATE, "delta_tokens is negative");
    for (int s = 0; s < n_seqs; s++) {
        if (c->plan.tail_fill[s] + c->delta_tokens >= c->C) {
            return fail(CA_ERR_STATE, "sequence " + std::to_string(s) + " has no free row in its last chunk: reserve and refresh first");
        }
        if (!positions && c->plan.seq_len[s] + c->delta_tokens >= max_position) {
            return fail(CA_ERR_INVALID, "sequence " + std::to_string(s) + " is longer than the cos/sin cache");
        }
    }
    const ca::LaunchArgs a = launch_args(c, nullptr, nullptr);
    ca::RotaryArgs r;
    r.positions = positions;
    r.query = q;
    r.cos_sin_cache = cos_sin_cache;
    r.rot_dim = rot_dim;
    r.max_position = max_position;
    r.is_neox = is_neox != 0;
    return launch_rc(ca::launch_rope_append(a, r, k, v,
                                            reinterpret_cast<const int32_t*>(c->dev_blob + c->off_seq_len),
                                            reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_slot),
                                            reinterpret_cast<const int32_t*>(c->dev_blob + c->off_tail_fill),
                                            n_seqs, static_cast<hipStream_t>(stream)), "rotary append launch");
}

int ca_scatter_kv(ca_ctx* c, const void* k, const void* v, int n_tokens, int tok_begin,
                  const int32_t* slots, int n_slots, void* stream) {
    if (!c || n_tokens < 0 || tok_begin < 0 || n_slots < 0) return fail(CA_ERR_INVALID, "bad argument");
    if (n_slots == 0 || tok_begin >= n_tokens) return CA_OK;
    if (!k || !v || !slots) return fail(CA_ERR_INVALID, "null pointer");
    if (int64_t(n_slots) * c->C < int64_t(n_tokens - tok_begin)) {
        return fail(CA_ERR_INVALID, "not enough chunks for the tokens to copy");
    }
    for (int i = 0; i < n_slots; i++) {
        if (slots[i] < 0 || slots[i] >= c->max_chunks) return fail(CA_ERR_INVALID, "slot outside the pool");
    }
    const ca::LaunchArgs a = launch_args(c, nullptr, nullptr);
    return launch_rc(ca::launch_scatter(a, k, v, n_tokens, tok_begin, slots, n_slots,
                                        static_cast<hipStream_t>(stream)), "scatter launch");
}

namespace {
int check_copy_pairs(const ca_ctx* c, const int32_t* src_dst, int n_pairs) {
    if (!c || n_pairs < 0) return fail(CA_ERR_INVALID, "bad argument");
    if (n_pairs > 0 && !src_dst) return fail(CA_ERR_INVALID, "null pointer");
    for (int i = 0; i < n_pairs; i++) {
        const int src = src_dst[2 * i], dst = src_dst[2 * i + 1];
        if (src < 0 || dst < 0 || src >= c->max_chunks || dst >= c->max_chunks) {
            return fail(CA_ERR_INVALID, "slot outside the pool");
        }
        if (src == dst) return fail(CA_ERR_INVALID, "a chunk cannot be copied onto itself");
        for (int j = 0; j < n_pairs; j++) {
            // one launch: a chunk written by one pair must not be read or written by another
            if (j != i && (src_dst[2 * j] == dst || (j < i && src_dst[2 * j + 1] == dst))) {
                return fail(CA_ERR_INVALID, "copy pairs overlap: a destination is also a source or written twice");
            }
        }
    }
    if ((size_t(c->H) * c->C * c->d * 2) % 16 != 0) return fail(CA_ERR_INVALID, "chunk size in bytes must be a multiple of 16");
    return CA_OK;
}

int check_row_targets(const ca_ctx* c, const void* k, const void* v, int n_rows, const int32_t* slot_row) {
    if (!c || n_rows < 0) return fail(CA_ERR_INVALID, "bad argument");
    if (n_rows == 0) return CA_OK;
    if (!k || !v || !slot_row) return fail(CA_ERR_INVALID, "null pointer");
    for (int i = 0; i < n_rows; i++) {
        if (slot_row[2 * i] < 0 || slot_row[2 * i] >= c->max_chunks || slot_row[2 * i + 1] < 0 ||
            slot_row[2 * i + 1] >= c->C) {
            return fail(CA_ERR_INVALID, "target " + std::to_string(i) + " is outside the pool or the chunk");
        }
    }
    return CA_OK;
}
}  // namespace

int ca_copy_chunks(ca_ctx* c, const int32_t* src_dst, int n_pairs, void* stream) {
    if (int rc = check_copy_pairs(c, src_dst, n_pairs)) return rc;
    if (n_pairs == 0) return CA_OK;
    const ca::LaunchArgs a = launch_args(c, nullptr, nullptr);
    return launch_rc(ca::launch_copy_chunks(a, src_dst, n_pairs, nullptr, nullptr, nullptr, 0,
                                            static_cast<hipStream_t>(stream)), "chunk copy launch");
}

int ca_copy_chunks_put_rows(ca_ctx* c, const int32_t* src_dst, int n_pairs, const void* k, const void* v, int n_rows,
                            const int32_t* slot_row, void* stream) {
    if (int rc = check_copy_pairs(c, src_dst, n_pairs)) return rc;
    if (int rc = check_row_targets(c, k, v, n_rows, slot_row)) return rc;
    if (n_pairs == 0 && n_rows == 0) return CA_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const ca::LaunchArgs a = launch_args(c, nullptr, nullptr);
    // One launch does both when the rows can simply be left out of the copies: the rows fit one
    // launch's argument block, a written row of a source chunk is written in its destination
    // chunk as well (else the copy would have to carry the row's old contents over while another
    // workgroup overwrites them), no chunk gets more than two rows, and no row is written twice.
    bool one_launch = n_rows <= 64 && n_pairs <= 64 && c->d % 8 == 0;
    for (int p = 0; one_launch && p < n_pairs; p++) {
        int rows_seen[2] = { -1, -1 };
        for (int r = 0; one_launch && r < n_rows; r++) {
            const int slot = slot_row[2 * r], row = slot_row[2 * r + 1];
            if (slot != src_dst[2 * p] && slot != src_dst[2 * p + 1]) continue;
            if (slot == src_dst[2 * p]) {
                bool also_in_dst = false;
                for (int q = 0; q < n_rows; q++) also_in_dst |= slot_row[2 * q] == src_dst[2 * p + 1] && slot_row[2 * q + 1] == row;
                one_launch &= also_in_dst;
            }
            if (rows_seen[0] < 0 || rows_seen[0] == row) rows_seen[0] = row;
            else if (rows_seen[1] < 0 || rows_seen[1] == row) rows_seen[1] = row;
            else one_launch = false;
        }
    }
    for (int r = 0; one_launch && r < n_rows; r++) {
        for (int q = 0; q < r; q++) one_launch &= !(slot_row[2 * q] == slot_row[2 * r] && slot_row[2 * q + 1] == slot_row[2 * r + 1]);
    }
    if (one_launch) {
        return launch_rc(ca::launch_copy_chunks(a, src_dst, n_pairs, k, v, slot_row, n_rows, st), "chunk copy and row write launch");
    }
    if (n_pairs > 0) {
        if (int rc = launch_rc(ca::launch_copy_chunks(a, src_dst, n_pairs, nullptr, nullptr, nullptr, 0, st), "chunk copy launch")) return rc;
    }
    if (n_rows == 0) return CA_OK;
    return launch_rc(ca::launch_put_rows(a, k, v, slot_row, n_rows, st), "row write launch");
}

int ca_copy_chunk(ca_ctx* c, int src_slot, int dst_slot, void* stream) {
    const int32_t pair[2] = { src_slot, dst_slot };
    return ca_copy_chunks(c, pair, 1, stream);
}

int ca_put_kv_rows(ca_ctx* c, const void* k, const void* v, int n_rows, const int32_t* slot_row, void* stream) {
    if (int rc = check_row_targets(c, k, v, n_rows, slot_row)) return rc;
    if (n_rows == 0) return CA_OK;
    const ca::LaunchArgs a = launch_args(c, nullptr, nullptr);
    return launch_rc(ca::launch_put_rows(a, k, v, slot_row, n_rows, static_cast<hipStream_t>(stream)), "row write launch");
}

int ca_ctx_set_plan(ca_ctx* c, int shared_seg_chunks, int stream_chunks) {
    if (!c || shared_seg_chunks < 0 || stream_chunks < 0) return fail(CA_ERR_INVALID, "bad argument");
    c->seg_chunks = shared_seg_chunks;
    c->stream_chunks = stream_chunks;
    c->valid = false;
    return CA_OK;
}

int ca_ctx_set_stream_hint(ca_ctx* c, int mode) {
    if (!c || mode < 0 || mode > 2) return fail(CA_ERR_INVALID, "stream hint must be 0, 1 or 2");
    c->stream_hint = mode;
    return CA_OK;
}

int ca_ctx_set_replan(ca_ctx* c, int percent) {
    if (!c || percent < 0) return fail(CA_ERR_INVALID, "replan threshold must be 0 (never) or a positive percentage");
    c->replan_percent = percent;
    return CA_OK;
}

int ca_ctx_table_stats(const ca_ctx* c, int64_t* full_builds, int64_t* patches) {
    if (!c) return fail(CA_ERR_INVALID, "null context");
    if (full_builds) *full_builds = c->full_builds;
    if (patches) *patches = c->patches;
    return CA_OK;
}

int ca_ctx_set_schedule(ca_ctx* c, int mode) {
    if (!c || mode < 0 || mode > 1) return fail(CA_ERR_INVALID, "schedule mode must be 0 or 1");
    c->schedule = mode;
    return CA_OK;
}

int ca_ctx_plan_info(const ca_ctx* c, ca_plan_info* info) {
    if (!c || !info) return fail(CA_ERR_INVALID, "bad argument");
    return guarded([&]() -> int {
        const ca::RefTables& ref = ref_tables(c);
        info->n_seqs = c->n_seqs;
        info->n_chunks = ref.n_chunks;
        info->n_shared_chunks = ref.n_shared;
        info->ref_partial_rows = ref.partial_rows;
        info->max_seq_n_chunks = ref.max_seq_n_chunks;
        info->n_shared_items = static_cast<int>(c->plan.shared_items.size());
        info->n_stream_items = static_cast<int>(c->plan.stream_items.size());
        info->n_part_rows = c->plan.n_part_rows;
        info->shared_tokens = c->plan.shared_tokens;
        info->stream_tokens = c->plan.stream_tokens;
        info->stream_per_wave = c->plan.stream_per_wave ? 1 : 0;
        info->reserved = 0;
        return CA_OK;
    });
}

int ca_ctx_ref_tables(const ca_ctx* c, int32_t* final_idx, int32_t* slots, int32_t* begins,
                      int32_t* ends, int32_t* offsets, int32_t* seq_n_tokens,
                      int32_t* seq_chunk_map) {
    if (!c) return fail(CA_ERR_INVALID, "null context");
    auto copy = [](int32_t* dst, const std::vector<int32_t>& src) {
        if (dst && !src.empty()) std::memcpy(dst, src.data(), src.size() * 4);
    };
    return guarded([&]() -> int {
        const ca::RefTables& ref = ref_tables(c);
        copy(final_idx, ref.final_idx);
        copy(slots, ref.slots);
        copy(begins, ref.begins);
        copy(ends, ref.ends);
        copy(offsets, ref.offsets);
        copy(seq_n_tokens, ref.seq_n_tokens);
        copy(seq_chunk_map, ref.seq_chunk_map);
        return CA_OK;
    });
}

int ca_ctx_export_partials(ca_ctx* c, float* maxs, float* sums, float* attns, void* stream) {
    if (!c || !c->valid) return fail(CA_ERR_STATE, "kernel context is not valid");
    if (c->partition != 0) return fail(CA_ERR_STATE, "partials are exported for partition 0 only");
    return guarded([&]() -> int {
        const ca::Plan& p = c->plan;
        // one item group per shared chunk, in shared-chunk order, is what the layout needs
        int n_units = 0;
        for (const auto& it : p.shared_items) {
            if (it.n_chunks != 1) return fail(CA_ERR_STATE, "export needs tables built with shared_seg_chunks = 1");
            n_units++;
        }
        (void)n_units;
        const size_t bytes = size_t(p.n_part_rows) * c->H * ca::PART_STRIDE * 4;
        std::vector<float> host(bytes / 4);
        hipStream_t st = static_cast<hipStream_t>(stream);
        if (bytes) CA_HIP(hipMemcpyAsync(host.data(), c->part, bytes, hipMemcpyDeviceToHost, st));
        CA_HIP(hipStreamSynchronize(st));
        const float ln2 = 0.6931471805599453f;
        // With one chunk per segment the shared items come in shared-chunk order (several
        // items per chunk when it covers more than one tile of sequences).  Sequence s keeps
        // the partial of an item at row part_ptr[s] + item.part_row.
        int chunk = -1, prev_slot_first = -1;
        for (const auto& it : p.shared_items) {
            if (it.slot_first != prev_slot_first) {
                chunk++;
                prev_slot_first = it.slot_first;
            }
            const ca::RefTables& ref = ref_tables(c);
            if (chunk >= ref.n_shared) return fail(CA_ERR_STATE, "shared items do not match the shared chunks");
            const int off = ref.offsets[chunk];
            const int b = ref.begins[chunk];
            const int n = ref.ends[chunk] - b;
            for (int h = 0; h < c->H; h++) {
                for (int r = 0; r < it.n_rows; r++) {
                    const int s = it.seq_begin + r;
                    const float* src = host.data() + (size_t(p.part_ptr[s] + it.part_row) * c->H + h) * ca::PART_STRIDE;
                    const size_t dst = size_t(off) * c->H + size_t(h) * n + (s - b);
                    if (maxs) maxs[dst] = src[0] * ln2;
                    if (sums) sums[dst] = src[1];
                    if (attns) std::memcpy(attns + dst * c->d, src + 4, sizeof(float) * c->d);
                }
            }
        }
        return CA_OK;
    });
}

int ca_ctx_read_partials_raw(ca_ctx* c, float* out, int64_t n_floats, void* stream) {
    if (!c || !out || n_floats < 0) return fail(CA_ERR_INVALID, "bad argument");
    const int64_t have = int64_t(c->plan.n_part_rows) * c->H * ca::PART_STRIDE;
    const int64_t n = std::min(n_floats, have);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (n > 0) CA_HIP(hipMemcpyAsync(out, c->part, size_t(n) * 4, hipMemcpyDeviceToHost, st));
    CA_HIP(hipStreamSynchronize(st));
    return CA_OK;
}

// ---- measurement aids (not for callers) ------------------------------------------------------

int ca_bench_decode_launch(ca_ctx* c, const void* q, void* out, int n_seqs, int what, void* stream) {
    if (what < 0 || what > 2) return fail(CA_ERR_INVALID, "what must be 0 (whole decode launch), 1 (stream items) or 2 (shared items)");
    if (int rc = check_ready(c, q, n_seqs)) return rc;
    if (int rc = check_attention_shape(c)) return rc;
    if (n_seqs > 0 && !out) return fail(CA_ERR_INVALID, "null device pointer");
    if (n_seqs == 0) return CA_OK;
    if (c->partition != 0 || c->schedule != 0 || c->plan_schedule != 0) {
        return fail(CA_ERR_STATE, "the tables were built for another partition or schedule");
    }
    const ca::LaunchArgs a = launch_args(c, q, out);
    const int n_shared = what == 1 ? 0 : static_cast<int>(c->plan.shared_items.size());
    const int n_stream = what == 2 ? 0 : static_cast<int>(c->plan.stream_items.size());
    return launch_rc(ca::launch_decode(a, n_shared, n_stream, false, static_cast<hipStream_t>(stream)), "decode launch");
}

int ca_bench_read_probe(ca_ctx* c, const void* dev, size_t bytes, int wgs_per_cu, void* stream) {
    if (!c || !dev || bytes < 16 || (reinterpret_cast<uintptr_t>(dev) & 15)) return fail(CA_ERR_INVALID, "bad argument");
    if (wgs_per_cu < 1 || wgs_per_cu > 8) return fail(CA_ERR_INVALID, "wgs_per_cu must be 1 .. 8");
    return guarded([&]() -> int {
        void* sink = ca::probe_sink_ptr(c->device);
        if (!sink) return fail(CA_ERR_STATE, "the static device buffers were not set up on this device");
        return launch_rc(ca::launch_read_probe(dev, bytes, c->n_cus * wgs_per_cu, sink, static_cast<hipStream_t>(stream)), "read probe");
    });
}

}  // extern "C"
