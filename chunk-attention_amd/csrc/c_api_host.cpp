// C-ABI of the decode path, host-only half: the table builder (ca_tables_*) and the prefix-tree
// chunk manager (ca_tree_*), plus the per-thread error message.  Nothing here touches a device or
// includes a HIP header, so this file, tables.cpp and prefix_tree.cpp also build with a plain C++
// compiler -- which is how the sanitizer build of the host logic is made (build.py --host-sanitize).
// Declarations and their reference counterparts are in include/chunk_attn_hip.h.
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "c_api_common.h"
#include "prefix_tree.h"
#include "tables.h"

namespace ca {
namespace abi {
namespace {
thread_local std::string g_last_error;
}
int fail(int code, const std::string& msg) {
    g_last_error = msg;
    return code;
}
const char* last_error() { return g_last_error.c_str(); }
}  // namespace abi
}  // namespace ca

using ca::abi::fail;
using ca::abi::guarded;

extern "C" {

const char* ca_last_error(void) { return ca::abi::last_error(); }

// ---- host-only table builder ---------------------------------------------------------------

struct ca_tables {
    ca::RefTables ref;
    ca::Plan plan;
    ca::PlanParams params;
    int n_seqs = 0;
    int chunk_size = 0;
};

namespace {
int tables_build(ca_tables** out, const ca_tables* like, const ca_chunk_row* rows, int n_rows, int n_seqs,
                 int chunk_size, int tpp_threshold, int partition, int shared_seg_chunks, int stream_chunks,
                 int n_heads, int n_cus) {
    if (!out || n_rows < 0 || n_seqs < 0 || (n_rows > 0 && !rows) || chunk_size <= 0) {
        return fail(CA_ERR_INVALID, "bad argument");
    }
    if (partition < 0 || partition > 2) return fail(CA_ERR_INVALID, "Unsupported partition type");
    return guarded([&]() -> int {
        auto t = new ca_tables();
        t->n_seqs = n_seqs;
        t->chunk_size = chunk_size;
        const ca::ChunkRow* r = reinterpret_cast<const ca::ChunkRow*>(rows);
        ca::PlanParams& pp = t->params;
        pp.tpp_threshold = tpp_threshold;
        pp.partition = partition;
        pp.shared_seg_chunks = shared_seg_chunks;
        pp.stream_chunks = stream_chunks;
        pp.n_heads = n_heads;
        pp.n_cus = n_cus;
        ca::PlanHints keep;
        if (like) {
            keep = like->plan.hints;
            pp.keep = &keep;
        }
        try {
            ca::build_ref_tables(r, n_rows, n_seqs, chunk_size, tpp_threshold, &t->ref);
            ca::build_plan(r, n_rows, n_seqs, chunk_size, pp, &t->plan);
        } catch (...) {
            delete t;
            throw;
        }
        pp.keep = nullptr;  // pointed at a local
        *out = t;
        return CA_OK;
    });
}
}  // namespace

int ca_tables_build(ca_tables** out, const ca_chunk_row* rows, int n_rows, int n_seqs,
                    int chunk_size, int tpp_threshold, int partition, int shared_seg_chunks,
                    int stream_chunks, int n_heads, int n_cus) {
    return tables_build(out, nullptr, rows, n_rows, n_seqs, chunk_size, tpp_threshold, partition,
                        shared_seg_chunks, stream_chunks, n_heads, n_cus);
}

int ca_tables_build_like(ca_tables** out, const ca_tables* like, const ca_chunk_row* rows, int n_rows,
                         int n_seqs) {
    if (!like) return fail(CA_ERR_INVALID, "bad argument");
    const ca::PlanParams& pp = like->params;
    return tables_build(out, like, rows, n_rows, n_seqs, like->chunk_size, pp.tpp_threshold, pp.partition,
                        pp.shared_seg_chunks, pp.stream_chunks, pp.n_heads, pp.n_cus);
}

int ca_tables_roll_tails(ca_tables* t, int delta_tokens, const int32_t* seq_idx, const int32_t* new_slots, int n) {
    if (!t) return fail(CA_ERR_INVALID, "bad argument");
    return guarded([&]() -> int {
        ca::roll_tails(&t->plan, t->chunk_size, t->params, delta_tokens, seq_idx, new_slots, n);
        return CA_OK;
    });
}

int ca_tables_stale(const ca_tables* t, int percent, int64_t extra_tokens) {
    return t && ca::plan_is_stale(t->plan, percent, extra_tokens) ? 1 : 0;
}

void ca_tables_destroy(ca_tables* t) { delete t; }

int ca_tables_info(const ca_tables* t, ca_plan_info* info) {
    if (!t || !info) return fail(CA_ERR_INVALID, "bad argument");
    info->n_seqs = t->n_seqs;
    info->n_chunks = t->ref.n_chunks;
    info->n_shared_chunks = t->ref.n_shared;
    info->ref_partial_rows = t->ref.partial_rows;
    info->max_seq_n_chunks = t->ref.max_seq_n_chunks;
    info->n_shared_items = static_cast<int>(t->plan.shared_items.size());
    info->n_stream_items = static_cast<int>(t->plan.stream_items.size());
    info->n_part_rows = t->plan.n_part_rows;
    info->shared_tokens = t->plan.shared_tokens;
    info->stream_tokens = t->plan.stream_tokens;
    info->stream_per_wave = t->plan.stream_per_wave ? 1 : 0;
    info->reserved = 0;
    return CA_OK;
}

int ca_tables_plan_sizes(const ca_tables* t, int* n_slots) {
    if (!t) return fail(CA_ERR_INVALID, "bad argument");
    if (n_slots) *n_slots = static_cast<int>(t->plan.slots.size());
    return CA_OK;
}

static void copy_i32(int32_t* dst, const std::vector<int32_t>& src) {
    if (dst && !src.empty()) std::memcpy(dst, src.data(), src.size() * 4);
}

int ca_tables_ref(const ca_tables* t, int32_t* final_idx, int32_t* slots, int32_t* begins,
                  int32_t* ends, int32_t* offsets, int32_t* seq_n_tokens, int32_t* seq_chunk_map) {
    if (!t) return fail(CA_ERR_INVALID, "bad argument");
    copy_i32(final_idx, t->ref.final_idx);
    copy_i32(slots, t->ref.slots);
    copy_i32(begins, t->ref.begins);
    copy_i32(ends, t->ref.ends);
    copy_i32(offsets, t->ref.offsets);
    copy_i32(seq_n_tokens, t->ref.seq_n_tokens);
    copy_i32(seq_chunk_map, t->ref.seq_chunk_map);
    return CA_OK;
}

int ca_tables_plan(const ca_tables* t, ca_work_item* shared_items, ca_work_item* stream_items,
                   int32_t* slots, int32_t* seq_len, int32_t* part_ptr, int32_t* tail_slot,
                   int32_t* tail_fill) {
    if (!t) return fail(CA_ERR_INVALID, "bad argument");
    static_assert(sizeof(ca_work_item) == sizeof(ca::WorkItem), "work item layouts must agree");
    if (shared_items && !t->plan.shared_items.empty()) {
        std::memcpy(shared_items, t->plan.shared_items.data(), t->plan.shared_items.size() * sizeof(ca::WorkItem));
    }
    if (stream_items && !t->plan.stream_items.empty()) {
        std::memcpy(stream_items, t->plan.stream_items.data(), t->plan.stream_items.size() * sizeof(ca::WorkItem));
    }
    copy_i32(slots, t->plan.slots);
    copy_i32(seq_len, t->plan.seq_len);
    copy_i32(part_ptr, t->plan.part_ptr);
    copy_i32(tail_slot, t->plan.tail_slot);
    copy_i32(tail_fill, t->plan.tail_fill);
    return CA_OK;
}

// ---- prefix-tree manager -------------------------------------------------------------------

struct ca_tree {
    GPT::PrefixTree tree;
    ca_tree(int c, int max_chunks, bool share) : tree(c, max_chunks, share, 0) {}
};

int ca_tree_create(ca_tree** out, int chunk_size, int max_chunks, int share_prefix) {
    if (!out || chunk_size <= 0 || max_chunks < 0) return fail(CA_ERR_INVALID, "bad argument");
    return guarded([&]() -> int {
        *out = new ca_tree(chunk_size, max_chunks, share_prefix != 0);
        return CA_OK;
    });
}

void ca_tree_destroy(ca_tree* t) { delete t; }

int ca_tree_max_chunks_for(int memory_mb, int chunk_size, int n_heads, int d_head, int elem_bytes) {
    return GPT::ChunkAllocator::max_chunks_for(memory_mb, chunk_size, n_heads, d_head, elem_bytes);
}

int ca_tree_add_seq(ca_tree* t, const int32_t* tokens, int n_tokens, int* seq_idx, int* tok_begin,
                    int32_t* new_slots, int cap, int* n_new) {
    if (!t || n_tokens < 0 || (n_tokens > 0 && !tokens)) return fail(CA_ERR_INVALID, "bad argument");
    return guarded([&]() -> int {
        std::vector<int> ids(tokens, tokens + n_tokens);
        std::vector<GPT::CopyJob> jobs;
        const int idx = t->tree.add_seq(ids, &jobs);
        if (seq_idx) *seq_idx = idx;
        if (tok_begin) *tok_begin = jobs.empty() ? n_tokens : jobs.front().tok_begin;
        if (n_new) *n_new = static_cast<int>(jobs.size());
        for (int i = 0; i < static_cast<int>(jobs.size()) && i < cap && new_slots; i++) new_slots[i] = jobs[i].slot;
        return CA_OK;
    });
}

int ca_tree_remove_seq(ca_tree* t, int seq_idx) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    return guarded([&]() -> int {
        t->tree.remove_seq(seq_idx);
        return CA_OK;
    });
}

int ca_tree_clear(ca_tree* t) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    return guarded([&]() -> int {
        t->tree.clear();
        return CA_OK;
    });
}

int ca_tree_reserve(ca_tree* t, int* n_new) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    return guarded([&]() -> int {
        const auto fresh = t->tree.reserve();
        if (n_new) *n_new = static_cast<int>(fresh.size());
        return CA_OK;
    });
}

int ca_tree_reserve_tails(ca_tree* t, int32_t* seq_idx, int32_t* new_slots, int cap, int* n_new) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    return guarded([&]() -> int {
        std::vector<int> seqs;
        const auto fresh = t->tree.reserve(&seqs);
        if (n_new) *n_new = static_cast<int>(fresh.size());
        for (int i = 0; i < static_cast<int>(fresh.size()) && i < cap; i++) {
            if (seq_idx) seq_idx[i] = seqs[i];
            if (new_slots) new_slots[i] = fresh[i]->slot();
        }
        return CA_OK;
    });
}

int ca_tree_append_token(ca_tree* t, const int32_t* tokens, int n_tokens, int* n_new) {
    if (!t || n_tokens < 0 || (n_tokens > 0 && !tokens)) return fail(CA_ERR_INVALID, "bad argument");
    return guarded([&]() -> int {
        if (static_cast<int>(t->tree.tails().size()) != n_tokens) {
            throw std::runtime_error("num of seqs is not equal to num of tokens");
        }
        const auto fresh = t->tree.reserve();
        t->tree.append_token_ids(std::vector<int>(tokens, tokens + n_tokens));
        if (n_new) *n_new = static_cast<int>(fresh.size());
        return CA_OK;
    });
}

int ca_tree_get_chunks(const ca_tree* t, ca_chunk_row* rows, int cap, int* n_rows) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    return guarded([&]() -> int {
        const auto infos = t->tree.get_chunks();
        if (n_rows) *n_rows = static_cast<int>(infos.size());
        for (int i = 0; i < static_cast<int>(infos.size()) && i < cap && rows; i++) {
            rows[i] = { infos[i].chunk->slot(), infos[i].chunk->n_tokens(), infos[i].seq_idx_begin, infos[i].seq_idx_end };
        }
        return CA_OK;
    });
}

int ca_tree_n_seqs(const ca_tree* t) { return t ? t->tree.n_seqs() : 0; }
int ca_tree_used_chunks(const ca_tree* t) { return t ? t->tree.allocator().used_chunks() : 0; }
uint64_t ca_tree_version(const ca_tree* t) { return t ? t->tree.version() : 0; }

int ca_tree_duplicate(ca_tree* t, int seq_idx, int copies, int32_t* copy_pairs, int cap_pairs, int* n_pairs) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    if (n_pairs) *n_pairs = 0;
    if (copies < 1) return CA_OK;
    if (!copy_pairs || cap_pairs < copies) return fail(CA_ERR_INVALID, "copy_pairs holds fewer than `copies` pairs");
    return guarded([&]() -> int {
        std::vector<std::pair<int, int>> pairs;
        t->tree.duplicate(seq_idx, copies, &pairs);
        for (size_t i = 0; i < pairs.size(); i++) {
            copy_pairs[2 * i] = pairs[i].first;
            copy_pairs[2 * i + 1] = pairs[i].second;
        }
        if (n_pairs) *n_pairs = static_cast<int>(pairs.size());
        return CA_OK;
    });
}

int ca_tree_append_completion(ca_tree* t, int seq_idx, const int32_t* tokens, int n_tokens,
                              int32_t* copy_pairs, int cap_pairs, int* n_pairs, int32_t* targets) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    if (n_pairs) *n_pairs = 0;
    if (n_tokens < 0 || (n_tokens > 0 && (!tokens || !targets))) return fail(CA_ERR_INVALID, "bad argument");
    if (n_tokens > 1 && (!copy_pairs || cap_pairs < n_tokens - 1)) {
        return fail(CA_ERR_INVALID, "copy_pairs holds fewer than n_tokens - 1 pairs");
    }
    return guarded([&]() -> int {
        std::vector<std::pair<int, int>> pairs;
        std::vector<GPT::PrefixTree::RowTarget> rows;
        t->tree.append_completion(seq_idx, std::vector<int>(tokens, tokens + n_tokens), &pairs, &rows);
        for (size_t i = 0; i < pairs.size(); i++) {
            copy_pairs[2 * i] = pairs[i].first;
            copy_pairs[2 * i + 1] = pairs[i].second;
        }
        for (size_t i = 0; i < rows.size(); i++) {
            targets[2 * i] = rows[i].slot;
            targets[2 * i + 1] = rows[i].row;
        }
        if (n_pairs) *n_pairs = static_cast<int>(pairs.size());
        return CA_OK;
    });
}

int ca_tree_tails(const ca_tree* t, int32_t* slots, int cap, int* n) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    const auto& tails = t->tree.tails();
    if (n) *n = static_cast<int>(tails.size());
    for (int i = 0; i < static_cast<int>(tails.size()) && i < cap && slots; i++) slots[i] = tails[i]->slot();
    return CA_OK;
}

int ca_tree_dump(const ca_tree* t, int32_t* nodes, int node_cap, int* n_nodes, int32_t* tokens,
                 int token_cap, int* n_tokens) {
    if (!t) return fail(CA_ERR_INVALID, "null tree");
    return guarded([&]() -> int {
        int nn = 0, nt = 0;
        std::vector<std::pair<int, const GPT::Chunk*>> stack;
        stack.emplace_back(0, const_cast<ca_tree*>(t)->tree.root());
        while (!stack.empty()) {
            const auto [depth, node] = stack.back();
            stack.pop_back();
            if (nodes && nn < node_cap) {
                nodes[4 * nn + 0] = depth;
                nodes[4 * nn + 1] = node->n_seqs;
                nodes[4 * nn + 2] = node->n_tokens();
                nodes[4 * nn + 3] = node->slot();
            }
            nn++;
            for (int tok : node->tokens) {
                if (tokens && nt < token_cap) tokens[nt] = tok;
                nt++;
            }
            for (auto it = node->children.rbegin(); it != node->children.rend(); ++it) {
                stack.emplace_back(depth + 1, *it);
            }
        }
        if (n_nodes) *n_nodes = nn;
        if (n_tokens) *n_tokens = nt;
        return CA_OK;
    });
}

}  // extern "C"
