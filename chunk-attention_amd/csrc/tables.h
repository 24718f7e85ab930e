// Flattening of the prefix tree into device tables.
//
// Two forms are built from the same get_chunks() rows:
//   * RefTables: the reference's own table set (kernel_cuda.cu:1331-1445 of the reference)
//     with K/V pointers replaced by pool slot ids.  Kept for bit-exact structure checks.
//   * Plan: the packed work list the HIP kernels consume -- shared "segments" (runs of
//     consecutive shared chunks covering the same sequence range, cut into pieces), per-
//     sequence "stream" items over the chunks only that sequence reads, and per-sequence
//     lists of the partial rows to merge.
#pragma once

#include <cstdint>
#include <vector>

namespace ca {

struct ChunkRow {
    int32_t slot;
    int32_t n_tokens;
    int32_t seq_begin;
    int32_t seq_end;
};

struct RefTables {
    int n_chunks = 0;
    int n_shared = 0;
    int partial_rows = 0;       // sum of n over shared chunks
    int max_seq_n_chunks = 0;   // width of seq_chunk_map
    std::vector<int32_t> final_idx;      // per row: chunk id after shared-first renumbering
    std::vector<int32_t> slots;          // per final chunk id (stands for keys_values)
    std::vector<int32_t> begins, ends, offsets;  // per shared chunk
    std::vector<int32_t> seq_n_tokens;   // per sequence
    std::vector<int32_t> seq_chunk_map;  // [n_seqs, max_seq_n_chunks], -1 where unwritten
};

void build_ref_tables(const ChunkRow* rows, int n_rows, int n_seqs, int chunk_size,
                      int tpp_threshold, RefTables* out);

// One unit of kernel work: 16 x int32, read with one 64-byte scalar load.  The sequence length
// and the first chunk slots sit in the item itself so that a workgroup can issue its first K/V
// loads after a single memory round trip.
constexpr int kInlineSlots = 8;
// No item holds more chunks than a wavefront has lanes: every wave keeps its item's slot ids in
// one register, chunk k in lane k.
constexpr int kMaxItemChunks = 64;
struct WorkItem {
    int32_t seq_begin;   // first sequence (row of q) this item attends for
    int32_t n_rows;      // sequences covered (1 for stream items, <= kMaxRows for shared,
                         // <= kWideRows for wide shared items)
    int32_t slot_first;  // index into Plan::slots of the item's first chunk
    int32_t n_chunks;    // consecutive entries of Plan::slots, <= kMaxItemChunks
    int32_t part_row;    // which of its sequence's partial rows the item writes: row
                         // part_ptr[seq] + part_row (for every covered sequence of a shared
                         // item); -1: the item writes the final output directly
    int32_t pos0;        // position of the first chunk on the sequence's root->leaf path
    int32_t len0;        // tokens (when the tables were built) of the sequence whose length
                         // bounds the valid tokens of these chunks
    int32_t flags;       // kItemWide: shared item in the row-split form (up to kWideRows sequences)
    int32_t inl[kInlineSlots];  // slots of the first chunks (same as Plan::slots[slot_first ..])
};
static_assert(sizeof(WorkItem) == 64, "WorkItem must stay 64 bytes");

// Decisions build_plan derives from the size of the whole step.  A plan patched after tails
// rolled over keeps them (ca::roll_tails), and a rebuild can be told to (PlanParams::keep), so
// that both give the same tables.
struct PlanHints {
    int base_tiles = 0;     // length of a shared segment in 64-token tiles before per-run adjustments
    int stream_chunks = 0;  // chunks per stream item
    int taper_chunks = 0;   // chunks per stream item of the last sequences, 0: no taper
    int64_t built_tokens = 0;  // tokens one forward attended (shared once, private per owner) when
                               // these sizes were derived: how far a patched plan has drifted from them
};

struct PlanParams {
    const PlanHints* keep = nullptr;  // reuse these instead of deriving them from the step's size
    int tpp_threshold = 1;
    int partition = 0;        // 0: shared chunks chunk-first, rest streamed; 1: all chunk-first;
                              // 2: everything streamed per sequence
    int shared_seg_chunks = 0;  // max chunks per shared segment, 0 = choose from n_cus
    int stream_chunks = 0;      // max chunks per stream item, 0 = choose from n_cus
    int n_heads = 32;
    int n_cus = 256;
    bool allow_per_wave = true;  // the launch schedule can run stream items one per wave
};

constexpr int kMaxRows = 32;    // sequences per shared work item (M tile)
constexpr int kWideRows = 128;  // sequences per wide shared work item
constexpr int kWideMin = 96;    // chunks covering at least this many sequences use wide items
constexpr int kWideMinLong = 33;       // ... and from this many on (more than one M tile) when they belong to a long run:
constexpr int kWideLongTokens = 2048;  // a run of at least this many tokens
constexpr int32_t kItemWide = 1;

struct Plan {
    int n_seqs = 0;
    int n_part_rows = 0;
    int max_parts_per_seq = 0;
    bool stream_per_wave = false;  // stream items are short and many: one per wave, four per workgroup
    bool shared_narrow = false;    // no shared item is wide or covers more than 16 sequences
    bool tails_streamed = false;   // every sequence's last chunk is the last chunk of a stream item
                                   // (what the fused decode step needs)
    int64_t shared_tokens = 0;   // physical tokens attended chunk-first (per head)
    int64_t stream_tokens = 0;   // tokens attended by stream items (per head, at build time)
    std::vector<WorkItem> shared_items;
    std::vector<WorkItem> stream_items;
    std::vector<int32_t> slots;      // chunk slot lists the items index into
    std::vector<int32_t> seq_len;    // tokens per sequence when the plan was built
    std::vector<int32_t> part_ptr;   // [n_seqs + 1]: sequence s owns partial rows part_ptr[s] .. part_ptr[s+1]
    std::vector<int32_t> tail_slot;  // per sequence: slot of its last chunk
    std::vector<int32_t> tail_fill;  // per sequence: tokens in that chunk when built
    std::vector<int32_t> tail_width; // per sequence: sequences covered by that chunk (host-side only)

    // host-side state from which the stream items are (re)generated
    PlanHints hints;
    int partition = 0;                          // partition the plan was built for
    int n_shared_slots = 0;                     // slots[0 .. n_shared_slots) belong to shared items
    std::vector<std::vector<int32_t>> own;      // per sequence: slots of the chunks it streams, path order
    std::vector<int32_t> own_pos0;              // per sequence: path position of own[s][0]
    std::vector<int32_t> shared_parts;          // per sequence: partial rows written by shared items
};

void build_plan(const ChunkRow* rows, int n_rows, int n_seqs, int chunk_size,
                const PlanParams& params, Plan* out);

// The tables after `delta_tokens` tokens were appended to every sequence since the plan was
// built and the sequences seqs[i], whose last chunk is thereby full, each got the fresh empty
// chunk new_slots[i] as new last chunk (reference Attention::reserve, attention.cpp:116-131).
// Gives exactly what build_plan gives for the rows of the tree in that state with
// PlanParams::keep = the plan's own hints: every length advances by delta_tokens, the rolled
// sequences' stream items are cut again, partial-row numbering follows; shared items keep their
// segments.  Only for plans in which no last chunk is attended chunk-first (partition 0 or 2
// with tpp_threshold >= 1).  Throws std::invalid_argument when that does not hold or an argument
// does not fit the plan (also: the last chunk of a rolled sequence covers other sequences too, which
// only rows handed in by hand can produce); the plan is unchanged then.
void roll_tails(Plan* plan, int chunk_size, const PlanParams& params, int delta_tokens,
                const int32_t* seqs, const int32_t* new_slots, int n);

// Re-planning policy for long decodes.  A patched plan keeps the work-item sizes that were derived
// from the step's size at the last full build (PlanHints); they are worth deriving again once the
// tokens a forward attends differ from what they were then by more than `percent` per cent
// (`extra_tokens`: tokens appended since the plan was last patched, i.e. delta_tokens * n_seqs).
// percent <= 0: never.
bool plan_is_stale(const Plan& plan, int percent, int64_t extra_tokens = 0);

}  // namespace ca
