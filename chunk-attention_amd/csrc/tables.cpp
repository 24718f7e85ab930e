#include "tables.h"

#include <algorithm>
#include <stdexcept>

namespace ca {

void build_ref_tables(const ChunkRow* rows, int n_rows, int n_seqs, int chunk_size,
                      int tpp_threshold, RefTables* out) {
    RefTables& t = *out;
    t = RefTables();
    // rows come from outside the library: every sequence range is checked before it indexes anything
    for (int i = 0; i < n_rows; i++) {
        if (rows[i].seq_begin < 0 || rows[i].seq_end > n_seqs || rows[i].seq_begin >= rows[i].seq_end) {
            throw std::invalid_argument("tables: chunk row with a bad sequence range");
        }
    }
    if (chunk_size <= 0) throw std::invalid_argument("tables: chunk size must be positive");
    t.n_chunks = n_rows;
    // shared = covers more than tpp_threshold sequences (reference kernel_cuda.cu:1343-1349)
    for (int i = 0; i < n_rows; i++) {
        const int n = rows[i].seq_end - rows[i].seq_begin;
        if (n > tpp_threshold) {
            t.begins.push_back(rows[i].seq_begin);
            t.ends.push_back(rows[i].seq_end);
            t.offsets.push_back(t.partial_rows);  // exclusive prefix sum (:1358-1369)
            t.partial_rows += n;
        }
    }
    t.n_shared = static_cast<int>(t.begins.size());

    t.seq_n_tokens.assign(n_seqs, 0);  // :1371-1377
    for (int i = 0; i < n_rows; i++)
        for (int s = rows[i].seq_begin; s < rows[i].seq_end; s++)
            t.seq_n_tokens[s] += rows[i].n_tokens;
    int max_len = 0;
    for (int s = 0; s < n_seqs; s++) max_len = std::max(max_len, t.seq_n_tokens[s]);
    t.max_seq_n_chunks = max_len / chunk_size + 1;  // :1382

    // shared chunks are numbered first, both groups in row order (:1393-1410)
    t.final_idx.resize(n_rows);
    t.slots.assign(n_rows, -1);
    t.seq_chunk_map.assign(size_t(n_seqs) * t.max_seq_n_chunks, -1);
    std::vector<int> filled(n_seqs, 0);
    int next_shared = 0, next_private = t.n_shared;
    for (int i = 0; i < n_rows; i++) {
        const int n = rows[i].seq_end - rows[i].seq_begin;
        const int id = (n > tpp_threshold) ? next_shared++ : next_private++;
        t.final_idx[i] = id;
        t.slots[id] = rows[i].slot;
        for (int s = rows[i].seq_begin; s < rows[i].seq_end; s++) {
            if (filled[s] >= t.max_seq_n_chunks) {
                throw std::logic_error("tables: a sequence has more chunks than its length allows");
            }
            t.seq_chunk_map[size_t(s) * t.max_seq_n_chunks + filled[s]++] = id;
        }
    }
}

namespace {
int ceil_div(int a, int b) { return (a + b - 1) / b; }
}  // namespace

namespace {

// Second stage of build_plan, also run on its own by roll_tails: cuts every sequence's private
// chunks (Plan::own) into stream items, numbers the partial rows and decides the launch form.
// Uses only what the plan holds, so that a patched plan and a rebuilt one agree.
void build_stream_items(Plan& p, int chunk_size, const PlanParams& params) {
    const int n_seqs = p.n_seqs;
    p.slots.resize(p.n_shared_slots);
    p.stream_items.clear();
    std::vector<int32_t> n_parts = p.shared_parts;
    const int stream_chunks = p.hints.stream_chunks, taper_chunks = p.hints.taper_chunks;
    int n_streaming = 0;  // sequences that stream anything
    for (int s = 0; s < n_seqs; s++) n_streaming += p.own[s].empty() ? 0 : 1;
    const int generation = std::max(1, 2 * params.n_cus / std::max(params.n_heads, 1));
    const int n_tapered = std::min(n_streaming / 2, std::max(n_streaming / 4, generation));
    int rank = 0;
    for (int s = 0; s < n_seqs; s++) {
        const auto& own = p.own[s];
        if (own.empty()) continue;
        const int item_chunks = (taper_chunks > 0 && rank >= n_streaming - n_tapered) ? taper_chunks : stream_chunks;
        rank++;
        const int total = static_cast<int>(own.size());
        // the last chunk is the sequence's tail, usually far from full: it rides along with
        // the item before it instead of opening a new one
        const int n_items = std::max(1, ceil_div(total - 1, item_chunks));
        for (int g = 0; g < n_items; g++) {
            const int c0 = int(int64_t(total) * g / n_items);
            const int c1 = int(int64_t(total) * (g + 1) / n_items);
            WorkItem it{};
            it.seq_begin = s;
            it.n_rows = 1;
            it.slot_first = static_cast<int>(p.slots.size());
            it.n_chunks = c1 - c0;
            it.pos0 = p.own_pos0[s] + c0;
            it.len0 = p.seq_len[s];
            for (int k = c0; k < c1; k++) {
                if (k - c0 < kInlineSlots) it.inl[k - c0] = own[k];
                p.slots.push_back(own[k]);
            }
            it.part_row = n_parts[s]++;
            p.stream_items.push_back(it);
        }
    }

    // Many short runs (a long shared prompt, a few private tokens each): a workgroup per run
    // would spend most of its life starting up, and only some of its waves would have a tile.
    // When every item is at most three 64-token tiles and there are enough of them to fill the
    // device at one item per wave, each wave takes an item of its own.
    {
        int max_tiles = 0;
        for (const WorkItem& it : p.stream_items) max_tiles = std::max(max_tiles, ceil_div(it.n_chunks * chunk_size, 64));
        const int64_t tasks = int64_t(p.stream_items.size()) * std::max(params.n_heads, 1);
        p.stream_per_wave = params.allow_per_wave && !p.stream_items.empty() && max_tiles <= 3 &&
                            tasks >= int64_t(3) * 2 * params.n_cus;
    }

    // a sequence whose only partial comes from a stream item needs no merge: that item
    // writes the final output itself and its partial row is dropped from the merge list
    for (auto& it : p.stream_items) {
        if (n_parts[it.seq_begin] == 1) {
            it.part_row = -1;
            n_parts[it.seq_begin] = 0;
        }
    }

    p.part_ptr.assign(n_seqs + 1, 0);
    p.max_parts_per_seq = 0;
    for (int s = 0; s < n_seqs; s++) {
        p.part_ptr[s + 1] = p.part_ptr[s] + n_parts[s];
        p.max_parts_per_seq = std::max(p.max_parts_per_seq, n_parts[s]);
    }
    p.n_part_rows = p.part_ptr[n_seqs];

    // the fused decode step lets the stream item that ends a sequence write the new token's row
    p.tails_streamed = n_seqs > 0;
    for (int s = 0; s < n_seqs; s++) {
        if (p.own[s].empty() || p.own[s].back() != p.tail_slot[s]) p.tails_streamed = false;
    }
    p.shared_narrow = true;
    for (const WorkItem& it : p.shared_items) {
        if ((it.flags & kItemWide) || it.n_rows > 16) p.shared_narrow = false;
    }

    // what the kernels assume about every item
    for (const auto* list : { &p.shared_items, &p.stream_items }) {
        for (const WorkItem& it : *list) {
            if (it.n_chunks < 1 || it.n_chunks > kMaxItemChunks) {
                throw std::logic_error("tables: work item with an unsupported number of chunks");
            }
        }
    }
}

}  // namespace

void build_plan(const ChunkRow* rows, int n_rows, int n_seqs, int chunk_size,
                const PlanParams& params, Plan* out) {
    Plan& p = *out;
    p = Plan();
    p.n_seqs = n_seqs;
    p.partition = params.partition;
    p.seq_len.assign(n_seqs, 0);
    p.tail_slot.assign(n_seqs, -1);
    p.tail_fill.assign(n_seqs, 0);
    p.tail_width.assign(n_seqs, 0);

    auto is_shared = [&](const ChunkRow& r) {
        if (params.partition == 2) return false;
        if (params.partition == 1) return true;
        return (r.seq_end - r.seq_begin) > params.tpp_threshold;
    };

    // position of every row on its root->leaf path = number of chunks above it.  Rows come
    // in pre-order, so a row's parent is the nearest earlier row whose range contains it;
    // since every non-leaf chunk is full, position p also means "p*chunk_size tokens above".
    std::vector<int> pos(n_rows, 0);
    {
        std::vector<int> depth_of_seq(n_seqs, 0);  // chunks seen so far on each sequence's path
        for (int i = 0; i < n_rows; i++) {
            const ChunkRow& r = rows[i];
            if (r.seq_begin < 0 || r.seq_end > n_seqs || r.seq_begin >= r.seq_end) {
                throw std::invalid_argument("tables: chunk row with a bad sequence range");
            }
            pos[i] = depth_of_seq[r.seq_begin];
            for (int s = r.seq_begin; s < r.seq_end; s++) {
                depth_of_seq[s]++;
                p.seq_len[s] += r.n_tokens;
                p.tail_slot[s] = r.slot;  // the last row covering s is its tail
                p.tail_fill[s] = r.n_tokens;
                p.tail_width[s] = r.seq_end - r.seq_begin;
            }
        }
    }

    // ---- shared runs -> segments ---------------------------------------------------------
    struct Run { int first_row, count; };
    std::vector<Run> runs;
    for (int i = 0; i < n_rows;) {
        if (!is_shared(rows[i])) { i++; continue; }
        int j = i + 1;
        while (j < n_rows && is_shared(rows[j]) && rows[j].seq_begin == rows[i].seq_begin &&
               rows[j].seq_end == rows[i].seq_end && pos[j] == pos[j - 1] + 1) {
            j++;
        }
        runs.push_back({ i, j - i });
        i = j;
    }
    // Which runs take the row-split wide form.  From kWideMin sequences on it always pays: each
    // K/V byte is fetched once per 128 sequences instead of once per 32.  Between kWideMinLong and
    // kWideMin it replaces two or three 32-row workgroups per segment by one whose tiles take
    // longer (~2 us against ~1.4 us), which halves the slot time the run takes from the streaming
    // but lengthens its chain: worth it on long runs only (measured with 64 sequences: a 64-chunk
    // run 28.4 -> 26.6 us per forward, a 48-chunk run 175.4 -> 168.9 us, 32- and 16-chunk runs
    // under long private parts unchanged, the 16-chunk root of a two-level tree 37.2 -> 38.6 us;
    // with 48 sequences, 48 shared chunks and 1024 private tokens 133.6 -> 130.3 us, 40 sequences,
    // 64 chunks and 512 tokens 72.0 -> 66.7 us, 56 sequences sharing all 64 chunks 27.0 -> 23.6 us).
    // Where "long" begins, from 40 and 64 sequences with 128, 512 and 2048 private tokens: at 2048
    // shared tokens the wide form is 0-8 % faster in all six cases, at 1024 it ranges from 6 %
    // faster to 7 % slower.
    auto run_wide = [&](const Run& run) {
        const int n = rows[run.first_row].seq_end - rows[run.first_row].seq_begin;
        return n >= kWideMin || (n >= kWideMinLong && int64_t(run.count) * chunk_size >= kWideLongTokens);
    };
    // Segment length.  A shared workgroup may run for a good part of the step's expected
    // duration (bytes at ~6.4 TB/s) but must not outlast it.  Long segments mean fewer
    // workgroups (each pays its start-up and final merge once), fewer partial rows to write and
    // merge, and fewer slots taken from the streaming workgroups; measured per 64-token tile,
    // unloaded: ~1.4 us for a 32-row item, ~2 us for a wide one, and up to twice that next to
    // streaming workgroups.  When the step is short but the shared work is not (everything
    // shared, little to stream), the tile count grows until the shared workgroups fit the
    // device's slots (two per compute unit, one for wide items) in one go (measured, 64 sequences
    // sharing all 64 chunks: 8 wide segments of 8 chunks 24.5 us per forward, 16 of 4: 26.5,
    // 11 of 6: 26.4, 6 of 11: 26.0, 4 of 16: 31.8).
    int64_t all_tokens = 0;
    for (int i = 0; i < n_rows; i++) {
        all_tokens += int64_t(rows[i].n_tokens) * (is_shared(rows[i]) ? 1 : rows[i].seq_end - rows[i].seq_begin);
    }
    const double step_us = double(all_tokens) * 4.0 * std::max(params.n_heads, 1) * 128.0 / 6.4e6;
    auto shared_wgs_with = [&](int n_tiles) {   // shared workgroups if every run used n_tiles per segment
        int64_t wgs = 0;
        for (const Run& run : runs) {
            const int n = rows[run.first_row].seq_end - rows[run.first_row].seq_begin;
            const int seg = std::clamp(n_tiles * 64 / chunk_size, 1, kMaxItemChunks);
            const int n_segs = std::max({ 1, (run.count + seg / 2) / seg, ceil_div(run.count, kMaxItemChunks) });
            // a wide workgroup counts for two: it keeps a compute unit's vector and matrix units
            // busy by itself, and a second one beside it only makes both take twice as long
            const bool wide = run_wide(run);
            wgs += int64_t(n_segs) * ceil_div(n, wide ? kWideRows : kMaxRows) * std::max(params.n_heads, 1) * (wide ? 2 : 1);
        }
        return wgs;
    };
    int base_tiles = std::max(static_cast<int>(0.3 * step_us), 4);
    while (base_tiles < 32 && shared_wgs_with(base_tiles) > int64_t(2) * params.n_cus) base_tiles++;
    if (params.keep) base_tiles = params.keep->base_tiles;
    p.hints.base_tiles = base_tiles;
    p.hints.built_tokens = params.keep ? params.keep->built_tokens : all_tokens;
    auto seg_chunks_for = [&](bool wide) {
        if (params.shared_seg_chunks > 0) return std::min(params.shared_seg_chunks, kMaxItemChunks);
        const int n_tiles = std::min(base_tiles, wide ? 64 : 32);  // 64-token tiles
        return std::clamp(n_tiles * 64 / chunk_size, 1, kMaxItemChunks);
    };

    std::vector<int32_t> n_parts(n_seqs, 0);  // partial rows handed out per sequence so far
    // segments per run: nearest, not ceiling; but never more chunks in a segment than an item holds
    std::vector<int> run_segs(runs.size());
    for (size_t r = 0; r < runs.size(); r++) {
        const int seg = seg_chunks_for(run_wide(runs[r]));
        run_segs[r] = std::max({ 1, (runs[r].count + seg / 2) / seg, ceil_div(runs[r].count, kMaxItemChunks) });
    }
    // Runs of different widths (a root shared by everyone, groups below it): a tile costs more
    // with more sequences on it (relative, alone: 1.0 up to 16 rows, 1.4 up to 32, 2.0 in the wide
    // form), and the workgroups with the longest chains keep their slots from the streaming
    // longest.  Runs whose segments would outlast what most shared workgroups take (the median
    // segment cost, weighted by workgroups) by more than a quarter are cut finer, at most twice as
    // fine (measured: two-level workload, root run 2 -> 3 segments, 39.4 -> 37.4 us per forward).
    if (params.shared_seg_chunks <= 0 && runs.size() > 1) {
        auto run_cost = [&](size_t r) {
            const int n = rows[runs[r].first_row].seq_end - rows[runs[r].first_row].seq_begin;
            const double per_tile = run_wide(runs[r]) ? 2.0 : (n > 16 ? 1.4 : 1.0);
            return per_tile * runs[r].count * chunk_size / 64.0;
        };
        std::vector<std::pair<double, int64_t>> seg_cost;  // (cost of one segment, workgroups per head)
        int64_t total_weight = 0;
        for (size_t r = 0; r < runs.size(); r++) {
            const int n = rows[runs[r].first_row].seq_end - rows[runs[r].first_row].seq_begin;
            const int64_t wgs = int64_t(run_segs[r]) * ceil_div(n, run_wide(runs[r]) ? kWideRows : kMaxRows);
            seg_cost.emplace_back(run_cost(r) / run_segs[r], wgs);
            total_weight += wgs;
        }
        std::sort(seg_cost.begin(), seg_cost.end());
        double median = seg_cost.back().first;
        int64_t acc = 0;
        for (const auto& sc : seg_cost) {
            acc += sc.second;
            if (2 * acc >= total_weight) {
                median = sc.first;
                break;
            }
        }
        for (size_t r = 0; r < runs.size(); r++) {
            if (median <= 0.0 || run_cost(r) / run_segs[r] <= 1.25 * median) continue;
            const int want = static_cast<int>(run_cost(r) / median + 0.5);
            run_segs[r] = std::min({ std::max(want, run_segs[r]), 2 * run_segs[r], runs[r].count });
        }
    }
    for (size_t ri = 0; ri < runs.size(); ri++) {
        const Run& run = runs[ri];
        const ChunkRow& r0 = rows[run.first_row];
        const int n = r0.seq_end - r0.seq_begin;
        const int n_segs = run_segs[ri];
        for (int g = 0; g < n_segs; g++) {
            // spread chunks evenly over the segments of a run
            const int c0 = int(int64_t(run.count) * g / n_segs);
            const int c1 = int(int64_t(run.count) * (g + 1) / n_segs);
            const int slot_first = static_cast<int>(p.slots.size());
            for (int k = c0; k < c1; k++) {
                p.slots.push_back(rows[run.first_row + k].slot);
                p.shared_tokens += rows[run.first_row + k].n_tokens;
            }
            // every covered sequence has the same chunks above this one, so this segment is
            // the same ordinal among the partial rows of each of them
            const int ordinal = n_parts[r0.seq_begin];
            for (int s = 0; s < n; s++) {
                if (n_parts[r0.seq_begin + s] != ordinal) {
                    throw std::logic_error("tables: sequences of one shared chunk disagree on its position");
                }
                n_parts[r0.seq_begin + s]++;
            }
            const bool wide = run_wide(run);
            const int tile_rows = wide ? kWideRows : kMaxRows;
            for (int m0 = 0; m0 < n; m0 += tile_rows) {
                WorkItem it{};
                it.flags = wide ? kItemWide : 0;
                it.seq_begin = r0.seq_begin + m0;
                it.n_rows = std::min(tile_rows, n - m0);
                it.slot_first = slot_first;
                it.n_chunks = c1 - c0;
                it.part_row = ordinal;
                it.pos0 = pos[run.first_row + c0];
                it.len0 = p.seq_len[r0.seq_begin];
                for (int k = 0; k < kInlineSlots && k < c1 - c0; k++) it.inl[k] = p.slots[slot_first + k];
                p.shared_items.push_back(it);
            }
        }
    }

    // ---- per-sequence private chunk lists -------------------------------------------------
    p.n_shared_slots = static_cast<int>(p.slots.size());
    p.own.assign(n_seqs, {});
    p.own_pos0.assign(n_seqs, 0);
    p.shared_parts = n_parts;
    int64_t stream_chunk_total = 0;
    {
        std::vector<int> last_pos(n_seqs, -1);
        for (int i = 0; i < n_rows; i++) {
            if (is_shared(rows[i])) continue;
            for (int s = rows[i].seq_begin; s < rows[i].seq_end; s++) {
                // the chunks a sequence streams are the tail end of its path: consecutive positions
                if (p.own[s].empty()) {
                    p.own_pos0[s] = pos[i];
                } else if (pos[i] != last_pos[s] + 1) {
                    throw std::logic_error("tables: private chunks of a sequence are not consecutive");
                }
                last_pos[s] = pos[i];
                p.own[s].push_back(rows[i].slot);
                p.stream_tokens += rows[i].n_tokens;
                stream_chunk_total++;
            }
        }
    }
    // Stream item length.  Taper: the stream items of the last sequences are half as long -- of
    // as many sequences as fill the device's workgroup slots once (one "generation": 2 * n_cus /
    // n_heads), or of the last quarter if that is more, never of more than half.  Workgroups
    // start in item order, so these are the ones that run while the launch drains; with items of
    // one size the last generation is a partial one whose members start late and end together
    // (measured at 512 private tokens per sequence: 32 sequences 50.6 -> 49.5 us per forward, 48:
    // 71.2 -> 69.7, 64: 88.6 -> 87.3, 128: 169.7 -> 167.3; quarter-length items leave waves idle
    // and lose).
    int stream_chunks = params.stream_chunks;
    int taper_chunks = 0;
    if (stream_chunks <= 0) {
        // four waves per workgroup each take whole chunks, so prefer multiples of four;
        // shrink towards four when there would be too few workgroups to fill the device
        // (never below one 64-token tile per wave: 256 tokens, and four chunks)
        const int per_wg_tokens = 512;
        const int min_chunks = std::max(4, 256 / chunk_size);
        stream_chunks = std::max(min_chunks, per_wg_tokens / chunk_size);
        const int64_t heads = std::max(params.n_heads, 1);
        const int64_t target = int64_t(2) * params.n_cus;
        while (stream_chunks > min_chunks && (stream_chunk_total / stream_chunks) * heads < target) {
            stream_chunks /= 2;
        }
        // Longer items where the streaming is long enough to stay balanced with them: every item
        // but a sequence's only one leaves a partial row behind, and rows written while the launch
        // streams cost far more than their bytes (measured with the stores switched off: 64
        // sequences x 4096 private tokens 653 -> 608 us for 10.9 MB of rows, i.e. the memory turns
        // its bus around for dirty lines that leave the L2 a few at a time).  Up to 2048 tokens per
        // item as long as that leaves five fills of the device's workgroup slots (measured, 512 ->
        // 2048 tokens: 64 x 4096 private tokens 666 -> 636 us, 64 x (1024 shared + 3072) 494 -> 488,
        // 32 x 2560 private 207 -> 202; with fewer fills the last, partial one costs more than the
        // rows: 64 x (3072 shared + 1024) 169 -> 173 us at 1024 tokens).
        while (stream_chunks * 2 * chunk_size <= 2048 &&
               (stream_chunk_total / (stream_chunks * 2)) * heads >= int64_t(10) * params.n_cus) {
            stream_chunks *= 2;
        }
        if (stream_chunks / 2 >= min_chunks) taper_chunks = stream_chunks / 2;
    }
    stream_chunks = std::min(stream_chunks, kMaxItemChunks - 1);  // an item may take one chunk more
    if (taper_chunks >= stream_chunks) taper_chunks = 0;          // (after the cap: nothing to taper)
    if (params.keep) {
        stream_chunks = params.keep->stream_chunks;
        taper_chunks = params.keep->taper_chunks;
    }
    p.hints.stream_chunks = stream_chunks;
    p.hints.taper_chunks = taper_chunks;

    build_stream_items(p, chunk_size, params);
}

void roll_tails(Plan* plan, int chunk_size, const PlanParams& params, int delta_tokens,
                const int32_t* seqs, const int32_t* new_slots, int n) {
    Plan& p = *plan;
    if (p.partition == 1 || params.tpp_threshold < 1 || params.partition != p.partition) {
        throw std::invalid_argument("tables: this plan attends last chunks chunk-first, it cannot be patched");
    }
    if (delta_tokens < 0 || n < 0 || (n > 0 && (!seqs || !new_slots))) {
        throw std::invalid_argument("tables: bad argument");
    }
    // validate before touching anything: the plan must stay usable when this throws
    std::vector<char> rolls(p.n_seqs, 0);
    for (int i = 0; i < n; i++) {
        const int s = seqs[i];
        if (s < 0 || s >= p.n_seqs || rolls[s]) throw std::invalid_argument("tables: bad or repeated sequence index");
        if (p.tail_fill[s] + delta_tokens != chunk_size) {
            throw std::invalid_argument("tables: the last chunk of a rolled sequence is not full");
        }
        if (p.own[s].empty()) throw std::invalid_argument("tables: sequence without a private last chunk");
        // a streamed last chunk that covers several sequences (partition 2 or a threshold above 1):
        // where its successors belong among the rows is the tree's business, not the patch's
        if (p.tail_width[s] != 1) throw std::invalid_argument("tables: the last chunk of a rolled sequence is not its own");
        rolls[s] = 1;
    }
    for (int s = 0; s < p.n_seqs; s++) {
        if (!rolls[s] && p.tail_fill[s] + delta_tokens > chunk_size) {
            throw std::invalid_argument("tables: a last chunk would hold more than chunk_size tokens");
        }
    }
    for (WorkItem& it : p.shared_items) it.len0 += delta_tokens;
    for (int s = 0; s < p.n_seqs; s++) {
        p.seq_len[s] += delta_tokens;
        p.tail_fill[s] += delta_tokens;
    }
    p.stream_tokens += int64_t(delta_tokens) * p.n_seqs;
    for (int i = 0; i < n; i++) {
        const int s = seqs[i];
        p.own[s].push_back(new_slots[i]);
        p.tail_slot[s] = new_slots[i];
        p.tail_fill[s] = 0;
        p.tail_width[s] = 1;
    }
    build_stream_items(p, chunk_size, params);
}

bool plan_is_stale(const Plan& plan, int percent, int64_t extra_tokens) {
    if (percent <= 0 || plan.hints.built_tokens <= 0) return false;
    const int64_t now = plan.shared_tokens + plan.stream_tokens + extra_tokens;
    const int64_t then = plan.hints.built_tokens;
    const int64_t diff = now > then ? now - then : then - now;
    return diff * 100 > int64_t(percent) * then;
}

}  // namespace ca
