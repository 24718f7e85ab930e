/*
 * C-ABI of the MI355X ChunkAttention decode path (libchunkattn_hip.so).
 *
 * Plain C types and raw pointers only.  Pointers named *_dev / q / out / k / v / *_pool are
 * device (HBM) addresses; everything else is host memory.  `stream` is a hipStream_t passed
 * as void* (NULL = the default stream).  Every function returns 0 on success or a negative
 * CA_ERR_* code; ca_last_error() gives the message for the calling thread.
 *
 * Two groups of entry points:
 *   ca_ctx_*, ca_refresh_kernel_context, ca_attention, ca_attn_chunks_first,
 *   ca_attn_seqs_first, ca_append_kv: the kernel seam.  They replace the functions the
 *   reference declares in cpp/chunk_attn/kernel_cuda.h:57-71 and its KernelContext
 *   (kernel_cuda.h:9-55), with torch tensors replaced by pointers and chunk pointers by pool
 *   slot ids.
 *   ca_tree_*: the prefix-tree chunk manager (reference cpp/chunk_attn/attention.cpp), for
 *   hosts that do not link the C++ class.
 *
 * Layouts (fp16, d_head = 128):
 *   q, out          [n_seqs, n_heads, d_head]
 *   k, v (add)      [n_tokens, n_heads, d_head]
 *   k, v (append)   [n_seqs, n_heads, d_head]
 *   k_pool, v_pool  [max_chunks][n_heads][chunk_size][d_head]; chunk `slot` starts at element
 *                   slot * n_heads * chunk_size * d_head
 */
#ifndef CHUNK_ATTN_HIP_H
#define CHUNK_ATTN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CA_OK 0
#define CA_ERR_INVALID (-1)   /* bad argument / unsupported shape */
#define CA_ERR_HIP (-2)       /* a HIP runtime call failed */
#define CA_ERR_STATE (-3)     /* tables not valid, sizes do not match the tables, ... */
#define CA_ERR_CAPACITY (-4)  /* chunk pool exhausted */
#define CA_ERR_RUNTIME (-5)   /* other manager errors (message says which) */

const char* ca_last_error(void);

/* ---- kernel context ------------------------------------------------------------------- */

typedef struct ca_ctx ca_ctx;

/* One flattened-tree row: reference ChunkInfo (cpp/chunk_attn/chunk_info.h:6-15) with the
 * Chunk* replaced by the chunk's pool slot and token count. */
typedef struct ca_chunk_row {
    int32_t slot;
    int32_t n_tokens;
    int32_t seq_begin;
    int32_t seq_end;
} ca_chunk_row;

/* Replaces KernelContext's constructor (kernel_cuda.h:10-31).  Any shape is accepted here;
 * the attention entry points need d_head 128 and chunk_size 32, 64 or 128 and fail with
 * CA_ERR_INVALID otherwise, as the reference's do (kernel_cuda.cu:1199, 1256-1265).
 * The pools stay owned by the caller and must outlive the context. */
int ca_ctx_create(ca_ctx** out, int n_heads, int d_head, int chunk_size, void* k_pool,
                  void* v_pool, int max_chunks, int tpp_threshold);
void ca_ctx_destroy(ca_ctx* ctx);

/* Replaces refresh_kernel_context(ctx, chunk_infos, n_seqs) (kernel_cuda.cu:1331-1445):
 * flattens the rows (in get_chunks order) into device tables, sizes the partial-result
 * buffer, resets delta_tokens to 0 and marks the context valid. */
int ca_refresh_kernel_context(ca_ctx* ctx, const ca_chunk_row* rows, int n_rows, int n_seqs,
                              void* stream);

/* The refresh for the common decode-step case, without a tree walk: since the tables were built,
 * delta_tokens tokens were appended to every sequence and nothing else changed, except that the
 * sequences seq_idx[i] (whose last chunk is full now) each got the fresh empty chunk new_slots[i]
 * as their new last chunk (what reference Attention::reserve does, attention.cpp:116-131; the
 * reference then rebuilds every table, kernel_cuda.cu:1331-1445).  Patches the lengths, the rolled
 * sequences' work items and the partial-row numbering in place, uploads, and resets delta_tokens
 * to 0: the tables equal those of a full refresh that keeps the same work-item sizes.  n may be 0
 * (folds delta_tokens into the tables).  CA_ERR_STATE when the tables cannot be patched (not
 * valid, every chunk attended chunk-first, a listed chunk not full): they are left as they were,
 * call ca_refresh_kernel_context instead. */
int ca_ctx_roll_tails(ca_ctx* ctx, const int32_t* seq_idx, const int32_t* new_slots, int n,
                      void* stream);

/* KernelContext::valid / delta_tokens (kernel_cuda.h:42-45). */
int ca_ctx_valid(const ca_ctx* ctx);
void ca_ctx_invalidate(ca_ctx* ctx);
int ca_ctx_delta_tokens(const ca_ctx* ctx);
/* delta_tokens < 0 is rejected (CA_ERR_INVALID): it would address rows in front of a chunk. */
int ca_ctx_set_delta_tokens(ca_ctx* ctx, int delta_tokens);

/* Replaces attention(ctx, q, out, partition) (kernel_cuda.cu:1320-1329).  partition 0:
 * chunks covering more than tpp_threshold sequences are attended chunk-first, the rest per
 * sequence; 1: every chunk chunk-first; 2: every chunk per sequence (the meaning the
 * reference's CPU path gives the argument, kernel_cpu_mkl.cpp:364-372). */
int ca_attention(ca_ctx* ctx, const void* q, void* out, int n_seqs, int partition,
                 void* stream);

/* ca_attention (partition 0, default schedule) for callers that cannot allocate: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the
 * reference.  It calls no hipMalloc / hipFree or other allocating routine: the partial rows go to
 * a static device array of CA_NOALLOC_SCRATCH_BYTES that the library holds on every GPU it runs
 * on until the process ends, instead of the context's own buffer.  Fails with CA_ERR_INVALID when
 * the forward's partial rows (n_part_rows * n_heads * 640 bytes, see ca_ctx_plan_info) exceed
 * that, and with CA_ERR_STATE when the tables are not those of partition 0 in the default
 * schedule (it never rebuilds them).  All contexts on one GPU share the array: calls that
 * overlap on one GPU (different streams or threads) race; calls on one stream are safe.  Nothing
 * in the array needs clearing between calls (every row read is written first).
 * Under graph capture: delta_tokens and the table addresses are kernel arguments of the captured
 * launches, so a captured forward replays the sequence lengths it was captured with.  Capture
 * again after every ca_append_kv / ca_decode_step, ca_ctx_roll_tails or refresh. */
#define CA_NOALLOC_SCRATCH_BYTES (32u << 20)
int ca_attention_noalloc(ca_ctx* ctx, const void* q, void* out, int n_seqs, void* stream);

/* Replaces attn_chunks_first(ctx, q) (kernel_cuda.cu:1118-1193): partial (max, sum, P.V)
 * of every shared segment into the context's partial buffer. */
int ca_attn_chunks_first(ca_ctx* ctx, const void* q, int n_seqs, void* stream);

/* Replaces attn_seqs_first(ctx, q, out) (kernel_cuda.cu:1195-1271): streams every
 * sequence's own chunks, merges them with the partials of ca_attn_chunks_first and writes
 * the normalised output. */
int ca_attn_seqs_first(ca_ctx* ctx, const void* q, void* out, int n_seqs, void* stream);

/* Replaces append_kv(ctx, keys, values) (kernel_cuda.cu:1273-1318): writes one new K/V row
 * per sequence at position seq_len + delta_tokens.  Does not change delta_tokens. */
int ca_append_kv(ca_ctx* ctx, const void* k, const void* v, int n_seqs, void* stream);

/* One decode step of the reference's attention layer in one call: Attention::append_token's
 * device half (attention.cpp:80-114 -> append_kv, kernel_cuda.cu:1273-1318) followed by
 * forward (attention.cpp:57-78 -> attention, kernel_cuda.cu:1320-1329), i.e. exactly
 *   ca_append_kv(k, v); ca_ctx_set_delta_tokens(delta_tokens + 1); ca_attention(q, out, partition 0)
 * with the same results in `out` and in the pools, bit for bit.  k, v: the new token's rows
 * [n_seqs, n_heads, d_head]; q attends every token including the new one.  When every sequence's
 * last chunk is streamed per sequence (always, with trees built by ca_tree_* / the Attention class
 * and tpp_threshold >= 1) no append launch is made: the workgroup that streams a sequence's last
 * chunk takes the new row from k / v, and the merge launch writes the rows into the pool behind
 * its merges.  Otherwise the two launches are made here.  Same preconditions as ca_append_kv (a free row in every last chunk:
 * reserve and refresh / ca_ctx_roll_tails first); delta_tokens is advanced by one on success. */
int ca_decode_step(ca_ctx* ctx, const void* q, const void* k, const void* v, void* out, int n_seqs,
                   void* stream);

/* Replaces rotary_embedding(positions, query, key, head_size, cos_sin_cache, is_neox)
 * (cpp/chunk_attn/pos_encoding_kernels.cu:94-139, bound as chunk_attn.ops.rotary_embedding in
 * cpp/chunk_attn/python_exports_ops.cpp:13): rotates query and key rows in place, fp16 only.
 * positions: n_tokens int64 on the device.  query: n_tokens rows of n_heads*head_size halves,
 * query_stride elements apart; key likewise with n_kv_heads (key may be NULL with
 * n_kv_heads 0).  cos_sin_cache: [max_position, rot_dim] halves, rot_dim/2 cosines then
 * rot_dim/2 sines per position.  is_neox != 0 pairs element r with r + rot_dim/2 (GPT-NeoX),
 * else 2r with 2r+1 (GPT-J).  Products are formed in fp32 and rounded to fp16 once; positions
 * outside [0, max_position) are clamped into the cache instead of read out of bounds. */
int ca_rotary_embedding(const int64_t* positions_dev, void* query, void* key,
                        const void* cos_sin_cache, int64_t n_tokens, int n_heads,
                        int n_kv_heads, int head_size, int rot_dim, int max_position,
                        int64_t query_stride, int64_t key_stride, int is_neox, void* stream);

/* Replace rms_norm(out, input, weight, epsilon) and fused_add_rms_norm(input, residual, weight,
 * epsilon) (cpp/chunk_attn/layernorm_kernels.cu:66-117, bound in python_exports_ops.cpp:16-18):
 * fp16 rows [n_tokens, hidden_size], contiguous, fp32 statistics.
 *   ca_rms_norm:            out = fp16(x * rsqrt(mean(x^2) + epsilon)) * weight   (out may equal input)
 *   ca_fused_add_rms_norm:  residual = fp16(input + residual);
 *                           input = fp16(residual * rsqrt(mean((input + residual)^2) + epsilon)) * weight */
int ca_rms_norm(void* out, const void* input, const void* weight, float epsilon, int64_t n_tokens,
                int hidden_size, void* stream);
int ca_fused_add_rms_norm(void* input, void* residual, const void* weight, float epsilon,
                          int64_t n_tokens, int hidden_size, void* stream);

/* The decode step of the reference's attention layer
 * (src/chunk_attn/models/llama_hf/modeling_llama.py:62,91-95: rotary_embedding on the new
 * query/key rows, then append_token -> append_kv) as one launch: q [n_seqs, n_heads, d_head]
 * is rotated in place, k is rotated on its way into the free row of each sequence's last
 * chunk (k itself is left untouched), v is copied beside it.  positions_dev may be NULL: the
 * position of a sequence is then its current length, seq_len + delta_tokens, checked against
 * max_position on the host.  Same preconditions and delta_tokens behaviour as ca_append_kv;
 * rot_dim must be a multiple of 16 (NeoX) or 8 (GPT-J) and at most d_head. */
int ca_rope_append_kv(ca_ctx* ctx, const int64_t* positions_dev, void* q, const void* k,
                      const void* v, const void* cos_sin_cache, int max_position, int rot_dim,
                      int is_neox, int n_seqs, void* stream);

/* Copy-in of an inserted sequence's K/V (what the reference does with two tensor slice
 * assignments per chunk, cpp/chunk_attn/chunk.cpp:63-72): token rows
 * [tok_begin, tok_begin + n_slots*chunk_size) clipped to n_tokens go to the listed chunks,
 * chunk_size rows each, starting at row 0.  k, v: [n_tokens, n_heads, d_head]. */
int ca_scatter_kv(ca_ctx* ctx, const void* k, const void* v, int n_tokens, int tok_begin,
                  const int32_t* slots, int n_slots, void* stream);

/* Device copy of one chunk's K and V (reference Chunk::deep_copy, chunk.cpp:93-107). */
int ca_copy_chunk(ca_ctx* ctx, int src_slot, int dst_slot, void* stream);
/* The same for n_pairs chunks in one launch (per 64 pairs): chunk src_dst[2i] is copied onto chunk
 * src_dst[2i+1] in both pools (host array; what the loops over deep_copy in reference
 * Attention::duplicate and append_completion do, attention.cpp:227-261,287-313).  No destination
 * may be the source or the destination of another pair (CA_ERR_INVALID). */
int ca_copy_chunks(ca_ctx* ctx, const int32_t* src_dst, int n_pairs, void* stream);

/* K/V rows to explicit places, one launch: row i of k and v ([n_rows, n_heads, d_head] on the
 * device) goes to row slot_row[2i+1] of chunk slot_row[2i] (host array).  The device half of the
 * row appends in reference Attention::append_completion (attention.cpp:243,253 ->
 * Chunk::append_tokens, chunk.cpp:63-72: one tensor slice assignment per candidate and pool). */
int ca_put_kv_rows(ca_ctx* ctx, const void* k, const void* v, int n_rows, const int32_t* slot_row,
                   void* stream);

/* ca_copy_chunks followed by ca_put_kv_rows -- the whole device half of one beam-search step
 * (reference Attention::append_completion, attention.cpp:227-261: deep copies of the last chunk,
 * then one row per candidate) -- with the result of making the copies first and the row writes
 * second.  One launch when the written rows can be left out of the copies (always in a beam
 * step: every candidate's row has the same index in its own copy of the chunk), two otherwise. */
int ca_copy_chunks_put_rows(ca_ctx* ctx, const int32_t* src_dst, int n_pairs, const void* k,
                            const void* v, int n_rows, const int32_t* slot_row, void* stream);

/* Work-list shaping.  0 = choose from the device's compute-unit count and the step's size.
 * shared_seg_chunks = 1 gives one partial row set per shared chunk, the granularity of the
 * reference's partial buffers.  A work item never holds more than 64 chunks: larger values are
 * cut down to that (63 for stream_chunks, whose last item may take one chunk more). */
int ca_ctx_set_plan(ca_ctx* ctx, int shared_seg_chunks, int stream_chunks);

/* How the private (per-sequence) chunks are read.  0 (default): with the non-temporal hint when
 * one forward attends more K/V than the 256 MiB last-level cache holds, plainly otherwise (a
 * caller that repeats forwards over a small cache finds part of it there again).  1: always with
 * the hint -- for a model whose layers each own a cache, so that nothing attended is still cached
 * when its layer comes round again.  2: never.  Results do not depend on it.  No counterpart in
 * the reference (its kernels use plain loads, kernel_cuda.cu:885-1086). */
int ca_ctx_set_stream_hint(ca_ctx* ctx, int mode);

/* Re-planning policy for long decodes.  ca_ctx_roll_tails keeps the work-item sizes (length of a
 * shared segment, of a stream item) that the last full build derived from the size of the step, so
 * that patched and rebuilt tables are the same tables; the reference rebuilds everything at every
 * roll-over instead (kernel_cuda.cu:1331-1445) and its tables never drift.  Once the tokens one
 * forward attends differ by more than `percent` per cent from what they were at the last full
 * build, ca_ctx_roll_tails rebuilds from its own rows (sizes derived afresh) instead of patching.
 * Default 25; 0: never.  ca_ctx_table_stats counts both kinds since the context was created. */
int ca_ctx_set_replan(ca_ctx* ctx, int percent);
int ca_ctx_table_stats(const ca_ctx* ctx, int64_t* full_builds, int64_t* patches);

/* How ca_attention is launched.  0 (default): one launch in which chunk-first and sequence-
 * first workgroups run side by side and write partial rows, then a merge launch.  1: a single
 * launch in which the workgroup that finishes the last partial of a (sequence, head) merges
 * them (completion counters; usually slower, kept for callers that need one launch). */
int ca_ctx_set_schedule(ca_ctx* ctx, int mode);

/* Timing of ca_attention with HIP events recorded on the stream the kernels are launched on
 * (the reference marks its phases with NVTX ranges, kernel_cuda.cu:1334-1433).
 * mode 0: off.  mode 1: ca_attention runs as it normally does with events around its launches;
 * ca_ctx_read_timing returns the accumulated milliseconds of the decode launch in *shared_ms
 * and of the merge launch in *merge_ms (*stream_ms stays 0).  mode 2: ca_attention runs as
 * three separately timed launches (chunk-first, sequence-first, merge) and the three
 * accumulators are filled; for phase analysis, slower than the normal forward.  Every mode
 * writes the complete output. */
int ca_ctx_set_timing(ca_ctx* ctx, int mode);
int ca_ctx_read_timing(ca_ctx* ctx, double* shared_ms, double* stream_ms, double* merge_ms,
                       int64_t* calls, int reset);

/* Named ranges around table refreshes, table patches, attention calls and K/V appends in a
 * profiler's marker trace (rocprofv3 --marker-trace), where the reference has NVTX ranges
 * (kernel_cuda.cu:1334-1433).  Process-wide, off by default.  Enabling loads the roctx library
 * at run time; CA_ERR_STATE when none is found. */
int ca_set_markers(int enable);

/* Numbers describing the current tables. */
typedef struct ca_plan_info {
    int32_t n_seqs;
    int32_t n_chunks;           /* rows given to the last refresh */
    int32_t n_shared_chunks;    /* reference n_shared_chunks */
    int32_t ref_partial_rows;   /* reference partial_attn_dim (sum of n over shared chunks) */
    int32_t max_seq_n_chunks;   /* width of the reference seq_chunk_map */
    int32_t n_shared_items;
    int32_t n_stream_items;
    int32_t n_part_rows;
    int64_t shared_tokens;      /* physical tokens attended chunk-first */
    int64_t stream_tokens;      /* tokens streamed per sequence (when the tables were built) */
    int32_t stream_per_wave;    /* 1: stream items run one per wave, four per workgroup (many short runs) */
    int32_t reserved;
} ca_plan_info;
int ca_ctx_plan_info(const ca_ctx* ctx, ca_plan_info* info);

/* Reference-form tables of the last refresh, copied into caller buffers (NULL = skip):
 *   final_idx [n_chunks], slots [n_chunks], begins/ends/offsets [n_shared_chunks],
 *   seq_n_tokens [n_seqs], seq_chunk_map [n_seqs * max_seq_n_chunks] (-1 = unwritten). */
int ca_ctx_ref_tables(const ca_ctx* ctx, int32_t* final_idx, int32_t* slots, int32_t* begins,
                      int32_t* ends, int32_t* offsets, int32_t* seq_n_tokens,
                      int32_t* seq_chunk_map);

/* Copies the chunk-first partials to host buffers in the reference's layout
 * (kernel_cuda.cu:830-838): for shared chunk i with n covered sequences and row offset
 * off = offsets[i]:  maxs/sums[off*H + h*n + r], attns[(off*H + h*n + r)*d ...], maxima in
 * natural-log units of score/sqrt(d).  Needs tables built with shared_seg_chunks = 1 and
 * partition 0.  Synchronises the stream. */
int ca_ctx_export_partials(ca_ctx* ctx, float* maxs, float* sums, float* attns, void* stream);

/* Raw copy of the partial-row buffer ([n_part_rows][n_heads][160] floats: max, sum, 2 unused,
 * 128 acc in base-2 units, 28 unused) to the host, for inspection.  Synchronises the stream. */
int ca_ctx_read_partials_raw(ca_ctx* ctx, float* out, int64_t n_floats, void* stream);

/* ---- measurement aids: for benchmarks, not for callers --------------------------------- */

/* Parts of a forward launched alone so that a benchmark can time a back-to-back train of them
 * between two events of its own.  The output is NOT complete afterwards (sequences whose output
 * needs the merge launch get none).  what 0: the decode launch without the merge launch; 1: only
 * its sequence-first workgroups (the stream items); 2: only its chunk-first workgroups.  Needs
 * tables of partition 0 in the default schedule; never rebuilds them.  No counterpart in the
 * reference. */
int ca_bench_decode_launch(ca_ctx* ctx, const void* q, void* out, int n_seqs, int what, void* stream);

/* One launch on `stream` that reads `bytes` of device memory at `dev` (16-byte aligned, at least 16
 * bytes) with non-temporal 16-byte loads, wgs_per_cu (1 .. 8) workgroups of 256 threads per compute
 * unit, eight loads per lane in flight, and keeps nothing: the read rate a kernel with no structure
 * reaches on this GPU, for benchmarks to quote beside the published peak.  No counterpart in the
 * reference. */
int ca_bench_read_probe(ca_ctx* ctx, const void* dev, size_t bytes, int wgs_per_cu, void* stream);

/* ---- host-only table builder (no device needed) ---------------------------------------- */

/* The flattening ca_refresh_kernel_context performs, exposed for structure checks: builds
 * the reference-form tables (kernel_cuda.cu:1331-1445) and the packed work list from the
 * rows, entirely on the host. */
typedef struct ca_tables ca_tables;

/* One unit of kernel work (see csrc/tables.h). */
typedef struct ca_work_item {
    int32_t seq_begin, n_rows, slot_first, n_chunks, part_row, pos0, len0, flags;
    int32_t inl[8]; /* slots of the item's first chunks */
} ca_work_item;

int ca_tables_build(ca_tables** out, const ca_chunk_row* rows, int n_rows, int n_seqs,
                    int chunk_size, int tpp_threshold, int partition, int shared_seg_chunks,
                    int stream_chunks, int n_heads, int n_cus);
/* the same for other rows, reusing the work-item sizes `like` was built with instead of deriving
 * them from the new rows (what a patched table keeps), and `like`'s other parameters */
int ca_tables_build_like(ca_tables** out, const ca_tables* like, const ca_chunk_row* rows,
                         int n_rows, int n_seqs);
/* host half of ca_ctx_roll_tails on a built table set (the reference-form tables are not patched) */
int ca_tables_roll_tails(ca_tables* t, int delta_tokens, const int32_t* seq_idx,
                         const int32_t* new_slots, int n);
/* 1 when the policy of ca_ctx_set_replan would rebuild these tables: the tokens they attend, plus
 * extra_tokens appended since, differ from those at their (last full) build by more than percent */
int ca_tables_stale(const ca_tables* t, int percent, int64_t extra_tokens);
void ca_tables_destroy(ca_tables* t);
/* sizes: fills the same struct ca_ctx_plan_info fills */
int ca_tables_info(const ca_tables* t, ca_plan_info* info);
/* length of the plan's slot list */
int ca_tables_plan_sizes(const ca_tables* t, int* n_slots);
/* reference-form tables, same buffers as ca_ctx_ref_tables */
int ca_tables_ref(const ca_tables* t, int32_t* final_idx, int32_t* slots, int32_t* begins,
                  int32_t* ends, int32_t* offsets, int32_t* seq_n_tokens, int32_t* seq_chunk_map);
/* packed plan: shared_items [n_shared_items], stream_items [n_stream_items], slots [n_slots],
 * seq_len / tail_slot / tail_fill [n_seqs], part_ptr [n_seqs + 1] (sequence s owns partial
 * rows part_ptr[s] .. part_ptr[s+1]-1; an item writes row part_ptr[seq] + item.part_row) */
int ca_tables_plan(const ca_tables* t, ca_work_item* shared_items, ca_work_item* stream_items,
                   int32_t* slots, int32_t* seq_len, int32_t* part_ptr, int32_t* tail_slot,
                   int32_t* tail_fill);

/* ---- prefix-tree chunk manager -------------------------------------------------------- */

typedef struct ca_tree ca_tree;

/* reference Attention's tree state + ChunkAllocator (attention.cpp:8-37,
 * chunk_allocator.cpp:8-56), without tensors. */
int ca_tree_create(ca_tree** out, int chunk_size, int max_chunks, int share_prefix);
void ca_tree_destroy(ca_tree* tree);
/* reference ChunkAllocator's capacity rule (chunk_allocator.cpp:32-35). */
int ca_tree_max_chunks_for(int memory_mb, int chunk_size, int n_heads, int d_head,
                           int elem_bytes);

/* reference Attention::add_seq (attention.cpp:141-193).  *seq_idx: index the sequence was
 * inserted at.  new_slots (capacity cap) receives the slots of the chunks that need K/V
 * copied in, in order; they hold tokens [*tok_begin, n_tokens).  *n_new may exceed cap, in
 * which case only cap entries were written. */
int ca_tree_add_seq(ca_tree* tree, const int32_t* tokens, int n_tokens, int* seq_idx,
                    int* tok_begin, int32_t* new_slots, int cap, int* n_new);
/* reference Attention::remove_seq (attention.cpp:263-278) */
int ca_tree_remove_seq(ca_tree* tree, int seq_idx);
int ca_tree_clear(ca_tree* tree);
/* reference Attention::reserve (attention.cpp:116-131); *n_new = chunks added */
int ca_tree_reserve(ca_tree* tree, int* n_new);
/* ca_tree_reserve that also reports, for each chunk added (up to cap), the index of the sequence
 * it became the last chunk of and its slot: the arguments of ca_ctx_roll_tails */
int ca_tree_reserve_tails(ca_tree* tree, int32_t* seq_idx, int32_t* new_slots, int cap, int* n_new);
/* host half of reference Attention::append_token (attention.cpp:80-114): reserve, then
 * record one token id per sequence.  Returns *n_new like ca_tree_reserve. */
int ca_tree_append_token(ca_tree* tree, const int32_t* tokens, int n_tokens, int* n_new);
/* reference Attention::get_chunks (attention.cpp:342-372).  Writes up to cap rows and
 * returns the total number of rows in *n_rows. */
int ca_tree_get_chunks(const ca_tree* tree, ca_chunk_row* rows, int cap, int* n_rows);
int ca_tree_n_seqs(const ca_tree* tree);
int ca_tree_used_chunks(const ca_tree* tree);
uint64_t ca_tree_version(const ca_tree* tree);
/* Tree half of reference Attention::duplicate (attention.cpp:287-313): `copies` more sequences
 * identical to seq_idx, inserted right after it (indices seq_idx+1 ..).  Every new sequence
 * shares the path and owns a copy of the tail chunk: copy_pairs (capacity cap_pairs >= copies
 * pairs) receives (source slot, destination slot) per copy, for ca_copy_chunk.  Unlike the
 * reference, the tail list is updated as well. */
int ca_tree_duplicate(ca_tree* tree, int seq_idx, int copies, int32_t* copy_pairs, int cap_pairs,
                      int* n_pairs);
/* Tree half of reference Attention::append_completion (attention.cpp:227-261), one beam-search
 * step: candidate 0 continues sequence seq_idx with tokens[0]; candidates 1 .. n_tokens-1 become
 * copies of its tail right after it, each continued with its own token.  copy_pairs (capacity
 * cap_pairs >= n_tokens - 1) receives the (source, destination) slots to copy first; targets
 * [n_tokens][2] receives (slot, row) where candidate i's K/V row belongs (sequence seq_idx + i).
 * Unlike the reference, sequence counts and the tail list stay consistent, and a full tail gets
 * its empty child first instead of tripping an assertion. */
int ca_tree_append_completion(ca_tree* tree, int seq_idx, const int32_t* tokens, int n_tokens,
                              int32_t* copy_pairs, int cap_pairs, int* n_pairs, int32_t* targets);
/* slot of the tail chunk of every sequence, in sequence order (reference tails()) */
int ca_tree_tails(const ca_tree* tree, int32_t* slots, int cap, int* n);
/* Pre-order dump (children first-to-last) of the whole tree for structure checks: per node
 * 4 ints (depth, n_seqs, n_tokens, slot; the root has slot -1) and its tokens appended to
 * `tokens`.  Returns counts in *n_nodes / *n_tokens; writes at most the given capacities. */
int ca_tree_dump(const ca_tree* tree, int32_t* nodes, int node_cap, int* n_nodes,
                 int32_t* tokens, int token_cap, int* n_tokens);

#ifdef __cplusplus
}
#endif
#endif /* CHUNK_ATTN_HIP_H */
