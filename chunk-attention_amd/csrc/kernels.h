// Launch interface between the C-ABI context (host code) and the HIP kernels.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "tables.h"

namespace ca {

constexpr int PART_STRIDE = 160;  // floats per partial row: max, sum, 2 pad, 128 acc, pad to 5 x 128 B

struct LaunchArgs {
    const void* q = nullptr;      // [n_seqs, H, 128] fp16
    void* out = nullptr;          // [n_seqs, H, 128] fp16
    const void* kpool = nullptr;  // [max_chunks, H, C, 128] fp16
    const void* vpool = nullptr;
    float* part = nullptr;        // [n_part_rows, H, PART_STRIDE]
    const WorkItem* shared_items = nullptr;
    const WorkItem* stream_items = nullptr;
    const int32_t* slots = nullptr;
    const int32_t* part_ptr = nullptr;
    int32_t* counters = nullptr;  // [n_seqs * H], zero between launches
    int delta_tokens = 0;
    int H = 0;
    int C = 0;
    int d = 128;
    float scale_log2 = 0.f;  // log2(e) / sqrt(d_head)
    // Read the per-sequence (private) chunks with the non-temporal hint.  Worth it when one
    // forward streams more than the last-level cache holds: the data cannot be found there
    // again, and without the hint it only displaces what could be.
    bool stream_nt = false;
    // Every wave of a stream workgroup takes a stream item of its own (four consecutive items per
    // workgroup): set by the plan when there are many short runs.  Not with fuse_merge.
    bool stream_per_wave = false;
    // No shared item of the work list covers more than 16 sequences and none is wide: the launch
    // can take the form of the kernel without the 32-row and wide matrix-core paths.
    bool shared_narrow = false;
    // Fused decode step: rows [n_seqs, H, 128] of the token appended by this step (delta_tokens
    // already counts it).  The decode launch attends them from here, the merge launch writes them
    // into the pool.  Needs a work list in which every sequence's last chunk is streamed.
    const void* k_new = nullptr;
    const void* v_new = nullptr;
    const int32_t* tail_slot = nullptr;  // device tables: slot of every sequence's last chunk and the
    const int32_t* tail_fill = nullptr;  // tokens it held when the plan was built (fused step's row writes)
};

// Static device scratch for the entry point that allocates nothing: a file-scope __device__
// array (kScratchBytes per GPU, held until the process ends) that stands in for the partial-row
// buffer.  scratch_setup resolves its address on `device`, which must be the current device
// (every GPU has its own copy at its own address); scratch_ptr returns what it found, or null.
constexpr size_t kScratchBytes = size_t(32) << 20;
int scratch_setup(int device);   // 0 or a positive hipError_t
float* scratch_ptr(int device);
// 16 bytes of device memory of its own for the read probe's never-taken store (resolved by
// scratch_setup as well)
void* probe_sink_ptr(int device);

// All return 0, -1 for an unsupported shape, or a positive hipError_t.
// One launch over the first n_shared_items shared items and the first n_stream_items stream
// items.  fuse_merge: the workgroup finishing the last partial of a (sequence, head) writes
// its output; otherwise only partial rows (and direct outputs) are written.
int launch_decode(const LaunchArgs& a, int n_shared_items, int n_stream_items, bool fuse_merge,
                  hipStream_t st);
// The second launch of a forward: merges the partial rows of every (sequence, head) when `merge`,
// and, for a fused decode step (a.k_new set), writes the step's new K/V rows into the pool
// (a.tail_slot / a.tail_fill, row tail_fill + delta_tokens - 1).
int launch_merge(const LaunchArgs& a, int n_seqs, bool merge, hipStream_t st);
int launch_fill(int32_t* p, int n, int32_t value, hipStream_t st);
// Copies `bytes` (a multiple of 16) from pinned host memory to device memory with a kernel on
// `st`.  For the table upload: a copy-engine transfer in the middle of a decode step costs the
// stream several microseconds of hand-over between queues, a small kernel does not.
int launch_upload(void* dst_dev, const void* src_pinned, size_t bytes, hipStream_t st);
// Measurement aid: n_wgs workgroups read `bytes` of device memory (from a 16-byte aligned
// address) with non-temporal 16-byte loads and keep nothing; `sink` is 4 writable bytes of
// device memory.
int launch_read_probe(const void* dev, size_t bytes, int n_wgs, void* sink, hipStream_t st);
int launch_append(const LaunchArgs& a, const void* k, const void* v, const int32_t* tail_slot,
                  const int32_t* tail_fill, int n_seqs, hipStream_t st);
int launch_scatter(const LaunchArgs& a, const void* k, const void* v, int n_tokens, int tok_begin,
                   const int32_t* slots, int n_slots, hipStream_t st);
// chunk src_dst[2i] of both pools copied onto chunk src_dst[2i+1], i < n_pairs (host array), one
// launch per 64 pairs; the pairs must not overlap.  With n_rows > 0 (at most 64) the same launch
// also does what launch_put_rows does for rows i < n_rows of k / v; the token rows it writes are
// left out of the copies (at most two different rows per pair), so the caller makes sure that a
// written row of a source chunk is written in the destination chunk too.
int launch_copy_chunks(const LaunchArgs& a, const int32_t* src_dst, int n_pairs, const void* k, const void* v,
                       const int32_t* slot_row, int n_rows, hipStream_t st);
// rows i < n of k/v ([n, H, d]) to row slot_row[2i+1] of chunk slot_row[2i] (host array)
int launch_put_rows(const LaunchArgs& a, const void* k, const void* v, const int32_t* slot_row, int n,
                    hipStream_t st);

// Rotary position embedding (fp16).  cos_sin_cache is [max_position, rot_dim]: rot_dim/2 cosines
// then rot_dim/2 sines per position; positions outside the cache are clamped into it.
struct RotaryArgs {
    const int64_t* positions = nullptr;  // device, one per token; may be null for launch_rope_append
    void* query = nullptr;               // rotated in place
    void* key = nullptr;                 // rotated in place (launch_rotary only; may be null with n_kv_heads 0)
    const void* cos_sin_cache = nullptr;
    int64_t n_tokens = 0;
    int n_heads = 0, n_kv_heads = 0, head_size = 0, rot_dim = 0, max_position = 0;
    int64_t query_stride = 0, key_stride = 0;  // elements between consecutive tokens
    bool is_neox = true;
};
int launch_rotary(const RotaryArgs& r, hipStream_t st);
// One launch for a decode step's new rows: r.query ([n_seqs, H, d]) is rotated in place, k is
// rotated on its way into the free row of each sequence's last chunk, v is copied beside it.
// The position of sequence s is r.positions[s] or, when that is null, seq_len[s] + delta_tokens.
int launch_rope_append(const LaunchArgs& a, const RotaryArgs& r, const void* k, const void* v,
                       const int32_t* seq_len, const int32_t* tail_slot, const int32_t* tail_fill,
                       int n_seqs, hipStream_t st);

// RMS normalisation of fp16 rows ([n_tokens, hidden], contiguous).  residual == nullptr:
// out = norm(input) * weight.  Otherwise the fused form: residual += input (rounded to fp16),
// input = norm(residual) * weight, `out` unused.  vec8: hidden % 8 == 0 and all pointers 16-byte
// aligned.
int launch_rms_norm(void* out, void* input, void* residual, const void* weight, float epsilon,
                    int64_t n_tokens, int hidden, bool vec8, hipStream_t st);

}  // namespace ca
