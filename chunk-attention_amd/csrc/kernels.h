// Launch interface between the C-ABI context (host code) and the HIP kernels.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "tables.h"

namespace ca {

constexpr int PART_STRIDE = 132;  // floats per partial row: max, sum, 2 pad, 128 acc

struct LaunchArgs {
    const void* q = nullptr;      // [n_seqs, H, 128] fp16
    void* out = nullptr;          // [n_seqs, H, 128] fp16
    const void* kpool = nullptr;  // [max_chunks, H, C, 128] fp16
    const void* vpool = nullptr;
    float* part = nullptr;        // [n_part_rows, H, PART_STRIDE]
    const int32_t* slots = nullptr;
    const int32_t* seq_len = nullptr;
    int delta_tokens = 0;
    int H = 0;
    int C = 0;
    int d = 128;
    float scale_log2 = 0.f;  // log2(e) / sqrt(d_head)
};

// All return 0, -1 for an unsupported shape, or a positive hipError_t.
int launch_stream(const LaunchArgs& a, const WorkItem* items, int n_items, hipStream_t st);
// mb: 16-row blocks per item (1, 2 or 4); every item of the launch has n_rows <= 16*mb
int launch_shared(const LaunchArgs& a, const WorkItem* items, int n_items, int mb, hipStream_t st);
int launch_merge(const LaunchArgs& a, const int32_t* part_ptr, const int32_t* part_rows,
                 int n_seqs, hipStream_t st);
int launch_append(const LaunchArgs& a, const void* k, const void* v, const int32_t* tail_slot,
                  const int32_t* tail_fill, int n_seqs, hipStream_t st);
int launch_scatter(const LaunchArgs& a, const void* k, const void* v, int n_tokens, int tok_begin,
                   const int32_t* slots, int n_slots, hipStream_t st);

}  // namespace ca
