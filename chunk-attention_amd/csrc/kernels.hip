// HIP kernels of the ChunkAttention decode path for gfx950 (MI355X), fp16 K/V/Q, d_head 128.
//
//   decode_kernel   one launch for a whole forward.  Its first workgroups run the chunk-first
//                   phase (shared_path): a segment of shared chunks is attended for up to 32
//                   sequences at once on the matrix cores (S^T = K.Q^T, O^T = V^T.P^T), one
//                   partial (max, sum, acc) row per sequence.  The others run the sequence-
//                   first phase (stream_path): a run of one sequence's own chunks is streamed
//                   at HBM speed (16-byte coalesced loads, fp32 online softmax) into one
//                   partial row, or straight into the output when nothing else is merged.
//                   Chunks covering many sequences (from about 100 on, and from 33 on in long
//                   shared runs: the work list says which) take the row-split wide_path.
//   merge_kernel    merges the partial rows of every (sequence, head) and writes the normalised
//                   output: the second launch of a forward.  (In the single-launch schedule the
//                   decode workgroup that completes the last partial of a (sequence, head) does
//                   this merge itself.)
//   append_kernel / scatter_kernel / put_rows_kernel   K/V row writes into the chunk pool.
//
// Partial rows live in base-2 units: max holds score*log2(e)/sqrt(d), sums and acc are
// relative to 2^max.  Row layout: [0] max, [1] sum, [4..131] acc (fp32); rows are 640 B apart so
// that no 128-byte line holds data of two writers.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>
#include <type_traits>

#include "kernels.h"

namespace ca {
namespace {

typedef _Float16 half_t;
typedef half_t h2 __attribute__((ext_vector_type(2)));
typedef half_t h4 __attribute__((ext_vector_type(4)));
typedef half_t h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

constexpr int D = 128;                 // d_head
constexpr int WG = 256;                // threads per workgroup (4 wavefronts of 64)
constexpr int NW = WG / 64;
constexpr float NEG_INF = -__builtin_huge_valf();

// Debug builds only (-DCA_TIMELINE): every workgroup of the decode launch leaves four stamps of the
// device's 100 MHz clock -- start, first K/V data consumed, end -- and its kind, read back through
// ca_debug_timeline.  Never compiled into the library that ships.
#ifdef CA_TIMELINE
__device__ unsigned long long ca_timeline[65536 * 4];
#define CA_STAMP(slot) do { if (threadIdx.x == 0) ca_timeline[(blockIdx.x & 65535) * 4 + (slot)] = wall_clock64(); } while (0)
#define CA_STAMP_VALUE(slot, v) do { if (threadIdx.x == 0) ca_timeline[(blockIdx.x & 65535) * 4 + (slot)] = (v); } while (0)
#else
#define CA_STAMP(slot) do {} while (0)
#define CA_STAMP_VALUE(slot, v) do {} while (0)
#endif

__device__ __forceinline__ float shfl_xor(float v, int mask) { return __shfl_xor(v, mask, 64); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, shfl_xor(v, m));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += shfl_xor(v, m);
    return v;
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Partial rows are written by one workgroup and read by another, possibly on a different XCD
// whose L2 is not coherent with the writer's.  When both happen in one launch (single-launch
// schedule) they are therefore moved with device-scope relaxed atomics (write-through stores,
// L2-bypassing loads): no cache-wide fence is needed, only "stores done" (a workgroup barrier)
// before the completion counter is bumped.
// Before a workgroup announces its partial rows through the completion counter, every wave
// waits until its own stores have been acknowledged: a workgroup barrier alone orders waves
// but does not wait for their outstanding global stores.
__device__ __forceinline__ void wait_own_stores() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) expcnt(0) lgkmcnt(0)
}
// coherent = the rows are read during this launch (single-launch schedule).  When a later launch
// reads them, ordinary stores do: the end of the launch makes them visible, and they leave the L2
// as whole lines instead of being written through 8 bytes at a time.
__device__ __forceinline__ void part_store(float* p, float v, bool coherent) {
    if (coherent) {
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        *p = v;
    }
}
__device__ __forceinline__ void part_store2(float* p, float a, float b, bool coherent) {
    if (coherent) {
        union { f2 f; uint64_t u; } x;
        x.f = f2{ a, b };
        __hip_atomic_store(reinterpret_cast<uint64_t*>(p), x.u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        *reinterpret_cast<f2*>(p) = f2{ a, b };
    }
}
__device__ __forceinline__ float part_load(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ f2 part_load2(const float* p) {
    union { f2 f; uint64_t u; } x;
    x.u = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return x.f;
}

typedef unsigned int u4v __attribute__((ext_vector_type(4)));
// 16-byte load with the non-temporal hint: K/V rows are read once and should not displace
// what the caches hold.
__device__ __forceinline__ uint4 nt_load16(const uint4* p) {
    const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}

// LDS transpose read (gfx950): within each group of 16 lanes, lane L supplies the address of four
// consecutive halves; with lane L pointing at row L/4, columns 4*(L%4).. of a 4 x 16 patch, lane i
// receives column i of the patch (rows 0..3).  That is the V^T operand of the matrix cores,
// lane (i = dim, g = token group), straight from a row-major V tile.
__device__ __forceinline__ h4 lds_read_tr(const half_t* p) {
    // p points into LDS: the cast narrows the generic pointer to the LDS address space
    typedef short s4v __attribute__((ext_vector_type(4)));
    const s4v raw = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4v __attribute__((address_space(3)))*)p);
    return __builtin_bit_cast(h4, raw);
}

__device__ __forceinline__ float dot8(const h8& a, const h8& b, float acc) {
    acc = __builtin_amdgcn_fdot2(h2{ a[0], a[1] }, h2{ b[0], b[1] }, acc, false);
    acc = __builtin_amdgcn_fdot2(h2{ a[2], a[3] }, h2{ b[2], b[3] }, acc, false);
    acc = __builtin_amdgcn_fdot2(h2{ a[4], a[5] }, h2{ b[4], b[5] }, acc, false);
    acc = __builtin_amdgcn_fdot2(h2{ a[6], a[7] }, h2{ b[6], b[7] }, acc, false);
    return acc;
}

// NV values per lane, one per 4-row group; the 16 lanes of a row group each hold a partial
// dot product of the same NV rows.  Returns, in lane j of each group, the full sum for value
// index (j % NV): a halving butterfly, so NV-1 (+ log2(16/NV)*NV) shuffles instead of 4*NV.
template <int NV>
__device__ __forceinline__ float reduce_rows16(float (&v)[NV], int j) {
    static_assert(NV == 16 || NV == 8, "row groups of 8 or 16 loads");
    if constexpr (NV == 8) {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] += shfl_xor(v[i], 8);
    }
    if constexpr (NV == 16) {
        const bool up = j & 8;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float send = up ? v[i] : v[i + 8];
            const float keep = up ? v[i + 8] : v[i];
            v[i] = keep + shfl_xor(send, 8);
        }
    }
    {
        const bool up = j & 4;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float send = up ? v[i] : v[i + 4];
            const float keep = up ? v[i + 4] : v[i];
            v[i] = keep + shfl_xor(send, 4);
        }
    }
    {
        const bool up = j & 2;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const float send = up ? v[i] : v[i + 2];
            const float keep = up ? v[i + 2] : v[i];
            v[i] = keep + shfl_xor(send, 2);
        }
    }
    {
        const bool up = j & 1;
        const float send = up ? v[0] : v[1];
        const float keep = up ? v[1] : v[0];
        v[0] = keep + shfl_xor(send, 1);
    }
    return v[0];
}

// ---------------------------------------------------------------------------------------
// Every wave fetches the slot ids of its item's chunks (at most 64: kMaxItemChunks) with one
// load, chunk k into lane k, when it starts.  Looking a slot up in memory right before the
// chunk's K/V loads would put a dependent round trip in front of every tile, and waiting for
// that load (the counter of outstanding loads is in-order) would also wait for every K/V load
// issued before it.  chunk_slot reads the id back from the register.
__device__ __forceinline__ int preload_slots(const WorkItem* __restrict__ gi, int slot_first, int n_chunks,
                                             const int32_t* __restrict__ slots, int lane) {
    // the item's inline slots do not wait for the item's header: they arrive with it
    int v = 0;
    if (lane < kInlineSlots) {
        v = gi->inl[lane];
    } else if (lane < n_chunks) {
        v = slots[slot_first + lane];
    }
    return v;
}
// k < 64, the same in every lane of the wave.
__device__ __forceinline__ int chunk_slot(int slotv, int k) { return __builtin_amdgcn_readlane(slotv, k); }

// Everything a workgroup needs besides its work item.
struct DecodeArgs {
    const half_t* q;
    const half_t* kpool;
    const half_t* vpool;
    half_t* out;
    float* part;
    const WorkItem* shared_items;
    const WorkItem* stream_items;
    const int32_t* slots;
    const int32_t* part_ptr;  // sequence s owns partial rows part_ptr[s] .. part_ptr[s+1]-1
    int32_t* counters;  // [n_seqs * H] partial rows completed so far, 0 between launches
    int n_shared_wgs;   // workgroups [0, n_shared_wgs) run shared items
    int delta_tokens;
    int H;
    float scale_log2;
    int fuse_merge;  // 1: the last workgroup to finish a (sequence, head) merges its partials
    int n_stream_items;   // stream items in the list
    int stream_per_wave;  // 1: every wave of a stream workgroup takes an item of its own (needs fuse_merge 0)
    int stream_nt;   // 1: private chunks are read with the non-temporal hint (see LaunchArgs)
    // Fused decode step (STEP kAppend): the newest token of every sequence, [n_seqs, H, D].
    // delta_tokens already counts it; its row in the pool is written by the merge launch.
    const half_t* k_new;
    const half_t* v_new;
};

// Decode launches come in two kinds.  kForward: attention over what the pool holds.  kAppend:
// the fused decode step (see stream_path).
constexpr int kForward = 0, kAppend = 1;

// Wave-level merge of the partial rows p0 .. p1-1 of one (sequence, head): lane l owns output
// dims 2l, 2l+1.  Rows are taken NB at a time with all their loads in flight together and
// folded with a running maximum, so a typical merge costs one memory round trip (NB = 16 in the
// merge launch, 8 inside the decode launch, where registers are scarce).
// COHERENT: rows may have been written during this launch by other workgroups (device-scope
// loads); otherwise they come from an earlier launch and plain loads do.
template <bool COHERENT, int NB = 8>
__device__ __forceinline__ void merge_rows(const float* __restrict__ part, int p0, int p1, int h,
                                           int H, half_t* __restrict__ out_row, int l) {
    float m_run = NEG_INF, lsum = 0.f;
    f2 o = f2{ 0.f, 0.f };
    for (int pb = p0; pb < p1; pb += NB) {
        f2 ml[NB], v[NB];
#pragma unroll
        for (int u = 0; u < NB; u++) {
            ml[u] = f2{ NEG_INF, 0.f };
            v[u] = f2{ 0.f, 0.f };
            if (pb + u < p1) {
                const float* r = part + (size_t(pb + u) * H + h) * PART_STRIDE;
                if constexpr (COHERENT) {
                    ml[u] = part_load2(r);
                    v[u] = part_load2(r + 4 + 2 * l);
                } else {
                    ml[u] = *reinterpret_cast<const f2*>(r);
                    v[u] = *reinterpret_cast<const f2*>(r + 4 + 2 * l);
                }
            }
        }
        float mb = m_run;
#pragma unroll
        for (int u = 0; u < NB; u++) mb = fmaxf(mb, ml[u][0]);
        if (mb == NEG_INF) continue;  // nothing but empty rows so far
        const float fa = (m_run == NEG_INF) ? 0.f : fast_exp2(m_run - mb);
        o *= fa;
        lsum *= fa;
        m_run = mb;
#pragma unroll
        for (int u = 0; u < NB; u++) {
            const float w = (ml[u][0] == NEG_INF) ? 0.f : fast_exp2(ml[u][0] - mb);
            o += w * v[u];
            lsum += w * ml[u][1];
        }
    }
    const float r = lsum > 0.f ? 1.f / lsum : 0.f;
    *reinterpret_cast<h2*>(out_row + 2 * l) = h2{ half_t(o[0] * r), half_t(o[1] * r) };
}

// LDS of one workgroup, shared by the two paths.
constexpr int VPITCH = D + 16;  // halves per LDS row of a V block: 288 B puts the 32-byte pieces of
                                // four consecutive token rows into four different bank groups,
                                // and rows stay 16-byte aligned for whole-vector writes
constexpr int OPITCH = D + 4;  // floats per row of the cross-wave accumulation buffer
// MBT: 16-row blocks per shared item (2: items of up to 32 sequences, 1: up to 16)
template <int MBT>
struct SharedPathLds {
    half_t v[NW][16 * VPITCH];
    float o[16 * MBT * OPITCH];
    float m[NW][16 * MBT];
    float l[NW][16 * MBT];
    int last[16 * MBT];
    int row[16 * MBT];  // partial row of each covered sequence
};
struct StreamPathLds {
    float p[NW][64];
    float o[NW][D];
    float m[NW];
    float l[NW];
    int state;  // workgroup-uniform decision flags
};
// K tiles use the same 288-byte row pitch: a 16-byte-per-lane read is served for lanes 0-7 of two
// neighbouring 16-lane groups at a time, and with rows 288 B apart those sixteen pieces (rows i,
// 16-byte columns g and g+1) fall into sixteen different 16-byte bank groups.  (272 B, which only
// separates the rows of one group, costs every such read a second pass: measured with the LDS
// bank-conflict counter.)
constexpr int WROWS = 128;  // sequences per wide item: 32 per wave
struct WidePathLds {
    half_t k[1][64 * VPITCH];
    half_t v[1][64 * VPITCH];
    int last[WROWS];
};
// The decode kernel exists in three forms, chosen on the host from what the work list holds, so
// that launches without the wide matrix-core path are not held to its register and LDS budget
// (two workgroups per compute unit) and run three per compute unit instead:
//   kMixFull    every path;
//   kMixStream  stream items only (nothing shared, or partition 2);
//   kMixNarrow  stream items and shared items of at most 16 sequences, none wide.
constexpr int kMixFull = 0, kMixStream = 1, kMixNarrow = 2;
constexpr int kNarrowLookahead = 1;  // blocks on their way in the narrow form (three workgroups per CU: 168 registers)
template <int MIX> union DecodeLds;
template <> union __attribute__((aligned(16))) DecodeLds<kMixFull> {
    SharedPathLds<2> sh;
    SharedPathLds<1> sh1;
    StreamPathLds st;
    WidePathLds wd;
};
template <> union __attribute__((aligned(16))) DecodeLds<kMixStream> {
    StreamPathLds st;
};
template <> union __attribute__((aligned(16))) DecodeLds<kMixNarrow> {
    SharedPathLds<1> sh;
    StreamPathLds st;
};

// ---------------------------------------------------------------------------------------
// stream_path: an item = a run of one sequence's own chunks.  Wave w of the workgroup takes
// tiles w, w+4, ... of the item (a tile = one chunk, or two chunks at chunk size 32) and reads
// them as 64-token sub-tiles.  Lane l = 16*g + j reads, for load i, the 16 bytes at offset
// 1024*i + 16*l of a sub-tile: row 4*i + g, dims 8*j..8*j+7, so every load instruction covers
// 1 KiB of contiguous memory and 32 of them (K, then V) are in flight per wave.
// ---------------------------------------------------------------------------------------
// PER_WAVE: the wave works alone on its own item (all tiles, no cross-wave combine, no barrier):
// the form for many short runs, where a workgroup per run would spend its life starting up.
// STEP kAppend (APPEND below): the fused decode step.  The newest token of the
// sequence (position len - 1) has no row in the pool yet: the wave whose tile holds that position
// takes the row from k_new / v_new instead, and the arithmetic is that of a forward over a pool
// the row was appended to beforehand.  The row itself is written into the pool by the merge launch
// that follows (merge_kernel's append workgroups), not here: stores scattered through a launch
// that streams at the memory's speed cost it 9 % of its duration (256 sequences: 192 -> 209 us;
// dirty lines leave the L2 in dribs and drabs and turn the memory bus around each time), the same
// rows written by a launch of their own, or at the end of the merge launch, cost 1-3 us.
template <int C, bool PER_WAVE, int STEP>
__device__ __forceinline__ void stream_path(const DecodeArgs& A, const WorkItem* __restrict__ gi,
                                            int h, StreamPathLds& sm) {
    WorkItem it;  // header only: the inline slots are read from global memory where needed
    it.seq_begin = gi->seq_begin; it.n_rows = gi->n_rows; it.slot_first = gi->slot_first;
    it.n_chunks = gi->n_chunks; it.part_row = gi->part_row; it.pos0 = gi->pos0;
    it.len0 = gi->len0; it.flags = gi->flags;
    const half_t* __restrict__ q = A.q;
    const half_t* __restrict__ kpool = A.kpool;
    const half_t* __restrict__ vpool = A.vpool;
    const int32_t* __restrict__ slots = A.slots;
    const int H = A.H;
    const float scale_log2 = A.scale_log2;
    const bool coh = A.fuse_merge != 0;  // partial rows are read during this launch
    // A wave works on 64-token sub-tiles: one chunk at chunk size 64, half a chunk at 128, two
    // consecutive chunks of the item at 32 (their loads go out together, so a wave has the same
    // 32 KiB in flight at every chunk size).
    constexpr int SUB = 64;                        // tokens per sub-tile
    constexpr int NL = SUB / 4;                    // 16-byte loads per lane per sub-tile
    constexpr int CPT = (C < SUB) ? SUB / C : 1;   // chunks per tile
    constexpr int NSUB = (C > SUB) ? C / SUB : 1;  // sub-tiles per tile
    constexpr int LPC = NL / CPT;                  // loads per lane that one chunk supplies
    static_assert(C == 32 || C == 64 || C == 128, "chunk sizes of the decode kernels");

    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, known uniform
    const int l = tid & 63, g = l >> 4, j = l & 15;
    const int slotv = preload_slots(gi, it.slot_first, it.n_chunks, slots, l);
    const int seq = it.seq_begin;
    const int len = it.len0 + A.delta_tokens;

    constexpr bool APPEND = STEP != kForward;
    const h8 qv = *reinterpret_cast<const h8*>(q + (size_t(seq) * H + h) * D + 8 * j);

    float m_run = NEG_INF, l_lane = 0.f;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;

    // Folding in the other partial rows of this (sequence, head).  Once every other partial
    // is complete (the counter says so and stays so until this workgroup resets it), wave w
    // folds rows w, w+4, ... of the list straight into its running softmax state, so nothing
    // is published and nothing remains to merge.  Each wave tries once after its first tile,
    // when the row loads hide behind the streaming; the rest happens at the end.
    const bool can_fold = !PER_WAVE && A.fuse_merge && it.part_row >= 0;
    const int p0 = (it.part_row >= 0) ? A.part_ptr[seq] : 0;
    const int p1 = (it.part_row >= 0) ? A.part_ptr[seq + 1] : 0;
    const int own = p0 + it.part_row;  // this workgroup's partial row
    int* counter = A.counters + (seq * H + h);
    bool folded = !can_fold;
    auto fold_rows = [&]() {
        for (int pb = p0 + w; pb < p1; pb += 2 * NW) {
            // two rows per round so that their loads overlap
            float rm[2], rl[2];
            f2 rv[2][4];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int p = pb + u * NW;
                rm[u] = NEG_INF;
                rl[u] = 0.f;
                if (p < p1 && p != own) {
                    const float* r = A.part + (size_t(p) * H + h) * PART_STRIDE;
                    const f2 ml = part_load2(r);
                    rm[u] = ml[0];
                    rl[u] = ml[1];
#pragma unroll
                    for (int e = 0; e < 4; e++) rv[u][e] = part_load2(r + 4 + 8 * j + 2 * e);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) rv[u][e] = f2{ 0.f, 0.f };
                }
            }
#pragma unroll
            for (int u = 0; u < 2; u++) {
                if (rm[u] == NEG_INF) continue;  // empty or absent row (wave-uniform)
                const float mn = fmaxf(m_run, rm[u]);
                const float fa = (m_run == NEG_INF) ? 0.f : fast_exp2(m_run - mn);
                const float fb = fast_exp2(rm[u] - mn);
                const float fo = (g == 0) ? fb : 0.f;  // the row is added once, by lane group 0
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    acc[2 * e] = acc[2 * e] * fa + fo * rv[u][e][0];
                    acc[2 * e + 1] = acc[2 * e + 1] * fa + fo * rv[u][e][1];
                }
                l_lane = l_lane * fa + ((l == 0) ? fb * rl[u] : 0.f);
                m_run = mn;
            }
        }
        folded = true;
    };
    bool tried = !can_fold;

    for (int t = (PER_WAVE ? 0 : w) * CPT; t < it.n_chunks; t += (PER_WAVE ? 1 : NW) * CPT) {
        int valid = len - (it.pos0 + t) * C;
        if (valid <= 0) break;  // chunks are in path order: everything after is empty too
        // tokens of this tile: bounded by the sequence's end and by the item's last chunk (the
        // sequence may go on in another item)
        const int n_here = (it.n_chunks - t < CPT) ? it.n_chunks - t : CPT;
        // the sequence ends inside this tile: the tile of its newest token
        const bool tile_has_new = APPEND && valid <= n_here * C;
        valid = valid < n_here * C ? valid : n_here * C;
        size_t base[CPT];
#pragma unroll
        for (int cc = 0; cc < CPT; cc++) {
            const int tc = (cc < n_here) ? t + cc : t;  // a missing second chunk is never loaded
            base[cc] = (size_t(chunk_slot(slotv, tc)) * H + h) * size_t(C) * D;
        }
#pragma unroll
        for (int sub = 0; sub < NSUB; sub++) {
            const int vsub = valid - sub * SUB;  // valid rows in this sub-tile
            if (vsub <= 0) break;
            const bool new_here = tile_has_new && vsub <= SUB;  // the newest token is row vsub - 1
            const bool masked = vsub < SUB || new_here;
            // load i of the sub-tile: 1 KiB at offset (i % LPC) KiB of chunk i / LPC
            const uint4* kp[CPT];
            const uint4* vp[CPT];
#pragma unroll
            for (int cc = 0; cc < CPT; cc++) {
                kp[cc] = reinterpret_cast<const uint4*>(kpool + base[cc] + size_t(sub) * SUB * D) + l;
                vp[cc] = reinterpret_cast<const uint4*>(vpool + base[cc] + size_t(sub) * SUB * D) + l;
            }
            uint4 kr[NL], vr[NL];
            if (!masked) {
#pragma unroll
                for (int i = 0; i < NL; i++) {
                    const uint4* p = kp[i / LPC] + 64 * (i % LPC);
                    kr[i] = A.stream_nt ? nt_load16(p) : *p;
                }
#pragma unroll
                for (int i = 0; i < NL; i++) {
                    const uint4* p = vp[i / LPC] + 64 * (i % LPC);
                    vr[i] = A.stream_nt ? nt_load16(p) : *p;
                }
            } else {
                // rows past the end of the sequence hold stale data: never read into the math
                const int vmem = (APPEND && new_here) ? vsub - 1 : vsub;  // rows that the pool holds
                // The newest token's pieces are requested in front of the tile's own loads: loads
                // return in order, so they are there when the tile is, at no round trip of their own.
                uint4 kn = make_uint4(0, 0, 0, 0), vn = make_uint4(0, 0, 0, 0);
                if constexpr (APPEND) {
                    if (new_here) {
                        const size_t new_off = (size_t(seq) * H + h) * D;
                        kn = *(reinterpret_cast<const uint4*>(A.k_new + new_off) + j);
                        vn = *(reinterpret_cast<const uint4*>(A.v_new + new_off) + j);
                    }
                }
#pragma unroll
                for (int i = 0; i < NL; i++) {
                    const bool ok = 4 * i + g < vmem;
                    kr[i] = ok ? kp[i / LPC][64 * (i % LPC)] : make_uint4(0, 0, 0, 0);
                    vr[i] = ok ? vp[i / LPC][64 * (i % LPC)] : make_uint4(0, 0, 0, 0);
                }
                if constexpr (APPEND) {
                    if (new_here) {
                        // row vsub - 1 = 4 * i_new + g_new is the newest token: lanes (g_new, j) take
                        // piece j of it from the caller's rows, as if it had been loaded from the pool
                        const int i_new = (vsub - 1) >> 2;
                        const bool mine = ((vsub - 1) & 3) == g;
#pragma unroll
                        for (int i = 0; i < NL; i++) {
                            if (i == i_new && mine) {
                                kr[i] = kn;
                                vr[i] = vn;
                            }
                        }
                    }
                }
            }
            float sc[NL];
#pragma unroll
            for (int i = 0; i < NL; i++) {
                sc[i] = dot8(*reinterpret_cast<const h8*>(&kr[i]), qv, 0.f);
            }
            // lane (g, j) now owns the score of row 4*(j % NL) + g
            float s = reduce_rows16<NL>(sc, j) * scale_log2;
#ifdef CA_TIMELINE
            if (t == 0 && sub == 0) CA_STAMP(1);
#endif
            const int row = 4 * (j % NL) + g;
            if (row >= vsub || j >= NL) s = NEG_INF;
            const float m_new = fmaxf(m_run, wave_max(s));
            const float alpha = fast_exp2(m_run - m_new);
            const float p = fast_exp2(s - m_new);
            m_run = m_new;
            l_lane = l_lane * alpha + p;
            sm.p[w][l] = p;
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] *= alpha;
            __builtin_amdgcn_wave_barrier();
            float pr[NL];
#pragma unroll
            for (int i = 0; i < NL; i += 4) {
                const f4 t4 = *reinterpret_cast<const f4*>(&sm.p[w][16 * g + i]);
                pr[i] = t4[0]; pr[i + 1] = t4[1]; pr[i + 2] = t4[2]; pr[i + 3] = t4[3];
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int i = 0; i < NL; i++) {
                const h8 vv = *reinterpret_cast<const h8*>(&vr[i]);
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e] = __builtin_fmaf(pr[i], float(vv[e]), acc[e]);
            }
        }
        if (!tried) {
            tried = true;
            const int done = __builtin_amdgcn_readfirstlane(
              __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            if (done == p1 - p0 - 1) fold_rows();
        }
    }

    // end of streaming: one workgroup-uniform look at the counter decides between folding the
    // remaining rows now and publishing this workgroup's partial.  The barrier in front makes
    // the look later than every wave's own early look, so "complete" seen there is seen here.
    if (can_fold) {
        __syncthreads();
        if (tid == 0) {
            sm.state = (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p1 - p0 - 1);
        }
        __syncthreads();
        if (sm.state && !folded) fold_rows();
    }
    const bool complete = can_fold && sm.state;

    // wave result: rows are spread over the four 16-lane groups
    const float l_wave = wave_sum(l_lane);
#pragma unroll
    for (int e = 0; e < 8; e++) {
        acc[e] += shfl_xor(acc[e], 16);
        acc[e] += shfl_xor(acc[e], 32);
    }
    if constexpr (PER_WAVE) {
        // lanes of group 0 hold dims 8j..8j+7 of the wave's (= the item's) result
        if (g == 0) {
            if (it.part_row < 0) {
                const float r = l_wave > 0.f ? 1.f / l_wave : 0.f;
                h8 o8;
#pragma unroll
                for (int e = 0; e < 8; e++) o8[e] = half_t(acc[e] * r);
                *reinterpret_cast<h8*>(A.out + (size_t(seq) * H + h) * D + 8 * j) = o8;
            } else {
                float* own_row = A.part + (size_t(own) * H + h) * PART_STRIDE;
#pragma unroll
                for (int e = 0; e < 8; e += 2) part_store2(own_row + 4 + 8 * j + e, acc[e], acc[e + 1], coh);
                if (j == 0) part_store2(own_row, m_run, l_wave, coh);
            }
        }
        return;
    }
    if (g == 0) {
#pragma unroll
        for (int e = 0; e < 8; e++) sm.o[w][8 * j + e] = acc[e];
    }
    if (l == 0) {
        sm.m[w] = m_run;
        sm.l[w] = l_wave;
    }
    __syncthreads();

    // combine the four waves: thread tid < 128 owns output dim tid
    float m = sm.m[0];
#pragma unroll
    for (int k = 1; k < NW; k++) m = fmaxf(m, sm.m[k]);
    float o = 0.f, lsum = 0.f;
    if (tid < D) {
#pragma unroll
        for (int k = 0; k < NW; k++) {
            const float f = (sm.m[k] == NEG_INF) ? 0.f : fast_exp2(sm.m[k] - m);
            o += f * sm.o[k][tid];
            lsum += f * sm.l[k];
        }
    }
    if (it.part_row < 0 || complete) {  // nothing (left) to merge: final output
        if (tid < D) {
            const float r = lsum > 0.f ? 1.f / lsum : 0.f;
            A.out[(size_t(seq) * H + h) * D + tid] = half_t(o * r);
        }
        if (complete && tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    float* own_row = A.part + (size_t(own) * H + h) * PART_STRIDE;
    if (tid < D) part_store(own_row + 4 + tid, o, coh);
    if (tid == 0) part_store2(own_row, m, lsum, coh);
    if (!A.fuse_merge) return;

    // publish, count, and let whoever arrives last merge from memory
    wait_own_stores();
    __syncthreads();  // every store of the row has completed
    if (tid == 0) {
        const int done = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm.state = (done == p1 - p0 - 1);
    }
    __syncthreads();
    if (sm.state && w == 0) {
        merge_rows<true>(A.part, p0, p1, h, H, A.out + (size_t(seq) * H + h) * D, l);
        if (l == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---------------------------------------------------------------------------------------
// shared_path: an item = (segment of chunks, up to 32 sequences).  The segment is one token
// stream cut into 16-token blocks; wave w takes blocks w, w+4, ... and keeps its own online-
// softmax state, so waves never wait for each other until the final merge.  The K and V of the
// next LA blocks are on their way while the current one is consumed: LA + 1 register sets used
// in turn (the loop body is unrolled LA + 1 times, so that every set has a fixed name and no
// block is ever copied from one set to another -- a copy would have to wait for the block it
// copies).  Every step of the loop issues exactly one block's loads, unconditionally: past the
// wave's last block it requests that block again (cached, never used).  With a conditional
// request the compiler cannot know how many loads are outstanding where the paths join and waits
// for all of them, which serialises request and use.
//
// Matrix-core operand layout (v_mfma_f32_16x16x*: lane l = 16*g + i):
//   A holds row i, B holds column i, each with the k-slice of group g; D holds rows 4g..4g+3
//   of column i.  S^T block = K_blk(16 tokens x 128) . Q^T  -> lane owns scores of tokens
//   4g..4g+3 for sequence i, which is exactly the B operand of O^T = V^T . P^T (k = 16
//   tokens), so probabilities never leave registers.  V^T comes from a wave-private LDS copy
//   of the 16 x 128 V block through the LDS transpose read (lds_read_tr).
// ---------------------------------------------------------------------------------------
template <int C, int MBT, int LA>
__device__ __forceinline__ void shared_path(const DecodeArgs& A, const WorkItem* __restrict__ gi,
                                            int h, SharedPathLds<MBT>& sm) {
    constexpr int MB = MBT;  // 16-row blocks of the item
    constexpr int R = LA + 1;  // register sets
    WorkItem it;
    it.seq_begin = gi->seq_begin; it.n_rows = gi->n_rows; it.slot_first = gi->slot_first;
    it.n_chunks = gi->n_chunks; it.part_row = gi->part_row; it.pos0 = gi->pos0;
    it.len0 = gi->len0; it.flags = gi->flags;
    const half_t* __restrict__ kpool = A.kpool;
    const half_t* __restrict__ vpool = A.vpool;
    const int32_t* __restrict__ slots = A.slots;
    const int H = A.H;
    const float scale_log2 = A.scale_log2;
    const bool coh = A.fuse_merge != 0;  // partial rows are read during this launch
    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, known uniform
    const int l = tid & 63, g = l >> 4, i = l & 15;
    const int slotv = preload_slots(gi, it.slot_first, it.n_chunks, slots, l);
    const int len = it.len0 + A.delta_tokens;
    const bool two = MB > 1 && it.n_rows > 16;  // second 16-row block in use (uniform)
    if (tid < it.n_rows) sm.row[tid] = A.part_ptr[it.seq_begin + tid] + it.part_row;

    // Q^T operand: sequence row mb*16+i, dims 32*ks + 8*g .. +7
    h8 qreg[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int row = mb * 16 + i;
        const half_t* qp = A.q + (size_t(it.seq_begin + row) * H + h) * D + 8 * g;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            qreg[mb][ks] = (row < it.n_rows) ? *reinterpret_cast<const h8*>(qp + 32 * ks) : h8{ 0, 0, 0, 0, 0, 0, 0, 0 };
        }
    }

    float m_run[MB], l_lane[MB];
    f4 oacc[MB][8];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        m_run[mb] = NEG_INF;
        l_lane[mb] = 0.f;
#pragma unroll
        for (int db = 0; db < 8; db++) oacc[mb][db] = f4{ 0.f, 0.f, 0.f, 0.f };
    }

    constexpr int BPC = C / 16;  // blocks per chunk
    // blocks of the item that hold tokens of the sequences: block tb has rem - 16 * tb of them
    const int rem = len - it.pos0 * C;
    const int n_blocks = min(it.n_chunks * BPC, (rem + 15) >> 4);
    auto block_base = [&](int tb) {
        return ((size_t(chunk_slot(slotv, tb / BPC)) * H + h) * size_t(C) + (tb % BPC) * 16) * D;
    };
    h8 kq[R][4];
    uint4 vq[R][4];
    // requests block tb of this wave; past its last block, that one again
    const int last_block = w + ((n_blocks - 1 - w) & ~(NW - 1));  // (only used when w < n_blocks)
    // ka, va: the lane's addresses, handed back so that the caller can keep them alive past the
    // block's use (see the loop)
    auto load_block = [&](int tb, h8 (&kr)[4], uint4 (&vr)[4], const half_t*& ka, const uint4*& va) {
        const size_t base = block_base(tb < n_blocks ? tb : last_block);
        ka = kpool + base + size_t(i) * D + 8 * g;
        va = reinterpret_cast<const uint4*>(vpool + base) + l;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) kr[ks] = *reinterpret_cast<const h8*>(ka + 32 * ks);
#pragma unroll
        for (int r = 0; r < 4; r++) vr[r] = va[64 * r];
    };
    // one block: scores, online softmax, O^T += V^T . P^T
    auto consume = [&](const h8 (&kreg)[4], const uint4 (&vraw)[4], int valid, bool first) {
        // V block -> LDS rows (row 4r+g, dims 8i..8i+7); stale rows past the end are zeroed
#pragma unroll
        for (int r = 0; r < 4; r++) {
            uint4 t = vraw[r];
            if (4 * r + g >= valid) t = make_uint4(0, 0, 0, 0);
            *reinterpret_cast<uint4*>(&sm.v[w][(4 * r + g) * VPITCH + 8 * i]) = t;
        }

        h4 pb[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            if (mb == 1 && !two) {
                pb[mb] = h4{ 0, 0, 0, 0 };
                continue;
            }
            f4 s = f4{ 0.f, 0.f, 0.f, 0.f };
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                s = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[ks], qreg[mb][ks], s, 0, 0, 0);
            }
            // raw-score maximum: the scale is positive and rides in the exponent's multiply-add.
            // Masking is a select, not a branch: no branch may sit between a matrix op and the
            // first use of its result (the compiler's wait states for that hazard do not reach
            // across a taken branch).
#pragma unroll
            for (int r = 0; r < 4; r++) {
                if (4 * g + r >= valid) s[r] = NEG_INF;
            }
            float mx = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
            mx = fmaxf(mx, shfl_xor(mx, 16));
            mx = fmaxf(mx, shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run[mb], mx * scale_log2);  // valid >= 1: mx is finite
            const float alpha = fast_exp2(m_run[mb] - m_new);
            m_run[mb] = m_new;
            float psum = 0.f;
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                p[r] = fast_exp2(__builtin_fmaf(s[r], scale_log2, -m_new));
                psum += p[r];
            }
            l_lane[mb] = l_lane[mb] * alpha + psum;
            pb[mb] = h4{ half_t(p[0]), half_t(p[1]), half_t(p[2]), half_t(p[3]) };
#pragma unroll
            for (int db = 0; db < 8; db++) oacc[mb][db] *= alpha;
        }

#ifdef CA_TIMELINE
        if (first) CA_STAMP(1);
#else
        (void)first;
#endif
        __builtin_amdgcn_wave_barrier();
        // O^T += V^T . P^T : A = V^T (row = dim 16*db + i, k = tokens 4g..4g+3)
#pragma unroll
        for (int db = 0; db < 8; db++) {
            const h4 a = lds_read_tr(&sm.v[w][(4 * g + (i >> 2)) * VPITCH + 16 * db + 4 * (i & 3)]);
            oacc[0][db] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, pb[0], oacc[0][db], 0, 0, 0);
            if constexpr (MB > 1) {
                if (two) oacc[1][db] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, pb[1], oacc[1][db], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    if (w < n_blocks) {
        const half_t* ka;
        const uint4* va;
        // (the first blocks in order, oldest first: the waits inside the loop are the minimum over
        // the ways into it, and a reordered start would make every round's first step wait longer)
#pragma unroll
        for (int j = 0; j < LA; j++) {
            load_block(w + NW * j, kq[j], vq[j], ka, va);
            __builtin_amdgcn_sched_barrier(0);
        }
        // Rounds of R steps with the loop's only exit after a round: a step past the wave's last
        // block still requests (its last block again: cached, never used) and skips the use.  On
        // every way to a use the same loads have been issued since the block's own, so the wait
        // in front of it is exact; with an exit inside the round, the compiler's single-exit form
        // of the loop would add ways that are never taken but shorten the count.
        int tb = w;
        do {
#pragma unroll
            for (int u = 0; u < R; u++) {
                load_block(tb + NW * LA, kq[(u + LA) % R], vq[(u + LA) % R], ka, va);
                if (tb < n_blocks) consume(kq[u], vq[u], rem - 16 * tb, tb == 0);
                // the address registers stay in use until here: were they free once the loads are
                // issued, the register allocator would make them the destination of the last load,
                // and writing the next block's address would wait for that load
                asm volatile("" ::"v"(ka), "v"(va));
                tb += NW;
            }
        } while (tb < n_blocks);
    }

    // ---- merge the four waves ------------------------------------------------------------
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        l_lane[mb] += shfl_xor(l_lane[mb], 16);
        l_lane[mb] += shfl_xor(l_lane[mb], 32);
        if (g == 0) sm.m[w][mb * 16 + i] = m_run[mb];
    }
    __syncthreads();
    float m_all[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        float m = sm.m[0][mb * 16 + i];
#pragma unroll
        for (int k = 1; k < NW; k++) m = fmaxf(m, sm.m[k][mb * 16 + i]);
        m_all[mb] = m;
        const float f = (m_run[mb] == NEG_INF) ? 0.f : fast_exp2(m_run[mb] - m);
        if (g == 0) sm.l[w][mb * 16 + i] = l_lane[mb] * f;
#pragma unroll
        for (int db = 0; db < 8; db++) oacc[mb][db] *= f;
    }
    for (int k = 0; k < NW; k++) {
        if (w == k) {
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
#pragma unroll
                for (int db = 0; db < 8; db++) {
                    // lane owns dims 16*db + 4*g .. +3 of sequence row mb*16 + i
                    f4* dst = reinterpret_cast<f4*>(&sm.o[(mb * 16 + i) * OPITCH + 16 * db + 4 * g]);
                    *dst = (k == 0) ? oacc[mb][db] : (*dst + oacc[mb][db]);
                }
            }
        }
        __syncthreads();
    }

    // ---- write the partial rows ------------------------------------------------------------
    for (int idx = tid; idx < it.n_rows * (D / 4); idx += WG) {
        const int row = idx / (D / 4), c4 = idx % (D / 4);
        float* dst = A.part + (size_t(sm.row[row]) * H + h) * PART_STRIDE + 4 + 4 * c4;
        const f4 v = *reinterpret_cast<const f4*>(&sm.o[row * OPITCH + 4 * c4]);
        part_store2(dst, v[0], v[1], coh);
        part_store2(dst + 2, v[2], v[3], coh);
    }
    if (w == 0 && g == 0) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            const int row = mb * 16 + i;
            if (row < it.n_rows) {
                float lsum = 0.f;
#pragma unroll
                for (int k = 0; k < NW; k++) lsum += sm.l[k][row];
                part_store2(A.part + (size_t(sm.row[row]) * H + h) * PART_STRIDE, m_all[mb], lsum, coh);
            }
        }
    }
    if (!A.fuse_merge) return;

    // count one finished partial for every covered sequence (after the barrier: all stores of
    // the rows have completed); merge the completed ones
    wait_own_stores();
    __syncthreads();
    if (tid < it.n_rows) {
        const int s = it.seq_begin + tid;
        const int done = __hip_atomic_fetch_add(&A.counters[s * H + h], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm.last[tid] = (done == A.part_ptr[s + 1] - A.part_ptr[s] - 1);
    }
    __syncthreads();
    for (int r = w; r < it.n_rows; r += NW) {
        if (sm.last[r]) {
            const int s = it.seq_begin + r;
            merge_rows<true>(A.part, A.part_ptr[s], A.part_ptr[s + 1], h, H,
                             A.out + (size_t(s) * H + h) * D, l);
            if (l == 0) __hip_atomic_store(&A.counters[s * H + h], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------------------
// wide_path: chunk-first for chunks shared by many sequences.  An item covers up to 128
// sequences; wave w owns rows 32w .. 32w+31, or 16w .. 16w+15 when the item has at most 64 (MBW
// = 16-row blocks per wave; Q^T and the output accumulators stay in the wave's registers for the
// whole segment), and attends every token.  The segment is walked in 64-token
// tiles: all 256 threads stage the K and V tile in LDS once (the next tile is already on its way
// in registers), then each wave runs the same MFMA scheme as shared_path with K operands read
// from LDS.  Every K/V byte is fetched once per 128 sequences and no cross-wave merge is needed.
//
// What keeps the vector unit's share of a tile small (it, not the matrix cores, bounds the tile):
//   * tiles that are wholly inside the sequence (all but at most the last) take a path with no
//     validity tests at all; the last, partial tile zeroes the missing rows while staging and
//     starts the score accumulators at -inf for the missing tokens instead of selecting afterwards;
//   * row maxima cross the four 16-lane groups with the lane-swap instructions, not through LDS;
//   * the running maximum only moves (and the accumulators are only rescaled) when some row of
//     the wave finds a larger score: a wave-uniform test, false for most tiles after the first few;
//   * the row sums come from one more matrix op per token pair (an all-ones A operand), which
//     also sums exactly the fp16 probabilities that P.V uses.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float max_over_groups(float v) {
    // lanes l, l^16, l^32, l^48 hold values of the same sequence: maximum of the four, in all four.
    // The swap instructions exchange whole 16-lane rows between two registers (16: the odd rows
    // of the first with the even rows of the second; 32: the upper half of the first with the lower
    // half of the second); with two copies of one value the two results hold each lane's own value
    // and its partner's.  (The result elements are copied out before the bit casts: a bit cast
    // applied to a vector element directly reads element 0 whatever the index.)
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned a0 = a[0], a1 = a[1];
    const float m16 = fmaxf(__builtin_bit_cast(float, a0), __builtin_bit_cast(float, a1));
    const unsigned w = __builtin_bit_cast(unsigned, m16);
    const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    const unsigned b0 = b[0], b1 = b[1];
    return fmaxf(__builtin_bit_cast(float, b0), __builtin_bit_cast(float, b1));
}

template <int C, int MBW>
__device__ __forceinline__ void wide_path(const DecodeArgs& A, const WorkItem* __restrict__ gi,
                                          int h, WidePathLds& sm) {
    static_assert(MBW == 1 || MBW == 2, "one or two 16-row blocks per wave");
    constexpr int MB = MBW;  // shadows the file-level constant inside this function
    WorkItem it;
    it.seq_begin = gi->seq_begin; it.n_rows = gi->n_rows; it.slot_first = gi->slot_first;
    it.n_chunks = gi->n_chunks; it.part_row = gi->part_row; it.pos0 = gi->pos0;
    it.len0 = gi->len0; it.flags = gi->flags;
    const half_t* __restrict__ kpool = A.kpool;
    const half_t* __restrict__ vpool = A.vpool;
    const int32_t* __restrict__ slots = A.slots;
    const int H = A.H;
    const float scale_log2 = A.scale_log2;
    const bool coh = A.fuse_merge != 0;  // partial rows are read during this launch
    const int tid = threadIdx.x;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave index, known uniform
    const int l = tid & 63, g = l >> 4, i = l & 15;
    const int slotv = preload_slots(gi, it.slot_first, it.n_chunks, slots, l);
    const int len = it.len0 + A.delta_tokens;
    const int row_base = 16 * MB * w;               // first item row of this wave
    const bool active = row_base < it.n_rows;       // wave has sequences (uniform per wave)

    h8 qreg[MB][4];
    int prow[MB];  // partial row of this lane's sequence (needed at the very end: asked for now)
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int row = row_base + mb * 16 + i;
        const half_t* qp = A.q + (size_t(it.seq_begin + row) * H + h) * D + 8 * g;
        prow[mb] = (row < it.n_rows) ? A.part_ptr[it.seq_begin + row] + it.part_row : -1;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            qreg[mb][ks] = (row < it.n_rows) ? *reinterpret_cast<const h8*>(qp + 32 * ks) : h8{ 0, 0, 0, 0, 0, 0, 0, 0 };
        }
    }
    float m_run[MB];
    f4 oacc[MB][8], lacc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        m_run[mb] = NEG_INF;
        lacc[mb] = f4{ 0.f, 0.f, 0.f, 0.f };
#pragma unroll
        for (int db = 0; db < 8; db++) oacc[mb][db] = f4{ 0.f, 0.f, 0.f, 0.f };
    }

    // The segment's tokens exist as a prefix: `have` of them, in n_full whole 64-token tiles and
    // one partial tile of `rem` tokens.
    const int total_tokens = it.n_chunks * C;
    int have = len - it.pos0 * C;
    have = have < total_tokens ? have : total_tokens;
    have = have > 0 ? have : 0;
    const int n_full = have >> 6, rem = have & 63;
    const int n_tiles = n_full + (rem ? 1 : 0);

    // Thread tid stages pieces tid + 256r (r = 0..3) of the K and of the V tile: piece p = token
    // row p/16 of the tile, dims 8*(p%16) .. +7.  Sixteen token rows never straddle a chunk.
    const int srow = tid >> 4, spiece = tid & 15;
    const int lds_w = srow * VPITCH + 8 * spiece;
    uint4 kst[4], vst[4];
    auto fetch_tile = [&](int t) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            int ck, crow;  // chunk of the item and token row inside it
            if constexpr (C == 64) {
                ck = t; crow = srow + 16 * r;
            } else if constexpr (C == 128) {
                ck = t >> 1; crow = 64 * (t & 1) + srow + 16 * r;
            } else {
                ck = 2 * t + (r >> 1); crow = srow + 16 * (r & 1);
            }
            // a chunk index past the item's last chunk reads lane values that were preloaded as
            // slot 0: valid memory, and only ever for tokens the partial-tile path zeroes
            const size_t off = ((size_t(chunk_slot(slotv, ck & 63)) * H + h) * size_t(C) + crow) * D + 8 * spiece;
            kst[r] = *reinterpret_cast<const uint4*>(kpool + off);
            vst[r] = *reinterpret_cast<const uint4*>(vpool + off);
        }
    };
    h8 ones;
#pragma unroll
    for (int e = 0; e < 8; e++) ones[e] = half_t(1.f);

    // MASKED: the tile holds only `valid` (< 64) tokens.  Rows past them hold stale data: zeroed
    // on their way into LDS (V must not meet a NaN), their scores start at -inf.
    // stage the tile held in kst/vst into buffer `buf`; valid < 64: rows past the tile's tokens
    // are zeroed on their way in
    auto stage_tile = [&](int buf, int valid) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            uint4 kk = kst[r], vv = vst[r];
            if (srow + 16 * r >= valid) {
                kk = make_uint4(0, 0, 0, 0);
                vv = make_uint4(0, 0, 0, 0);
            }
            *reinterpret_cast<uint4*>(&sm.k[buf][lds_w + 16 * r * VPITCH]) = kk;
            *reinterpret_cast<uint4*>(&sm.v[buf][lds_w + 16 * r * VPITCH]) = vv;
        }
    };
    auto stage_full_tile = [&](int buf) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            *reinterpret_cast<uint4*>(&sm.k[buf][lds_w + 16 * r * VPITCH]) = kst[r];
            *reinterpret_cast<uint4*>(&sm.v[buf][lds_w + 16 * r * VPITCH]) = vst[r];
        }
    };

    // One tile: staged from kst/vst between two barriers, then the next tile is requested and this
    // one is attended.  (Staging the next tile into a second buffer while this one is read, one
    // barrier per tile, measured slower: 99.8 against 76.1 us for a 64-tile segment.)
    // MASKED: the tile holds only `valid` (< 64) tokens: their scores start at -inf (the staging
    // zeroed the rows, so stale NaNs never meet V).
    auto tile_body = [&](int t, auto masked_tag, int valid) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const half_t* __restrict__ kt = sm.k[0];
        const half_t* __restrict__ vt = sm.v[0];
        __syncthreads();
        if (MASKED) {
            stage_tile(0, valid);
        } else {
            stage_full_tile(0);
        }
        __syncthreads();
#ifdef CA_TIMELINE
        if (t == 0) CA_STAMP(1);
#endif
        if (t + 1 < n_tiles) fetch_tile(t + 1);
        if (active) {
            // scores of the 64 tokens for this wave's rows; lane (g, i) gets tokens 16tb + 4g .. +3
            // of sequence row i
            f4 sc[MB][4];
#pragma unroll
            for (int tb = 0; tb < 4; tb++) {
                h8 kop[4];
#pragma unroll
                for (int ks = 0; ks < 4; ks++) {
                    kop[ks] = *reinterpret_cast<const h8*>(&kt[(16 * tb + i) * VPITCH + 32 * ks + 8 * g]);
                }
                f4 init = f4{ 0.f, 0.f, 0.f, 0.f };
                if constexpr (MASKED) {
#pragma unroll
                    for (int r = 0; r < 4; r++) init[r] = (16 * tb + 4 * g + r >= valid) ? NEG_INF : 0.f;
                }
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    // rows past the item's last sequence carry zero queries: computed, never stored
                    f4 acc = init;
#pragma unroll
                    for (int ks = 0; ks < 4; ks++) {
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kop[ks], qreg[mb][ks], acc, 0, 0, 0);
                    }
                    sc[mb][tb] = acc;
                }
            }
            // Online softmax on the raw scores: the row maximum is taken before scaling (the scale is
            // positive) and the scale rides in the exponent's multiply-add.  No branch sits between a
            // matrix op and the first use of its result: the one branch below follows the maxima.
            float m_new[MB];
            bool grew = false;
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                float mx = fmaxf(fmaxf(sc[mb][0][0], sc[mb][0][1]), fmaxf(sc[mb][0][2], sc[mb][0][3]));
#pragma unroll
                for (int tb = 1; tb < 4; tb++) {
                    mx = fmaxf(mx, fmaxf(fmaxf(sc[mb][tb][0], sc[mb][tb][1]), fmaxf(sc[mb][tb][2], sc[mb][tb][3])));
                }
                mx = max_over_groups(mx);  // valid >= 1: finite
                m_new[mb] = fmaxf(m_run[mb], mx * scale_log2);
                grew |= m_new[mb] > m_run[mb];
            }
            if (__builtin_amdgcn_ballot_w64(grew) != 0) {
                // some row of the wave found a larger score: move the maxima, rescale what was summed
                // relative to the old ones (rows that did not move get a factor of exactly 1)
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    const float alpha = fast_exp2(m_run[mb] - m_new[mb]);
                    m_run[mb] = m_new[mb];
                    lacc[mb] *= alpha;
#pragma unroll
                    for (int db = 0; db < 8; db++) oacc[mb][db] *= alpha;
                }
            }
            // Per pair of 16-token blocks: probabilities, packed as the B operand of the 32-token-
            // deep P.V (k-slot (g, e) stands for token 4g + e of block 2*tp (e < 4) or 2*tp + 1
            // (e >= 4), which is where the S^T result layout already holds them), then the matrix ops
            // of that pair; the second pair's exponentials do not depend on the first pair's
            // matrix ops and stand between them in program order, so that they can overlap.
            h8 pp[MB][2];
            auto probabilities = [&](int tp) {
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    const float nm = -m_run[mb];
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        pp[mb][tp][e] = half_t(fast_exp2(__builtin_fmaf(sc[mb][2 * tp + (e >> 2)][e & 3], scale_log2, nm)));
                    }
                }
            };
            probabilities(0);
#pragma unroll
            for (int tp = 0; tp < 2; tp++) {
                // all eight V^T operands of this token pair are requested before the first matrix
                // op waits for one: the reads' latencies overlap instead of adding up
                h8 a[8];
#pragma unroll
                for (int db = 0; db < 8; db++) {
                    const half_t* p0 = &vt[(32 * tp + 4 * g + (i >> 2)) * VPITCH + 16 * db + 4 * (i & 3)];
                    const h4 lo = lds_read_tr(p0), hi = lds_read_tr(p0 + 16 * VPITCH);
                    a[db] = h8{ lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
                }
                if (tp == 0) probabilities(1);
#pragma unroll
                for (int mb = 0; mb < MB; mb++) {
                    // row sums: an all-ones A operand adds up the probabilities of every sequence
                    lacc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pp[mb][tp], lacc[mb], 0, 0, 0);
                }
#pragma unroll
                for (int db = 0; db < 8; db++) {
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) {
                        oacc[mb][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[db], pp[mb][tp], oacc[mb][db], 0, 0, 0);
                    }
                }
            }
        }
    };

    if (n_tiles > 0) fetch_tile(0);
    for (int t = 0; t < n_full; t++) tile_body(t, std::false_type{}, 64);
    if (rem) tile_body(n_full, std::true_type{}, rem);

    // ---- each wave writes the partial rows of its own sequences ----------------------------
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        if (prow[mb] >= 0) {
            float* dst = A.part + (size_t(prow[mb]) * H + h) * PART_STRIDE;
            // every lane of a sequence holds the same row sum (the matrix op summed over all tokens)
            if (g == 0) part_store2(dst, m_run[mb], lacc[mb][0], coh);
#pragma unroll
            for (int db = 0; db < 8; db++) {
                part_store2(dst + 4 + 16 * db + 4 * g, oacc[mb][db][0], oacc[mb][db][1], coh);
                part_store2(dst + 4 + 16 * db + 4 * g + 2, oacc[mb][db][2], oacc[mb][db][3], coh);
            }
        }
    }
    if (!A.fuse_merge) return;

    wait_own_stores();
    __syncthreads();
    for (int r = tid; r < it.n_rows; r += WG) {
        const int s = it.seq_begin + r;
        const int done = __hip_atomic_fetch_add(&A.counters[s * H + h], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        sm.last[r] = (done == A.part_ptr[s + 1] - A.part_ptr[s] - 1);
    }
    __syncthreads();
    for (int r = w; r < it.n_rows; r += NW) {
        if (sm.last[r]) {
            const int s = it.seq_begin + r;
            merge_rows<true>(A.part, A.part_ptr[s], A.part_ptr[s + 1], h, H,
                             A.out + (size_t(s) * H + h) * D, l);
            if (l == 0) __hip_atomic_store(&A.counters[s * H + h], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// grid = (n_shared_items + n_stream_items) * H workgroups, shared items first: they have the
// longest dependent chains and are sized to about one per compute unit, so they are done long
// before the streaming is and the merge falls to stream workgroups, one row each.
// What a workgroup needs before its first loads can go out comes as the leading scalar
// arguments: with kernel-argument preload they arrive in scalar registers with the wave (the
// first 14 dwords), so the work item's header is requested at once instead of after a round trip to the
// argument buffer; a struct passed by value is never preloaded.  The rest is wanted later.
struct DecodeRest {
    const int32_t* slots;
    half_t* out;
    float* part;
    const int32_t* part_ptr;
    int32_t* counters;
    const half_t* k_new;  // fused decode step only
    const half_t* v_new;
};
constexpr int kFlagFuseMerge = 1, kFlagPerWave = 2, kFlagStreamNt = 4;

// Workgroup b of a launch runs on XCD b % 8 of this part, and every XCD has an L2 of its own.
// The row tiles of one (shared segment, head) read the same K/V: they should meet in one L2 and
// run at about the same time.  Shared workgroup b therefore takes unit
//   u = (b % 8) * ceil-share + b / 8      (XCD x works through a contiguous range of units)
// of the head-major order u = head * n_items + item, in which the row tiles of a segment (adjacent
// in the item list) are neighbours -- whatever the number of heads is.
__device__ __forceinline__ int xcd_unit(int b, int n) {
    const int x = b & 7, q = n >> 3, r = n & 7;
    return x * q + (x < r ? x : r) + (b >> 3);
}

template <int C, int MIX, int STEP>
__global__ __launch_bounds__(WG, (MIX == kMixFull || C == 128 || STEP != kForward) ? 2 : 3) void decode_kernel(
    const WorkItem* stream_items, const WorkItem* shared_items, const half_t* kpool, const half_t* vpool,
    const half_t* q, int n_shared_wgs, int H, int delta_tokens, int flags, float scale_log2,
    int n_stream_items, const DecodeRest rest) {
    DecodeArgs A;
    A.q = q; A.kpool = kpool; A.vpool = vpool; A.out = rest.out; A.part = rest.part;
    A.shared_items = shared_items; A.stream_items = stream_items; A.slots = rest.slots;
    A.part_ptr = rest.part_ptr; A.counters = rest.counters; A.n_shared_wgs = n_shared_wgs;
    A.delta_tokens = delta_tokens; A.H = H; A.scale_log2 = scale_log2;
    A.fuse_merge = (flags & kFlagFuseMerge) ? 1 : 0;
    A.n_stream_items = n_stream_items;
    A.stream_per_wave = (flags & kFlagPerWave) ? 1 : 0;
    A.stream_nt = (flags & kFlagStreamNt) ? 1 : 0;
    A.k_new = rest.k_new; A.v_new = rest.v_new;
    __shared__ DecodeLds<MIX> lds;
    const int bid = blockIdx.x;
    CA_STAMP(0);
    CA_STAMP_VALUE(2, (unsigned long long)(bid < A.n_shared_wgs ? 0 : 2));
    if (MIX != kMixStream && bid < A.n_shared_wgs) {
        if constexpr (MIX != kMixStream) {
            const int unit = xcd_unit(bid, A.n_shared_wgs);
            const int n_items = A.n_shared_wgs / A.H;
            const int h = unit / n_items;
            const WorkItem* gi = A.shared_items + (unit - h * n_items);
            if constexpr (MIX == kMixFull) {
                if (gi->flags & kItemWide) {
                    // up to 64 sequences: 16 rows per wave keep all four waves busy
                    if (gi->n_rows <= 64) {
                        wide_path<C, 1>(A, gi, h, lds.wd);
                    } else {
                        wide_path<C, 2>(A, gi, h, lds.wd);
                    }
                } else if (gi->n_rows <= 16) {
                    shared_path<C, 1, 3>(A, gi, h, lds.sh1);
                } else {
                    shared_path<C, 2, 1>(A, gi, h, lds.sh);
                }
            } else {
                shared_path<C, 1, kNarrowLookahead>(A, gi, h, lds.sh);
            }
        }
    } else {
        const int sid = bid - A.n_shared_wgs;
        if (A.stream_per_wave) {
            // four consecutive items per workgroup, one per wave, same head
            const int item = 4 * (sid / A.H) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
            if (item < A.n_stream_items) stream_path<C, true, STEP>(A, A.stream_items + item, sid % A.H, lds.st);
        } else {
            stream_path<C, false, STEP>(A, A.stream_items + sid / A.H, sid % A.H, lds.st);
        }
    }
    CA_STAMP(3);
}

// What the merge launch of a fused decode step needs to write the step's new K/V rows.
struct MergeAppend {
    const half_t* k_new;  // [n_seqs, H, D]; null: nothing to append
    const half_t* v_new;
    half_t* kpool;
    half_t* vpool;
    const int32_t* tail_slot;
    const int32_t* tail_fill;
    int delta_before;         // delta_tokens before the step: the row is tail_fill + delta_before
    int C;
};

// Workgroups [0, n_merge_wgs): one wave per (sequence, head), merging its partial rows.
// Workgroups behind them (fused decode step only): the new token's K and V rows into the pool,
// one thread per 16-byte piece.
__global__ __launch_bounds__(WG) void merge_kernel(const float* __restrict__ part,
                                                   half_t* __restrict__ out,
                                                   const int32_t* __restrict__ part_ptr,
                                                   int n_seqs, int H, int n_merge_wgs, MergeAppend ap) {
    if (int(blockIdx.x) >= n_merge_wgs) {
        constexpr int pieces = D / 8;
        const int idx = (blockIdx.x - n_merge_wgs) * WG + threadIdx.x;
        if (idx >= n_seqs * H * pieces) return;
        const int piece = idx % pieces, sh = idx / pieces, h = sh % H, seq = sh / H;
        const int row = ap.tail_fill[seq] + ap.delta_before;
        if (row < 0 || row >= ap.C) return;  // host guarantees a free row; never write outside the chunk
        const size_t src = size_t(sh) * D + 8 * piece;
        const size_t dst = ((size_t(ap.tail_slot[seq]) * H + h) * ap.C + row) * D + 8 * piece;
        *reinterpret_cast<h8*>(ap.kpool + dst) = *reinterpret_cast<const h8*>(ap.k_new + src);
        *reinterpret_cast<h8*>(ap.vpool + dst) = *reinterpret_cast<const h8*>(ap.v_new + src);
        return;
    }
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    const int sh = blockIdx.x * NW + w;
    if (sh >= n_seqs * H) return;
    const int seq = sh / H, h = sh % H;
    const int p0 = part_ptr[seq], p1 = part_ptr[seq + 1];
    if (p0 == p1) return;  // written directly by a stream item
    merge_rows<false, 16>(part, p0, p1, h, H, out + (size_t(seq) * H + h) * D, l);
}

__global__ __launch_bounds__(WG) void fill_kernel(int32_t* __restrict__ p, int n, int32_t value) {
    const int idx = blockIdx.x * WG + threadIdx.x;
    if (idx < n) p[idx] = value;
}

__global__ __launch_bounds__(WG) void upload_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, int n) {
    const int idx = blockIdx.x * WG + threadIdx.x;
    if (idx < n) dst[idx] = src[idx];
}

// ---------------------------------------------------------------------------------------
// K/V row writes.  One thread moves one piece (16 bytes when d_head allows, else 2) of K and V.
// ---------------------------------------------------------------------------------------
// Measurement aid: reads n16 16-byte units and keeps nothing.  Workgroup b, thread t reads unit
// 256*b + t, then strides by the whole grid: at any moment the grid reads a few contiguous
// megabytes, eight non-temporal loads per lane in flight.  What a read with no structure at
// all reaches on this GPU: the yardstick beside the published peak.
__global__ __launch_bounds__(WG) void read_probe_kernel(const uint4* __restrict__ p, size_t n16,
                                                        uint32_t* __restrict__ sink) {
    constexpr int U = 8;
    const size_t stride = size_t(gridDim.x) * WG;
    size_t i = size_t(blockIdx.x) * WG + threadIdx.x;
    uint32_t acc = 0;
    for (; i + (U - 1) * stride < n16; i += U * stride) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = nt_load16(p + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const uint4 v = nt_load16(p + i);
        acc += v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u) sink[0] = acc;  // keeps the loads alive; practically never stores
}

template <typename T>
__global__ __launch_bounds__(WG) void append_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                                    T* __restrict__ kpool, T* __restrict__ vpool,
                                                    const int32_t* __restrict__ tail_slot,
                                                    const int32_t* __restrict__ tail_fill,
                                                    int delta_tokens, int n_seqs, int H, int C,
                                                    int pieces) {
    const int idx = blockIdx.x * WG + threadIdx.x;
    if (idx >= n_seqs * H * pieces) return;
    const int piece = idx % pieces, sh = idx / pieces, h = sh % H, seq = sh / H;
    const int row = tail_fill[seq] + delta_tokens;
    if (row < 0 || row >= C) return;  // host guarantees a free row; never write outside the chunk
    const size_t dst = ((size_t(tail_slot[seq]) * H + h) * C + row) * pieces + piece;
    kpool[dst] = k[idx];
    vpool[dst] = v[idx];
}

constexpr int SCATTER_SLOTS = 64;
struct ScatterArgs {
    int32_t slots[SCATTER_SLOTS];
};

template <typename T>
__global__ __launch_bounds__(WG) void scatter_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                                     T* __restrict__ kpool, T* __restrict__ vpool,
                                                     ScatterArgs args, int tok_begin, int n_copy,
                                                     int H, int C, int pieces) {
    const int64_t idx = int64_t(blockIdx.x) * WG + threadIdx.x;
    if (idx >= int64_t(n_copy) * H * pieces) return;
    const int piece = idx % pieces;
    const int h = (idx / pieces) % H;
    const int t = idx / (int64_t(pieces) * H);  // token within this launch
    const int slot = args.slots[t / C];
    const size_t dst = ((size_t(slot) * H + h) * C + (t % C)) * pieces + piece;
    const size_t src = (size_t(tok_begin + t) * H + h) * pieces + piece;
    kpool[dst] = k[src];
    vpool[dst] = v[src];
}

// K/V rows to explicit places: row i of k and v goes to row targets.row[i] of chunk
// targets.slot[i] (the beam-search step's row writes, one launch for all candidates).
constexpr int PUT_ROWS = 64;
struct PutTargets {
    int32_t slot[PUT_ROWS];
    int32_t row[PUT_ROWS];
};
template <typename T>
__global__ __launch_bounds__(WG) void put_rows_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                                      T* __restrict__ kpool, T* __restrict__ vpool,
                                                      PutTargets targets, int first, int n, int H, int C,
                                                      int pieces) {
    const int idx = blockIdx.x * WG + threadIdx.x;
    if (idx >= n * H * pieces) return;
    const int piece = idx % pieces, ih = idx / pieces, h = ih % H, i = ih / H;
    const size_t dst = ((size_t(targets.slot[i]) * H + h) * C + targets.row[i]) * pieces + piece;
    const size_t src = (size_t(first + i) * H + h) * pieces + piece;
    kpool[dst] = k[src];
    vpool[dst] = v[src];
}

// Whole-chunk copies, all pairs in one launch (the beam-search step's tail copies): workgroups
// (x, y) with y < n_pairs copy pair y of both pools, 16 bytes per thread and step.  Token rows
// pairs.skip[y][0..1] (-1: none) are left out, in source and destination alike: the same launch
// writes them.  Workgroups with y >= n_pairs are the row writers: row i of k and v goes to row
// put.row[i] of chunk put.slot[i] (what put_rows_kernel does).
constexpr int COPY_PAIRS = 64;
struct CopyPairs {
    int32_t src[COPY_PAIRS];
    int32_t dst[COPY_PAIRS];
    int32_t skip[COPY_PAIRS][2];
};
__global__ __launch_bounds__(WG) void copy_chunks_kernel(uint4* __restrict__ kpool, uint4* __restrict__ vpool,
                                                         CopyPairs pairs, int n_pairs, int units_per_chunk,
                                                         int units_per_row, int C, const uint4* __restrict__ k,
                                                         const uint4* __restrict__ v, PutTargets put, int n_put, int H) {
    if (int(blockIdx.y) >= n_pairs) {
        const int idx = (blockIdx.y - n_pairs) * gridDim.x * WG + blockIdx.x * WG + threadIdx.x;
        if (idx >= n_put * H * units_per_row) return;
        const int piece = idx % units_per_row, ih = idx / units_per_row, h = ih % H, i = ih / H;
        const size_t dst = ((size_t(put.slot[i]) * H + h) * C + put.row[i]) * units_per_row + piece;
        kpool[dst] = k[idx];
        vpool[dst] = v[idx];
        return;
    }
    const size_t src = size_t(pairs.src[blockIdx.y]) * units_per_chunk;
    const size_t dst = size_t(pairs.dst[blockIdx.y]) * units_per_chunk;
    const int skip0 = pairs.skip[blockIdx.y][0], skip1 = pairs.skip[blockIdx.y][1];
    for (int u = blockIdx.x * WG + threadIdx.x; u < units_per_chunk; u += gridDim.x * WG) {
        const int row = (u / units_per_row) % C;
        if (row == skip0 || row == skip1) continue;
        const uint4 kk = kpool[src + u], vv = vpool[src + u];
        kpool[dst + u] = kk;
        vpool[dst + u] = vv;
    }
}

// Partial rows of the allocation-free forward.  In host code this name is only a handle for
// hipGetSymbolAddress: the kernels get the resolved device address as an argument.
static __device__ __align__(256) float scratch[kScratchBytes / sizeof(float)];
// Where the read probe would store (it practically never does): its own word, so that a probe on
// another stream cannot touch a partial row.
static __device__ __align__(16) uint32_t probe_sink[4];

constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;  // contexts may be created from several threads
float* g_scratch_ptr[kMaxDevices] = {};
void* g_probe_sink_ptr[kMaxDevices] = {};

}  // namespace

int scratch_setup(int device) {
    if (device < 0 || device >= kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (g_scratch_ptr[device] && g_probe_sink_ptr[device]) return 0;
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    void* sink = nullptr;
    e = hipGetSymbolAddress(&sink, HIP_SYMBOL(probe_sink));
    if (e != hipSuccess) return static_cast<int>(e);
    g_probe_sink_ptr[device] = sink;
    g_scratch_ptr[device] = static_cast<float*>(ptr);
    return 0;
}

#ifdef CA_TIMELINE
extern "C" int ca_debug_timeline(unsigned long long* out, int n_wgs) {
    if (!out || n_wgs < 0 || n_wgs > 65536) return -1;
    return static_cast<int>(hipMemcpyFromSymbol(out, HIP_SYMBOL(ca_timeline), size_t(n_wgs) * 4 * sizeof(unsigned long long)));
}
#endif

float* scratch_ptr(int device) {
    if (device < 0 || device >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    return g_scratch_ptr[device];
}

void* probe_sink_ptr(int device) {
    if (device < 0 || device >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    return g_probe_sink_ptr[device];
}

// ---- launchers -----------------------------------------------------------------------------

#define CA_LAUNCH_CHECK()                                        \
    do {                                                         \
        hipError_t e_ = hipGetLastError();                       \
        if (e_ != hipSuccess) return static_cast<int>(e_);       \
    } while (0)

static DecodeArgs decode_args(const LaunchArgs& a) {
    DecodeArgs d;
    d.q = static_cast<const half_t*>(a.q);
    d.kpool = static_cast<const half_t*>(a.kpool);
    d.vpool = static_cast<const half_t*>(a.vpool);
    d.out = static_cast<half_t*>(a.out);
    d.part = a.part;
    d.shared_items = a.shared_items;
    d.stream_items = a.stream_items;
    d.slots = a.slots;
    d.part_ptr = a.part_ptr;
    d.counters = a.counters;
    d.n_shared_wgs = 0;
    d.delta_tokens = a.delta_tokens;
    d.H = a.H;
    d.scale_log2 = a.scale_log2;
    d.fuse_merge = 0;
    d.n_stream_items = 0;
    d.stream_per_wave = 0;
    d.stream_nt = a.stream_nt ? 1 : 0;
    d.k_new = static_cast<const half_t*>(a.k_new);
    d.v_new = static_cast<const half_t*>(a.v_new);
    return d;
}

int launch_decode(const LaunchArgs& a, int n_shared_items, int n_stream_items, bool fuse_merge,
                  hipStream_t st) {
    if (a.stream_per_wave && fuse_merge) return -1;  // waves on their own never meet at a barrier
    const bool append = a.k_new != nullptr;
    if (append && (!a.v_new || fuse_merge)) return -1;
    const int step = append ? kAppend : kForward;
    const int stream_groups = a.stream_per_wave ? (n_stream_items + NW - 1) / NW : n_stream_items;
    const int64_t wgs = int64_t(n_shared_items + stream_groups) * a.H;
    if (wgs <= 0) return 0;
    DecodeArgs d = decode_args(a);
    d.n_shared_wgs = n_shared_items * a.H;
    d.fuse_merge = fuse_merge ? 1 : 0;
    d.n_stream_items = n_stream_items;
    d.stream_per_wave = a.stream_per_wave ? 1 : 0;
    const dim3 grid(static_cast<unsigned>(wgs)), block(WG);
    const DecodeRest rest{ d.slots, d.out, d.part, d.part_ptr, d.counters, d.k_new, d.v_new };
    const int flags = (d.fuse_merge ? kFlagFuseMerge : 0) | (d.stream_per_wave ? kFlagPerWave : 0) |
                      (d.stream_nt ? kFlagStreamNt : 0);
    // the lightest form of the kernel that holds every path this launch takes
    const int mix = (n_shared_items == 0) ? kMixStream : (a.shared_narrow ? kMixNarrow : kMixFull);
#define CA_DECODE_LAUNCH(CS, MIX, STEP)                                                                    \
    hipLaunchKernelGGL((decode_kernel<CS, MIX, STEP>), grid, block, 0, st, d.stream_items, d.shared_items, \
                       d.kpool, d.vpool, d.q, d.n_shared_wgs, d.H, d.delta_tokens, flags, d.scale_log2,     \
                       d.n_stream_items, rest)
#define CA_DECODE_STEP(CS, MIX)                                           \
    do {                                                                  \
        if (step == kForward) CA_DECODE_LAUNCH(CS, MIX, kForward);        \
        else CA_DECODE_LAUNCH(CS, MIX, kAppend);                          \
    } while (0)
#define CA_DECODE_MIX(CS)                                                 \
    do {                                                                  \
        if (mix == kMixStream) CA_DECODE_STEP(CS, kMixStream);            \
        else if (mix == kMixNarrow) CA_DECODE_STEP(CS, kMixNarrow);       \
        else CA_DECODE_STEP(CS, kMixFull);                                \
    } while (0)
    switch (a.C) {
        case 32: CA_DECODE_MIX(32); break;
        case 64: CA_DECODE_MIX(64); break;
        case 128: CA_DECODE_MIX(128); break;
        default: return -1;
    }
#undef CA_DECODE_MIX
#undef CA_DECODE_STEP
#undef CA_DECODE_LAUNCH
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_merge(const LaunchArgs& a, int n_seqs, bool merge, hipStream_t st) {
    if (n_seqs <= 0) return 0;
    const bool append = a.k_new != nullptr;
    if (!merge && !append) return 0;
    if (append && (!a.v_new || !a.tail_slot || !a.tail_fill || a.d != D)) return -1;
    const int merge_wgs = merge ? (n_seqs * a.H + NW - 1) / NW : 0;
    const int append_wgs = append ? (n_seqs * a.H * (D / 8) + WG - 1) / WG : 0;
    MergeAppend ap{};
    if (append) {
        ap.k_new = static_cast<const half_t*>(a.k_new);
        ap.v_new = static_cast<const half_t*>(a.v_new);
        ap.kpool = static_cast<half_t*>(const_cast<void*>(a.kpool));
        ap.vpool = static_cast<half_t*>(const_cast<void*>(a.vpool));
        ap.tail_slot = a.tail_slot;
        ap.tail_fill = a.tail_fill;
        ap.delta_before = a.delta_tokens - 1;
        ap.C = a.C;
    }
    hipLaunchKernelGGL(merge_kernel, dim3(merge_wgs + append_wgs), dim3(WG), 0, st, a.part,
                       static_cast<half_t*>(a.out), a.part_ptr, n_seqs, a.H, merge_wgs, ap);
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_fill(int32_t* p, int n, int32_t value, hipStream_t st) {
    if (n <= 0) return 0;
    hipLaunchKernelGGL(fill_kernel, dim3((n + WG - 1) / WG), dim3(WG), 0, st, p, n, value);
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_upload(void* dst_dev, const void* src_pinned, size_t bytes, hipStream_t st) {
    if (bytes == 0) return 0;
    if (bytes % 16 != 0 || bytes / 16 > size_t(1) << 30) return -1;
    const int n = static_cast<int>(bytes / 16);
    hipLaunchKernelGGL(upload_kernel, dim3((n + WG - 1) / WG), dim3(WG), 0, st, static_cast<uint4*>(dst_dev),
                       static_cast<const uint4*>(src_pinned), n);
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_read_probe(const void* dev, size_t bytes, int n_wgs, void* sink, hipStream_t st) {
    if (bytes < 16 || !sink) return -1;
    hipLaunchKernelGGL(read_probe_kernel, dim3(n_wgs > 0 ? n_wgs : 256), dim3(WG), 0, st,
                       static_cast<const uint4*>(dev), bytes / 16, static_cast<uint32_t*>(sink));
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_append(const LaunchArgs& a, const void* k, const void* v, const int32_t* tail_slot,
                  const int32_t* tail_fill, int n_seqs, hipStream_t st) {
    if (n_seqs <= 0) return 0;
    void* kp = const_cast<void*>(a.kpool);
    void* vp = const_cast<void*>(a.vpool);
    if (a.d % 8 == 0) {
        const int pieces = a.d / 8, total = n_seqs * a.H * pieces;
        hipLaunchKernelGGL(append_kernel<uint4>, dim3((total + WG - 1) / WG), dim3(WG), 0, st,
                           static_cast<const uint4*>(k), static_cast<const uint4*>(v),
                           static_cast<uint4*>(kp), static_cast<uint4*>(vp), tail_slot, tail_fill,
                           a.delta_tokens, n_seqs, a.H, a.C, pieces);
    } else {
        const int pieces = a.d, total = n_seqs * a.H * pieces;
        hipLaunchKernelGGL(append_kernel<uint16_t>, dim3((total + WG - 1) / WG), dim3(WG), 0, st,
                           static_cast<const uint16_t*>(k), static_cast<const uint16_t*>(v),
                           static_cast<uint16_t*>(kp), static_cast<uint16_t*>(vp), tail_slot,
                           tail_fill, a.delta_tokens, n_seqs, a.H, a.C, pieces);
    }
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_scatter(const LaunchArgs& a, const void* k, const void* v, int n_tokens, int tok_begin,
                   const int32_t* slots, int n_slots, hipStream_t st) {
    void* kp = const_cast<void*>(a.kpool);
    void* vp = const_cast<void*>(a.vpool);
    for (int s0 = 0; s0 < n_slots; s0 += SCATTER_SLOTS) {
        const int ns = (n_slots - s0 < SCATTER_SLOTS) ? (n_slots - s0) : SCATTER_SLOTS;
        const int t0 = tok_begin + s0 * a.C;
        int n_copy = ns * a.C;
        if (t0 + n_copy > n_tokens) n_copy = n_tokens - t0;
        if (n_copy <= 0) break;
        ScatterArgs args;
        for (int i = 0; i < SCATTER_SLOTS; i++) args.slots[i] = (i < ns) ? slots[s0 + i] : 0;
        if (a.d % 8 == 0) {
            const int pieces = a.d / 8;
            const int64_t total = int64_t(n_copy) * a.H * pieces;
            hipLaunchKernelGGL(scatter_kernel<uint4>, dim3(static_cast<unsigned>((total + WG - 1) / WG)),
                               dim3(WG), 0, st, static_cast<const uint4*>(k), static_cast<const uint4*>(v),
                               static_cast<uint4*>(kp), static_cast<uint4*>(vp), args, t0, n_copy, a.H,
                               a.C, pieces);
        } else {
            const int pieces = a.d;
            const int64_t total = int64_t(n_copy) * a.H * pieces;
            hipLaunchKernelGGL(scatter_kernel<uint16_t>, dim3(static_cast<unsigned>((total + WG - 1) / WG)),
                               dim3(WG), 0, st, static_cast<const uint16_t*>(k),
                               static_cast<const uint16_t*>(v), static_cast<uint16_t*>(kp),
                               static_cast<uint16_t*>(vp), args, t0, n_copy, a.H, a.C, pieces);
        }
        CA_LAUNCH_CHECK();
    }
    return 0;
}

int launch_copy_chunks(const LaunchArgs& a, const int32_t* src_dst, int n_pairs, const void* k, const void* v,
                       const int32_t* slot_row, int n_rows, hipStream_t st) {
    const size_t chunk_bytes = size_t(a.H) * a.C * a.d * 2;
    if (chunk_bytes % 16 != 0 || chunk_bytes / 16 > 0x7fffffff || (a.d * 2) % 16 != 0) return -1;
    if (n_rows > PUT_ROWS || (n_rows > 0 && (!k || !v || !slot_row))) return -1;
    const int units = static_cast<int>(chunk_bytes / 16), units_per_row = a.d * 2 / 16;
    uint4* kp = static_cast<uint4*>(const_cast<void*>(a.kpool));
    uint4* vp = static_cast<uint4*>(const_cast<void*>(a.vpool));
    PutTargets put;
    for (int i = 0; i < PUT_ROWS; i++) {
        put.slot[i] = (i < n_rows) ? slot_row[2 * i] : 0;
        put.row[i] = (i < n_rows) ? slot_row[2 * i + 1] : 0;
    }
    // enough workgroups per pair to fill the device with a handful of pairs, two 16-byte
    // pieces of each pool per thread at least
    int per_pair = (units + 2 * WG - 1) / (2 * WG);
    if (per_pair > 128) per_pair = 128;
    if (per_pair < 1) per_pair = 1;
    for (int i0 = 0; i0 < n_pairs || (i0 == 0 && n_rows > 0); i0 += COPY_PAIRS) {
        const int m = (n_pairs - i0 < COPY_PAIRS) ? (n_pairs - i0) : COPY_PAIRS;
        CopyPairs pairs;
        for (int i = 0; i < COPY_PAIRS; i++) {
            pairs.src[i] = (i < m) ? src_dst[2 * (i0 + i)] : 0;
            pairs.dst[i] = (i < m) ? src_dst[2 * (i0 + i) + 1] : 0;
            pairs.skip[i][0] = pairs.skip[i][1] = -1;
            // rows of this pair's chunks that the row writers own
            for (int r = 0; i < m && r < n_rows; r++) {
                if (put.slot[r] != pairs.src[i] && put.slot[r] != pairs.dst[i]) continue;
                if (pairs.skip[i][0] < 0 || pairs.skip[i][0] == put.row[r]) {
                    pairs.skip[i][0] = put.row[r];
                } else if (pairs.skip[i][1] < 0 || pairs.skip[i][1] == put.row[r]) {
                    pairs.skip[i][1] = put.row[r];
                } else {
                    return -1;  // more than two written rows in one pair's chunks: not a beam step
                }
            }
        }
        // the row writers ride along with the first launch
        const int put_here = (i0 == 0) ? n_rows : 0;
        const int put_wgs = (put_here * a.H * units_per_row + per_pair * WG - 1) / (per_pair * WG);
        hipLaunchKernelGGL(copy_chunks_kernel, dim3(per_pair, m + put_wgs), dim3(WG), 0, st, kp, vp, pairs, m, units,
                           units_per_row, a.C, static_cast<const uint4*>(k), static_cast<const uint4*>(v), put,
                           put_here, a.H);
        CA_LAUNCH_CHECK();
    }
    return 0;
}

int launch_put_rows(const LaunchArgs& a, const void* k, const void* v, const int32_t* slot_row, int n,
                    hipStream_t st) {
    void* kp = const_cast<void*>(a.kpool);
    void* vp = const_cast<void*>(a.vpool);
    for (int i0 = 0; i0 < n; i0 += PUT_ROWS) {
        const int m = (n - i0 < PUT_ROWS) ? (n - i0) : PUT_ROWS;
        PutTargets t;
        for (int i = 0; i < PUT_ROWS; i++) {
            t.slot[i] = (i < m) ? slot_row[2 * (i0 + i)] : 0;
            t.row[i] = (i < m) ? slot_row[2 * (i0 + i) + 1] : 0;
        }
        if (a.d % 8 == 0) {
            const int pieces = a.d / 8, total = m * a.H * pieces;
            hipLaunchKernelGGL(put_rows_kernel<uint4>, dim3((total + WG - 1) / WG), dim3(WG), 0, st,
                               static_cast<const uint4*>(k), static_cast<const uint4*>(v), static_cast<uint4*>(kp),
                               static_cast<uint4*>(vp), t, i0, m, a.H, a.C, pieces);
        } else {
            const int pieces = a.d, total = m * a.H * pieces;
            hipLaunchKernelGGL(put_rows_kernel<uint16_t>, dim3((total + WG - 1) / WG), dim3(WG), 0, st,
                               static_cast<const uint16_t*>(k), static_cast<const uint16_t*>(v),
                               static_cast<uint16_t*>(kp), static_cast<uint16_t*>(vp), t, i0, m, a.H, a.C, pieces);
        }
        CA_LAUNCH_CHECK();
    }
    return 0;
}

}  // namespace ca
