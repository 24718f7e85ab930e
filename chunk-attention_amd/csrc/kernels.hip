// HIP kernels of the ChunkAttention decode path for gfx950 (MI355X), fp16 K/V/Q, d_head 128.
//
//   shared_kernel   chunk-first phase: one workgroup attends a segment of shared chunks for up
//                   to 64 sequences at once on the matrix cores (S^T = K.Q^T, O^T = V^T.P^T)
//                   and writes one partial (max, sum, acc) row per sequence.
//   stream_kernel   sequence-first phase: one workgroup streams a run of one sequence's own
//                   chunks at HBM speed (16-byte coalesced loads, fp32 online softmax) and
//                   writes one partial row, or the final output when nothing else is merged.
//   merge_kernel    combines the partial rows of every (sequence, head) and normalises.
//   append_kernel / scatter_kernel   K/V row writes into the chunk pool.
//
// Partial rows live in base-2 units: max holds score*log2(e)/sqrt(d), sums and acc are
// relative to 2^max.  Row layout: [0] max, [1] sum, [4..131] acc (fp32).
#include <hip/hip_runtime.h>

#include <cstdint>

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
// stream_kernel: grid = n_items * H workgroups.  Wave w of a workgroup takes chunks
// w, w+4, ... of the item; a chunk is read as 64-token sub-tiles (32 for chunk_size 32).
// Lane l = 16*g + j reads, for load i, the 16 bytes at offset 1024*i + 16*l of a sub-tile:
// row 4*i + g, dims 8*j..8*j+7, so every load instruction covers 1 KiB of contiguous memory.
// ---------------------------------------------------------------------------------------
template <int C>
__global__ __launch_bounds__(WG) void stream_kernel(
  const half_t* __restrict__ q, const half_t* __restrict__ kpool,
  const half_t* __restrict__ vpool, half_t* __restrict__ out, float* __restrict__ part,
  const WorkItem* __restrict__ items, const int32_t* __restrict__ slots,
  const int32_t* __restrict__ seq_len, int delta_tokens, int H, float scale_log2) {
    constexpr int SUB = (C < 64) ? C : 64;  // tokens per sub-tile
    constexpr int NL = SUB / 4;             // 16-byte loads per lane per sub-tile
    constexpr int NSUB = C / SUB;

    const int h = blockIdx.x % H;
    const WorkItem it = items[blockIdx.x / H];
    const int tid = threadIdx.x;
    const int w = tid >> 6, l = tid & 63, g = l >> 4, j = l & 15;
    const int seq = it.seq_begin;
    const int len = seq_len[it.len_seq] + delta_tokens;

    __shared__ float sm_p[NW][64];
    __shared__ float sm_o[NW][D];
    __shared__ float sm_m[NW], sm_l[NW];

    const h8 qv = *reinterpret_cast<const h8*>(q + (size_t(seq) * H + h) * D + 8 * j);

    float m_run = NEG_INF, l_lane = 0.f;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;

    for (int t = w; t < it.n_chunks; t += NW) {
        int valid = len - (it.pos0 + t) * C;
        if (valid <= 0) break;  // chunks are in path order: everything after is empty too
        valid = valid < C ? valid : C;
        const int slot = slots[it.slot_first + t];
        const size_t base = (size_t(slot) * H + h) * size_t(C) * D;
#pragma unroll
        for (int sub = 0; sub < NSUB; sub++) {
            const int vsub = valid - sub * SUB;  // valid rows in this sub-tile
            if (vsub <= 0) break;
            const bool masked = vsub < SUB;
            const uint4* kp = reinterpret_cast<const uint4*>(kpool + base + size_t(sub) * SUB * D) + l;
            const uint4* vp = reinterpret_cast<const uint4*>(vpool + base + size_t(sub) * SUB * D) + l;
            uint4 kr[NL], vr[NL];
            if (!masked) {
#pragma unroll
                for (int i = 0; i < NL; i++) kr[i] = kp[64 * i];
#pragma unroll
                for (int i = 0; i < NL; i++) vr[i] = vp[64 * i];
            } else {
                // rows past the end of the sequence hold stale data: never read into the math
#pragma unroll
                for (int i = 0; i < NL; i++) {
                    const bool ok = 4 * i + g < vsub;
                    kr[i] = ok ? kp[64 * i] : make_uint4(0, 0, 0, 0);
                    vr[i] = ok ? vp[64 * i] : make_uint4(0, 0, 0, 0);
                }
            }
            float sc[NL];
#pragma unroll
            for (int i = 0; i < NL; i++) {
                sc[i] = dot8(*reinterpret_cast<const h8*>(&kr[i]), qv, 0.f);
            }
            // lane (g, j) now owns the score of row 4*(j % NL) + g
            float s = reduce_rows16<NL>(sc, j) * scale_log2;
            const int row = 4 * (j % NL) + g;
            if (row >= vsub || j >= NL) s = NEG_INF;
            const float m_new = fmaxf(m_run, wave_max(s));
            const float alpha = fast_exp2(m_run - m_new);
            const float p = fast_exp2(s - m_new);
            m_run = m_new;
            l_lane = l_lane * alpha + p;
            sm_p[w][l] = p;
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] *= alpha;
            __builtin_amdgcn_wave_barrier();
            float pr[NL];
#pragma unroll
            for (int i = 0; i < NL; i += 4) {
                const f4 t4 = *reinterpret_cast<const f4*>(&sm_p[w][16 * g + i]);
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
    }

    // wave result: rows are spread over the four 16-lane groups
    const float l_wave = wave_sum(l_lane);
#pragma unroll
    for (int e = 0; e < 8; e++) {
        acc[e] += shfl_xor(acc[e], 16);
        acc[e] += shfl_xor(acc[e], 32);
    }
    if (g == 0) {
#pragma unroll
        for (int e = 0; e < 8; e++) sm_o[w][8 * j + e] = acc[e];
    }
    if (l == 0) {
        sm_m[w] = m_run;
        sm_l[w] = l_wave;
    }
    __syncthreads();

    if (tid < D) {
        float m = sm_m[0];
#pragma unroll
        for (int k = 1; k < NW; k++) m = fmaxf(m, sm_m[k]);
        float o = 0.f, lsum = 0.f;
#pragma unroll
        for (int k = 0; k < NW; k++) {
            const float f = (sm_m[k] == NEG_INF) ? 0.f : fast_exp2(sm_m[k] - m);
            o += f * sm_o[k][tid];
            lsum += f * sm_l[k];
        }
        if (it.part_row >= 0) {
            float* row = part + (size_t(it.part_row) * H + h) * PART_STRIDE;
            row[4 + tid] = o;
            if (tid == 0) {
                row[0] = m;
                row[1] = lsum;
            }
        } else {
            const float r = lsum > 0.f ? 1.f / lsum : 0.f;
            out[(size_t(seq) * H + h) * D + tid] = half_t(o * r);
        }
    }
}

// ---------------------------------------------------------------------------------------
// shared_kernel: grid = n_items * H workgroups; an item = (segment of chunks, up to 16*MB
// sequences).  The segment is one token stream cut into 16-token blocks; wave w takes blocks
// w, w+4, ...  and keeps its own online-softmax state, so waves never wait for each other
// until the final merge.
//
// Matrix-core operand layout (v_mfma_f32_16x16x*: lane l = 16*g + i):
//   A holds row i, B holds column i, each with the k-slice of group g; D holds rows 4g..4g+3
//   of column i.  S^T block = K_blk(16 tokens x 128) . Q^T  -> lane owns scores of tokens
//   4g..4g+3 for sequence i, which is exactly the B operand of O^T = V^T . P^T (k = 16
//   tokens), so probabilities never leave registers.  V^T comes from a wave-private LDS copy
//   of the 16 x 128 V block read column-wise.
// ---------------------------------------------------------------------------------------
constexpr int VPITCH = D + 4;  // halves per LDS row of the V block: 264 B keeps the four
                               // token groups on disjoint banks for 2-byte column reads
constexpr int OPITCH = D + 4;  // floats per row of the cross-wave accumulation buffer

template <int C, int MB>
__global__ __launch_bounds__(WG) void shared_kernel(
  const half_t* __restrict__ q, const half_t* __restrict__ kpool,
  const half_t* __restrict__ vpool, float* __restrict__ part,
  const WorkItem* __restrict__ items, const int32_t* __restrict__ slots,
  const int32_t* __restrict__ seq_len, int delta_tokens, int H, float scale_log2) {
    const int h = blockIdx.x % H;
    const WorkItem it = items[blockIdx.x / H];
    const int tid = threadIdx.x;
    const int w = tid >> 6, l = tid & 63, g = l >> 4, i = l & 15;
    const int len = seq_len[it.len_seq] + delta_tokens;

    __shared__ __attribute__((aligned(16))) half_t sm_v[NW][16 * VPITCH];
    __shared__ __attribute__((aligned(16))) float sm_o[MB * 16 * OPITCH];
    __shared__ float sm_m[NW][MB * 16];
    __shared__ float sm_l[NW][MB * 16];

    // Q^T operand: sequence row mb*16+i, dims 32*ks + 8*g .. +7
    h8 qreg[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int row = mb * 16 + i;
        const half_t* qp = q + (size_t(it.seq_begin + row) * H + h) * D + 8 * g;
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

    const int n_blocks = it.n_chunks * (C / 16);
    for (int tb = w; tb < n_blocks; tb += NW) {
        const int ck = tb / (C / 16);
        const int row0 = (tb % (C / 16)) * 16;
        int valid = len - (it.pos0 + ck) * C - row0;  // valid tokens in this block
        if (valid <= 0) break;
        const int slot = slots[it.slot_first + ck];
        const size_t base = ((size_t(slot) * H + h) * size_t(C) + row0) * D;

        h8 kreg[4];
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            kreg[ks] = *reinterpret_cast<const h8*>(kpool + base + size_t(i) * D + 32 * ks + 8 * g);
        }
        uint4 vraw[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            vraw[r] = *(reinterpret_cast<const uint4*>(vpool + base) + 64 * r + l);
            if (4 * r + g >= valid) vraw[r] = make_uint4(0, 0, 0, 0);  // stale rows past the end
        }
        // V block -> LDS rows (row 4r+g, dims 8i..8i+7)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            uint2* dst = reinterpret_cast<uint2*>(&sm_v[w][(4 * r + g) * VPITCH + 8 * i]);
            dst[0] = make_uint2(vraw[r].x, vraw[r].y);
            dst[1] = make_uint2(vraw[r].z, vraw[r].w);
        }

        h4 pb[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            f4 s = f4{ 0.f, 0.f, 0.f, 0.f };
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                s = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg[ks], qreg[mb][ks], s, 0, 0, 0);
            }
            float mx = NEG_INF;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                s[r] = (4 * g + r < valid) ? s[r] * scale_log2 : NEG_INF;
                mx = fmaxf(mx, s[r]);
            }
            mx = fmaxf(mx, shfl_xor(mx, 16));
            mx = fmaxf(mx, shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run[mb], mx);
            const float alpha = fast_exp2(m_run[mb] - m_new);
            m_run[mb] = m_new;
            float psum = 0.f;
            float p[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                p[r] = fast_exp2(s[r] - m_new);
                psum += p[r];
            }
            l_lane[mb] = l_lane[mb] * alpha + psum;
            pb[mb] = h4{ half_t(p[0]), half_t(p[1]), half_t(p[2]), half_t(p[3]) };
#pragma unroll
            for (int db = 0; db < 8; db++) oacc[mb][db] *= alpha;
        }

        __builtin_amdgcn_wave_barrier();
        // O^T += V^T . P^T : A = V^T (row = dim 16*db + i, k = tokens 4g..4g+3)
#pragma unroll
        for (int db = 0; db < 8; db++) {
            const half_t* col = &sm_v[w][(4 * g) * VPITCH + 16 * db + i];
            const h4 a = h4{ col[0], col[VPITCH], col[2 * VPITCH], col[3 * VPITCH] };
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                oacc[mb][db] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, pb[mb], oacc[mb][db], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }

    // ---- merge the four waves ------------------------------------------------------------
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        l_lane[mb] += shfl_xor(l_lane[mb], 16);
        l_lane[mb] += shfl_xor(l_lane[mb], 32);
        if (g == 0) sm_m[w][mb * 16 + i] = m_run[mb];
    }
    __syncthreads();
    float m_all[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        float m = sm_m[0][mb * 16 + i];
#pragma unroll
        for (int k = 1; k < NW; k++) m = fmaxf(m, sm_m[k][mb * 16 + i]);
        m_all[mb] = m;
        const float f = (m_run[mb] == NEG_INF) ? 0.f : fast_exp2(m_run[mb] - m);
        if (g == 0) sm_l[w][mb * 16 + i] = l_lane[mb] * f;
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
                    f4* dst = reinterpret_cast<f4*>(&sm_o[(mb * 16 + i) * OPITCH + 16 * db + 4 * g]);
                    *dst = (k == 0) ? oacc[mb][db] : (*dst + oacc[mb][db]);
                }
            }
        }
        __syncthreads();
    }

    // ---- write the partial rows ------------------------------------------------------------
    for (int idx = tid; idx < it.n_rows * (D / 4); idx += WG) {
        const int row = idx / (D / 4), c4 = idx % (D / 4);
        float* dst = part + (size_t(it.part_row + row) * H + h) * PART_STRIDE;
        *reinterpret_cast<f4*>(dst + 4 + 4 * c4) = *reinterpret_cast<const f4*>(&sm_o[row * OPITCH + 4 * c4]);
    }
    if (w == 0 && g == 0) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            const int row = mb * 16 + i;
            if (row < it.n_rows) {
                float lsum = 0.f;
#pragma unroll
                for (int k = 0; k < NW; k++) lsum += sm_l[k][row];
                float* dst = part + (size_t(it.part_row + row) * H + h) * PART_STRIDE;
                dst[0] = m_all[mb];
                dst[1] = lsum;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// merge_kernel: one wave per (sequence, head); lane owns two output dims.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(WG) void merge_kernel(const float* __restrict__ part,
                                                   half_t* __restrict__ out,
                                                   const int32_t* __restrict__ part_ptr,
                                                   const int32_t* __restrict__ part_rows,
                                                   int n_seqs, int H) {
    const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
    const int sh = blockIdx.x * NW + w;
    if (sh >= n_seqs * H) return;
    const int seq = sh / H, h = sh % H;
    const int p0 = part_ptr[seq], p1 = part_ptr[seq + 1];
    if (p0 == p1) return;  // written directly by a stream item

    float m = NEG_INF;
    for (int p = p0 + l; p < p1; p += 64) {
        m = fmaxf(m, part[(size_t(part_rows[p]) * H + h) * PART_STRIDE]);
    }
    m = wave_max(m);
    float lsum = 0.f;
    f2 o = f2{ 0.f, 0.f };
    for (int p = p0; p < p1; p++) {
        const float* row = part + (size_t(part_rows[p]) * H + h) * PART_STRIDE;
        const float mp = row[0];
        const float f = (mp == NEG_INF) ? 0.f : fast_exp2(mp - m);
        lsum += f * row[1];
        const f2 v = *reinterpret_cast<const f2*>(row + 4 + 2 * l);
        o += f * v;
    }
    const float r = lsum > 0.f ? 1.f / lsum : 0.f;
    h2* dst = reinterpret_cast<h2*>(out + (size_t(seq) * H + h) * D + 2 * l);
    *dst = h2{ half_t(o[0] * r), half_t(o[1] * r) };
}

// ---------------------------------------------------------------------------------------
// K/V row writes.  One thread moves one piece (16 bytes when d_head allows, else 2) of K and V.
// ---------------------------------------------------------------------------------------
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
    if (row >= C) return;  // host guarantees a free row; never write outside the chunk
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

}  // namespace

// ---- launchers -----------------------------------------------------------------------------

#define CA_LAUNCH_CHECK()                                        \
    do {                                                         \
        hipError_t e_ = hipGetLastError();                       \
        if (e_ != hipSuccess) return static_cast<int>(e_);       \
    } while (0)

int launch_stream(const LaunchArgs& a, const WorkItem* items, int n_items, hipStream_t st) {
    if (n_items <= 0) return 0;
    const dim3 grid(static_cast<unsigned>(n_items) * a.H), block(WG);
    const half_t* q = static_cast<const half_t*>(a.q);
    const half_t* kp = static_cast<const half_t*>(a.kpool);
    const half_t* vp = static_cast<const half_t*>(a.vpool);
    half_t* out = static_cast<half_t*>(a.out);
    switch (a.C) {
        case 32:
            hipLaunchKernelGGL(stream_kernel<32>, grid, block, 0, st, q, kp, vp, out, a.part, items,
                               a.slots, a.seq_len, a.delta_tokens, a.H, a.scale_log2);
            break;
        case 64:
            hipLaunchKernelGGL(stream_kernel<64>, grid, block, 0, st, q, kp, vp, out, a.part, items,
                               a.slots, a.seq_len, a.delta_tokens, a.H, a.scale_log2);
            break;
        case 128:
            hipLaunchKernelGGL(stream_kernel<128>, grid, block, 0, st, q, kp, vp, out, a.part, items,
                               a.slots, a.seq_len, a.delta_tokens, a.H, a.scale_log2);
            break;
        default:
            return -1;
    }
    CA_LAUNCH_CHECK();
    return 0;
}

template <int C>
static int launch_shared_c(const LaunchArgs& a, const WorkItem* items, int n_items, int mb,
                           hipStream_t st) {
    const dim3 grid(static_cast<unsigned>(n_items) * a.H), block(WG);
    const half_t* q = static_cast<const half_t*>(a.q);
    const half_t* kp = static_cast<const half_t*>(a.kpool);
    const half_t* vp = static_cast<const half_t*>(a.vpool);
    switch (mb) {
        case 1:
            hipLaunchKernelGGL((shared_kernel<C, 1>), grid, block, 0, st, q, kp, vp, a.part, items,
                               a.slots, a.seq_len, a.delta_tokens, a.H, a.scale_log2);
            break;
        case 2:
            hipLaunchKernelGGL((shared_kernel<C, 2>), grid, block, 0, st, q, kp, vp, a.part, items,
                               a.slots, a.seq_len, a.delta_tokens, a.H, a.scale_log2);
            break;
        case 4:
            hipLaunchKernelGGL((shared_kernel<C, 4>), grid, block, 0, st, q, kp, vp, a.part, items,
                               a.slots, a.seq_len, a.delta_tokens, a.H, a.scale_log2);
            break;
        default:
            return -1;
    }
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_shared(const LaunchArgs& a, const WorkItem* items, int n_items, int mb,
                  hipStream_t st) {
    if (n_items <= 0) return 0;
    switch (a.C) {
        case 32: return launch_shared_c<32>(a, items, n_items, mb, st);
        case 64: return launch_shared_c<64>(a, items, n_items, mb, st);
        case 128: return launch_shared_c<128>(a, items, n_items, mb, st);
        default: return -1;
    }
}

int launch_merge(const LaunchArgs& a, const int32_t* part_ptr, const int32_t* part_rows,
                 int n_seqs, hipStream_t st) {
    if (n_seqs <= 0) return 0;
    const int waves = n_seqs * a.H;
    hipLaunchKernelGGL(merge_kernel, dim3((waves + NW - 1) / NW), dim3(WG), 0, st, a.part,
                       static_cast<half_t*>(a.out), part_ptr, part_rows, n_seqs, a.H);
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

}  // namespace ca
