// Rotary position embedding for gfx950 (MI355X), fp16 data, fp32 arithmetic rounded once.
//
//   rotary_kernel        the in-place operator on query and key rows of any head size
//                        (reference: cpp/chunk_attn/pos_encoding_kernels.cu:24-92).
//   rope_append_kernel   the decode step's three memory passes in one launch: rotate the new
//                        query rows in place, rotate the new key rows on their way into each
//                        sequence's last chunk, and copy the value rows beside them
//                        (reference sequence: src/chunk_attn/models/llama_hf/modeling_llama.py:62,
//                        91-95 = rotary_embedding, then append_token -> append_kv_kernel,
//                        cpp/chunk_attn/kernel_cuda.cu:1088-1115).
//
// cos_sin_cache row p holds cos(p * f_r), r < rot_dim/2, then sin(p * f_r).  NeoX style pairs
// element r with r + rot_dim/2; GPT-J style pairs 2r with 2r+1.  Elements past rot_dim pass
// through unchanged.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernels.h"
#include "rotary_math.h"

namespace ca {
namespace {

using rotary::clamp_pos;
using rotary::h4;
using rotary::h8;
using rotary::half_t;
using rotary::rot_elem;

constexpr int WG = 256;

// One thread rotates one (x, y) pair.  rows: query rows first, then key rows.
template <bool IS_NEOX>
__global__ __launch_bounds__(WG) void rotary_kernel(const int64_t* __restrict__ positions,
                                                    half_t* __restrict__ query,
                                                    half_t* __restrict__ key,
                                                    const half_t* __restrict__ cache,
                                                    int64_t n_tokens, int n_heads, int n_kv_heads,
                                                    int head_size, int rot_dim, int max_position,
                                                    int64_t query_stride, int64_t key_stride) {
    const int embed = rot_dim / 2;
    const int64_t per_token = int64_t(n_heads + n_kv_heads) * embed;
    const int64_t idx = int64_t(blockIdx.x) * WG + threadIdx.x;
    if (idx >= n_tokens * per_token) return;
    const int64_t token = idx / per_token;
    const int rem = static_cast<int>(idx % per_token);
    const int head = rem / embed, r = rem % embed;
    half_t* row = (head < n_heads) ? query + token * query_stride + int64_t(head) * head_size
                                   : key + token * key_stride + int64_t(head - n_heads) * head_size;
    const half_t* cs = cache + clamp_pos(positions[token], max_position) * rot_dim;
    const float c = float(cs[r]), s = float(cs[embed + r]);
    const int xi = IS_NEOX ? r : 2 * r;
    const int yi = IS_NEOX ? embed + r : 2 * r + 1;
    const float x = float(row[xi]), y = float(row[yi]);
    row[xi] = half_t(rot_elem(x, y, c, s, true));
    row[yi] = half_t(rot_elem(y, x, c, s, false));
}

// The same operator for rows made of whole 16-byte pieces (head_size, strides and, NeoX style,
// rot_dim / 2 multiples of 8; GPT-J style rot_dim a multiple of 8; 16-byte aligned pointers): one
// thread rotates 8 pairs (NeoX: the pieces at r0 and r0 + rot_dim/2) or 4 pairs (GPT-J: one
// piece), so every load and store moves 16 bytes per lane.  Same arithmetic as rotary_kernel.
template <bool IS_NEOX>
__global__ __launch_bounds__(WG) void rotary_vec_kernel(const int64_t* __restrict__ positions,
                                                        half_t* __restrict__ query,
                                                        half_t* __restrict__ key,
                                                        const half_t* __restrict__ cache,
                                                        int64_t n_tokens, int n_heads, int n_kv_heads,
                                                        int head_size, int rot_dim, int max_position,
                                                        int64_t query_stride, int64_t key_stride) {
    const int embed = rot_dim / 2;
    const int units = IS_NEOX ? embed / 8 : rot_dim / 8;  // work units per head
    const int64_t per_token = int64_t(n_heads + n_kv_heads) * units;
    const int64_t idx = int64_t(blockIdx.x) * WG + threadIdx.x;
    if (idx >= n_tokens * per_token) return;
    const int64_t token = idx / per_token;
    const int rem = static_cast<int>(idx % per_token);
    const int head = rem / units, u = rem % units;
    half_t* row = (head < n_heads) ? query + token * query_stride + int64_t(head) * head_size
                                   : key + token * key_stride + int64_t(head - n_heads) * head_size;
    const half_t* cs = cache + clamp_pos(positions[token], max_position) * rot_dim;
    if constexpr (IS_NEOX) {
        const int r0 = 8 * u;
        h8 x = *reinterpret_cast<const h8*>(row + r0);
        h8 y = *reinterpret_cast<const h8*>(row + embed + r0);
        const h8 c8 = *reinterpret_cast<const h8*>(cs + r0);
        const h8 s8 = *reinterpret_cast<const h8*>(cs + embed + r0);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float xf = float(x[e]), yf = float(y[e]), c = float(c8[e]), sn = float(s8[e]);
            x[e] = half_t(rot_elem(xf, yf, c, sn, true));
            y[e] = half_t(rot_elem(yf, xf, c, sn, false));
        }
        *reinterpret_cast<h8*>(row + r0) = x;
        *reinterpret_cast<h8*>(row + embed + r0) = y;
    } else {
        h8 v = *reinterpret_cast<const h8*>(row + 8 * u);
        const h4 c4 = *reinterpret_cast<const h4*>(cs + 4 * u);
        const h4 s4 = *reinterpret_cast<const h4*>(cs + embed + 4 * u);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float xf = float(v[2 * e]), yf = float(v[2 * e + 1]), c = float(c4[e]), sn = float(s4[e]);
            v[2 * e] = half_t(rot_elem(xf, yf, c, sn, true));
            v[2 * e + 1] = half_t(rot_elem(yf, xf, c, sn, false));
        }
        *reinterpret_cast<h8*>(row + 8 * u) = v;
    }
}

// One thread owns 8 consecutive elements of one (sequence, head) row of q, k or v:
// units [0, n) are query rows, [n, 2n) key rows, [2n, 3n) value rows, n = n_seqs * H * d/8.
// Requires d % 8 == 0 and, NeoX style, rot_dim % 16 == 0 (the pairing partner is then another
// whole 8-element piece); GPT-J pairs stay inside a piece.
template <bool IS_NEOX>
__global__ __launch_bounds__(WG) void rope_append_kernel(
    const int64_t* __restrict__ positions, const int32_t* __restrict__ seq_len,
    half_t* __restrict__ q, const half_t* __restrict__ k, const half_t* __restrict__ v,
    half_t* __restrict__ kpool, half_t* __restrict__ vpool, const half_t* __restrict__ cache,
    const int32_t* __restrict__ tail_slot, const int32_t* __restrict__ tail_fill, int delta_tokens,
    int n_seqs, int H, int C, int d, int rot_dim, int max_position) {
    const int pieces = d / 8;
    const int n = n_seqs * H * pieces;
    const int idx = blockIdx.x * WG + threadIdx.x;
    if (idx >= 3 * n) return;
    const int role = idx / n, unit = idx % n;  // 0 q, 1 k, 2 v
    const int piece = unit % pieces, sh = unit / pieces, h = sh % H, seq = sh / H;
    const int row = tail_fill[seq] + delta_tokens;
    const size_t src = size_t(sh) * d + 8 * piece;
    const size_t dst = ((size_t(tail_slot[seq]) * H + h) * C + row) * d + 8 * piece;
    if (role == 2) {
        if (row >= 0 && row < C) *reinterpret_cast<h8*>(vpool + dst) = *reinterpret_cast<const h8*>(v + src);
        return;
    }
    const half_t* in = (role == 0) ? q : k;
    h8 own = *reinterpret_cast<const h8*>(in + src);
    if (8 * piece < rot_dim) {
        const int64_t pos = positions ? positions[seq] : int64_t(seq_len[seq]) + delta_tokens;
        const half_t* cs = cache + clamp_pos(pos, max_position) * rot_dim;
        // NeoX style: the partner piece is read before any lane of this wave stores (one wave holds
        // whole rows: d/8 lanes per row divide 64), so rotating q in place is safe
        own = rotary::rotate_piece<IS_NEOX>(in + size_t(sh) * d, 8 * piece, own, cs, rot_dim);
    }
    if (role == 0) {
        *reinterpret_cast<h8*>(q + src) = own;
    } else if (row >= 0 && row < C) {  // host guarantees a free row; never write outside the chunk
        *reinterpret_cast<h8*>(kpool + dst) = own;
    }
}

}  // namespace

#define CA_LAUNCH_CHECK()                                        \
    do {                                                         \
        hipError_t e_ = hipGetLastError();                       \
        if (e_ != hipSuccess) return static_cast<int>(e_);       \
    } while (0)

int launch_rotary(const RotaryArgs& r, hipStream_t st) {
    half_t* q = static_cast<half_t*>(r.query);
    half_t* k = static_cast<half_t*>(r.key);
    const half_t* cache = static_cast<const half_t*>(r.cos_sin_cache);
    auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool pieces = r.head_size % 8 == 0 && r.rot_dim % (r.is_neox ? 16 : 8) == 0 &&
                        r.query_stride % 8 == 0 && r.key_stride % 8 == 0 && aligned16(q) && aligned16(k) &&
                        aligned16(cache);
    if (pieces) {
        const int units = r.is_neox ? r.rot_dim / 16 : r.rot_dim / 8;
        const int64_t total = r.n_tokens * int64_t(r.n_heads + r.n_kv_heads) * units;
        if (total <= 0) return 0;
        if (total > int64_t(0x7fffffff) * WG) return -1;
        const dim3 grid(static_cast<unsigned>((total + WG - 1) / WG)), block(WG);
        if (r.is_neox) {
            hipLaunchKernelGGL(rotary_vec_kernel<true>, grid, block, 0, st, r.positions, q, k, cache, r.n_tokens,
                               r.n_heads, r.n_kv_heads, r.head_size, r.rot_dim, r.max_position,
                               r.query_stride, r.key_stride);
        } else {
            hipLaunchKernelGGL(rotary_vec_kernel<false>, grid, block, 0, st, r.positions, q, k, cache, r.n_tokens,
                               r.n_heads, r.n_kv_heads, r.head_size, r.rot_dim, r.max_position,
                               r.query_stride, r.key_stride);
        }
        CA_LAUNCH_CHECK();
        return 0;
    }
    const int64_t total = r.n_tokens * int64_t(r.n_heads + r.n_kv_heads) * (r.rot_dim / 2);
    if (total <= 0) return 0;
    if (total > int64_t(0x7fffffff) * WG) return -1;
    const dim3 grid(static_cast<unsigned>((total + WG - 1) / WG)), block(WG);
    if (r.is_neox) {
        hipLaunchKernelGGL(rotary_kernel<true>, grid, block, 0, st, r.positions, q, k, cache, r.n_tokens,
                           r.n_heads, r.n_kv_heads, r.head_size, r.rot_dim, r.max_position,
                           r.query_stride, r.key_stride);
    } else {
        hipLaunchKernelGGL(rotary_kernel<false>, grid, block, 0, st, r.positions, q, k, cache, r.n_tokens,
                           r.n_heads, r.n_kv_heads, r.head_size, r.rot_dim, r.max_position,
                           r.query_stride, r.key_stride);
    }
    CA_LAUNCH_CHECK();
    return 0;
}

int launch_rope_append(const LaunchArgs& a, const RotaryArgs& r, const void* k, const void* v,
                       const int32_t* seq_len, const int32_t* tail_slot, const int32_t* tail_fill,
                       int n_seqs, hipStream_t st) {
    if (n_seqs <= 0) return 0;
    if (a.d % 8 != 0 || r.rot_dim % (r.is_neox ? 16 : 8) != 0 || r.rot_dim > a.d) return -1;
    if ((64 % (a.d / 8)) != 0) return -1;  // whole rows per wave (in-place query rotation)
    const int64_t total = int64_t(3) * n_seqs * a.H * (a.d / 8);
    if (total > 0x7fffffff) return -1;
    const dim3 grid(static_cast<unsigned>((total + WG - 1) / WG)), block(WG);
    half_t* kp = static_cast<half_t*>(const_cast<void*>(a.kpool));
    half_t* vp = static_cast<half_t*>(const_cast<void*>(a.vpool));
    half_t* q = static_cast<half_t*>(r.query);
    const half_t* cache = static_cast<const half_t*>(r.cos_sin_cache);
    if (r.is_neox) {
        hipLaunchKernelGGL(rope_append_kernel<true>, grid, block, 0, st, r.positions, seq_len, q,
                           static_cast<const half_t*>(k), static_cast<const half_t*>(v), kp, vp, cache,
                           tail_slot, tail_fill, a.delta_tokens, n_seqs, a.H, a.C, a.d, r.rot_dim,
                           r.max_position);
    } else {
        hipLaunchKernelGGL(rope_append_kernel<false>, grid, block, 0, st, r.positions, seq_len, q,
                           static_cast<const half_t*>(k), static_cast<const half_t*>(v), kp, vp, cache,
                           tail_slot, tail_fill, a.delta_tokens, n_seqs, a.H, a.C, a.d, r.rot_dim,
                           r.max_position);
    }
    CA_LAUNCH_CHECK();
    return 0;
}

}  // namespace ca
