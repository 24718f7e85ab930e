// The arithmetic of the rotary position embedding, shared by the rotary kernels and by the decode
// kernel's fused step (which rotates the new query and key rows in registers): fp16 data, fp32
// arithmetic rounded once.  cos_sin_cache row p holds cos(p * f_r), r < rot_dim/2, then
// sin(p * f_r).  NeoX style pairs element r with r + rot_dim/2; GPT-J style pairs 2r with 2r+1.
// Elements past rot_dim pass through unchanged.
// (reference: cpp/chunk_attn/pos_encoding_kernels.cu:24-92)
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace ca {
namespace rotary {

typedef _Float16 half_t;
typedef half_t h4 __attribute__((ext_vector_type(4)));
typedef half_t h8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ int64_t clamp_pos(int64_t p, int max_position) {
    // never read outside the cache, whatever the caller's positions hold
    return p < 0 ? 0 : (p >= max_position ? int64_t(max_position) - 1 : p);
}

// Every kernel forms the rotation with the same two fp32 operations per element, a rounded
// product and a fused multiply-add:
//   x' = fma(x, cos, -(y * sin)),  y' = fma(y, cos, x * sin)
__device__ __forceinline__ float rot_elem(float own, float other, float c, float s, bool is_x) {
    const float t = other * s;
    return __builtin_fmaf(own, c, is_x ? -t : t);
}

// The 8 consecutive elements `own` = row[d0 .. d0+7] (d0 a multiple of 8) rotated for the position
// whose cos/sin row is `cs`.  NeoX style reads the partner piece from `row`; needs rot_dim a
// multiple of 16 (NeoX) or 8 (GPT-J).
template <bool IS_NEOX>
__device__ __forceinline__ h8 rotate_piece(const half_t* __restrict__ row, int d0, h8 own,
                                           const half_t* __restrict__ cs, int rot_dim) {
    if (d0 >= rot_dim) return own;
    const int embed = rot_dim / 2;
    if constexpr (IS_NEOX) {
        const bool is_x = d0 < embed;
        const int r0 = is_x ? d0 : d0 - embed;
        const h8 other = *reinterpret_cast<const h8*>(row + (is_x ? r0 + embed : r0));
        const h8 c8 = *reinterpret_cast<const h8*>(cs + r0);
        const h8 s8 = *reinterpret_cast<const h8*>(cs + embed + r0);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            own[e] = half_t(rot_elem(float(own[e]), float(other[e]), float(c8[e]), float(s8[e]), is_x));
        }
    } else {
        const h4 c4 = *reinterpret_cast<const h4*>(cs + d0 / 2);
        const h4 s4 = *reinterpret_cast<const h4*>(cs + embed + d0 / 2);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float x = float(own[2 * e]), y = float(own[2 * e + 1]);
            const float c = float(c4[e]), s = float(s4[e]);
            own[2 * e] = half_t(rot_elem(x, y, c, s, true));
            own[2 * e + 1] = half_t(rot_elem(y, x, c, s, false));
        }
    }
    return own;
}

}  // namespace rotary
}  // namespace ca
