// RMS normalisation for gfx950 (MI355X), fp16 rows, fp32 statistics: the two operators the
// reference exports beside rotary_embedding (cpp/chunk_attn/layernorm_kernels.cu:23-117,
// python_exports_ops.cpp:16-18).  One workgroup per token row; 16-byte accesses when the row
// length allows; the second pass re-reads the row from cache.
//
//   rms_norm            out = fp16(x * rsqrt(mean(x^2) + eps)) * weight
//   fused_add_rms_norm  residual = fp16(input + residual);  input = fp16(residual * rsqrt(...)) * weight
//                       with the mean taken over the unrounded fp32 sums, as the reference does
// Rounding points are the reference's: the normalised value is rounded to fp16, then multiplied
// by the weight in fp16.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "kernels.h"

namespace ca {
namespace {

typedef _Float16 half_t;
typedef half_t h8 __attribute__((ext_vector_type(8)));

constexpr int WG = 256;

__device__ __forceinline__ float block_sum(float v, float* sm) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) sm[w] = v;
    __syncthreads();
    return sm[0] + sm[1] + sm[2] + sm[3];
}

// VEC = 8: rows are multiples of 8 elements and 16-byte aligned; VEC = 1: any row length.
// With VEC = 8 a thread keeps the first KEEP pieces it reads (rows of up to KEEP * 2048 elements
// entirely) in registers between the two passes, so the row is read from memory once; longer rows
// re-read the rest.
constexpr int KEEP = 4;

// One 8-element piece of the first pass: returns its contribution to the sum of squares and
// leaves in x what the second pass normalises (with ADD: the rounded sum, also written to residual).
template <bool ADD>
__device__ __forceinline__ float first_pass8(h8& x, half_t* __restrict__ residual_piece) {
    float ss = 0.f;
    if constexpr (ADD) {
        const h8 r = *reinterpret_cast<const h8*>(residual_piece);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float s = float(x[e]) + float(r[e]);
            ss += s * s;
            x[e] = half_t(s);
        }
        *reinterpret_cast<h8*>(residual_piece) = x;
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) ss += float(x[e]) * float(x[e]);
    }
    return ss;
}

__device__ __forceinline__ h8 second_pass8(const h8 x, const h8 w, float inv) {
    h8 y;
#pragma unroll
    for (int e = 0; e < 8; e++) y[e] = half_t(float(x[e]) * inv) * w[e];
    return y;
}

template <int VEC, bool ADD>
__global__ __launch_bounds__(WG) void rms_norm_kernel(half_t* __restrict__ out, half_t* __restrict__ input,
                                                      half_t* __restrict__ residual,
                                                      const half_t* __restrict__ weight, float epsilon,
                                                      int hidden) {
    __shared__ float sm[4];
    const size_t row = size_t(blockIdx.x) * hidden;
    const half_t* src = ADD ? residual : input;
    half_t* dst = ADD ? input : out;
    float ss = 0.f;
    if constexpr (VEC == 8) {
        h8 kept[KEEP];
#pragma unroll
        for (int it = 0; it < KEEP; it++) {  // the loads of all kept pieces go out together
            const int idx = (threadIdx.x + it * WG) * 8;
            if (idx < hidden) kept[it] = *reinterpret_cast<const h8*>(input + row + idx);
        }
#pragma unroll
        for (int it = 0; it < KEEP; it++) {
            const int idx = (threadIdx.x + it * WG) * 8;
            if (idx < hidden) ss += first_pass8<ADD>(kept[it], ADD ? residual + row + idx : nullptr);
        }
        for (int idx = (threadIdx.x + KEEP * WG) * 8; idx < hidden; idx += WG * 8) {
            h8 x = *reinterpret_cast<const h8*>(input + row + idx);
            ss += first_pass8<ADD>(x, ADD ? residual + row + idx : nullptr);
        }
        const float inv = __builtin_amdgcn_rsqf(block_sum(ss, sm) / float(hidden) + epsilon);
#pragma unroll
        for (int it = 0; it < KEEP; it++) {
            const int idx = (threadIdx.x + it * WG) * 8;
            if (idx < hidden) {
                *reinterpret_cast<h8*>(dst + row + idx) =
                  second_pass8(kept[it], *reinterpret_cast<const h8*>(weight + idx), inv);
            }
        }
        // (with ADD, a thread re-reads here only what it wrote above itself)
        for (int idx = (threadIdx.x + KEEP * WG) * 8; idx < hidden; idx += WG * 8) {
            *reinterpret_cast<h8*>(dst + row + idx) =
              second_pass8(*reinterpret_cast<const h8*>(src + row + idx), *reinterpret_cast<const h8*>(weight + idx), inv);
        }
    } else {
        for (int idx = threadIdx.x; idx < hidden; idx += WG) {
            float s = float(input[row + idx]);
            if constexpr (ADD) {
                s += float(residual[row + idx]);
                residual[row + idx] = half_t(s);
            }
            ss += s * s;
        }
        const float inv = __builtin_amdgcn_rsqf(block_sum(ss, sm) / float(hidden) + epsilon);
        for (int idx = threadIdx.x; idx < hidden; idx += WG) {
            dst[row + idx] = half_t(float(src[row + idx]) * inv) * weight[idx];
        }
    }
}

}  // namespace

int launch_rms_norm(void* out, void* input, void* residual, const void* weight, float epsilon,
                    int64_t n_tokens, int hidden, bool vec8, hipStream_t st) {
    if (n_tokens <= 0 || hidden <= 0) return 0;
    if (n_tokens > 0x7fffffff) return -1;
    const dim3 grid(static_cast<unsigned>(n_tokens)), block(WG);
    half_t* o = static_cast<half_t*>(out);
    half_t* in = static_cast<half_t*>(input);
    half_t* res = static_cast<half_t*>(residual);
    const half_t* w = static_cast<const half_t*>(weight);
    if (residual) {
        if (vec8) hipLaunchKernelGGL((rms_norm_kernel<8, true>), grid, block, 0, st, o, in, res, w, epsilon, hidden);
        else hipLaunchKernelGGL((rms_norm_kernel<1, true>), grid, block, 0, st, o, in, res, w, epsilon, hidden);
    } else {
        if (vec8) hipLaunchKernelGGL((rms_norm_kernel<8, false>), grid, block, 0, st, o, in, res, w, epsilon, hidden);
        else hipLaunchKernelGGL((rms_norm_kernel<1, false>), grid, block, 0, st, o, in, res, w, epsilon, hidden);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : static_cast<int>(e);
}

}  // namespace ca
