// kv_producer_util.hpp -- per-head RMSNorm and rotary embedding of one head vector held by one wave
// (lane l: coordinates l and l + 64), with the reference's roundings (qk_norm_batch_kernel, kernels.cu:880-923;
// rope_batch_kernel, 927-961; rope_kernel, 193-235).  Shared by kv_producer.hip and kv_decode_fused.hip.
//
// Every product is rounded to fp32 before anything else happens to it, as in the reference's separate
// kernels: no fused multiply-add where the source has none, and no multiply fused into the conversion to
// fp16 (one rounding instead of two changes a result in a few hundred thousand).
#pragma once

#include "kv_common.hpp"

namespace twkv {

// sum over the 128 coordinates of a head in the reference's order; lane l passes (x[l], x[l + 64])
__device__ __forceinline__ float head_tree_sum(float a, float b) {
#pragma clang fp contract(off)
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) {     // lanes 0 and 32 end up with the sums of their 32 coordinates
        a += __shfl_down(a, off, 32);
        b += __shfl_down(b, off, 32);
    }
    const float t = a + b;                        // lane 0: s0 + s2, lane 32: s1 + s3
    return __shfl(t, 0, 64) + __shfl(t, 32, 64);
}

struct HeadXform {
    const half_t* weight;   // NULL: no RMSNorm
    float eps;
    int biased;
    const half_t* cos_row;  // NULL: no rotation; row of rope_dim / 2 entries for this position
    const half_t* sin_row;
    int rope_dim;
    int single_order;       // second output as fma(x1, c, x0 * s)
};

// RMSNorm and rotation of one head held as (x0 = coordinate lane, x1 = coordinate lane + 64), with the
// fp16 rounding after each step
__device__ __forceinline__ void xform_head(float& x0, float& x1, int lane, const HeadXform& t) {
#pragma clang fp contract(off)
    if (t.weight) {
        const float sum = head_tree_sum(x0 * x0, x1 * x1);
        const float rms = 1.0f / sqrtf(sum / (float)kHeadDim + t.eps);
        float w0 = (float)t.weight[lane], w1 = (float)t.weight[lane + 64];
        if (t.biased) { w0 += 1.0f; w1 += 1.0f; }
        x0 = as_half_value((x0 * rms) * w0);
        x1 = as_half_value((x1 * rms) * w1);
    }
    if (t.cos_row) {
        const int half = t.rope_dim >> 1;
        if (half == 64) {
            const float c = (float)t.cos_row[lane], s = (float)t.sin_row[lane];
            const float o0 = __builtin_fmaf(x0, c, -(x1 * s));
            const float o1 = t.single_order ? __builtin_fmaf(x1, c, x0 * s) : __builtin_fmaf(x0, s, x1 * c);
            x0 = as_half_value(o0);
            x1 = as_half_value(o1);
        } else {
            // coordinate d < rope_dim pairs with d + half (d < half) or d - half; only x0's coordinates
            // (d = lane < 64) can be inside a partial rotation
            const bool first = lane < half, inside = lane < t.rope_dim;
            const int partner = first ? lane + half : lane - half;
            const float other = __shfl(x0, inside ? partner : lane, 64);
            if (inside) {
                const int j = first ? lane : partner;
                const float c = (float)t.cos_row[j], s = (float)t.sin_row[j];
                const float a = first ? x0 : other, b = first ? other : x0;      // (x_d, x_{d + half})
                const float o = first ? __builtin_fmaf(a, c, -(b * s))
                                      : (t.single_order ? __builtin_fmaf(b, c, a * s) : __builtin_fmaf(a, s, b * c));
                x0 = as_half_value(o);
            }
        }
    }
}

}  // namespace twkv
