// kv_rotate_util.hpp -- pieces shared by the kernels that apply the 128x128 rotation with
// v_mfma_f32_16x16x4_f32 (kv_rotate.hip, kv_decode_fused.hip).  Lane (i = lane % 16, kk = lane / 16) of a wave
// holds, for one row of R and one vector, the coordinates 4s + kk, s = 0..31.
#pragma once

#include "kv_common.hpp"

namespace twkv {

// fp16 at index (4s + kk) of a row held as 16 x (8 halves): s = 2*q + e picks dword (2e + kk/2) of 16-byte
// piece q, half kk%2.
__device__ __forceinline__ float pick_half(const uint4& piece, int e, int kk) {
    uint32_t lo = e ? piece.z : piece.x;
    uint32_t hi = e ? piece.w : piece.y;
    uint32_t w = (kk & 2) ? hi : lo;
    w = (kk & 1) ? (w >> 16) : (w & 0xffffu);
    union { uint16_t u; half_t h; } cv;
    cv.u = (uint16_t)w;
    return (float)cv.h;
}

// Sum of squares of a vector held as xv[s] = coordinate 4s + kk, in the reference's order (kernels.cu:1509-1520):
// a 32-lane shuffle-down tree per group of 32 coordinates -- its offsets 16, 8 and 4 combine coordinates that are
// congruent mod 4, which one lane owns (local j and j+4, j+2, j+1 of the group's 8 registers); offsets 2 and 1
// cross the lane groups kk -- then (s0 + s2) + (s1 + s3) over the four groups.  Every lane of a vector gets the sum.
__device__ __forceinline__ float rotation_tree_sum_sq(const float (&xv)[32]) {
    float sgrp[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        float t[8];
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = xv[8 * w + j] * xv[8 * w + j];
        float a0 = t[0] + t[4], a1 = t[1] + t[5], a2 = t[2] + t[6], a3 = t[3] + t[7];
        float b0 = a0 + a2, b1 = a1 + a3;
        float c = b0 + b1;                                   // c_kk of the tree
        float d = c + __shfl_xor(c, 32, 64);                 // offset 2: c0+c2 | c1+c3
        sgrp[w] = d + __shfl_xor(d, 16, 64);                 // offset 1: d0+d1
    }
    return (sgrp[0] + sgrp[2]) + (sgrp[1] + sgrp[3]);
}

}  // namespace twkv
