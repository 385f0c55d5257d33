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

// An operand tile in LDS: 16 rows of 128 halves (4 KB) regrouped so that lane kk * 16 + i finds its 32 halves
// (coordinates 4s + kk of row i) in one 64-byte row, row number = lane.  The four 16-byte pieces of a row are
// stored swizzled (piece p of row r at p ^ ((r / 4) % 4)): 16 lanes reading the same piece of 16 consecutive rows
// then touch all 64 banks once.
constexpr int kOperandTileDwords = 64 * 16;

__device__ __forceinline__ int operand_tile_dword(int row, int q) {
    return row * 16 + ((((q >> 2) ^ (row >> 2)) & 3) << 2) + (q & 3);
}

// raw[j] = 16-byte piece j * 64 + lane of the tile as it lies in memory (piece q = lane % 16 of row 4j + lane / 16):
// its halves e and 4 + e go to row e * 16 + (4j + lane / 16), dword q.
__device__ __forceinline__ void stage_operand_tile(uint32_t* tile, const uint4 (&raw)[4], int lane) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = 4 * j + (lane >> 4), q = lane & 15;
        tile[operand_tile_dword(0 * 16 + i, q)] = (raw[j].x & 0xffffu) | (raw[j].z << 16);
        tile[operand_tile_dword(1 * 16 + i, q)] = (raw[j].x >> 16) | (raw[j].z & 0xffff0000u);
        tile[operand_tile_dword(2 * 16 + i, q)] = (raw[j].y & 0xffffu) | (raw[j].w << 16);
        tile[operand_tile_dword(3 * 16 + i, q)] = (raw[j].y >> 16) | (raw[j].w & 0xffff0000u);
    }
}

// Lane kk * 16 + i reads row kk * 16 + i: out[s] = coordinate 4s + kk of row i of the tile.
__device__ __forceinline__ void read_operand_tile(const uint32_t* tile, int lane, float (&out)[32]) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const uint4 p = *reinterpret_cast<const uint4*>(tile + operand_tile_dword(lane, 4 * t));
        const uint32_t w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            union { uint32_t u; half_t h[2]; } cv;
            cv.u = w[e];
            out[8 * t + 2 * e] = (float)cv.h[0];
            out[8 * t + 2 * e + 1] = (float)cv.h[1];
        }
    }
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
