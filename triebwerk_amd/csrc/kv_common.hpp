// kv_common.hpp -- shared device helpers for the gfx950 KV-cache kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace twkv {

constexpr int kHeadDim = 128;   // the reference kernels hard-size to 128 (kernels.cu:1504)
constexpr int kWave = 64;       // CDNA wavefront
constexpr int kPageTokens = 16; // tokens per cache page in the paged layout

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// Lloyd-Max tables of the reference (kernels.cu:1426-1445).
__device__ __constant__ const float kCentroids2[4] = {-0.13351f, -0.04003f, 0.04003f, 0.13351f};
__device__ __constant__ const float kBounds2[3] = {-0.08677f, 0.0f, 0.08677f};
__device__ __constant__ const float kCentroids4[16] = {
    -0.24155f, -0.18293f, -0.14304f, -0.11099f, -0.08330f, -0.05806f, -0.03432f, -0.01135f,
    0.01135f,  0.03432f,  0.05806f,  0.08330f,  0.11099f,  0.14304f,  0.18293f,  0.24155f};
__device__ __constant__ const float kBounds4[15] = {
    -0.21224f, -0.16299f, -0.12701f, -0.09715f, -0.07068f, -0.04619f, -0.02284f, 0.00000f,
    0.02284f,  0.04619f,  0.07068f,  0.09715f,  0.12701f,  0.16299f,  0.21224f};

// Host-side copies for building lookup tables.
static const float kCentroids2Host[4] = {-0.13351f, -0.04003f, 0.04003f, 0.13351f};
static const float kCentroids4Host[16] = {
    -0.24155f, -0.18293f, -0.14304f, -0.11099f, -0.08330f, -0.05806f, -0.03432f, -0.01135f,
    0.01135f,  0.03432f,  0.05806f,  0.08330f,  0.11099f,  0.14304f,  0.18293f,  0.24155f};

// turbo_quantize of the reference (kernels.cu:1448-1473) with the boundaries as immediates.  The reference walks a
// tree of strict `<` comparisons for 4 bits (a value on a boundary goes up, NaN -> 15) and counts `>=` for 2 bits
// (NaN -> 0).  The tree's answer is the number of boundaries b, in their sorted order, with !(val < b) -- the values
// below a boundary form a lower set -- and that count is what is computed here: 15 compare-and-add pairs without a
// branch, where the tree as written costs a wave whose lanes disagree every one of its 15 nodes with the branching
// around them (2 us per decode launch for the four values per lane of a rotation).
__device__ __forceinline__ int turbo_quantize(float val, int bits) {
    if (bits == 4) {
        constexpr float kB[15] = {-0.21224f, -0.16299f, -0.12701f, -0.09715f, -0.07068f, -0.04619f, -0.02284f, 0.00000f,
                                  0.02284f,  0.04619f,  0.07068f,  0.09715f,  0.12701f,  0.16299f,  0.21224f};
        int idx = 0;
#pragma unroll
        for (int i = 0; i < 15; i++) idx += !(val < kB[i]) ? 1 : 0;
        return idx;
    }
    return (int)(val >= -0.08677f) + (int)(val >= 0.0f) + (int)(val >= 0.08677f);
}

// Cache row of position p of sequence g: the reference's g*msl + p
// (kernels.cu:973, 1629, 1690), or the paged indirection.
__device__ __forceinline__ long long cache_row(const int* __restrict__ block_table, int bt_stride,
                                               long long seq_stride_rows, int g, int p) {
    if (block_table) {
        int page = block_table[(long long)g * bt_stride + (p / kPageTokens)];
        return (long long)page * kPageTokens + (p % kPageTokens);
    }
    return (long long)g * seq_stride_rows + p;
}

// Chunk c of nsplit of a sequence of n tokens: the sequence's 32-token tiles are dealt
// out evenly, so every chunk of one sequence has the same length to within one tile
// whatever max_seq_len the caller allocated.  Empty (t0 >= t1) when n has fewer tiles
// than nsplit.
// Chunks 2j and 2j+1 do not split their tiles in halves but kPairShare : 64 - kPairShare.
// The MFMA scan runs an even and the following odd chunk on the two wave groups of one CU,
// and the group in the upper wave slots gets ~5 % less of the CU (measured; s_setprio does
// not change it), so an even split leaves the lower group idle at the end.
constexpr unsigned kPairShare = 33;
__device__ __forceinline__ unsigned chunk_boundary(unsigned tiles, unsigned c, unsigned nsplit) {
    if (c >= nsplit) return tiles;
    if ((c & 1u) == 0) return (c * tiles) / nsplit;             // tiles * nsplit < 2^32 (nsplit <= 64)
    const unsigned lo = ((c - 1) * tiles) / nsplit;
    const unsigned hi = c + 1 >= nsplit ? tiles : ((c + 1) * tiles) / nsplit;
    return lo + ((hi - lo) * kPairShare + 32u) / 64u;
}
__device__ __forceinline__ void chunk_range(int n, int c, int nsplit, int& t0, int& t1) {
    const unsigned tiles = (unsigned)(n + 31) >> 5;
    t0 = 32 * (int)chunk_boundary(tiles, (unsigned)c, (unsigned)nsplit);
    int e = 32 * (int)chunk_boundary(tiles, (unsigned)c + 1u, (unsigned)nsplit);
    t1 = e < n ? e : n;
}
// Does chunk c hold any token?  Always when the sequence has at least nsplit tiles.
__device__ __forceinline__ bool chunk_nonempty(int n, int c, int nsplit) {
    const unsigned tiles = (unsigned)(n + 31) >> 5;
    if (tiles >= (unsigned)nsplit) return true;
    return chunk_boundary(tiles, (unsigned)c + 1u, (unsigned)nsplit) > chunk_boundary(tiles, (unsigned)c, (unsigned)nsplit);
}

// The same for the fp16 whole-row scan (AttnArgs::even_chunks): units of 8 tokens, one per wave of its workgroups,
// dealt out evenly with no shares; units * nsplit < 2^32.
__device__ __forceinline__ void even_chunk_range(int n, int c, int nsplit, int& t0, int& t1) {
    const unsigned units = (unsigned)(n + 7) >> 3;
    t0 = 8 * (int)(((unsigned)c * units) / (unsigned)nsplit);
    const int e = 8 * (int)((((unsigned)c + 1u) * units) / (unsigned)nsplit);
    t1 = e < n ? e : n;
}
__device__ __forceinline__ bool even_chunk_nonempty(int n, int c, int nsplit) {
    const unsigned units = (unsigned)(n + 7) >> 3;
    return (((unsigned)c + 1u) * units) / (unsigned)nsplit > ((unsigned)c * units) / (unsigned)nsplit;
}

// fp32 -> fp16 of a value that must first exist as a rounded fp32 number.  Without the barrier the
// compiler folds a preceding multiply or fused multiply-add into the conversion (v_fma_mixlo_f16: one
// rounding instead of two), which changes a result in a few hundred thousand.
__device__ __forceinline__ float as_half_value(float x) {
    asm volatile("" : "+v"(x));
    return (float)(half_t)x;
}

// sigmoid_gate_batch_kernel's arithmetic (kernels.cu:2993-2994) on an output that has already been rounded to fp16
__device__ __forceinline__ half_t gated(half_t out, half_t gate) {
    return (half_t)((float)out / (1.0f + expf(-(float)gate)));
}

// Workgroup barrier that orders LDS accesses only: global loads and stores issued before it stay in flight
// (__syncthreads also waits for every one of them).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace twkv
