// kv_mfma_util.hpp -- constants and helpers shared by the MFMA attention kernels
// (kv_attention_mfma.hip: decode scan, kv_prefill_mfma.hip: causal prefill).
#pragma once

#include "kv_common.hpp"
#include "kv_kernels.hpp"

namespace twkv {

constexpr int kGroupWaves = 8;        // KV heads (waves) that walk one item together
constexpr int kMaxWaves = 16;         // waves per workgroup: one workgroup per CU, two groups
constexpr int kMaxBalanceSeqs = 4096; // sequences (blocks) the balanced walk can index (16 KB of LDS)
constexpr int kTableWords = 256 * 64; // 64 KB
constexpr float kNegBig = -1e30f;
// fp16(kAlpha4 * c) has max relative rounding error 1.05e-4 over the 4-bit table
// (exhaustive search over the fp32 values of one octave).
constexpr float kAlpha4 = 19.391284942626953f;
// the same for the 2-bit table: 1.1e-7
constexpr float kAlpha2 = 25.46918296813965f;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kInvSqrtD = 0.08838834764831845f;

__device__ __forceinline__ int seq_pos(const AttnArgs& a, int g) {
    if (a.pos_mode == kPosArray) return a.positions[g];
    if (a.pos_mode == kPosScalar) return a.pos_scalar;
    return g;
}

__device__ __forceinline__ float h2f_bits(uint32_t bits16) {
    union { uint16_t u; half_t h; } cv;
    cv.u = (uint16_t)bits16;
    return (float)cv.h;
}

__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }

typedef uint32_t uint32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint32x2_t __attribute__((ext_vector_type(2)));

// Buffer descriptor over [base, base + bytes).  Every input is forced into scalar
// registers: a descriptor held in vector registers makes each load a serialising loop.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const char* base, int bytes) {
    uint64_t p = reinterpret_cast<uint64_t>(base);
    uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(p >> 32));
    char* q = reinterpret_cast<char*>(((uint64_t)hi << 32) | lo);
    return __builtin_amdgcn_make_buffer_rsrc(q, 0, __builtin_amdgcn_readfirstlane(bytes), 0x00020000);
}

// Cache policy (the aux operand of the raw buffer loads) of the loads that stream the cache: bit 1 = nt,
// "non-temporal".  A decode scan reads every cache byte once per launch and a layer's cache is far larger than
// any cache level, so nothing is gained by keeping the lines; with the hint a launch that only reads 554 MB
// takes 78-82 us instead of 88-90 us on MI355X (7.0 instead of 6.2 TB/s).
// Only for lines that one load instruction of one wave covers in full: a line touched by two instructions (two
// waves, or two half-line loads of one wave) is fetched twice, and the launch gets slower than without the hint.
constexpr int kStreamCodes = 2;
// the norm rows (16 bytes per token for 8 heads) are shared by the workgroups of a sequence: kept in the caches
constexpr int kStreamNorms = 0;

// compute units of the current device (cached; kv_attention_mfma.hip)
int compute_units();

// The dequantization table of the MFMA scans, built by the nthreads threads of a workgroup: entry e (a cache byte)
// fills 256 bytes with replicas of its centroids as fp16 -- 4 bit: 64 replicas of (low code, high code); 2 bit: 32
// replicas of the byte's four codes, in their own order (NATURAL) or as 0, 2, 1, 3.  The centroids come out of a
// register by wave shuffle (lane c holds centroid c, scaled): indexing the constant arrays with a per-lane index is a
// dependent memory load per look-up, microseconds for this loop.  Lower lanes run at least as many rounds as higher
// ones, so the lanes the shuffles read (0..15) are active whenever any lane is.
template <int BITS, bool NATURAL>
__device__ __forceinline__ void build_centroid_table(uint32_t* tab_s, float alpha, int tid, int nthreads) {
    const int lane = tid & 63;
    const float cent_lane = alpha * (BITS == 4 ? kCentroids4[lane & 15] : kCentroids2[lane & 3]);
    auto cent = [&](int c) -> half_t { return (half_t)__shfl(cent_lane, c, 64); };
    for (int i = tid * 4; i < kTableWords; i += nthreads * 4) {
        const int e = i >> 6;
        if constexpr (BITS == 4) {
            half2_t p = {cent(e & 15), cent(e >> 4)};
            const uint32_t w = *reinterpret_cast<uint32_t*>(&p);
            *reinterpret_cast<uint4*>(&tab_s[i]) = uint4{w, w, w, w};
        } else {
            constexpr int f1 = NATURAL ? 2 : 4, f2 = NATURAL ? 4 : 2;
            half2_t p0 = {cent(e & 3), cent((e >> f1) & 3)};
            half2_t p1 = {cent((e >> f2) & 3), cent((e >> 6) & 3)};
            const uint32_t w0 = *reinterpret_cast<uint32_t*>(&p0), w1 = *reinterpret_cast<uint32_t*>(&p1);
            *reinterpret_cast<uint4*>(&tab_s[i]) = uint4{w0, w1, w0, w1};
        }
    }
}

}  // namespace twkv
