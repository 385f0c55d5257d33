// kv_attention_mfma.hip -- GQA decode attention over the 4-bit compressed cache
// for gfx950: codes are expanded to fp16 centroids in registers and the two
// contractions (q.K^T and P.V) run on the matrix cores.
//
// Same mathematics as turbo_gqa_attention_batch_kernel of the reference
// (kernels.cu:1641-1776): q_rot = R q; s_p = (q_rot . c(K codes_p)) * kn_p / sqrt(D);
// softmax over p <= pos with "+1e-8" in the denominator; acc = sum_p w_p vn_p c(V codes_p);
// out = R^T acc.  Three launches: rotate_kernel in kv_rotate.hip (q_rot, once per sequence and
// head), attention_mfma4_kernel (the context scan, below), attention_merge_kernel
// (split merge, normalisation, rotate-back).
//
// Why MFMA for a bandwidth-bound scan: at 5.6 TB/s of 4-bit codes one CU must
// consume ~18 codes per clock for K and V together, and with two query heads per
// KV head that is ~4 vector-ALU operations per code (extract, look up, two FMAs)
// against a budget of 64 lane-operations per clock per CU.  Moving the FMAs to
// MFMA leaves one v_perm_b32 (LDS address) and one ds_read_b32 per BYTE of codes.
//
// Mapping (one wave = one KV head of one sequence, 32 tokens per iteration):
//   K: lane (t = lane%16, kg = lane/16) loads 16 bytes = dims [32kg, 32kg+32) of
//      token t.  Dword j of it is the B operand of MFMA j (v_mfma_f32_16x16x32_f16),
//      columns = tokens; the A operand holds q_rot for the GQA group's heads in the
//      matching dimension order, rows = heads.  Result S[head][token]: a lane holds
//      the scores of ONE token (its lane%16) for the group's heads.
//   softmax: online, per head, in base 2 (q_rot is pre-scaled by log2(e)/sqrt(D)).
//      One v_permlane32_swap per head brings the two 16-token sub-tiles into the two
//      halves of the wave, so a lane does the exponentials of exactly one token; the
//      running maximum is only raised when a score exceeds it by more than 2^5
//      (then every accumulator is rescaled), which keeps it uniform over the wave.
//      The probabilities go through a 1 KB LDS tile into the A-operand layout
//      P[head][token] of the second contraction (4 ds_write_b16 + 1 ds_read_b128).
//   V: lane (n = lane%16, kg = lane/16) loads, for tokens 4kg..4kg+3, the dword
//      that holds dims 8n..8n+7.  Nibbles of two tokens are interleaved with
//      v_bfi_b32 so that one table look-up yields the fp16 pair (token, token+1) for
//      one dim, which is the B-operand order of O[head][dim] += P[head][token] V[token][dim].
//   dequantization: a 256-entry table byte -> (centroid[lo nibble], centroid[hi nibble])
//      as packed fp16, replicated per lane in LDS (64 KB) so that every ds_read_b32 of
//      a wave is bank-conflict free; the address is one v_perm_b32.
//   addressing: every load is (scalar base of the 16-token sub-tile) + (per-lane
//      offset fixed for the whole kernel); pages of the paged layout only change
//      the scalar base.
//   scheduling: workgroups are persistent (two per CU) and walk a list of
//      (sequence, chunk, head group) items, so the 64 KB table is built once per
//      workgroup; waves never synchronise after that.
//   precision: fp16 operands would cost ~5e-4 relative error each for q_rot and for
//      the probabilities.  Both are split into hi + lo fp16 parts that ride in MFMA
//      rows the GQA group leaves empty (head n -> row n and n+8), so the split costs
//      no extra MFMA; the two halves are added after the contraction.
//      The centroid table is stored as fp16(alpha * c) with alpha chosen so that all
//      eight magnitudes round with <= 1.1e-4 relative error (3.6e-4 without it);
//      1/alpha is folded into q_rot and into the final accumulator.
// The partial (acc[128], max, sum) per (sequence, head, chunk) goes to the split
// workspace; attention_merge_kernel combines, normalises and rotates back.

#include "kv_common.hpp"
#include "kv_kernels.hpp"

#include <cstring>

#ifndef TW_EXP
#define TW_EXP 0
#endif
#ifndef TW_DEPTH
#define TW_DEPTH 1
#endif
#define TW_LUT(addr) ((TW_EXP == 3 || TW_EXP == 4) ? ((uint32_t)(addr) & 0x33ffu) : *reinterpret_cast<const uint32_t*>(tab_lane + (addr)))
#define TW_LUTK(addr) ((TW_EXP == 1) ? ((uint32_t)(addr) & 0x33ffu) : TW_LUT(addr))
#define TW_LUTV(addr) ((TW_EXP == 2) ? ((uint32_t)(addr) & 0x33ffu) : TW_LUT(addr))

namespace twkv {

namespace {

constexpr int kMaxWaves = 8;          // KV heads per workgroup
constexpr int kMaxGroup = 4;          // query heads per KV head handled by this kernel
constexpr int kTableWords = 256 * 64; // 64 KB
constexpr float kNegBig = -1e30f;
// fp16(kAlpha4 * c) has max relative rounding error 1.05e-4 over the 4-bit table
// (exhaustive search over the fp32 values of one octave).
constexpr float kAlpha4 = 19.391284942626953f;
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

}  // namespace

template <bool PAGED, int R, int DEPTH>
__global__ void __launch_bounds__(kMaxWaves * kWave, (DEPTH <= 1 ? 4 : 2))
attention_mfma4_kernel(AttnArgs a, int total_items, int hgroups) {
    __shared__ __attribute__((aligned(16))) uint32_t tab_s[kTableWords];
    // per wave: P[row][k] as fp16, rows 0..R-1 = heads, rows 8..8+R-1 = rounding remainders
    __shared__ __attribute__((aligned(16))) half_t p_s[kMaxWaves][16][32];

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;   // wave index is wave-uniform: keep it scalar
    const int ln = lane & 15, kg = lane >> 4;
    const int waves = nthreads / kWave;
    const int Hk = a.num_kv_heads;

    const char* tab_lane = reinterpret_cast<const char*>(tab_s);
    const uint32_t lane4 = (uint32_t)lane * 4u;
    const uint32_t kvp = (uint32_t)Hk * 64u;           // bytes per cache row (all heads)
    const uint32_t nrow = (uint32_t)Hk * 2u;           // bytes per norm row
    // per-lane byte offsets inside a 16-token sub-tile, fixed for the whole kernel
    const uint32_t koff = (uint32_t)ln * kvp + 16u * (uint32_t)kg;
    uint32_t voff[4];
#pragma unroll
    for (int i = 0; i < 4; i++) voff[i] = (uint32_t)(4 * kg + i) * kvp + 4u * (uint32_t)ln;
    const uint32_t sub_bytes = 16u * kvp;              // sub-tile b follows sub-tile a when contiguous
    // After the sub-tile swap a lane owns token ln of sub-tile (kg >> 1); lanes with odd kg idle.
    const int my_sub = kg >> 1;
    const bool useful = (kg & 1) == 0;
    const uint32_t noff = (uint32_t)ln * nrow + (PAGED ? 0u : (uint32_t)my_sub * 16u * nrow);
    // slot of that token in the k order of the P.V contraction: k = 8*(t/4) + 4*sub + t%4
    half_t* p_w = &p_s[wave][0][8 * (ln >> 2) + 4 * my_sub + (ln & 3)];
    const uint4* p_r = reinterpret_cast<const uint4*>(&p_s[wave][ln][8 * kg]);
    constexpr float kRaise = 5.0f;                     // raise the running max only past 2^5

    bool table_ready = false;
    for (int item = blockIdx.x; item < total_items; item += gridDim.x) {
        const int hg = item % hgroups;
        const int chunk = (item / hgroups) % a.nsplit;
        const int g = item / (hgroups * a.nsplit);
        const int h = hg * waves + wave;                      // KV head of this wave
        const int n = uniform(seq_pos(a, g)) + 1;
        int t0, t1;
        chunk_range(n, chunk, a.nsplit, t0, t1);
        if (t0 >= t1) continue;                               // uniform

        // scalar bases of this wave's head
        const char* kseq = reinterpret_cast<const char*>(a.k) + (long long)h * 64;
        const char* vseq = reinterpret_cast<const char*>(a.v) + (long long)h * 64;
        const char* knseq = reinterpret_cast<const char*>(a.k_norms) + (long long)h * 2;
        const char* vnseq = reinterpret_cast<const char*>(a.v_norms) + (long long)h * 2;
        const int* bt = PAGED ? a.block_table + (long long)g * a.bt_stride : nullptr;
        const long long seq_row0 = (long long)g * a.seq_stride_rows;

        // Buffer descriptors: base = first cache row of the tile (contiguous cache) or of the
        // 16-token page (paged cache), extent = the rows that exist, so lanes past the end
        // of the sequence read zeros instead of foreign memory.  All scalar.
        auto page_row = [&](int ts) -> long long {   // paged: past the end re-read the last page (masked)
            return (long long)uniform(bt[min(ts, t1 - 1) >> 4]) * kPageTokens;
        };
        auto issue_k = [&](uint4 (&kreg)[2], int tile) {
            if (PAGED) {
#pragma unroll
                for (int sub = 0; sub < 2; sub++) {
                    __amdgpu_buffer_rsrc_t r = make_rsrc(kseq + page_row(tile + 16 * sub) * kvp, kPageTokens * (int)kvp);
                    uint32x4_t q = __builtin_amdgcn_raw_buffer_load_b128(r, (int)koff, 0, 0);
                    kreg[sub] = uint4{q[0], q[1], q[2], q[3]};
                }
            } else {
                __amdgpu_buffer_rsrc_t r = make_rsrc(kseq + (seq_row0 + tile) * kvp, max(min(n - tile, 32), 0) * (int)kvp);
                uint32x4_t q0 = __builtin_amdgcn_raw_buffer_load_b128(r, (int)koff, 0, 0);
                uint32x4_t q1 = __builtin_amdgcn_raw_buffer_load_b128(r, (int)(koff + sub_bytes), 0, 0);
                kreg[0] = uint4{q0[0], q0[1], q0[2], q0[3]};
                kreg[1] = uint4{q1[0], q1[1], q1[2], q1[3]};
            }
        };
        auto issue_v = [&](uint32_t (&vreg)[2][4], int tile) {
            if (PAGED) {
#pragma unroll
                for (int sub = 0; sub < 2; sub++) {
                    __amdgpu_buffer_rsrc_t r = make_rsrc(vseq + page_row(tile + 16 * sub) * kvp, kPageTokens * (int)kvp);
#pragma unroll
                    for (int i = 0; i < 4; i++) vreg[sub][i] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff[i], 0, 0);
                }
            } else {
                __amdgpu_buffer_rsrc_t r = make_rsrc(vseq + (seq_row0 + tile) * kvp, max(min(n - tile, 32), 0) * (int)kvp);
#pragma unroll
                for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        vreg[sub][i] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)(voff[i] + sub * sub_bytes), 0, 0);
                }
            }
        };
        // fp16 bits of kn (low half) and vn (high half) of this lane's token.  When a norm row
        // (all KV heads of one token) is a multiple of 16 bytes the lane fetches the 16 bytes
        // that hold its head with one b128 load (rows of consecutive tokens are contiguous, so
        // the 32 useful lanes read one contiguous run) and picks its half-word; a 2-byte gather
        // over the same rows costs ~15 % of the whole scan's bandwidth.
        auto pick = [&](const uint32x4_t& q) -> uint32_t {
            const int dw = (h & 7) >> 1;
            uint32_t w = dw == 0 ? q[0] : dw == 1 ? q[1] : dw == 2 ? q[2] : q[3];
            return (h & 1) ? (w >> 16) : (w & 0xffffu);
        };
        auto issue_n = [&](int tile) -> uint32_t {
            const bool wide = (nrow & 15u) == 0;
            const uint32_t hgrp = (uint32_t)(h >> 3) * 16u;          // 16-byte group of this head inside a row
            if (PAGED) {
                long long r0 = page_row(tile), r1 = page_row(tile + 16);
                const long long rr = my_sub ? r1 : r0;
                if (wide) {
                    uint32x4_t kq = {0, 0, 0, 0}, vq = {0, 0, 0, 0};
                    if (useful) {
                        const char* kp = reinterpret_cast<const char*>(a.k_norms) + (rr + ln) * nrow + hgrp;
                        const char* vp = reinterpret_cast<const char*>(a.v_norms) + (rr + ln) * nrow + hgrp;
                        kq = *reinterpret_cast<const uint32x4_t*>(kp);
                        vq = *reinterpret_cast<const uint32x4_t*>(vp);
                    }
                    return pick(kq) | (pick(vq) << 16);
                }
                uint32_t kk = *reinterpret_cast<const uint16_t*>(knseq + (rr + ln) * nrow);
                uint32_t vv = *reinterpret_cast<const uint16_t*>(vnseq + (rr + ln) * nrow);
                return kk | (vv << 16);
            }
            const long long row = seq_row0 + tile;
            const int rows = max(min(n - tile, 32), 0);
            if (wide) {
                __amdgpu_buffer_rsrc_t rk = make_rsrc(reinterpret_cast<const char*>(a.k_norms) + row * nrow, rows * (int)nrow);
                __amdgpu_buffer_rsrc_t rv = make_rsrc(reinterpret_cast<const char*>(a.v_norms) + row * nrow, rows * (int)nrow);
                uint32x4_t kq = {0, 0, 0, 0}, vq = {0, 0, 0, 0};
                if (useful) {
                    kq = __builtin_amdgcn_raw_buffer_load_b128(rk, (int)(noff + hgrp), 0, 0);
                    vq = __builtin_amdgcn_raw_buffer_load_b128(rv, (int)(noff + hgrp), 0, 0);
                }
                return pick(kq) | (pick(vq) << 16);
            }
            __amdgpu_buffer_rsrc_t rk = make_rsrc(knseq + row * nrow, rows * (int)nrow);
            __amdgpu_buffer_rsrc_t rv = make_rsrc(vnseq + row * nrow, rows * (int)nrow);
            uint32_t kk = __builtin_amdgcn_raw_buffer_load_b16(rk, (int)noff, 0, 0);
            uint32_t vv = __builtin_amdgcn_raw_buffer_load_b16(rv, (int)noff, 0, 0);
            return kk | (vv << 16);
        };

        float4_t o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = float4_t{0.f, 0.f, 0.f, 0.f};
        float m_run[R], l_run[R];
#pragma unroll
        for (int r = 0; r < R; r++) { m_run[r] = kNegBig; l_run[r] = 0.0f; }

        // DEPTH tiles of loads are in flight per wave; a slot is re-issued (for the tile DEPTH
        // further on) as soon as its contents have been expanded.
        const int ntiles = (t1 - t0 + 31) >> 5;
        uint4 kring[DEPTH][2];
        uint32_t vring[DEPTH][2][4];
        uint32_t nring[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            if (d < ntiles && TW_EXP != 5) {
                issue_k(kring[d], t0 + 32 * d);
                nring[d] = issue_n(t0 + 32 * d);
                issue_v(vring[d], t0 + 32 * d);
            }
        }

        // The first loads are already in flight while the workgroup builds its table.
        if (!table_ready) {
        // ---- dequantization table, once per workgroup: entry e, 64 identical words
        for (int i = tid * 4; i < kTableWords; i += nthreads * 4) {
            int e = i >> 6;
            half2_t p = {(half_t)(kAlpha4 * kCentroids4[e & 15]), (half_t)(kAlpha4 * kCentroids4[e >> 4])};
            uint32_t w = *reinterpret_cast<uint32_t*>(&p);
            *reinterpret_cast<uint4*>(&tab_s[i]) = uint4{w, w, w, w};
        }
        for (int i = tid; i < kMaxWaves * 16 * 32 / 2; i += nthreads) reinterpret_cast<uint32_t*>(p_s)[i] = 0u;
        __syncthreads();
            table_ready = true;
        }

        // A operand of the score MFMAs: q_rot[head][32kg + 8j + i]; row m carries the
        // fp16 value of head m, row m + 8 what the rounding left over.
        half8_t aq[4];
        {
            const int hq = ln & 7;
            const bool lo_part = (ln & 8) != 0;
            const float* qr = a.qrot + ((long long)g * a.num_heads + (long long)h * R + (hq < R ? hq : 0)) * a.ws_stride + 32 * kg;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float4 v0 = *reinterpret_cast<const float4*>(qr + 8 * j);
                float4 v1 = *reinterpret_cast<const float4*>(qr + 8 * j + 4);
                float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    float x = (hq < R) ? v[i] : 0.0f;
                    half_t hi = (half_t)x;
                    half_t lo = (half_t)(x - (float)hi);
                    aq[j][i] = lo_part ? lo : hi;
                }
            }
        }


        for (int it0 = 0; it0 < ntiles; it0 += DEPTH) {
#pragma unroll
          for (int d = 0; d < DEPTH; d++) {
            const int it = it0 + d;
            if (it >= ntiles) break;
            uint4 (&kreg)[2] = kring[d];
            uint32_t (&vreg)[2][4] = vring[d];
            uint32_t& nreg = nring[d];
            const int tile = t0 + 32 * it;
            const int next_tile = tile + 32 * DEPTH;
            const bool more = it + DEPTH < ntiles;

#if TW_EXP == 5
            {   // loads only, plain global loads with per-lane 64-bit pointers
                const char* kp = kseq + (seq_row0 + tile) * kvp + koff;
                const char* vp = vseq + (seq_row0 + tile) * kvp;
                uint4 ka = *reinterpret_cast<const uint4*>(kp);
                uint4 kb2 = *reinterpret_cast<const uint4*>(kp + sub_bytes);
                uint32_t f = ka.x ^ ka.w ^ kb2.y ^ kb2.z;
#pragma unroll
                for (int sub = 0; sub < 2; sub++)
#pragma unroll
                    for (int i = 0; i < 4; i++) f ^= *reinterpret_cast<const uint32_t*>(vp + voff[i] + sub * sub_bytes);
                if (useful) {
                    const char* np_ = reinterpret_cast<const char*>(a.k_norms) + (seq_row0 + tile) * nrow + noff;
                    const char* nq_ = reinterpret_cast<const char*>(a.v_norms) + (seq_row0 + tile) * nrow + noff;
                    uint4 n1 = *reinterpret_cast<const uint4*>(np_);
                    uint4 n2 = *reinterpret_cast<const uint4*>(nq_);
                    f ^= n1.x ^ n2.w;
                }
                o[0][0] += __uint_as_float(f & 0x3fffffu);
                continue;
            }
#endif
#if TW_EXP == 4
            {   // loads only: fold the loaded words into one accumulator and re-issue
                uint32_t f = kreg[0].x ^ kreg[0].y ^ kreg[0].z ^ kreg[0].w ^ kreg[1].x ^ kreg[1].y ^ kreg[1].z ^ kreg[1].w ^ nreg;
#pragma unroll
                for (int sub = 0; sub < 2; sub++)
#pragma unroll
                    for (int i = 0; i < 4; i++) f ^= vreg[sub][i];
                o[0][0] += __uint_as_float(f & 0x3fffffu);
                if (more) { issue_k(kreg, next_tile); nreg = issue_n(next_tile); issue_v(vreg, next_tile); }
                continue;
            }
#endif
            // ---- scores S[head][token] for both sub-tiles
            float4_t s[2];
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                const uint32_t w[4] = {kreg[sub].x, kreg[sub].y, kreg[sub].z, kreg[sub].w};
                union { uint32_t u[4]; half8_t h; } kv[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    kv[j].u[0] = TW_LUTK(__builtin_amdgcn_perm(w[j], lane4, 0x0c0c0400u));
                    kv[j].u[1] = TW_LUTK(__builtin_amdgcn_perm(w[j], lane4, 0x0c0c0500u));
                    kv[j].u[2] = TW_LUTK(__builtin_amdgcn_perm(w[j], lane4, 0x0c0c0600u));
                    kv[j].u[3] = TW_LUTK(__builtin_amdgcn_perm(w[j], lane4, 0x0c0c0700u));
                }
                s[sub] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; j++) s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aq[j], kv[j].h, s[sub], 0, 0, 0);
            }
            if (more) issue_k(kreg, next_tile);

            // ---- online softmax (base 2): this lane owns token ln of sub-tile my_sub
            const float kn = h2f_bits(nreg & 0xffffu), vn = h2f_bits(nreg >> 16);
            if (more) nreg = issue_n(next_tile);
            const bool valid = useful && (tile + 16 * my_sub + ln < t1);
            float raw[R], x[R];
            bool raise = false;
#pragma unroll
            for (int r = 0; r < R; r++) {
                // rows r (hi part of q_rot) and r + 8 (lo part) sit 32 lanes apart; the swap also
                // moves sub-tile b into the upper half of the wave
                uint32x2_t sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(s[0][r]), __float_as_uint(s[1][r]), false, false);
                raw[r] = (__uint_as_float(sw[0]) + __uint_as_float(sw[1])) * kn;    // kernels.cu:1707
                x[r] = valid ? raw[r] - m_run[r] : kNegBig;
                raise = raise || (x[r] > kRaise);
            }
            if (__any(raise)) {                                         // rare after the first tiles
#pragma unroll
                for (int r = 0; r < R; r++) {
                    float m_new = fmaxf(m_run[r], wave_max(valid ? raw[r] : kNegBig));
                    float alpha = __builtin_amdgcn_exp2f(m_run[r] - m_new);
                    m_run[r] = m_new;
                    l_run[r] *= alpha;
                    x[r] = valid ? raw[r] - m_new : kNegBig;
#pragma unroll
                    for (int j = 0; j < 8; j++) o[j][r] *= alpha;       // rows r and r + 8 live in register r
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                float p = __builtin_amdgcn_exp2f(x[r]);
                l_run[r] += p;
                float pf = p * vn;                                      // (s * vn) * centroid, kernels.cu:1765
                half_t hi = (half_t)pf;
                half_t lo = (half_t)(pf - (float)hi);
                if (useful) {
                    p_w[r * 32] = hi;
                    p_w[(r + 8) * 32] = lo;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            union { uint4 q; half8_t h; } pa;
            pa.q = *p_r;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            __builtin_amdgcn_wave_barrier();

            // ---- O[head][dim 8ln + j] += P[head][token] V[token][dim]
            uint32_t xe[4], xo[4];   // [2*sub + pair]: index bytes for even / odd dims
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                for (int pr = 0; pr < 2; pr++) {
                    uint32_t wa = vreg[sub][2 * pr], wb = vreg[sub][2 * pr + 1];
                    xe[2 * sub + pr] = (wa & 0x0f0f0f0fu) | ((wb << 4) & 0xf0f0f0f0u);
                    xo[2 * sub + pr] = ((wa >> 4) & 0x0f0f0f0fu) | (wb & 0xf0f0f0f0u);
                }
            }
            if (more) issue_v(vreg, next_tile);
#pragma unroll
            for (int jp = 0; jp < 4; jp++) {         // two dims (even, odd) per step: 8 look-ups, 2 MFMAs
                const uint32_t sel = 0x0c0c0400u + ((uint32_t)jp << 8);
                union { uint32_t u[4]; half8_t h; } be, bo;
#pragma unroll
                for (int q4 = 0; q4 < 4; q4++) {
                    be.u[q4] = TW_LUTV(__builtin_amdgcn_perm(xe[q4], lane4, sel));
                    bo.u[q4] = TW_LUTV(__builtin_amdgcn_perm(xo[q4], lane4, sel));
                }
                o[2 * jp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, be.h, o[2 * jp], 0, 0, 0);
                o[2 * jp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, bo.h, o[2 * jp + 1], 0, 0, 0);
            }
          }
        }

        // ---- partial result of this (sequence, KV head, chunk)
#pragma unroll
        for (int r = 0; r < R; r++) {
            l_run[r] = wave_sum(l_run[r]);                                        // idle and masked lanes hold 0
#pragma unroll
            for (int j = 0; j < 8; j++) o[j][r] += __shfl_xor(o[j][r], 32, 64);   // row r + row r+8 (lo part of P)
        }
        if (kg == 0) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                float* part = a.ws + ((long long)g * a.num_heads + (long long)h * R + r) * a.ws_stride +
                              (long long)chunk * kPartialFloats;
#pragma unroll
                for (int j = 0; j < 8; j++) part[8 * ln + j] = o[j][r] * (1.0f / kAlpha4);
                if (ln == 0) {
                    part[kHeadDim] = m_run[r];
                    part[kHeadDim + 1] = l_run[r];
                }
            }
        }
    }
}

static int resident_groups() {
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached = (TW_DEPTH <= 1 ? 2 : 1) * cus;   // 64 KB of LDS and <= 128 VGPRs per workgroup of 8 waves: two per CU
    }
    return cached;
}

static int scan_waves(const AttnArgs& a) {
    int waves = a.num_kv_heads < kMaxWaves ? a.num_kv_heads : kMaxWaves;
    while (a.num_kv_heads % waves != 0) waves--;
    return waves;
}

float attention_mfma_q_scale(int bits) {
    (void)bits;
    return kLog2e * kInvSqrtD / kAlpha4;   // score scale of kernels.cu:1707 in base 2, table scale undone
}

// Shape check; with rotate_query also q_rot = R q (kernels.cu:1671-1681) into the workspace.
bool prepare_attention_mfma(AttnArgs& a, hipStream_t s, bool rotate_query) {
    const int R = a.num_heads / a.num_kv_heads;
    if (a.bits != 4) return false;
    if (R != 1 && R != 2 && R != 4) return false;
    // needs the split workspace with room for q_rot behind each block's partials
    if (!a.ws || !a.qrot) return false;
    if ((reinterpret_cast<uintptr_t>(a.qrot) & 15u) != 0 || (a.ws_stride & 3) != 0) return false;
    const long long items = (long long)a.G * a.nsplit * (a.num_kv_heads / scan_waves(a));
    if (items <= 0 || items > 0x7fffffff) return false;
    a.force_merge = 1;
    a.m_log2 = 1;
    if (rotate_query) {
        RotArgs r;
        memset(&r, 0, sizeof(r));
        r.nseg = 1;
        r.seg_src[0] = a.q;
        r.seg_stride[0] = a.q_stride;
        r.seg_heads[0] = a.num_heads;
        r.seg_nvec[0] = a.G * a.num_heads;
        r.seg_units[0] = (r.seg_nvec[0] + 15) / 16 * 8;
        r.seg_kind[0] = 1;
        r.rotation = a.rotation;
        r.qrot = a.qrot;
        r.qrot_stride = a.ws_stride;
        r.q_scale = attention_mfma_q_scale(a.bits);
        launch_rotate(r, a.bits, s);
    }
    return true;
}

void launch_attention_mfma_scan(const AttnArgs& a, hipStream_t s) {
    const int waves = scan_waves(a);
    const int hgroups = a.num_kv_heads / waves;
    const int items = a.G * a.nsplit * hgroups;
    int grid = resident_groups();
    if (items < grid) grid = items;
    const int R = a.num_heads / a.num_kv_heads;
    const dim3 g3(grid), b3(waves * kWave);
#ifndef TW_DEPTH
#define TW_DEPTH 1
#endif
#define TW_LAUNCH(P, RR) hipLaunchKernelGGL((attention_mfma4_kernel<P, RR, TW_DEPTH>), g3, b3, 0, s, a, items, hgroups)
    if (a.block_table) {
        if (R == 1) TW_LAUNCH(true, 1); else if (R == 2) TW_LAUNCH(true, 2); else TW_LAUNCH(true, 4);
    } else {
        if (R == 1) TW_LAUNCH(false, 1); else if (R == 2) TW_LAUNCH(false, 2); else TW_LAUNCH(false, 4);
    }
#undef TW_LAUNCH
}

}  // namespace twkv
