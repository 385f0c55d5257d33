// kv_pair_scan.hpp -- the 32-token tile of the 4-bit decode scan with TWO KV heads per wave, shared by the kernels
// that use it (kv_decode_fused.hip: the one-launch decode step; kv_attention_pair.hip: the stand-alone scan).
//
// Why pairs.  A 128-byte line of a compressed cache row is two 4-bit heads (2 x 64 bytes of codes).  With one head
// per wave two waves fetch every line, each for its half.  When a wave takes both halves every load instruction
// covers whole lines that no other instruction touches, and the loads can carry the non-temporal hint
// (kStreamCodes): a launch that only reads 554 MB then takes 78-82 us instead of 88-90 us on MI355X.  With
// half-line loads the hint doubles the fetches, so the two go together.
//
// Mathematics as turbo_gqa_attention_batch_kernel of the reference (kernels.cu:1688-1766): scores
// s_p = (q_rot . c(K codes_p)) * kn_p (q_rot pre-scaled by log2(e) / sqrt(D) / alpha), online softmax in base 2,
// acc += (w_p * vn_p) * c(V codes_p).  The operand conventions (table look-up by v_perm_b32 address, fp16 value +
// rounding remainder rows for q_rot and the probabilities, running maximum raised only past 2^5) are those of
// kv_attention_mfma.hip.
//
// Layout of a tile in a wave (lane = (pn = lane % 16, pkg = lane / 16), hd = pn / 8 the head of the pair):
//   loads    K: instruction c (0..3) covers tokens 8c .. 8c+7 whole, and every lane asks for the piece it multiplies:
//            lane (pn, pkg) the 16 bytes 16 (4 hd + pkg) .. of token 8c + pn % 8 of the pair's 128-byte row (an
//            instruction that covers the same lines in address order and a ds_bpermute per dword to hand the pieces
//            on costs 3 us of 104 at 64 x 8192 tokens: the scan has no LDS issue slots to spare).  V: lane (pn, pkg) loads 8 bytes (16 dims of head hd: dims 16 (pn % 8) ..) of tokens
//            4 pkg + i and 16 + 4 pkg + i, i = 0..3.  Norms: 4 bytes (the pair's two fp16) of tokens tok0 and tok0 + 16.
//   scores   MFMA set c: columns 0-7 = tokens 8c .. 8c+7 of the first head, columns 8-15 the same tokens of the second;
//            the A operand holds
//            the query heads of both KV heads: row 4 hd + r the fp16 value, row + 8 the rounding remainder.  A lane's
//            accumulator registers are the rows 4 pkg + i, so the first head's scores arrive in lane groups 0 (values)
//            and 2 (remainders), the second head's in groups 1 and 3, register r in both: no per-lane choice of a register.
//   softmax  two permlane32 swaps per query head add value and remainder rows and leave lane (pn, pkg) with the scores
//            of tokens tok0 = 8 (pkg / 2) + pn % 8 and tok0 + 16 of head hd; the lanes whose group holds the other
//            head's rows (pkg % 2 != hd) own nothing.
//   P.V      the probabilities times the V norms go through the wave's 1 KB LDS tile into A-operand order (rows as
//            above); MFMA j: columns 0-7 = dim 16 (pn % 8) + j of the first head, 8-15 of the second.
// A product of a row with a column of the other head is computed and never used.
//
// The 2-bit form (BITS = 2) is the same tile on rows of half the size: a pair of heads is 64 bytes of a token's row,
// K 4 x 8 bytes per lane (32 dims), V 8 x 4 bytes (16 dims of one token), the table maps a byte to its FOUR
// centroids (8 bytes, ds_read_b64, 32 replicas).  Half a line per load instruction, so no non-temporal hint.  For P.V
// the 2-bit fields of four tokens are transposed into bytes that hold one dim of the four (two v_bfi stages, one
// instruction per look-up), so that a look-up yields four consecutive contraction slots.
#pragma once

#include "kv_common.hpp"
#include "kv_mfma_util.hpp"

namespace twkv {

template <int BITS> struct PairBytes { static constexpr uint32_t head = BITS * 16u; };     // code bytes of one head and token

// What a lane knows about itself (derive once, after any code that would otherwise keep these alive in registers).
template <int R, int BITS = 4>
struct PairLane {
    int pn, pkg, hd;
    uint32_t nshift;        // 16 hd: where this lane's head sits in a dword of two fp16 norms
    uint32_t lane_rep;      // byte offset of the lane's replica inside a table entry
    bool useful;            // owns two (token, head) pairs of every tile
    int tok0;               // the first of them (the other: tok0 + 16)
    half_t* p_w;            // where its probabilities go in the wave's P tile (row 4 hd, column of tok0); with R < 4
                            // the lanes that own nothing write their zeros to the spare rows 4 hd + R + r instead
                            // of being masked off (four exec-mask regions less per tile)
    const uint4* p_r;       // its A operand of the P.V MFMAs
    const char* tab;        // the centroid table
    uint32_t koff_rows, koff_bytes;   // K: row pn % 8 and byte 16 (4 hd + pkg) inside a pair row
    uint32_t voff_rows, voff_bytes;   // V: row 4 pkg and byte 8 pn

    __device__ __forceinline__ void init(int lane, half_t (*p_tile)[32], const uint32_t* table) {
        pn = lane & 15; pkg = lane >> 4; hd = pn >> 3;
        nshift = 16u * (uint32_t)hd;
        lane_rep = BITS == 4 ? (uint32_t)lane * 4u : (uint32_t)(lane & 31) * 8u;
        useful = (pkg & 1) == hd;
        tok0 = 8 * (pkg >> 1) + (pn & 7);
        p_w = &p_tile[4 * hd + ((R < 4 && !useful) ? R : 0)][8 * (tok0 >> 2) + (tok0 & 3)];
        p_r = reinterpret_cast<const uint4*>(&p_tile[pn][8 * pkg]);
        tab = reinterpret_cast<const char*>(table);
        koff_rows = (uint32_t)(pn & 7); koff_bytes = (BITS == 4 ? 16u : 8u) * (uint32_t)(4 * hd + pkg);
        voff_rows = (uint32_t)(4 * pkg); voff_bytes = (BITS == 4 ? 8u : 4u) * (uint32_t)pn;
    }
    __device__ __forceinline__ uint32_t lut32(uint32_t addr) const { return *reinterpret_cast<const uint32_t*>(tab + addr); }
    __device__ __forceinline__ uint2 lut64(uint32_t addr) const { return *reinterpret_cast<const uint2*>(tab + addr); }
    // reductions over the lanes of this lane's head (lane groups of both parities included: those that own nothing
    // contribute the neutral element)
    __device__ __forceinline__ float head_max(float v) const {
        v = fmaxf(v, __shfl_xor(v, 1, 64)); v = fmaxf(v, __shfl_xor(v, 2, 64)); v = fmaxf(v, __shfl_xor(v, 4, 64));
        v = fmaxf(v, __shfl_xor(v, 16, 64)); v = fmaxf(v, __shfl_xor(v, 32, 64));
        return v;
    }
    __device__ __forceinline__ float head_sum(float v) const {
        v += __shfl_xor(v, 1, 64); v += __shfl_xor(v, 2, 64); v += __shfl_xor(v, 4, 64);
        v += __shfl_xor(v, 16, 64); v += __shfl_xor(v, 32, 64);
        return v;
    }
};

// The registers of one tile in flight.
template <int BITS> struct PairPieces;
template <> struct PairPieces<4> { typedef uint32x4_t k_t; typedef uint32x2_t v_t; };
template <> struct PairPieces<2> { typedef uint32x2_t k_t; typedef uint32_t v_t; };
template <int BITS = 4>
struct PairTileRegs {
    typename PairPieces<BITS>::k_t k[4];        // instruction c: 32 dims of one token and head
    typename PairPieces<BITS>::v_t v[2][4];     // [sub-tile][i]: 16 dims of one token and head
    uint32_t n[2][2];       // [token tok0 | tok0 + 16][K | V]: the pair's two fp16 norms
};

template <int R>
struct PairState {
    float4_t o[16];         // accumulator of P.V MFMA j
    float m_run[R], l_run[R];
    half8_t aq[4];          // A operand of the score MFMAs

    __device__ __forceinline__ void reset() {
#pragma unroll
        for (int j = 0; j < 16; j++) o[j] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < R; r++) { m_run[r] = kNegBig; l_run[r] = 0.0f; }
    }
    // q_rot of the pair's query heads: row(i) -> the 128 floats of query head i (i = hd * R + r, 0 <= i < 2 R)
    template <class Lane, class RowOf>
    __device__ __forceinline__ void load_query(const Lane& L, RowOf row_of) {
        const int m = L.pn & 7;                                // operand row m (and m + 8): head m / 4, query head m % 4
        const bool lo_part = (L.pn & 8) != 0;
        const bool live = (m & 3) < R;
        const float* qr = row_of(live ? (m >> 2) * R + (m & 3) : 0) + 32 * L.pkg;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float4 v0 = *reinterpret_cast<const float4*>(qr + 8 * j);
            float4 v1 = *reinterpret_cast<const float4*>(qr + 8 * j + 4);
            float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float x = live ? v[i] : 0.0f;
                half_t hi = (half_t)x;
                half_t lo = (half_t)(x - (float)hi);
                aq[j][i] = lo_part ? lo : hi;
            }
        }
    }
};

// One tile.  `tile` is its first token, `n` the tokens of the sequence; after_k / after_n / after_v are called as
// soon as the K, norm and V registers of `t` have been consumed (the caller re-issues them for a later tile there).
template <int R, int BITS, class AfterK, class AfterN, class AfterV>
__device__ __forceinline__ void pair_scan_tile(const PairLane<R, BITS>& L, PairState<R>& S, PairTileRegs<BITS>& t, int tile, int n,
                                               AfterK after_k, AfterN after_n, AfterV after_v) {
    constexpr float kRaise = 5.0f;                     // raise the running max only past 2^5
    // ---- scores: set c = tokens 8c .. 8c+7 of both heads
    float4_t s[4];
    if constexpr (BITS == 2) {
        // operand i = 4 c + j: bytes 2 (j % 2) and + 1 of dword j / 2 of the lane's 8 bytes of set c, dims 8j .. 8j + 7.
        // The look-ups run kAheadK operands ahead of the MFMAs (see the P.V loop below).
        constexpr int kAheadK = 4;
        uint2 klo[kAheadK], khi[kAheadK];
        auto look = [&](int i, uint2& lo, uint2& hi) {
            const uint32_t w = t.k[i >> 2][(i & 3) >> 1];
            const uint32_t sel = 0x0c0c0400u + ((uint32_t)(2 * (i & 1)) << 8);
            lo = L.lut64(__builtin_amdgcn_perm(w, L.lane_rep, sel));
            hi = L.lut64(__builtin_amdgcn_perm(w, L.lane_rep, sel + 0x100u));
        };
#pragma unroll
        for (int i = 0; i < kAheadK; i++) look(i, klo[i], khi[i]);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            union { uint32_t u[4]; half8_t h; } kv;
            kv.u[0] = klo[i % kAheadK].x; kv.u[1] = klo[i % kAheadK].y; kv.u[2] = khi[i % kAheadK].x; kv.u[3] = khi[i % kAheadK].y;
            if (i + kAheadK < 16) look(i + kAheadK, klo[i % kAheadK], khi[i % kAheadK]);
            asm volatile("" ::: "memory");
            if ((i & 3) == 0) s[i >> 2] = float4_t{0.f, 0.f, 0.f, 0.f};
            s[i >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(S.aq[i & 3], kv.h, s[i >> 2], 0, 0, 0);
        }
    } else {
#pragma unroll
    for (int c = 0; c < 4; c++) {
        union { uint32_t u[4]; half8_t h; } kv[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t w = t.k[c][j];
            kv[j].u[0] = L.lut32(__builtin_amdgcn_perm(w, L.lane_rep, 0x0c0c0400u));
            kv[j].u[1] = L.lut32(__builtin_amdgcn_perm(w, L.lane_rep, 0x0c0c0500u));
            kv[j].u[2] = L.lut32(__builtin_amdgcn_perm(w, L.lane_rep, 0x0c0c0600u));
            kv[j].u[3] = L.lut32(__builtin_amdgcn_perm(w, L.lane_rep, 0x0c0c0700u));
        }
        s[c] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++) s[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(S.aq[j], kv[j].h, s[c], 0, 0, 0);
    }
    }
    after_k();
    // Wave priority rises as the tile advances (scores 0, softmax 1, P.V 2): of the two waves of a SIMD the one
    // that is further along issues first, finishes its tile and puts its next loads on the way.  2.5 % at
    // 64 x 8192 tokens; raising it for the scores, or for scores and P.V alike, gains nothing.
    __builtin_amdgcn_s_setprio(1);

    // ---- online softmax (base 2): this lane owns tokens tok0 and tok0 + 16 of head hd
    float kn[2], vn[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        kn[i] = h2f_bits((t.n[i][0] >> L.nshift) & 0xffffu);
        vn[i] = h2f_bits((t.n[i][1] >> L.nshift) & 0xffffu);
    }
    after_n();
    const bool valid[2] = {L.useful && (tile + L.tok0 < n), L.useful && (tile + L.tok0 + 16 < n)};
    float raw[2][R], x[2][R];
    bool raise = false;
#pragma unroll
    for (int r = 0; r < R; r++) {
        // the row of (hd, r) is 4 hd + r: register r of lane group hd, its remainder 32 lanes further on
        float v[4];
#pragma unroll
        for (int c = 0; c < 4; c++) v[c] = s[c][r];
        uint32x2_t s01 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[0]), __float_as_uint(v[1]), false, false);
        uint32x2_t s23 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[2]), __float_as_uint(v[3]), false, false);
        raw[0][r] = (__uint_as_float(s01[0]) + __uint_as_float(s01[1])) * kn[0];    // kernels.cu:1707
        raw[1][r] = (__uint_as_float(s23[0]) + __uint_as_float(s23[1])) * kn[1];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            x[i][r] = valid[i] ? raw[i][r] - S.m_run[r] : kNegBig;
            raise = raise || (x[i][r] > kRaise);
        }
    }
    if (__any(raise)) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float mine = fmaxf(valid[0] ? raw[0][r] : kNegBig, valid[1] ? raw[1][r] : kNegBig);
            const float m_new = fmaxf(S.m_run[r], L.head_max(mine));
            const float alpha = __builtin_amdgcn_exp2f(S.m_run[r] - m_new);
            S.m_run[r] = m_new;
            S.l_run[r] *= alpha;
#pragma unroll
            for (int i = 0; i < 2; i++) x[i][r] = valid[i] ? raw[i][r] - m_new : kNegBig;
            // accumulator register r of a lane is row 4 pkg + r: query head r (of either KV head, value or remainder)
#pragma unroll
            for (int j = 0; j < 16; j++) S.o[j][r] *= alpha;
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const float pe = __builtin_amdgcn_exp2f(x[i][r]);
            S.l_run[r] += pe;
            const float pf = pe * vn[i];                            // (s * vn) * centroid, kernels.cu:1765
            const half_t hi = (half_t)pf;
            const half_t lo = (half_t)(pf - (float)hi);
            if (R < 4 || L.useful) {
                L.p_w[r * 32 + 4 * i] = hi;
                L.p_w[(r + 8) * 32 + 4 * i] = lo;
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    union { uint4 q; half8_t h; } pa;
    pa.q = *L.p_r;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    __builtin_amdgcn_s_setprio(2);
    // ---- O[row][dim 16 (pn % 8) + j of head pn / 8] += P[row][token] V[token][dim]
    if constexpr (BITS == 4) {
    uint32_t xe[2][4], xo[2][4];
#pragma unroll
    for (int dw = 0; dw < 2; dw++) {
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
#pragma unroll
            for (int pr = 0; pr < 2; pr++) {
                const uint32_t wa = t.v[sub][2 * pr][dw], wb = t.v[sub][2 * pr + 1][dw];
                xe[dw][2 * sub + pr] = (wa & 0x0f0f0f0fu) | ((wb << 4) & 0xf0f0f0f0u);
                xo[dw][2 * sub + pr] = ((wa >> 4) & 0x0f0f0f0fu) | (wb & 0xf0f0f0f0u);
            }
        }
    }
    after_v();
#pragma unroll
    for (int dw = 0; dw < 2; dw++) {
#pragma unroll
        for (int jp = 0; jp < 4; jp++) {
            const uint32_t sel = 0x0c0c0400u + ((uint32_t)jp << 8);
            union { uint32_t u[4]; half8_t h; } be, bo;
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                be.u[q4] = L.lut32(__builtin_amdgcn_perm(xe[dw][q4], L.lane_rep, sel));
                bo.u[q4] = L.lut32(__builtin_amdgcn_perm(xo[dw][q4], L.lane_rep, sel));
            }
            S.o[8 * dw + 2 * jp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, be.h, S.o[8 * dw + 2 * jp], 0, 0, 0);
            S.o[8 * dw + 2 * jp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, bo.h, S.o[8 * dw + 2 * jp + 1], 0, 0, 0);
        }
    }
    } else {
    // 2 bit: t.v[sub][i] holds the 16 codes (dims 0..15 of the lane's 16, field j at bit 2j) of token 4 pkg + i of
    // sub-tile `sub`.  y[sub][m]: bytes k = 0..3, byte k = the codes of the sub-tile's four tokens (token i at bit 2i)
    // for dim 4k + {0, 2, 1, 3}[m]: one look-up gives the four contraction slots 4 sub .. 4 sub + 3 of that dim.
    uint32_t y[2][4];
#pragma unroll
    for (int sub = 0; sub < 2; sub++) {
        const uint32_t w0 = t.v[sub][0], w1 = t.v[sub][1], w2 = t.v[sub][2], w3 = t.v[sub][3];
        // nibble k of xe: tokens (a, b) at dim 2k; of xo: at dim 2k + 1
        const uint32_t xe01 = (w0 & 0x33333333u) | ((w1 << 2) & 0xccccccccu), xo01 = ((w0 >> 2) & 0x33333333u) | (w1 & 0xccccccccu);
        const uint32_t xe23 = (w2 & 0x33333333u) | ((w3 << 2) & 0xccccccccu), xo23 = ((w2 >> 2) & 0x33333333u) | (w3 & 0xccccccccu);
        y[sub][0] = (xe01 & 0x0f0f0f0fu) | ((xe23 << 4) & 0xf0f0f0f0u);        // dims 0, 4, 8, 12
        y[sub][1] = ((xe01 >> 4) & 0x0f0f0f0fu) | (xe23 & 0xf0f0f0f0u);        // dims 2, 6, 10, 14
        y[sub][2] = (xo01 & 0x0f0f0f0fu) | ((xo23 << 4) & 0xf0f0f0f0u);        // dims 1, 5, 9, 13
        y[sub][3] = ((xo01 >> 4) & 0x0f0f0f0fu) | (xo23 & 0xf0f0f0f0u);        // dims 3, 7, 11, 15
    }
    after_v();
    // The look-ups run kAhead operands ahead of the MFMAs, held there by an empty asm statement the scheduler does not
    // move LDS reads across: left alone it sinks every look-up next to its MFMA and the wave waits out the LDS
    // latency sixteen times per tile.
    constexpr int kAhead = 4;
    uint2 qa[kAhead], qb[kAhead];
    auto look = [&](int j, uint2& a4, uint2& b4) {
        constexpr int kWhich[4] = {0, 2, 1, 3};
        const int m = kWhich[j & 3];
        const uint32_t sel = 0x0c0c0400u + ((uint32_t)(j >> 2) << 8);
        a4 = L.lut64(__builtin_amdgcn_perm(y[0][m], L.lane_rep, sel));
        b4 = L.lut64(__builtin_amdgcn_perm(y[1][m], L.lane_rep, sel));
    };
#pragma unroll
    for (int j = 0; j < kAhead; j++) look(j, qa[j], qb[j]);
#pragma unroll
    for (int j = 0; j < 16; j++) {
        union { uint32_t u[4]; half8_t h; } bv;
        bv.u[0] = qa[j % kAhead].x; bv.u[1] = qa[j % kAhead].y; bv.u[2] = qb[j % kAhead].x; bv.u[3] = qb[j % kAhead].y;
        if (j + kAhead < 16) look(j + kAhead, qa[j % kAhead], qb[j % kAhead]);
        asm volatile("" ::: "memory");
        S.o[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, bv.h, S.o[j], 0, 0, 0);
    }
    }
    __builtin_amdgcn_s_setprio(0);
}

// The wave's partial result per (head of the pair, query head): sink(hd, r, dims) is called by the 16 lanes that
// hold the rows of head hd with dims = the lane's 16 values of dim 16 (pn % 8) .. +15 (value + remainder rows added,
// 1 / alpha applied); all lanes end with l_run summed over the head.
template <int R, int BITS, class Sink>
__device__ __forceinline__ void pair_scan_finish(const PairLane<R, BITS>& L, PairState<R>& S, float inv_alpha, Sink sink) {
    const int khi = L.hd;                                       // lane group that holds the rows of head hd
#pragma unroll
    for (int r = 0; r < R; r++) {
        S.l_run[r] = L.head_sum(S.l_run[r]);
        float ov[16];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            float v = S.o[j][r];
            ov[j] = (v + __shfl_xor(v, 32, 64)) * inv_alpha;
        }
        if (L.pkg == khi) sink(L.hd, r, ov);
    }
}

}  // namespace twkv
