// kv_prefill_mfma.hip -- causal prefill attention over the 4-bit and 2-bit compressed
// caches for gfx950 (turbo_gqa_prefill_attention_kernel of the reference,
// kernels.cu:1874-1960: query token t attends cache rows 0..t of one sequence).
//
// The decode scan (kv_attention_mfma.hip, which documents the building blocks: LDS centroid
// table, K through ds_bpermute, value + remainder fp16 operands, lazy base-2 softmax, split
// partials) with the 16 MFMA rows filled: a wave takes a block of 8/R consecutive query
// tokens for the R query heads of its KV head (8 rows, plus 8 for the rounding remainders),
// so a tile of K and V codes is expanded once for 8/R query tokens instead of once per
// token.  Row m = 4*(kg%2) + i of the block sits in register i of the lanes with that
// kg%2: after v_permlane32_swap every lane owns one token for four rows.  Each row has its
// own causal limit.  Blocks differ in length by construction, so the work is always cut by
// the balanced walk (tiles of all blocks in one list, equal runs per group of waves).
// Same launches around it as for decode: rotate_kernel (q_rot) before, merge_rotate_kernel
// after; workspace block of query token t and head: ((t * num_heads + head) * ws_stride).

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"

#include <cstring>

namespace twkv {

namespace {

// reductions over the 32 lanes that hold the same rows (lanes with the same (lane / 16) % 2)
__device__ __forceinline__ float rows_max(float v) {
    v = fmaxf(v, __shfl_xor(v, 32, 64));
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float rows_sum(float v) {
    v += __shfl_xor(v, 32, 64);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace

template <int R, int BITS>
__global__ void __launch_bounds__(kMaxWaves * kWave)
prefill_mfma_kernel(AttnArgs a, int group_waves) {
    constexpr bool PAGED = false;
    constexpr int DEPTH = 1;
    constexpr int NQ = 8 / R;       // query tokens per block: 8 rows = NQ tokens x R heads
    constexpr int KW = BITS;        // dwords of K codes per lane and sub-tile (32 dims of one token)
    constexpr int VW = BITS;        // dwords of V codes per lane and sub-tile
    constexpr uint32_t kHeadBytes = BITS * 16;   // bytes of one head in a cache row
    constexpr float kAlpha = BITS == 4 ? kAlpha4 : kAlpha2;
    __shared__ __attribute__((aligned(16))) uint32_t tab_s[kTableWords];
    // per wave: P[row][k] as fp16, rows 0..7 = (query token, head), rows 8..15 = rounding remainders
    __shared__ __attribute__((aligned(16))) half_t p_s[kMaxWaves][16][32];
    // balanced walk: tiles of the sequences before g, and {tiles per group, total tiles}
    __shared__ int pre_s[kMaxBalanceSeqs + 1];
    __shared__ int bal_s[2];

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;   // wave index is wave-uniform: keep it scalar
    const int ln = lane & 15, kg = lane >> 4;
    // The workgroup's waves form groups of group_waves (one KV head each); a group walks its
    // own list of items and never synchronises with the others once the table is built.
    const int grp = wave / group_waves, wv = wave % group_waves;
    const int ngroups = (nthreads / kWave) / group_waves;
    const int Hk = a.num_kv_heads;

    const char* tab_lane = reinterpret_cast<const char*>(tab_s);
    // byte offset of this lane's replica inside a table entry (entries are 256 bytes apart)
    const uint32_t lane_rep = BITS == 4 ? (uint32_t)lane * 4u : (uint32_t)(lane & 31) * 8u;
    const uint32_t kvp = (uint32_t)Hk * kHeadBytes;    // bytes per cache row (all heads)
    const uint32_t nrow = (uint32_t)Hk * 2u;           // bytes per norm row
    // per-lane byte offsets inside a 16-token sub-tile, fixed for the whole kernel
    // K is loaded with lane l on token l/4, quarter l%4 of the head's row, so that four adjacent
    // lanes read one contiguous piece (a quarter of the cache accesses of loading in operand
    // order); ds_bpermute then moves it to operand order: lane (ln, kg) takes token ln, quarter kg.
    const uint32_t koff = (uint32_t)(lane >> 2) * kvp + (kHeadBytes / 4) * (uint32_t)(lane & 3);
    const int ksrc = 4 * (4 * ln + kg);                // byte address of the source lane for ds_bpermute
    uint32_t voff[VW];
#pragma unroll
    for (int i = 0; i < VW; i++) {
        if (BITS == 4) voff[i] = (uint32_t)(4 * kg + i) * kvp + 4u * (uint32_t)ln;
        else voff[i] = (uint32_t)(4 * kg + 2 * i + (ln & 1)) * kvp + 4u * (uint32_t)(ln >> 1);
    }
    // 2-bit V: which halves of its two dwords a lane keeps and which it hands to lane ^ 1
    const bool odd = (ln & 1) != 0;
    const uint32_t sel_keep = odd ? 0x07060302u : 0x05040100u;
    const uint32_t sel_send = odd ? 0x05040100u : 0x07060302u;
    const uint32_t sub_bytes = 16u * kvp;              // sub-tile b follows sub-tile a when contiguous
    // After the sub-tile swap a lane owns token ln of sub-tile (kg >> 1) for rows 4*(kg & 1) .. +3.
    const int my_sub = kg >> 1;
    const int row0 = 4 * (kg & 1);
    constexpr bool useful = true;
    const uint32_t noff = (uint32_t)ln * nrow + (PAGED ? 0u : (uint32_t)my_sub * 16u * nrow);
    // slot of that token in the k order of the P.V contraction: k = 8*(t/4) + 4*sub + t%4
    half_t* p_w = &p_s[wave][row0][8 * (ln >> 2) + 4 * my_sub + (ln & 3)];
    const uint4* p_r = reinterpret_cast<const uint4*>(&p_s[wave][ln][8 * kg]);
    constexpr float kRaise = 5.0f;                     // raise the running max only past 2^5

    auto lut32 = [&](uint32_t addr) -> uint32_t { return *reinterpret_cast<const uint32_t*>(tab_lane + addr); };
    auto lut64 = [&](uint32_t addr) -> uint2 { return *reinterpret_cast<const uint2*>(tab_lane + addr); };

    // ---- state of the piece in hand (wave-uniform): block of query tokens qb, keys [t0, t1)
    const int nblocks = (a.G + NQ - 1) / NQ;
    int chunk = 0, qb = 0, h = 0, n = 0, t0 = 0, t1 = 0, nseg = 0;
    const char *kseq = nullptr, *vseq = nullptr, *knseq = nullptr, *vnseq = nullptr;
    const int* bt = nullptr;
    constexpr long long seq_row0 = 0;                         // one sequence: cache row = key position
    // Balanced walk.  The 32-key tiles of all blocks form one list (block qb needs the keys
    // 0 .. its last query); every group of waves takes `quota` consecutive tiles of it, cut
    // where a block ends.  The piece of block qb that group number gb takes is partial
    // gb - (tiles before qb) / quota of each of the block's (query token, head) rows.
    int bal_cur = 0, bal_end = 0, bal_g = 0, bal_quota = 1, bal_gb = 0;
    auto next_piece = [&]() -> bool {
        if (bal_cur >= bal_end) return false;
        while (pre_s[bal_g + 1] <= bal_cur) bal_g++;
        qb = bal_g;
        const int first = pre_s[qb], last = pre_s[qb + 1];
        const int stop = min(bal_end, last);
        n = min(qb * NQ + NQ, a.G);                           // keys the block's last query attends
        t0 = 32 * (bal_cur - first);
        t1 = min(32 * (stop - first), n);
        chunk = bal_gb - first / bal_quota;
        nseg = (last - 1) / bal_quota - first / bal_quota + 1;
        bal_cur = stop;
        h = wv;
        kseq = reinterpret_cast<const char*>(a.k) + (long long)h * kHeadBytes;
        vseq = reinterpret_cast<const char*>(a.v) + (long long)h * kHeadBytes;
        knseq = reinterpret_cast<const char*>(a.k_norms) + (long long)h * 2;
        vnseq = reinterpret_cast<const char*>(a.v_norms) + (long long)h * 2;
        return true;
    };

    // Buffer descriptors: base = first cache row of the tile (contiguous cache) or of the
    // 16-token page (paged cache), extent = the rows that exist, so lanes past the end
    // of the sequence read zeros instead of foreign memory.  All scalar.
    auto page_row = [&](int ts) -> long long {   // paged: past the end re-read the last page (masked)
        return (long long)uniform(bt[min(ts, t1 - 1) >> 4]) * kPageTokens;
    };
    auto load_k = [&](__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t (&dst)[KW]) {
        if constexpr (BITS == 4) {
            uint32x4_t q = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
            dst[0] = q[0]; dst[1] = q[1]; dst[2] = q[2]; dst[3] = q[3];
        } else {
            uint32x2_t q = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
            dst[0] = q[0]; dst[1] = q[1];
        }
    };
    auto issue_k = [&](uint32_t (&kreg)[2][KW], int tile) {
        if (PAGED) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++)
                load_k(make_rsrc(kseq + page_row(tile + 16 * sub) * kvp, kPageTokens * (int)kvp), koff, kreg[sub]);
        } else {
            __amdgpu_buffer_rsrc_t r = make_rsrc(kseq + (seq_row0 + tile) * kvp, max(min(n - tile, 32), 0) * (int)kvp);
            load_k(r, koff, kreg[0]);
            load_k(r, koff + sub_bytes, kreg[1]);
        }
    };
    auto issue_v = [&](uint32_t (&vreg)[2][VW], int tile) {
        if (PAGED) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                __amdgpu_buffer_rsrc_t r = make_rsrc(vseq + page_row(tile + 16 * sub) * kvp, kPageTokens * (int)kvp);
#pragma unroll
                for (int i = 0; i < VW; i++) vreg[sub][i] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff[i], 0, 0);
            }
        } else {
            __amdgpu_buffer_rsrc_t r = make_rsrc(vseq + (seq_row0 + tile) * kvp, max(min(n - tile, 32), 0) * (int)kvp);
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                for (int i = 0; i < VW; i++)
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

    // DEPTH tiles of loads are in flight per wave; each register set is re-issued (for the
    // tile DEPTH further on) as soon as its contents have been expanded.
    uint32_t kring[DEPTH][2][KW];
    uint32_t vring[DEPTH][2][VW];
    uint32_t nring[DEPTH];
    auto issue_first = [&]() {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            if (d == 0 || t0 + 32 * d < t1) {
                issue_k(kring[d], t0 + 32 * d);
                nring[d] = issue_n(t0 + 32 * d);
                issue_v(vring[d], t0 + 32 * d);
            }
        }
    };

    // wave 0 leaves the prefix of tiles per block in LDS
    if (wave == 0) {
        int carry = 0, tmax = 0;
        for (int base = 0; base < nblocks; base += kWave) {
            const int gg = base + lane;
            const int t = gg < nblocks ? (min(gg * NQ + NQ, a.G) + 31) >> 5 : 0;
            tmax = max(tmax, t);
            int inc = t;
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                int up = __shfl_up(inc, off, 64);
                if (lane >= off) inc += up;
            }
            if (gg < nblocks) pre_s[gg + 1] = carry + inc;
            carry += __shfl(inc, kWave - 1, 64);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) tmax = max(tmax, __shfl_xor(tmax, off, 64));
        if (lane == 0) {
            pre_s[0] = 0;
            const int groups = (int)gridDim.x * ngroups;
            const int quota = (carry + groups - 1) / groups;
            const int by_slots = (tmax + a.max_slots - 2) / (a.max_slots - 1);   // a block gets <= max_slots pieces
            bal_s[0] = max(max(quota, by_slots), 1);
            bal_s[1] = carry;
        }
    }
    // ---- dequantization table, once per workgroup: entry e fills 256 bytes with replicas
    for (int i = tid * 4; i < kTableWords; i += nthreads * 4) {
        const int e = i >> 6;
        if constexpr (BITS == 4) {
            half2_t p = {(half_t)(kAlpha * kCentroids4[e & 15]), (half_t)(kAlpha * kCentroids4[e >> 4])};
            uint32_t w = *reinterpret_cast<uint32_t*>(&p);
            *reinterpret_cast<uint4*>(&tab_s[i]) = uint4{w, w, w, w};
        } else {
            half2_t p0 = {(half_t)(kAlpha * kCentroids2[e & 3]), (half_t)(kAlpha * kCentroids2[(e >> 4) & 3])};
            half2_t p1 = {(half_t)(kAlpha * kCentroids2[(e >> 2) & 3]), (half_t)(kAlpha * kCentroids2[(e >> 6) & 3])};
            uint32_t w0 = *reinterpret_cast<uint32_t*>(&p0), w1 = *reinterpret_cast<uint32_t*>(&p1);
            *reinterpret_cast<uint4*>(&tab_s[i]) = uint4{w0, w1, w0, w1};
        }
    }
    for (int i = tid; i < kMaxWaves * 16 * 32 / 2; i += nthreads) reinterpret_cast<uint32_t*>(p_s)[i] = 0u;
    __syncthreads();             // the only workgroup-wide barrier; every wave reaches it

    {
        bal_quota = bal_s[0];
        bal_gb = (int)blockIdx.x * ngroups + grp;
        const long long start = (long long)bal_gb * bal_quota;
        bal_cur = (int)min(start, (long long)bal_s[1]);
        bal_end = (int)min(start + bal_quota, (long long)bal_s[1]);
        int lo = 0, hi = nblocks;                             // last block that starts at or before bal_cur
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (pre_s[mid] <= bal_cur) lo = mid; else hi = mid;
        }
        bal_g = lo;
    }

    while (next_piece()) {
        issue_first();
        const int ntiles = (t1 - t0 + 31) >> 5;

        float4_t o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = float4_t{0.f, 0.f, 0.f, 0.f};
        float m_run[4], l_run[4];
        int lim[4];                                           // causal limit of row row0 + i: keys < lim
#pragma unroll
        for (int i = 0; i < 4; i++) {
            m_run[i] = kNegBig; l_run[i] = 0.0f;
            const int gq = qb * NQ + (row0 + i) / R;
            lim[i] = gq < a.G ? min(gq + 1, t1) : 0;
        }

        // A operand of the score MFMAs: row m < 8 = (query token qb*NQ + m/R, head h*R + m%R) carries
        // the fp16 value of q_rot[32kg + 8j + i], row m + 8 what the rounding left over.  The 2-bit
        // table returns the codes of a byte in the order 0,2,1,3.
        half8_t aq[4];
        {
            const int hq = ln & 7;
            const bool lo_part = (ln & 8) != 0;
            const int gq = qb * NQ + hq / R;
            const float* qr = a.qrot + ((long long)min(gq, a.G - 1) * a.num_heads + (long long)h * R + hq % R) * a.ws_stride + 32 * kg;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float4 v0 = *reinterpret_cast<const float4*>(qr + 8 * j);
                float4 v1 = *reinterpret_cast<const float4*>(qr + 8 * j + 4);
                float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const int src = BITS == 4 ? i : ((i & 4) | ((i & 1) << 1) | ((i & 2) >> 1));
                    float x = (gq < a.G) ? v[src] : 0.0f;
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
            if (DEPTH > 1 && it >= ntiles) break;
            uint32_t (&kreg)[2][KW] = kring[d];
            uint32_t (&vreg)[2][VW] = vring[d];
            uint32_t& nreg = nring[d];
            const int tile = t0 + 32 * it;
            const int next_tile = tile + 32 * DEPTH;
            const bool more = it + DEPTH < ntiles;

            // ---- scores S[head][token] for both sub-tiles
            float4_t s[2];
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                uint32_t kw[KW];
#pragma unroll
                for (int i = 0; i < KW; i++) kw[i] = (uint32_t)__builtin_amdgcn_ds_bpermute(ksrc, (int)kreg[sub][i]);
                union { uint32_t u[4]; half8_t h; } kv[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if constexpr (BITS == 4) {
                        const uint32_t w = kw[j];
                        kv[j].u[0] = lut32(__builtin_amdgcn_perm(w, lane_rep, 0x0c0c0400u));
                        kv[j].u[1] = lut32(__builtin_amdgcn_perm(w, lane_rep, 0x0c0c0500u));
                        kv[j].u[2] = lut32(__builtin_amdgcn_perm(w, lane_rep, 0x0c0c0600u));
                        kv[j].u[3] = lut32(__builtin_amdgcn_perm(w, lane_rep, 0x0c0c0700u));
                    } else {
                        const uint32_t w = kw[j >> 1];
                        const uint32_t sel = (j & 1) ? 0x0c0c0600u : 0x0c0c0400u;
                        uint2 l0 = lut64(__builtin_amdgcn_perm(w, lane_rep, sel));
                        uint2 l1 = lut64(__builtin_amdgcn_perm(w, lane_rep, sel + 0x100u));
                        kv[j].u[0] = l0.x; kv[j].u[1] = l0.y; kv[j].u[2] = l1.x; kv[j].u[3] = l1.y;
                    }
                }
                s[sub] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; j++) s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aq[j], kv[j].h, s[sub], 0, 0, 0);
            }
            if (more) issue_k(kreg, next_tile);

            // ---- online softmax (base 2): this lane owns key ln of sub-tile my_sub for rows row0 .. row0+3
            const float kn = h2f_bits(nreg & 0xffffu), vn = h2f_bits(nreg >> 16);
            if (more) nreg = issue_n(next_tile);
            const int key = tile + 16 * my_sub + ln;
            float raw[4], x[4];
            bool raise = false;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // rows m (value part of q_rot) and m + 8 (remainder) sit 32 lanes apart; the swap also
                // moves sub-tile b into the upper half of the wave
                uint32x2_t sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(s[0][i]), __float_as_uint(s[1][i]), false, false);
                raw[i] = (__uint_as_float(sw[0]) + __uint_as_float(sw[1])) * kn;    // kernels.cu:1707
                x[i] = key < lim[i] ? raw[i] - m_run[i] : kNegBig;
                raise = raise || (x[i] > kRaise);
            }
            if (__any(raise)) {                                         // rare after the first tiles
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float m_new = fmaxf(m_run[i], rows_max(key < lim[i] ? raw[i] : kNegBig));
                    float alpha = __builtin_amdgcn_exp2f(m_run[i] - m_new);
                    m_run[i] = m_new;
                    l_run[i] *= alpha;
                    x[i] = key < lim[i] ? raw[i] - m_new : kNegBig;
#pragma unroll
                    for (int j = 0; j < 8; j++) o[j][i] *= alpha;       // rows m and m + 8 live in the lanes with this kg % 2
                }
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float p = __builtin_amdgcn_exp2f(x[i]);
                l_run[i] += p;
                float pf = p * vn;                                      // (s * vn) * centroid, kernels.cu:1765
                half_t hi = (half_t)pf;
                half_t lo = (half_t)(pf - (float)hi);
                p_w[i * 32] = hi;
                p_w[(i + 8) * 32] = lo;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            union { uint4 q; half8_t h; } pa;
            pa.q = *p_r;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            __builtin_amdgcn_wave_barrier();

            // ---- O[head][dim 8ln + j] += P[head][token] V[token][dim]
            if constexpr (BITS == 4) {
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
                        be.u[q4] = lut32(__builtin_amdgcn_perm(xe[q4], lane_rep, sel));
                        bo.u[q4] = lut32(__builtin_amdgcn_perm(xo[q4], lane_rep, sel));
                    }
                    o[2 * jp] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, be.h, o[2 * jp], 0, 0, 0);
                    o[2 * jp + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, bo.h, o[2 * jp + 1], 0, 0, 0);
                }
            } else {
                // Per sub-tile: wa = 16-bit codes of tokens (4kg, 4kg+2), wb = of (4kg+1, 4kg+3) for
                // this lane's 8 dims.  ie/io: per byte, low nibble = token a dims (d, d+1), high
                // nibble = token b dims (d, d+1); bytes = (tokens 0,1 | d=0), (0,1 | d=4),
                // (2,3 | d=0), (2,3 | d=4) for ie and d = 2, 6 for io.
                uint32_t ie[2], io[2];
#pragma unroll
                for (int sub = 0; sub < 2; sub++) {
                    const uint32_t keep = __builtin_amdgcn_perm(vreg[sub][1], vreg[sub][0], sel_keep);
                    const uint32_t send = __builtin_amdgcn_perm(vreg[sub][1], vreg[sub][0], sel_send);
                    const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1, 0xf, 0xf, false);  // lane ^ 1
                    const uint32_t wa = odd ? recv : keep, wb = odd ? keep : recv;
                    ie[sub] = (wa & 0x0f0f0f0fu) | ((wb << 4) & 0xf0f0f0f0u);
                    io[sub] = ((wa >> 4) & 0x0f0f0f0fu) | (wb & 0xf0f0f0f0u);
                }
                if (more) issue_v(vreg, next_tile);
#pragma unroll
                for (int q = 0; q < 4; q++) {            // dims (2q, 2q+1): 4 look-ups, 2 MFMAs
                    const uint32_t x0 = (q & 1) ? io[0] : ie[0], x1 = (q & 1) ? io[1] : ie[1];
                    const uint32_t sel = 0x0c0c0400u + ((uint32_t)(q >> 1) << 8);
                    uint2 l00 = lut64(__builtin_amdgcn_perm(x0, lane_rep, sel));
                    uint2 l01 = lut64(__builtin_amdgcn_perm(x0, lane_rep, sel + 0x200u));
                    uint2 l10 = lut64(__builtin_amdgcn_perm(x1, lane_rep, sel));
                    uint2 l11 = lut64(__builtin_amdgcn_perm(x1, lane_rep, sel + 0x200u));
                    union { uint32_t u[4]; half8_t h; } be, bo;
                    be.u[0] = l00.x; be.u[1] = l01.x; be.u[2] = l10.x; be.u[3] = l11.x;
                    bo.u[0] = l00.y; bo.u[1] = l01.y; bo.u[2] = l10.y; bo.u[3] = l11.y;
                    o[2 * q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, be.h, o[2 * q], 0, 0, 0);
                    o[2 * q + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa.h, bo.h, o[2 * q + 1], 0, 0, 0);
                }
            }
            if (DEPTH > 1) __builtin_amdgcn_sched_barrier(0);   // keep the unrolled tiles from interleaving (register pressure)
          }
        }

        // ---- partial results of this piece: one per (query token, head) row
#pragma unroll
        for (int i = 0; i < 4; i++) {
            l_run[i] = rows_sum(l_run[i]);                                        // masked lanes hold 0
#pragma unroll
            for (int j = 0; j < 8; j++) o[j][i] += __shfl_xor(o[j][i], 32, 64);   // row m + row m+8 (remainder of P)
        }
        if (kg < 2) {                                          // lanes kg hold rows 4kg .. 4kg+3
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int m = 4 * kg + i;
                const int gq = qb * NQ + m / R;
                if (gq < a.G) {
                    float* part0 = a.ws + ((long long)gq * a.num_heads + (long long)h * R + m % R) * a.ws_stride;
                    float* part = part0 + (long long)chunk * kPartialFloats;
#pragma unroll
                    for (int j = 0; j < 8; j++) part[8 * ln + j] = o[j][i] * (1.0f / kAlpha);
                    if (ln == 0) {
                        part[kHeadDim] = m_run[i];
                        part[kHeadDim + 1] = l_run[i];
                        // the piece with key 0 tells the merge how many partials there are
                        if (t0 == 0) reinterpret_cast<int*>(part0)[kHeadDim + 2] = nseg;
                    }
                }
            }
        }
    }
}

// The prefill kernel serves: causal positions (query t attends 0..t), one wave per KV head with
// all KV heads in one group, room for the tile prefix of every block, >= 3 partial slots.
bool prefill_mfma_usable(const AttnArgs& a) {
    const int R = a.num_heads / a.num_kv_heads;
    if (a.pos_mode != kPosIota || a.block_table) return false;
    if (a.bits != 4 && a.bits != 2) return false;
    if (R != 1 && R != 2 && R != 4) return false;
    if (a.num_kv_heads > kGroupWaves || kMaxWaves % a.num_kv_heads != 0) return false;
    if ((a.G + 8 / R - 1) / (8 / R) > kMaxBalanceSeqs) return false;
    return a.max_slots >= 3 && a.ws && a.qrot;
}

void launch_prefill_mfma_scan(const AttnArgs& a, hipStream_t s) {
    const int waves = a.num_kv_heads;
    const int R = a.num_heads / a.num_kv_heads;
    const int ngroups = kMaxWaves / waves;
    // tiles in all blocks together; no more groups than tiles
    const long long nq = 8 / R, nblocks = (a.G + nq - 1) / nq;
    long long tiles = 0;
    for (long long b = 0; b < nblocks; b++) tiles += (((b + 1) * nq < a.G ? (b + 1) * nq : a.G) + 31) / 32;
    int grid = compute_units();
    if (tiles < (long long)grid * ngroups) grid = (int)((tiles + ngroups - 1) / ngroups);
    if (grid < 1) grid = 1;
    const dim3 g3(grid), b3(ngroups * waves * kWave);
    note_scan_kernel("prefill_mfma_kernel");
#define TW_LAUNCH_P(RR, BB) launch_scan_kernel(prefill_mfma_kernel<RR, BB>, g3, b3, s, a, waves)
    if (a.bits == 4) {
        if (R == 1) TW_LAUNCH_P(1, 4); else if (R == 2) TW_LAUNCH_P(2, 4); else TW_LAUNCH_P(4, 4);
    } else {
        if (R == 1) TW_LAUNCH_P(1, 2); else if (R == 2) TW_LAUNCH_P(2, 2); else TW_LAUNCH_P(4, 2);
    }
#undef TW_LAUNCH_P
}

}  // namespace twkv
