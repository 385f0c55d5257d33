// kv_attention_mfma2c.hip -- GQA decode attention over the 2-bit compressed cache for
// gfx950 with 8 KV heads: the waves of a group load whole cache rows together.
//
// Same mathematics, work cutting (even chunks / balanced walk), tile arithmetic and
// partials as attention_mfma_kernel (kv_attention_mfma.hip, which documents them).  What
// differs is how the bytes arrive.  A 2-bit head is 32 bytes per token, a quarter of a
// cache line, and with one head per wave four waves pull the same line at different
// moments: measured 4.4 TB/s for that pattern against 5.7-6.0 TB/s for this one.  Here the
// 8 waves of a group read a 32-token tile as what it is in memory, 8 KB of contiguous
// rows for K and 8 KB for V (wave w: rows 4w..4w+3, one 16-byte load per lane), plus the
// two 512-byte blocks of norms once per group instead of once per wave, and leave them
// in LDS; every wave then picks its head's bytes from there in MFMA operand order (no
// ds_bpermute).  The price is one workgroup barrier per tile: the two groups of a
// workgroup walk their items in lockstep, a round lasting as long as the longer item.
// Tiles are double-buffered: the loads of tile t+1 are issued before the arithmetic of
// tile t and stored to LDS after it.

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"

namespace twkv {

namespace {

constexpr int kCoopHeads = 8;                    // KV heads = waves per group; a cache row is 8 x 32 bytes
constexpr int kRowBytes = kCoopHeads * 32;
constexpr int kTileRow = kRowBytes + 16;         // LDS row stride: spreads the operand-order reads over the banks
constexpr int kCoopSeqs = 1024;                  // sequences the balanced walk can index here (LDS is nearly full)

}  // namespace

template <bool PAGED, int R>
__global__ void __launch_bounds__(kMaxWaves * kWave)
attention_mfma2c_kernel(AttnArgs a, int total_items) {
    constexpr float kAlpha = kAlpha2;
    __shared__ __attribute__((aligned(16))) uint32_t tab_s[kTableWords];
    // per wave: P[row][k] as fp16, rows 0..R-1 = heads, rows 8..8+R-1 = rounding remainders
    __shared__ __attribute__((aligned(16))) half_t p_s[kMaxWaves][16][32];
    // per group, double-buffered: the tile's K rows, V rows and norm rows (K norms, V norms)
    __shared__ __attribute__((aligned(16))) char kt_s[2][2][32 * kTileRow];
    __shared__ __attribute__((aligned(16))) char vt_s[2][2][32 * kTileRow];
    __shared__ __attribute__((aligned(16))) char nn_s[2][2][2][32 * 16];
    __shared__ int pre_s[kCoopSeqs + 1];
    __shared__ int bal_s[2];
    __shared__ int nt_s[2];                      // tiles of each group's item in this round

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;
    const int ln = lane & 15, kg = lane >> 4;
    const int grp = wave / kCoopHeads, wv = wave % kCoopHeads;     // wv = KV head of this wave
    const int ngroups = (nthreads / kWave) / kCoopHeads;

    const char* tab_lane = reinterpret_cast<const char*>(tab_s);
    const uint32_t lane_rep = (uint32_t)(lane & 31) * 8u;          // this lane's replica inside a 256-byte table entry
    // 2-bit V: which halves of its two dwords a lane keeps and which it hands to lane ^ 1
    const bool odd = (ln & 1) != 0;
    const uint32_t sel_keep = odd ? 0x07060302u : 0x05040100u;
    const uint32_t sel_send = odd ? 0x05040100u : 0x07060302u;
    // After the sub-tile swap a lane owns token ln of sub-tile (kg >> 1); lanes with odd kg idle.
    const int my_sub = kg >> 1;
    const bool useful = (kg & 1) == 0;
    // slot of that token in the k order of the P.V contraction: k = 8*(t/4) + 4*sub + t%4
    half_t* p_w = &p_s[wave][0][8 * (ln >> 2) + 4 * my_sub + (ln & 3)];
    const uint4* p_r = reinterpret_cast<const uint4*>(&p_s[wave][ln][8 * kg]);
    constexpr float kRaise = 5.0f;                                 // raise the running max only past 2^5

    // what this lane carries of a tile: 16 bytes of row 4wv + lane/16 (sub-tile wv/4)
    const uint32_t goff = (uint32_t)(PAGED ? (wv & 3) : wv) * 1024u + (uint32_t)lane * 16u;
    const int stash_off = (4 * wv + (lane >> 4)) * kTileRow + 16 * (lane & 15);
    // what it picks from a tile in LDS, in MFMA operand order
    int kro[2], vro[2][2];
#pragma unroll
    for (int sub = 0; sub < 2; sub++) {
        kro[sub] = (16 * sub + ln) * kTileRow + 32 * wv + 8 * kg;                       // dims 32kg..32kg+31 of token ln
#pragma unroll
        for (int i = 0; i < 2; i++)                                                     // tokens 4kg+2i+(ln&1), dims 16(ln/2)..
            vro[sub][i] = (16 * sub + 4 * kg + 2 * i + (ln & 1)) * kTileRow + 32 * wv + 4 * (ln >> 1);
    }
    const int nro = (16 * my_sub + ln) * 16 + 2 * wv;

    auto lut64 = [&](uint32_t addr) -> uint2 { return *reinterpret_cast<const uint2*>(tab_lane + addr); };

    // ---- state of the item in hand (uniform over the group)
    int chunk = 0, g = 0, n = 0, t0 = 0, t1 = 0, nseg = 0;
    const int h = wv;
    const int* bt = nullptr;
    long long seq_row0 = 0;
    auto decode = [&](int item) -> bool {                    // false: the chunk holds no token
        chunk = item % a.nsplit;
        g = item / a.nsplit;
        n = uniform(seq_pos(a, g)) + 1;
        // Even chunks of whole tiles (the two groups of a workgroup walk in lockstep, so equal shares
        // are the fastest); a sequence with fewer tiles than chunks gives its first chunks a tile each.
        // The live partials are 0 .. nseg-1 either way, and the merge is told nseg.
        const int tiles = (n + 31) >> 5;
        nseg = min(a.nsplit, tiles);
        const int b0 = tiles >= a.nsplit ? (int)(((long long)chunk * tiles) / a.nsplit) : min(chunk, tiles);
        const int b1 = tiles >= a.nsplit ? (int)(((long long)(chunk + 1) * tiles) / a.nsplit) : min(chunk + 1, tiles);
        t0 = 32 * b0;
        t1 = min(32 * b1, n);
        if (t0 >= t1) return false;
        bt = PAGED ? a.block_table + (long long)g * a.bt_stride : nullptr;
        seq_row0 = (long long)g * a.seq_stride_rows;
        return true;
    };
    int bal_cur = 0, bal_end = 0, bal_g = 0, bal_quota = 1, bal_gb = 0;
    auto next_piece = [&]() -> bool {                        // the balanced walk of attention_mfma_kernel
        if (bal_cur >= bal_end) return false;
        while (pre_s[bal_g + 1] <= bal_cur) bal_g++;
        g = bal_g;
        const int first = pre_s[g], last = pre_s[g + 1];
        const int stop = min(bal_end, last);
        n = uniform(seq_pos(a, g)) + 1;
        t0 = 32 * (bal_cur - first);
        t1 = min(32 * (stop - first), n);
        chunk = bal_gb - first / bal_quota;
        nseg = (last - 1) / bal_quota - first / bal_quota + 1;
        bal_cur = stop;
        bt = PAGED ? a.block_table + (long long)g * a.bt_stride : nullptr;
        seq_row0 = (long long)g * a.seq_stride_rows;
        return true;
    };

    // Global -> registers: this lane's share of the tile at `tile`.  Rows past the end of the
    // sequence are cut by the descriptors' extents and read as zeros.
    // Paged: the two block-table entries of a tile (even lanes: first page, odd lanes: second) are
    // fetched a tile ahead of its loads, so that no load waits for its page number.
    auto fetch_pages = [&](int tile) -> int { return bt[min(tile + 16 * (lane & 1), t1 - 1) >> 4]; };
    auto load_tile = [&](int tile, int pages, uint4& kr, uint4& vr, uint4& nr) {
        long long row;
        int rows;
        if (PAGED) {          // a page is one 16-token sub-tile; past the end the last page is re-read (masked)
            row = (long long)__builtin_amdgcn_readlane(pages, wv >> 2) * kPageTokens;
            rows = kPageTokens;
        } else {
            row = seq_row0 + tile;
            rows = max(min(n - tile, 32), 0);
        }
        __amdgpu_buffer_rsrc_t rk = make_rsrc(reinterpret_cast<const char*>(a.k) + row * kRowBytes, rows * kRowBytes);
        __amdgpu_buffer_rsrc_t rv = make_rsrc(reinterpret_cast<const char*>(a.v) + row * kRowBytes, rows * kRowBytes);
        uint32x4_t k4 = __builtin_amdgcn_raw_buffer_load_b128(rk, (int)goff, 0, kStreamCodes);
        uint32x4_t v4 = __builtin_amdgcn_raw_buffer_load_b128(rv, (int)goff, 0, kStreamCodes);
        kr = uint4{k4[0], k4[1], k4[2], k4[3]};
        vr = uint4{v4[0], v4[1], v4[2], v4[3]};
        if (wv < 2 && lane < 32) {                           // wave 0: the 32 K-norm rows, wave 1: the V-norm rows
            const char* nbase = reinterpret_cast<const char*>(wv ? a.v_norms : a.k_norms);
            if (PAGED) {      // pages are whole: a plain load, one page per half of the tile
                const int p0 = __builtin_amdgcn_readlane(pages, 0), p1 = __builtin_amdgcn_readlane(pages, 1);
                const long long prow = (long long)((lane & 16) ? p1 : p0) * kPageTokens + (lane & 15);
                nr = *reinterpret_cast<const uint4*>(nbase + prow * 16);
            } else {
                __amdgpu_buffer_rsrc_t rn = make_rsrc(nbase + (seq_row0 + tile) * 16, max(min(n - tile, 32), 0) * 16);
                uint32x4_t n4 = __builtin_amdgcn_raw_buffer_load_b128(rn, lane * 16, 0, kStreamCodes);
                nr = uint4{n4[0], n4[1], n4[2], n4[3]};
            }
        }
    };
    auto stash = [&](int buf, const uint4& kr, const uint4& vr, const uint4& nr) {
        *reinterpret_cast<uint4*>(&kt_s[grp][buf][stash_off]) = kr;
        *reinterpret_cast<uint4*>(&vt_s[grp][buf][stash_off]) = vr;
        if (wv < 2 && lane < 32) *reinterpret_cast<uint4*>(&nn_s[grp][buf][wv][lane * 16]) = nr;
    };

    // ---- even chunks or balanced walk (as in attention_mfma_kernel); wave 0 leaves the prefix of tiles in LDS
    bool balanced = false;
    if (a.balance && a.G <= kCoopSeqs) {
        int carry = 0, tmin = 0x7fffffff, tmax = 0;
        for (int base = 0; base < a.G; base += kWave) {
            const int gg = base + lane;
            const int t = gg < a.G ? (seq_pos(a, gg) + 1 + 31) >> 5 : 0;
            if (gg < a.G) { tmin = min(tmin, t); tmax = max(tmax, t); }
            if (wave == 0) {
                int inc = t;
#pragma unroll
                for (int off = 1; off < kWave; off <<= 1) {
                    int up = __shfl_up(inc, off, 64);
                    if (lane >= off) inc += up;
                }
                if (gg < a.G) pre_s[gg + 1] = carry + inc;
                carry += __shfl(inc, kWave - 1, 64);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            tmin = min(tmin, __shfl_xor(tmin, off, 64));
            tmax = max(tmax, __shfl_xor(tmax, off, 64));
        }
        balanced = uniform((tmax - tmin) * 8 > tmax ? 1 : 0) != 0;
        if (wave == 0 && lane == 0) {
            pre_s[0] = 0;
            const int groups = (int)gridDim.x * ngroups;
            const int quota = (carry + groups - 1) / groups;
            const int by_slots = (tmax + a.max_slots - 2) / (a.max_slots - 1);
            bal_s[0] = max(max(quota, by_slots), 1);
            bal_s[1] = carry;
        }
    }
    // ---- dequantization table: entry e (a byte = 4 codes) -> 4 fp16 centroids in the order 0, 2, 1, 3; 32 replicas
    for (int i = tid * 4; i < kTableWords; i += nthreads * 4) {
        const int e = i >> 6;
        half2_t p0 = {(half_t)(kAlpha * kCentroids2[e & 3]), (half_t)(kAlpha * kCentroids2[(e >> 4) & 3])};
        half2_t p1 = {(half_t)(kAlpha * kCentroids2[(e >> 2) & 3]), (half_t)(kAlpha * kCentroids2[(e >> 6) & 3])};
        uint32_t w0 = *reinterpret_cast<uint32_t*>(&p0), w1 = *reinterpret_cast<uint32_t*>(&p1);
        *reinterpret_cast<uint4*>(&tab_s[i]) = uint4{w0, w1, w0, w1};
    }
    for (int i = tid; i < kMaxWaves * 16 * 32 / 2; i += nthreads) reinterpret_cast<uint32_t*>(p_s)[i] = 0u;
    if (tid < 2) nt_s[tid] = 0;
    __syncthreads();

    const int item_step = (int)gridDim.x * ngroups;
    int item = (int)blockIdx.x * ngroups + grp;
    if (balanced) {
        bal_quota = bal_s[0];
        bal_gb = (int)blockIdx.x * ngroups + grp;
        const long long start = (long long)bal_gb * bal_quota;
        bal_cur = (int)min(start, (long long)bal_s[1]);
        bal_end = (int)min(start + bal_quota, (long long)bal_s[1]);
        int lo = 0, hi = a.G;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (pre_s[mid] <= bal_cur) lo = mid; else hi = mid;
        }
        bal_g = lo;
    }
    auto advance = [&]() -> bool {                           // the group's next item that holds tokens
        if (balanced) return next_piece();
        while (item < total_items) {
            const bool ok = decode(item);
            item += item_step;
            if (ok) return true;
        }
        return false;
    };

    // ---- rounds: every group takes its next item; all waves of the workgroup step through
    // max(tiles) tiles with one barrier per tile
    for (;;) {
        const bool have = advance();
        const int ntiles = have ? (t1 - t0 + 31) >> 5 : 0;
        uint4 ra[3] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
        int pages_next = 0;                                  // entries of the tile after the one being loaded
        if (have) {
            int pages = 0;
            if (PAGED) {
                pages = fetch_pages(t0);
                pages_next = fetch_pages(t0 + 32);
            }
            load_tile(t0, pages, ra[0], ra[1], ra[2]);
            stash(0, ra[0], ra[1], ra[2]);
        }
        if (wv == 0 && lane == 0) nt_s[grp] = ntiles;
        __syncthreads();
        const int round_tiles = max(nt_s[0], nt_s[1]);
        if (round_tiles == 0) break;                         // no group has anything left: uniform over the workgroup

        float4_t o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = float4_t{0.f, 0.f, 0.f, 0.f};
        float m_run[R], l_run[R];
#pragma unroll
        for (int r = 0; r < R; r++) { m_run[r] = kNegBig; l_run[r] = 0.0f; }

        // A operand of the score MFMAs: q_rot[head][32kg + 8j + i]; row m carries the fp16 value of
        // head m, row m + 8 what the rounding left over; the table returns a byte's codes in the order 0,2,1,3
        half8_t aq[4];
        if (have) {
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
                    const int src = (i & 4) | ((i & 1) << 1) | ((i & 2) >> 1);
                    float x = (hq < R) ? v[src] : 0.0f;
                    half_t hi = (half_t)x;
                    half_t lo = (half_t)(x - (float)hi);
                    aq[j][i] = lo_part ? lo : hi;
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) aq[j] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }

        auto compute = [&](int buf, int tile) {
            const char* ktb = &kt_s[grp][buf][0];
            const char* vtb = &vt_s[grp][buf][0];
            // ---- scores S[head][token] for both sub-tiles
            float4_t s[2];
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                const uint2 kw = *reinterpret_cast<const uint2*>(ktb + kro[sub]);
                s[sub] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t w = (j >> 1) ? kw.y : kw.x;
                    const uint32_t sel = (j & 1) ? 0x0c0c0600u : 0x0c0c0400u;
                    uint2 l0 = lut64(__builtin_amdgcn_perm(w, lane_rep, sel));
                    uint2 l1 = lut64(__builtin_amdgcn_perm(w, lane_rep, sel + 0x100u));
                    union { uint32_t u[4]; half8_t h; } kv;
                    kv.u[0] = l0.x; kv.u[1] = l0.y; kv.u[2] = l1.x; kv.u[3] = l1.y;
                    s[sub] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aq[j], kv.h, s[sub], 0, 0, 0);
                }
            }

            // (wave priority rises through the tile, as in kv_pair_scan.hpp: 1 % here, where a barrier per tile
            // keeps the waves closer together anyway)
            __builtin_amdgcn_s_setprio(1);
            // ---- online softmax (base 2): this lane owns token ln of sub-tile my_sub
            const float kn = h2f_bits(*reinterpret_cast<const uint16_t*>(&nn_s[grp][buf][0][nro]));
            const float vn = h2f_bits(*reinterpret_cast<const uint16_t*>(&nn_s[grp][buf][1][nro]));
            const bool valid = useful && (tile + 16 * my_sub + ln < t1);
            float raw[R], x[R];
            bool raise = false;
#pragma unroll
            for (int r = 0; r < R; r++) {
                // rows r (value of q_rot) and r + 8 (remainder) sit 32 lanes apart; the swap also moves
                // the second sub-tile into the upper half of the wave
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

            __builtin_amdgcn_s_setprio(2);
            // ---- O[head][dim 8ln + j] += P[head][token] V[token][dim]
            // Per sub-tile: wa = 16-bit codes of tokens (4kg, 4kg+2), wb = of (4kg+1, 4kg+3) for
            // this lane's 8 dims.  xe/xo: per byte, low nibble = token a dims (d, d+1), high
            // nibble = token b dims (d, d+1); bytes = (tokens 0,1 | d=0), (0,1 | d=4),
            // (2,3 | d=0), (2,3 | d=4) for xe and d = 2, 6 for xo.
            uint32_t xe[2], xo[2];
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                const uint32_t d0 = *reinterpret_cast<const uint32_t*>(vtb + vro[sub][0]);
                const uint32_t d1 = *reinterpret_cast<const uint32_t*>(vtb + vro[sub][1]);
                const uint32_t keep = __builtin_amdgcn_perm(d1, d0, sel_keep);
                const uint32_t send = __builtin_amdgcn_perm(d1, d0, sel_send);
                const uint32_t recv = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0xB1, 0xf, 0xf, false);  // lane ^ 1
                const uint32_t wa = odd ? recv : keep, wb = odd ? keep : recv;
                xe[sub] = (wa & 0x0f0f0f0fu) | ((wb << 4) & 0xf0f0f0f0u);
                xo[sub] = ((wa >> 4) & 0x0f0f0f0fu) | (wb & 0xf0f0f0f0u);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {            // dims (2q, 2q+1): 4 look-ups, 2 MFMAs
                const uint32_t x0 = (q & 1) ? xo[0] : xe[0], x1 = (q & 1) ? xo[1] : xe[1];
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
            __builtin_amdgcn_s_setprio(0);
        };
        // One tile: start the loads of the next tile, do the arithmetic of tile `it` from LDS, put the
        // tile that arrived into the other buffer, and meet the other waves.  (Two tiles of loads in
        // flight were measured: no faster.)
        for (int it = 0; it < round_tiles; it++) {
            if (it + 1 < ntiles) {
                const int pages = pages_next;
                if (PAGED && it + 2 < ntiles) pages_next = fetch_pages(t0 + 32 * (it + 2));
                load_tile(t0 + 32 * (it + 1), pages, ra[0], ra[1], ra[2]);
            }
            if (it < ntiles) compute(it & 1, t0 + 32 * it);
            if (it + 1 < ntiles) stash((it & 1) ^ 1, ra[0], ra[1], ra[2]);
            __syncthreads();
        }

        // ---- partial result of this (sequence, KV head, chunk or piece)
        if (have) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                l_run[r] = wave_sum(l_run[r]);                                        // idle and masked lanes hold 0
#pragma unroll
                for (int j = 0; j < 8; j++) o[j][r] += __shfl_xor(o[j][r], 32, 64);   // row r + row r+8 (remainder of P)
            }
            if (kg == 0) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    float* part = a.ws + ((long long)g * a.num_heads + (long long)h * R + r) * a.ws_stride +
                                  (long long)chunk * kPartialFloats;
#pragma unroll
                    for (int j = 0; j < 8; j++) part[8 * ln + j] = o[j][r] * (1.0f / kAlpha);
                    if (ln == 0) {
                        part[kHeadDim] = m_run[r];
                        part[kHeadDim + 1] = l_run[r];
                        // whoever holds the sequence's first token tells the merge, in the spare word of
                        // partial 0, how many partials there are
                        if (t0 == 0) reinterpret_cast<int*>(part - (long long)chunk * kPartialFloats)[kHeadDim + 2] = nseg;
                    }
                }
            }
        }
    }
}

// 2-bit codes, exactly 8 KV heads (a 256-byte row), GQA groups of 1, 2 or 4
bool attention_mfma2c_usable(const AttnArgs& a) {
    const int R = a.num_heads / a.num_kv_heads;
    return a.bits == 2 && a.num_kv_heads == kCoopHeads && (R == 1 || R == 2 || R == 4) &&
           !(a.balance && a.G > kCoopSeqs);
}

void launch_attention_mfma2c_scan(const AttnArgs& a, hipStream_t s) {
    const int items = a.G * a.nsplit;
    int ngroups = kMaxWaves / kCoopHeads;
    int grid = compute_units();
    if (items < grid * ngroups) {
        ngroups = (items + grid - 1) / grid;
        if (ngroups < 1) ngroups = 1;
        grid = (items + ngroups - 1) / ngroups;
    }
    const int R = a.num_heads / a.num_kv_heads;
    const dim3 g3(grid), b3(ngroups * kCoopHeads * kWave);
    note_scan_kernel("attention_mfma2c_kernel");
#define TW_LAUNCH_C(P, RR) launch_scan_kernel(attention_mfma2c_kernel<P, RR>, g3, b3, s, a, items)
    if (a.block_table) {
        if (R == 1) TW_LAUNCH_C(true, 1); else if (R == 2) TW_LAUNCH_C(true, 2); else TW_LAUNCH_C(true, 4);
    } else {
        if (R == 1) TW_LAUNCH_C(false, 1); else if (R == 2) TW_LAUNCH_C(false, 2); else TW_LAUNCH_C(false, 4);
    }
#undef TW_LAUNCH_C
}

}  // namespace twkv
