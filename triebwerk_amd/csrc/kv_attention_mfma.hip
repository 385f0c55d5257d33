// kv_attention_mfma.hip -- GQA decode attention over the 4-bit and 2-bit compressed
// caches for gfx950: codes are expanded to fp16 centroids in registers and the two
// contractions (q.K^T and P.V) run on the matrix cores.
//
// Same mathematics as turbo_gqa_attention_batch_kernel of the reference
// (kernels.cu:1641-1776): q_rot = R q; s_p = (q_rot . c(K codes_p)) * kn_p / sqrt(D);
// softmax over p <= pos with "+1e-8" in the denominator; acc = sum_p w_p vn_p c(V codes_p);
// out = R^T acc.  Three launches: rotate_kernel in kv_rotate.hip (q_rot, once per sequence and
// head), attention_mfma_kernel (the context scan, below), merge_rotate_kernel
// (split merge, normalisation, rotate-back).  The mapping is described for 4-bit codes;
// the 2-bit differences follow it.
//
// Why MFMA for a bandwidth-bound scan: at 5.6 TB/s of 4-bit codes one CU must
// consume ~18 codes per clock for K and V together, and with two query heads per
// KV head that is ~4 vector-ALU operations per code (extract, look up, two FMAs)
// against a budget of 64 lane-operations per clock per CU.  Moving the FMAs to
// MFMA leaves one v_perm_b32 (LDS address) and one ds_read_b32 per BYTE of codes.
//
// Mapping (one wave = one KV head of one sequence, 32 tokens per iteration):
//   K: lane (t = lane%16, kg = lane/16) holds 16 bytes = dims [32kg, 32kg+32) of
//      token t (loaded by lane 4t + kg, so that adjacent lanes read adjacent bytes, and
//      moved with ds_bpermute).  Dword j of it is the B operand of MFMA j (v_mfma_f32_16x16x32_f16),
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
//   scheduling: one persistent workgroup of 16 waves per CU.  Its waves form two groups of
//      8 (one KV head per wave); each group walks its own list of items, so the 64 KB table
//      is built once per CU and waves never synchronise after that.  Items are cut one of
//      two ways, chosen on the device from the positions: even chunks (every sequence into
//      nsplit chunks of 32-token tiles; item = sequence, chunk, head group) when the lengths
//      are within 1/8 of each other, else the balanced walk (all tiles of all sequences in
//      one list, an equal run per group, cut where a sequence ends), whose pieces number
//      the partials of a sequence 0, 1, 2, ...  Measured: the waves in the upper wave slots
//      of a CU (the second group, or a second workgroup) run ~5 % slower than the lower ones
//      whatever their s_setprio; chunk_range therefore gives even chunks 33/64 and odd
//      chunks 31/64 of a pair's tiles.
//   precision: fp16 operands would cost ~5e-4 relative error each for q_rot and for
//      the probabilities.  Both are split into hi + lo fp16 parts that ride in MFMA
//      rows the GQA group leaves empty (head n -> row n and n+8), so the split costs
//      no extra MFMA; the two halves are added after the contraction.
//      The centroid table is stored as fp16(alpha * c) with alpha chosen so that all
//      eight magnitudes round with <= 1.1e-4 relative error (3.6e-4 without it);
//      1/alpha is folded into q_rot and into the final accumulator.
//   2-bit codes: a cache row of one head is 32 bytes.  K: a lane loads 8 bytes (the same 32
//      dims).  The table maps a byte (4 codes) to 4 fp16 centroids, 8 bytes per entry and 32
//      replicas, read with ds_read_b64 (conflict free per half wave); entry order is
//      (code0, code2, code1, code3), matched by the order of q_rot in the A operand, because
//      that order is what V needs.  V: the 8 dims of a lane are 2 bytes per token; lanes n and
//      n^1 share dwords, so each loads the dword of two of the four tokens and they trade
//      halves with one DPP move.  Index bytes hold (token a dims d,d+1 | token b dims d,d+1),
//      so one look-up returns the B-operand dwords (a,b) of dim d and of dim d+1.
// The partial (acc[128], max, sum) per (sequence, head, chunk or piece) goes to the split
// workspace; merge_rotate_kernel combines, normalises and rotates back.  The wave that holds
// a sequence's first token also leaves, in a spare word of partial 0, how many partials the
// sequence has (0 = even chunks, where chunk_nonempty tells).

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"

#include <cstring>

namespace twkv {

namespace {

constexpr int kMaxGroup = 4;          // query heads per KV head handled by this kernel
// Tiles of loads in flight per wave.  Deeper is only safe while nothing spills: a spilled
// register is reloaded through the same in-order memory counter as the prefetched tiles,
// so every reload waits for all of them.
constexpr int kDepth4 = 1, kDepth2 = 1;

}  // namespace

template <bool PAGED, int R, int BITS, int DEPTH>
__global__ void __launch_bounds__(kMaxWaves * kWave)
attention_mfma_kernel(AttnArgs a, int total_items, int hgroups, int group_waves) {
    constexpr int KW = BITS;        // dwords of K codes per lane and sub-tile (32 dims of one token)
    constexpr int VW = BITS;        // dwords of V codes per lane and sub-tile
    constexpr uint32_t kHeadBytes = BITS * 16;   // bytes of one head in a cache row
    constexpr float kAlpha = BITS == 4 ? kAlpha4 : kAlpha2;
    __shared__ __attribute__((aligned(16))) uint32_t tab_s[kTableWords];
    // per wave: P[row][k] as fp16, rows 0..R-1 = heads, rows 8..8+R-1 = rounding remainders
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
    // After the sub-tile swap a lane owns token ln of sub-tile (kg >> 1); lanes with odd kg idle.
    const int my_sub = kg >> 1;
    const bool useful = (kg & 1) == 0;
    const uint32_t noff = (uint32_t)ln * nrow + (PAGED ? 0u : (uint32_t)my_sub * 16u * nrow);
    // slot of that token in the k order of the P.V contraction: k = 8*(t/4) + 4*sub + t%4
    half_t* p_w = &p_s[wave][0][8 * (ln >> 2) + 4 * my_sub + (ln & 3)];
    const uint4* p_r = reinterpret_cast<const uint4*>(&p_s[wave][ln][8 * kg]);
    constexpr float kRaise = 5.0f;                     // raise the running max only past 2^5

    auto lut32 = [&](uint32_t addr) -> uint32_t { return *reinterpret_cast<const uint32_t*>(tab_lane + addr); };
    auto lut64 = [&](uint32_t addr) -> uint2 { return *reinterpret_cast<const uint2*>(tab_lane + addr); };

    // ---- state of the item in hand (wave-uniform)
    int chunk = 0, g = 0, h = 0, n = 0, t0 = 0, t1 = 0;
    const char *kseq = nullptr, *vseq = nullptr, *knseq = nullptr, *vnseq = nullptr;
    const int* bt = nullptr;
    long long seq_row0 = 0;
    int nseg = 0;                                             // balanced walk: partials sequence g gets; 0 = even chunks
    auto set_bases = [&]() {                                  // scalar bases of this wave's head
        kseq = reinterpret_cast<const char*>(a.k) + (long long)h * kHeadBytes;
        vseq = reinterpret_cast<const char*>(a.v) + (long long)h * kHeadBytes;
        knseq = reinterpret_cast<const char*>(a.k_norms) + (long long)h * 2;
        vnseq = reinterpret_cast<const char*>(a.v_norms) + (long long)h * 2;
        bt = PAGED ? a.block_table + (long long)g * a.bt_stride : nullptr;
        seq_row0 = (long long)g * a.seq_stride_rows;
    };
    auto decode = [&](int item) -> bool {                    // false: the chunk holds no token
        const int hg = item % hgroups;
        chunk = (item / hgroups) % a.nsplit;
        g = item / (hgroups * a.nsplit);
        h = hg * group_waves + wv;                            // KV head of this wave
        n = uniform(seq_pos(a, g)) + 1;
        chunk_range(n, chunk, a.nsplit, t0, t1);
        if (t0 >= t1) return false;
        set_bases();
        return true;
    };
    // Balanced walk (ragged batches).  All 32-token tiles of all sequences form one list; every
    // group of waves takes `quota` consecutive tiles of it, cut where a sequence ends.  The piece
    // of sequence g that group number gb takes is partial gb - (tiles before g) / quota of g.
    int bal_cur = 0, bal_end = 0, bal_g = 0, bal_quota = 1, bal_gb = 0;
    auto next_piece = [&]() -> bool {
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
        h = wv;
        set_bases();
        return true;
    };

    // Buffer descriptors: base = first cache row of the tile (contiguous cache) or of the
    // 16-token page (paged cache), extent = the rows that exist, so lanes past the end
    // of the sequence read zeros instead of foreign memory.  All scalar.
    // Paged: the two block-table entries of a tile are fetched one tile ahead by a vector load
    // (even lanes: first page, odd lanes: second) that is issued before the loads of the tile in
    // between, so it has returned, in order, by the time that tile's codes are waited for, and the
    // wait for it holds up no load in flight.  Past the end the last page is re-read (masked).
    auto fetch_pages = [&](int ts) -> int { return bt[min(ts + 16 * (lane & 1), t1 - 1) >> 4]; };
    auto page_row = [&](int pages, int sub) -> long long {
        return (long long)__builtin_amdgcn_readlane(pages, sub) * kPageTokens;
    };
    int pages_next = 0;                          // entries of the tile whose loads are issued next in the loop
    auto load_k = [&](__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t (&dst)[KW]) {
        if constexpr (BITS == 4) {
            uint32x4_t q = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
            dst[0] = q[0]; dst[1] = q[1]; dst[2] = q[2]; dst[3] = q[3];
        } else {
            uint32x2_t q = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
            dst[0] = q[0]; dst[1] = q[1];
        }
    };
    auto issue_k = [&](uint32_t (&kreg)[2][KW], int tile, int pages) {
        if (PAGED) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++)
                load_k(make_rsrc(kseq + page_row(pages, sub) * kvp, kPageTokens * (int)kvp), koff, kreg[sub]);
        } else {
            __amdgpu_buffer_rsrc_t r = make_rsrc(kseq + (seq_row0 + tile) * kvp, max(min(n - tile, 32), 0) * (int)kvp);
            load_k(r, koff, kreg[0]);
            load_k(r, koff + sub_bytes, kreg[1]);
        }
    };
    auto issue_v = [&](uint32_t (&vreg)[2][VW], int tile, int pages) {
        if (PAGED) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                __amdgpu_buffer_rsrc_t r = make_rsrc(vseq + page_row(pages, sub) * kvp, kPageTokens * (int)kvp);
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
    auto issue_n = [&](int tile, int pages) -> uint32_t {
        const bool wide = (nrow & 15u) == 0;
        const uint32_t hgrp = (uint32_t)(h >> 3) * 16u;          // 16-byte group of this head inside a row
        if (PAGED) {
            const long long rr = my_sub ? page_row(pages, 1) : page_row(pages, 0);
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
        int pg[DEPTH + 1];
        if (PAGED) {
#pragma unroll
            for (int d = 0; d <= DEPTH; d++) pg[d] = fetch_pages(t0 + 32 * d);
            pages_next = pg[DEPTH];
        }
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            if (d == 0 || t0 + 32 * d < t1) {
                issue_k(kring[d], t0 + 32 * d, PAGED ? pg[d] : 0);
                nring[d] = issue_n(t0 + 32 * d, PAGED ? pg[d] : 0);
                issue_v(vring[d], t0 + 32 * d, PAGED ? pg[d] : 0);
            }
        }
    };

    // Even chunks or balanced walk?  Every wave looks at the spread of the sequence lengths
    // itself (cheap), so that in the even case its first loads are in flight while the
    // workgroup builds its table; wave 0 also leaves the prefix of tiles in LDS.
    bool balanced = false;
    if (a.balance) {
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
        balanced = uniform((tmax - tmin) * 8 > tmax ? 1 : 0) != 0;   // even chunks serve (nearly) equal lengths better
        if (wave == 0 && lane == 0) {
            pre_s[0] = 0;
            const int groups = (int)gridDim.x * ngroups;
            const int quota = (carry + groups - 1) / groups;
            const int by_slots = (tmax + a.max_slots - 2) / (a.max_slots - 1);   // a sequence gets <= max_slots pieces
            bal_s[0] = max(max(quota, by_slots), 1);
            bal_s[1] = carry;
        }
    }
    // The first loads of the first item are in flight while the workgroup builds its table
    // (not in the balanced walk, whose first piece is only known after the barrier).
    const int item_step = (int)gridDim.x * ngroups;
    int item = (int)blockIdx.x * ngroups + grp;
    bool ready = false;          // the item is decoded, holds tokens, and its first loads are issued
    if (!balanced && item < total_items && decode(item)) {
        issue_first();
        ready = true;
    }
    // ---- dequantization table, once per workgroup
    build_centroid_table<BITS, false>(tab_s, kAlpha, tid, nthreads);
    for (int i = tid; i < kMaxWaves * 16 * 32 / 2; i += nthreads) reinterpret_cast<uint32_t*>(p_s)[i] = 0u;
    __syncthreads();             // the only workgroup-wide barrier; every wave reaches it

    if (balanced) {
        bal_quota = bal_s[0];
        bal_gb = (int)blockIdx.x * ngroups + grp;
        const long long start = (long long)bal_gb * bal_quota;
        bal_cur = (int)min(start, (long long)bal_s[1]);
        bal_end = (int)min(start + bal_quota, (long long)bal_s[1]);
        int lo = 0, hi = a.G;                                 // last sequence that starts at or before bal_cur
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (pre_s[mid] <= bal_cur) lo = mid; else hi = mid;
        }
        bal_g = lo;
    }

    for (;;) {
        if (balanced) {
            if (!next_piece()) break;
            issue_first();
        } else {
            if (item >= total_items) break;
            if (!ready) {
                if (!decode(item)) { item += item_step; continue; }   // uniform over the wave
                issue_first();
            }
            ready = false;
            item += item_step;
        }
        const int ntiles = (t1 - t0 + 31) >> 5;

        float4_t o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) o[j] = float4_t{0.f, 0.f, 0.f, 0.f};
        float m_run[R], l_run[R];
#pragma unroll
        for (int r = 0; r < R; r++) { m_run[r] = kNegBig; l_run[r] = 0.0f; }

        // A operand of the score MFMAs: q_rot[head][32kg + 8j + i]; row m carries the
        // fp16 value of head m, row m + 8 what the rounding left over.  The 2-bit table
        // returns the codes of a byte in the order 0,2,1,3.
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
                    const int src = BITS == 4 ? i : ((i & 4) | ((i & 1) << 1) | ((i & 2) >> 1));
                    float x = (hq < R) ? v[src] : 0.0f;
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
            const int pages = pages_next;
            if (PAGED && more) pages_next = fetch_pages(next_tile + 32);

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
            if (more) issue_k(kreg, next_tile, pages);

            // ---- online softmax (base 2): this lane owns token ln of sub-tile my_sub
            const float kn = h2f_bits(nreg & 0xffffu), vn = h2f_bits(nreg >> 16);
            if (more) nreg = issue_n(next_tile, pages);
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
                if (more) issue_v(vreg, next_tile, pages);
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
                if (more) issue_v(vreg, next_tile, pages);
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
                for (int j = 0; j < 8; j++) part[8 * ln + j] = o[j][r] * (1.0f / kAlpha);
                if (ln == 0) {
                    part[kHeadDim] = m_run[r];
                    part[kHeadDim + 1] = l_run[r];
                    // whoever holds the sequence's first token tells the merge, in the spare word of
                    // partial 0, how many partials there are (0: even chunks)
                    if (t0 == 0) reinterpret_cast<int*>(part - (long long)chunk * kPartialFloats)[kHeadDim + 2] = balanced ? nseg : 0;
                }
            }
        }
    }
}

int compute_units() {
    static int cached = 0;
    if (cached == 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached = cus;
    }
    return cached;
}

// waves that walk one item together: the KV heads, at most kGroupWaves at a time
static int scan_waves(const AttnArgs& a) {
    int waves = a.num_kv_heads < kGroupWaves ? a.num_kv_heads : kGroupWaves;
    while (a.num_kv_heads % waves != 0) waves--;
    return waves;
}

float attention_mfma_q_scale(int bits) {
    // score scale of kernels.cu:1707 in base 2, table scale undone
    return kLog2e * kInvSqrtD / (bits == 4 ? kAlpha4 : kAlpha2);
}

namespace {
// a prompt over the compressed cache goes to the kernel that expands a tile once per workgroup
bool takes_prefill_tq(const AttnArgs& a) {
    return prefill_tq_mfma_usable(a) && !(prefill_form() == 4 && prefill_mfma_usable(a));
}
}  // namespace

// Shape check; with rotate_query also q_rot = R q (kernels.cu:1671-1681) into the workspace.
bool prepare_attention_mfma(AttnArgs& a, hipStream_t s, bool rotate_query) {
    const int R = a.num_heads / a.num_kv_heads;
    if (a.bits != 4 && a.bits != 2) return false;
    if (R != 1 && R != 2 && R != 4) return false;
    if (takes_prefill_tq(a)) return true;                  // that kernel needs no workspace and rotates its queries itself
    // needs the split workspace with room for q_rot behind each block's partials
    if (!a.ws || !a.qrot) return false;
    if ((reinterpret_cast<uintptr_t>(a.qrot) & 15u) != 0 || (a.ws_stride & 3) != 0) return false;
    const long long items = (long long)a.G * a.nsplit * (a.num_kv_heads / scan_waves(a));
    if (items <= 0 || items > 0x7fffffff) return false;
    a.force_merge = 1;
    a.m_log2 = 1;
    a.slots_from_ws = 1;
    // ragged batches: cut the work by tiles, not by sequence (decided on the device from the positions)
    a.balance = (a.num_kv_heads == scan_waves(a) && a.G <= kMaxBalanceSeqs && a.max_slots >= 3 && a.G > 1) ? 1 : 0;
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

// Returns whether the output is finished (the prompt kernel normalises and rotates back itself); otherwise the
// partials wait in the workspace for the merge.
bool launch_attention_mfma_scan(const AttnArgs& a, hipStream_t s) {
    if (takes_prefill_tq(a)) {
        launch_prefill_tq_mfma(a, s, prefill_form());
        return true;
    }
    if (prefill_mfma_usable(a)) {
        launch_prefill_mfma_scan(a, s);
        return false;
    }
    if (attention_variant() != 3 && attention_pair_usable(a)) {      // KV heads in pairs: two heads per wave
        launch_attention_pair_scan(a, s);
        return false;
    }
    const int waves = scan_waves(a);
    const int hgroups = a.num_kv_heads / waves;
    const int items = a.G * a.nsplit * hgroups;
    // One workgroup per CU (80 KB of LDS, <= 128 VGPRs), made of as many groups as fit in
    // kMaxWaves waves; fewer groups or workgroups when there are not that many items.
    int ngroups = kMaxWaves / waves;
    int grid = compute_units();
    if (items < grid * ngroups) {
        ngroups = (items + grid - 1) / grid;
        if (ngroups < 1) ngroups = 1;
        grid = (items + ngroups - 1) / ngroups;
    }
    const int R = a.num_heads / a.num_kv_heads;
    const dim3 g3(grid), b3(ngroups * waves * kWave);
    note_scan_kernel("attention_mfma_kernel");
#define TW_LAUNCH(P, RR, BB) launch_scan_kernel(attention_mfma_kernel<P, RR, BB, (BB == 4 ? kDepth4 : kDepth2)>, g3, b3, s, a, items, hgroups, waves)
#define TW_LAUNCH_R(P, BB) \
    do { if (R == 1) TW_LAUNCH(P, 1, BB); else if (R == 2) TW_LAUNCH(P, 2, BB); else TW_LAUNCH(P, 4, BB); } while (0)
    if (a.block_table) {
        if (a.bits == 4) TW_LAUNCH_R(true, 4); else TW_LAUNCH_R(true, 2);
    } else {
        if (a.bits == 4) TW_LAUNCH_R(false, 4); else TW_LAUNCH_R(false, 2);
    }
#undef TW_LAUNCH_R
#undef TW_LAUNCH
    return false;
}

}  // namespace twkv
