// kv_attention_pair.hip -- the stand-alone context scan of GQA decode attention over the compressed cache (4 and 2 bit)
// with two KV heads per wave (gfx950).  Same mathematics, workspace and partials as attention_mfma_kernel
// (kv_attention_mfma.hip; kernels.cu:1641-1776 of the reference) and the same two ways of cutting the work -- even
// chunks of every sequence, or the balanced walk over all tiles of a ragged batch -- but the tile is
// kv_pair_scan.hpp's: at 4 bit a wave reads whole 128-byte lines (two heads) with non-temporal loads, so the waves of a
// group (four pairs = 8 KV heads) read whole 512-byte cache rows between them and every byte is fetched once; at 2 bit
// a pair is half a line and the loads keep the ordinary policy.
// Contiguous and paged layout; launched between rotate_kernel (q_rot into the workspace) and merge_rotate_kernel.

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"
#include "kv_pair_scan.hpp"

namespace twkv {

namespace {
constexpr int kPairScanWaves = 8;      // waves per workgroup: 256 registers each, one workgroup per CU (64 KB table)
}  // namespace

template <bool PAGED, int R, int BITS>
__global__ void __launch_bounds__(kPairScanWaves * kWave)
attention_pair_kernel(AttnArgs a, int total_items, int hgroups, int group_waves) {
    constexpr float kAlpha = BITS == 4 ? kAlpha4 : kAlpha2;
    constexpr uint32_t kHeadBytes4 = BITS * 16;                      // bytes of one head in a cache row
    constexpr int kCodesAux = BITS == 4 ? kStreamCodes : 0;          // whole lines per instruction only at 4 bit
    __shared__ __attribute__((aligned(16))) uint32_t tab_s[kTableWords];
    __shared__ __attribute__((aligned(16))) half_t p_s[kPairScanWaves][16][32];
    // balanced walk: tiles of the sequences before g, and {tiles per group, total tiles}
    __shared__ int pre_s[kMaxBalanceSeqs + 1];
    __shared__ int bal_s[2];

    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;
    // The workgroup's waves form groups of group_waves (one pair of KV heads each); a group walks its own list of
    // items and never synchronises with the others once the table is built.
    const int grp = wave / group_waves, wv = wave % group_waves;
    const int ngroups = (nthreads / kWave) / group_waves;
    const int Hk = a.num_kv_heads;
    const uint32_t kvp = (uint32_t)Hk * kHeadBytes4;   // bytes per cache row (all heads)
    const uint32_t nrow = (uint32_t)Hk * 2u;           // bytes per norm row

    PairLane<R, BITS> L;
    L.init(lane, p_s[wave], tab_s);
    const uint32_t koff = L.koff_rows * kvp + L.koff_bytes;
    const uint32_t voff = L.voff_rows * kvp + L.voff_bytes;
    const uint32_t noff = (uint32_t)L.tok0 * nrow;

    // ---- state of the item in hand (wave-uniform)
    int chunk = 0, g = 0, h = 0, n = 0, t0 = 0, t1 = 0;
    const char *kpair = nullptr, *vpair = nullptr, *knpair = nullptr, *vnpair = nullptr;
    const int* bt = nullptr;
    int nseg = 0;                                             // balanced walk: partials sequence g gets; 0 = even chunks
    auto set_bases = [&]() {                                  // scalar bases of this wave's pair of heads
        // (contiguous cache: from the sequence's first row, which leaves one multiplication per tile and array)
        const long long row0 = PAGED ? 0 : (long long)g * a.seq_stride_rows;
        kpair = reinterpret_cast<const char*>(a.k) + row0 * kvp + (long long)h * kHeadBytes4;
        vpair = reinterpret_cast<const char*>(a.v) + row0 * kvp + (long long)h * kHeadBytes4;
        knpair = reinterpret_cast<const char*>(a.k_norms) + row0 * nrow + (long long)h * 2;
        vnpair = reinterpret_cast<const char*>(a.v_norms) + row0 * nrow + (long long)h * 2;
        bt = PAGED ? a.block_table + (long long)g * a.bt_stride : nullptr;
    };
    auto decode = [&](int item) -> bool {                    // false: the chunk holds no token
        const int hg = item % hgroups;
        chunk = (item / hgroups) % a.nsplit;
        g = item / (hgroups * a.nsplit);
        h = 2 * (hg * group_waves + wv);                      // first KV head of this wave's pair
        n = uniform(seq_pos(a, g)) + 1;
        chunk_range(n, chunk, a.nsplit, t0, t1);
        if (t0 >= t1) return false;
        set_bases();
        return true;
    };
    // Balanced walk (ragged batches), as in attention_mfma_kernel: all 32-token tiles of all sequences form one
    // list; every group takes `quota` consecutive tiles of it, cut where a sequence ends.
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
        h = 2 * wv;
        set_bases();
        return true;
    };

    // Loads of a tile.  Contiguous cache: one descriptor over the rows of the tile that exist (rows past the
    // sequence's end read as zeros, and so does a tile past the chunk's last one, which is asked for with no rows
    // rather than skipped by a branch).  Paged cache: a tile is two 16-token pages, each with its own descriptor; the
    // two block-table entries of a tile are fetched one tile ahead (even lanes the first page, odd lanes the second),
    // before the loads of the tile in between, so they have returned, in order, by the time they are needed.  Past
    // the end the last page is re-read (its tokens are masked).  After a chunk's last tile the loads are still issued,
    // through descriptors of no bytes (`live` false: zeros, no traffic), and the block table is read again at the
    // chunk's last entry: with every load of the loop unconditional the compiler knows how many are in flight when
    // the entries are needed and waits for exactly those before them -- with the loads under `if (more)` it waited
    // for all of them, the next tile's included, at the end of every tile (9 % of the 2-bit paged scan, 2 % at 4 bit).
    auto fetch_pages = [&](int ts) -> int { return bt[min(ts + 16 * (lane & 1), t1 - 1) >> 4]; };
    auto page_row = [&](int pages, int sub) -> long long {
        return (long long)__builtin_amdgcn_readlane(pages, sub) * kPageTokens;
    };
    int pages_next = 0;                          // entries of the tile whose loads are issued next in the loop
    // `pages`: paged cache, the tile's two block-table entries; contiguous cache, the rows of the tile that exist
    auto tile_rows = [&](int tile) -> int { return max(min(n - tile, 32), 0); };
    auto load_k = [&](__amdgpu_buffer_rsrc_t r, uint32_t off) {
        if constexpr (BITS == 4) return __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, kCodesAux);
        else return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, kCodesAux);
    };
    auto load_v = [&](__amdgpu_buffer_rsrc_t r, uint32_t off) {
        if constexpr (BITS == 4) return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, kCodesAux);
        else return __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, kCodesAux);
    };
    auto issue_k = [&](PairTileRegs<BITS>& t, int tile, int pages, bool live = true) {
        if (PAGED) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                __amdgpu_buffer_rsrc_t r = make_rsrc(kpair + page_row(pages, sub) * kvp, live ? kPageTokens * (int)kvp : 0);
                t.k[2 * sub] = load_k(r, koff);
                t.k[2 * sub + 1] = load_k(r, koff + 8u * kvp);
            }
        } else {
            __amdgpu_buffer_rsrc_t r = make_rsrc(kpair + (long long)tile * kvp, pages * (int)kvp);
#pragma unroll
            for (int c = 0; c < 4; c++) t.k[c] = load_k(r, koff + (uint32_t)(8 * c) * kvp);
        }
    };
    auto issue_v = [&](PairTileRegs<BITS>& t, int tile, int pages, bool live = true) {
        if (PAGED) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                __amdgpu_buffer_rsrc_t r = make_rsrc(vpair + page_row(pages, sub) * kvp, live ? kPageTokens * (int)kvp : 0);
#pragma unroll
                for (int j = 0; j < 4; j++) t.v[sub][j] = load_v(r, voff + (uint32_t)j * kvp);
            }
        } else {
            __amdgpu_buffer_rsrc_t r = make_rsrc(vpair + (long long)tile * kvp, pages * (int)kvp);
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    t.v[sub][j] = load_v(r, voff + (uint32_t)(16 * sub + j) * kvp);
            }
        }
    };
    // the pair's two fp16 norms of tokens tok0 and tok0 + 16, K and V
    auto issue_n = [&](PairTileRegs<BITS>& t, int tile, int pages, bool live = true) {
        if (PAGED) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                __amdgpu_buffer_rsrc_t rk = make_rsrc(knpair + page_row(pages, i) * nrow, live ? kPageTokens * (int)nrow : 0);
                __amdgpu_buffer_rsrc_t rv = make_rsrc(vnpair + page_row(pages, i) * nrow, live ? kPageTokens * (int)nrow : 0);
                t.n[i][0] = __builtin_amdgcn_raw_buffer_load_b32(rk, (int)noff, 0, kStreamNorms);
                t.n[i][1] = __builtin_amdgcn_raw_buffer_load_b32(rv, (int)noff, 0, kStreamNorms);
            }
        } else {
            // (every lane asks, also those that own no token: they repeat a neighbour's address)
            __amdgpu_buffer_rsrc_t rk = make_rsrc(knpair + (long long)tile * nrow, pages * (int)nrow);
            __amdgpu_buffer_rsrc_t rv = make_rsrc(vnpair + (long long)tile * nrow, pages * (int)nrow);
            t.n[0][0] = __builtin_amdgcn_raw_buffer_load_b32(rk, (int)noff, 0, kStreamNorms);
            t.n[1][0] = __builtin_amdgcn_raw_buffer_load_b32(rk, (int)(noff + 16u * nrow), 0, kStreamNorms);
            t.n[0][1] = __builtin_amdgcn_raw_buffer_load_b32(rv, (int)noff, 0, kStreamNorms);
            t.n[1][1] = __builtin_amdgcn_raw_buffer_load_b32(rv, (int)(noff + 16u * nrow), 0, kStreamNorms);
        }
    };

    // One tile of loads is in flight per wave; each register set is re-issued for the next tile as soon as its
    // contents have been expanded.  (A second set of registers with the tile after next in flight, the loop unrolled
    // over the two sets: 3 % slower at 2 bit, where the waves spend 45 % of their time waiting for loads and the set
    // costs 20 registers, on even and on ragged batches -- as at 4 bit, more requests in flight do not arrive sooner.
    // Two 2-bit tiles as ONE step of the loop -- both tiles' loads in flight, one pass of the online softmax over the
    // lane's four tokens, one decision about the maximum and one hand-over of the probabilities per 64 tokens, 203-237
    // registers: 71.6-72.1 against 67.3-67.8 us at 64 x 8192 tokens, 51.3 against 47.3 us on the ragged batch.)
    PairTileRegs<BITS> t;
    auto issue_first = [&]() {
        int pg0 = PAGED ? 0 : tile_rows(t0);
        if (PAGED) {
            pg0 = fetch_pages(t0);
            pages_next = fetch_pages(t0 + 32);
        }
        issue_k(t, t0, pg0);
        issue_n(t, t0, pg0);
        issue_v(t, t0, pg0);
    };

    // Even chunks or balanced walk?  Every wave looks at the spread of the sequence lengths itself (cheap), so that
    // in the even case its first loads are in flight while the workgroup builds its table; wave 0 also leaves the
    // prefix of tiles in LDS.
    bool balanced = false;
    if (a.balance) {
        int carry = 0, tmin = 0x7fffffff, tmax = 0;
        for (int base = 0; base < a.G; base += kWave) {
            const int gg = base + lane;
            const int tl = gg < a.G ? (seq_pos(a, gg) + 1 + 31) >> 5 : 0;
            if (gg < a.G) { tmin = min(tmin, tl); tmax = max(tmax, tl); }
            if (wave == 0) {
                int inc = tl;
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
    const int item_step = (int)gridDim.x * ngroups;
    int item = (int)blockIdx.x * ngroups + grp;
    bool ready = false;          // the item is decoded, holds tokens, and its first loads are issued
    if (!balanced && item < total_items && decode(item)) {
        issue_first();
        ready = true;
    }
    // ---- dequantization table, once per workgroup
    build_centroid_table<BITS, true>(tab_s, kAlpha, tid, nthreads);
    for (int i = tid; i < kPairScanWaves * 16 * 32 / 2; i += nthreads) reinterpret_cast<uint32_t*>(p_s)[i] = 0u;
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

    PairState<R> S;
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
        S.reset();
        S.load_query(L, [&](int i) -> const float* {
            return a.qrot + ((long long)g * a.num_heads + (long long)h * R + i) * a.ws_stride;
        });

        for (int tile = t0; tile < t1; tile += 32) {
            const bool more = tile + 32 < t1;
            int pages = 0;
            if (PAGED) {
                pages = pages_next;                                  // the next tile's pages, already here
                pages_next = fetch_pages(tile + 64);                 // and the one after: before the next tile's loads
            }
            if (PAGED) {
                pair_scan_tile<R>(L, S, t, tile, n, [&]() { issue_k(t, tile + 32, pages, more); },
                                  [&]() { issue_n(t, tile + 32, pages, more); }, [&]() { issue_v(t, tile + 32, pages, more); });
            } else {
                const int rows = more ? tile_rows(tile + 32) : 0;
                pair_scan_tile<R>(L, S, t, tile, n, [&]() { issue_k(t, tile + 32, rows); }, [&]() { issue_n(t, tile + 32, rows); },
                                  [&]() { issue_v(t, tile + 32, rows); });
            }
        }

        // ---- partial results of this (sequence, pair of KV heads, chunk)
        pair_scan_finish<R>(L, S, 1.0f / kAlpha, [&](int hd, int r, const float (&ov)[16]) {
            float* base = a.ws + ((long long)g * a.num_heads + (long long)(h + hd) * R + r) * a.ws_stride;
            float* part = base + (long long)chunk * kPartialFloats;
#pragma unroll
            for (int j4 = 0; j4 < 4; j4++)
                *reinterpret_cast<float4*>(part + 16 * (L.pn & 7) + 4 * j4) = float4{ov[4 * j4], ov[4 * j4 + 1], ov[4 * j4 + 2], ov[4 * j4 + 3]};
            if ((L.pn & 7) == 0) {
                part[kHeadDim] = S.m_run[r];
                part[kHeadDim + 1] = S.l_run[r];
                // whoever holds the sequence's first token tells the merge, in the spare word of partial 0, how many
                // partials there are (0: even chunks)
                if (t0 == 0) reinterpret_cast<int*>(base)[kHeadDim + 2] = balanced ? nseg : 0;
            }
        });
    }
}

// pairs that walk one item together: half the KV heads, at most four at a time
static int pair_scan_waves(const AttnArgs& a) {
    int waves = a.num_kv_heads / 2 < 4 ? a.num_kv_heads / 2 : 4;
    while (waves > 1 && (a.num_kv_heads / 2) % waves != 0) waves--;
    return waves;
}

bool attention_pair_usable(const AttnArgs& a) {
    const int R = a.num_kv_heads > 0 ? a.num_heads / a.num_kv_heads : 0;
    if ((a.bits != 4 && a.bits != 2) || (a.num_kv_heads & 1) != 0 || (R != 1 && R != 2 && R != 4)) return false;
    if (a.pos_mode == kPosIota || !a.ws || !a.qrot) return false;
    auto al = [](const void* p, unsigned m) { return (reinterpret_cast<uintptr_t>(p) & m) == 0; };
    if (!al(a.k, a.bits == 4 ? 15 : 7) || !al(a.v, a.bits == 4 ? 15 : 7) || !al(a.k_norms, 3) || !al(a.v_norms, 3)) return false;
    if (!al(a.ws, 15) || (a.ws_stride & 3) != 0) return false;       // 16-byte stores of the partials
    const long long items = (long long)a.G * a.nsplit * (a.num_kv_heads / (2 * pair_scan_waves(a)));
    return items > 0 && items <= 0x7fffffff;
}

// the balanced walk is for batches whose 8 (or fewer) KV heads one group of waves covers
bool attention_pair_balances(const AttnArgs& a) { return a.num_kv_heads == 2 * pair_scan_waves(a); }

void launch_attention_pair_scan(const AttnArgs& a, hipStream_t s) {
    const int waves = pair_scan_waves(a);
    const int hgroups = a.num_kv_heads / (2 * waves);
    const int items = a.G * a.nsplit * hgroups;
    int ngroups = kPairScanWaves / waves;
    int grid = compute_units();
    if (items < grid * ngroups) {
        ngroups = (items + grid - 1) / grid;
        if (ngroups < 1) ngroups = 1;
        grid = (items + ngroups - 1) / ngroups;
    }
    const int R = a.num_heads / a.num_kv_heads;
    const dim3 g3(grid), b3(ngroups * waves * kWave);
    note_scan_kernel("attention_pair_kernel");
#define TW_LAUNCH(P, RR, BB) launch_scan_kernel(attention_pair_kernel<P, RR, BB>, g3, b3, s, a, items, hgroups, waves)
#define TW_LAUNCH_R(P, BB) do { if (R == 1) TW_LAUNCH(P, 1, BB); else if (R == 2) TW_LAUNCH(P, 2, BB); else TW_LAUNCH(P, 4, BB); } while (0)
    if (a.bits == 4) { if (a.block_table) TW_LAUNCH_R(true, 4); else TW_LAUNCH_R(false, 4); }
    else { if (a.block_table) TW_LAUNCH_R(true, 2); else TW_LAUNCH_R(false, 2); }
#undef TW_LAUNCH_R
#undef TW_LAUNCH
}

}  // namespace twkv
