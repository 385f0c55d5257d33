// kv_decode_fused.hip -- one decode step of one layer over the compressed cache in ONE launch (gfx950):
// append K and V of the new token (turbo_kv_quantize_batch_kernel, kernels.cu:1563-1636), rotate the query
// (1671-1681), scan the context (1688-1766), merge the parts of the context, normalise and rotate back
// (1746, 1769-1775).  forward_layer_batch does this with three launches (engine.cpp:1985-2006) and the
// three-kernel path of this library (rotate_kernel, attention_pair_kernel or attention_mfma_kernel,
// merge_rotate_kernel) does too;
// each of those small launches costs ~4.5 us before it does anything and the scan another ~6 us to start
// and drain, which is a third of a layer at contexts of a few hundred tokens.
//
// A workgroup owns one sequence and HKW of its KV heads (HKW = 1, 2, 4 or 8) together with their query heads, so
// nothing is handed from one workgroup to another.  Two forms: PAIR (HKW even) -- 8 waves, each scanning two KV heads
// with the tile of kv_pair_scan.hpp (256 registers per wave, two waves per SIMD either way); otherwise 16 waves with
// one KV head each, described here:
//   1. all threads stage the unit's vectors (K heads, V heads, query heads of the new token) in LDS and fill
//      the centroid table; with producers one wave per K or query vector applies RMSNorm and rotary embedding
//      there (kernels.cu:880-961).  Waves 0-7 (all 16 when the unit has more than 16 vectors) then rotate the
//      vectors exactly as rotate_kernel does -- lane i16 = vector, wave = block of 16 output coordinates, the
//      same v_mfma_f32_16x16x4_f32 chain, so the codes have the same bits -- and store codes and norms in the
//      cache, the scaled q_rot in LDS;
//   2. after the barrier wave w scans every SPLIT-th tile of the context (SPLIT = 16 / HKW, starting at tile
//      w / HKW) for head w % HKW with the loop of attention_mfma_kernel (the table look-ups, MFMA tiling,
//      online softmax are described there).  All its loads are issued after the barrier: the new token's row
//      was stored by this workgroup (same CU, same L1), which a workgroup-scope barrier makes visible;
//   3. the partial results meet in LDS: merge (log-sum-exp), "+1e-8" normalisation, and R^T on fp16 MFMAs (value +
//      remainder of the normalised output; the output tolerates a different order of additions, the codes did
//      not); output gate as in merge_rotate_kernel.
// The waves in the upper wave slots of a CU run ~5 % slower (see kv_common.hpp: kPairShare), so the parts
// of the upper eight waves get 31/64 of the tiles.
//
// One sequence is one workgroup's work whatever its length: right for batches of similar lengths (a
// rollout's decode steps) and for short contexts; the three-kernel path with its balanced walk stays the
// choice for ragged long contexts, and the only one for the paged layout.
// (Tried at batch 64: workgroups of all 8 KV heads, four per sequence with a quarter of the context each, so that a
// workgroup's waves read whole cache rows side by side -- a plain read of the cache in that pattern runs at 6.8
// instead of 6.4 TB/s -- and the quarters' sums meeting in a workspace, finished by whichever workgroup takes the
// last arrival ticket.  The agent-scope release and acquire fences around that hand-over, each a write-back or an
// invalidation of the XCD's L2, cost 34 us per launch; with no fence at all, which is not correct, the launch took
// 99 us against 97: the scan is not held up by the access pattern.)

#include <atomic>
#include <cmath>
#include <cstring>

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"
#include "kv_pair_scan.hpp"
#include "kv_producer_util.hpp"
#include "kv_rotate_util.hpp"

namespace twkv {

namespace {

constexpr int kFusedWaves = 16;
constexpr int kPairWaves = 8;                  // waves of a workgroup whose waves scan two KV heads each
constexpr unsigned kFusedShare = 33;           // 64ths of a sequence's tiles that go to the lower eight waves
constexpr unsigned kPairTileShare = 32;        // the same with eight waves in all: two per SIMD, no upper slots
constexpr int kFusedMaxQ = 32;                 // query heads of a unit: HKW * R <= 8 * 4
constexpr int kRowFloats = kHeadDim + 4;       // LDS row of a vector: conflict-free 16-byte accesses
constexpr int kStageStride = 2 * kHeadDim + 16;   // bytes per staged fp16 vector
constexpr int kMaxShares = 8;                  // workgroups that may share one sequence's context
static_assert(8 * (2 + 4) * kStageStride <= kFusedMaxQ * kRowFloats * 4, "staged vectors fit the output rows");

}  // namespace

// EARLY (PAIR only): waves ask for their first tile in the middle of the prologue; for launches whose waves have few
// tiles (the host decides from what it knows of the context lengths).  A template parameter because the mere presence
// of that path, never taken, made the long-context launch 2 us slower.
// SHARES: f.shares (2, 4 or 8) workgroups share the context of a unit -- for batches whose units alone leave compute units
// idle.  Share c scans the c-th of f.shares even runs of the sequence's tiles; the last share appends the new row.  Each
// leaves its unnormalised sums in memory, draws a ticket, and the workgroup with the last ticket merges all of them (in
// share order, all read back from memory: the result does not depend on who was last) and finishes the unit.  The
// hand-over uses device-scope accesses only where they are needed -- the partial sums and the ticket -- and no
// cache-wide fence: stores with device scope are written through to where every compute unit's device-scope loads look
// (a release / acquire pair at device scope writes back and invalidates a whole L2 and costs 20 us per launch where this
// costs 4-9 us with every workgroup of a full-size launch taking part, measured with a stand-alone probe).
template <int R, int BITS, bool PROD, bool PAIR, bool EARLY, bool SHARES = false>
__global__ void __launch_bounds__((PAIR ? kPairWaves : kFusedWaves) * kWave)
decode_fused_kernel(AttnArgs a, FusedArgs f) {
    constexpr int NW = PAIR ? kPairWaves : kFusedWaves;        // waves of the workgroup
    constexpr int KW = BITS, VW = BITS;
    constexpr uint32_t kHeadBytes = BITS * 16;
    constexpr float kAlpha = BITS == 4 ? kAlpha4 : kAlpha2;
    __shared__ __attribute__((aligned(16))) uint32_t tab_s[kTableWords];
    // the scan's probabilities and partials; before the scan the same space holds R as 8 operand tiles
    constexpr int kParts = PAIR ? 2 * NW : NW;                 // (part, head) partials: a wave leaves one per head it scans
    constexpr int kRotGroups = NW / 8;                         // groups of eight waves that rotate (a wave = 16 output coordinates)
    constexpr int kPBytes = NW * 16 * 32 * 2, kPartBytes = kParts * R * kRowFloats * 4;
    constexpr int kRotBytes = 8 * kOperandTileDwords * 4;
    __shared__ __attribute__((aligned(16))) char scan_s[kPBytes + kPartBytes > kRotBytes ? kPBytes + kPartBytes : kRotBytes];
    half_t (*p_s)[16][32] = reinterpret_cast<half_t (*)[16][32]>(scan_s);
    float (*part_s)[R][kRowFloats] = reinterpret_cast<float (*)[R][kRowFloats]>(scan_s + kPBytes);
    uint32_t* rot_s = reinterpret_cast<uint32_t*>(scan_s);
    __shared__ __attribute__((aligned(16))) float qrot_s[kFusedMaxQ][kHeadDim];
    __shared__ __attribute__((aligned(16))) float o_s[kFusedMaxQ][kRowFloats];
    __shared__ __attribute__((aligned(16))) half_t prod_s[4][kHeadDim];   // k_weight, q_weight, cos row, sin row

    const int tid = threadIdx.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;
    const int ln = lane & 15, kg = lane >> 4;          // names of the scan; the rotations call them i16, kk
    const int Hk = a.num_kv_heads;
    const int HKW = f.hkw;
    const int nhg = Hk / HKW;
    const int SPLIT = kParts / HKW;                    // parts of the context per head

    // ---- unit of this workgroup.  Workgroups are dealt to the 8 XCDs in turn; the units of one sequence
    // go to one XCD so that the norm rows they all read (16 bytes per token for 8 heads) come out of one L2.
    int g, hg, share = 0;
    const int nshares = SHARES ? f.shares : 1;
    {
        int b = (int)blockIdx.x;
        if ((a.G & 7) == 0) {
            const int xcd = b & 7;
            int j = b >> 3;
            if (SHARES) { share = j % nshares; j /= nshares; }      // the shares of a unit on one XCD as well
            g = (j / nhg) * 8 + xcd;
            hg = j % nhg;
        } else {
            if (SHARES) { share = b % nshares; b /= nshares; }
            g = b / nhg;
            hg = b % nhg;
        }
    }
    const bool appends = !SHARES || share == nshares - 1;          // the share that holds the sequence's last tile
    // ---- operands of the rotations first: nothing about them depends on the position.  The unit's vectors
    // (K heads, V heads, query heads) are fetched once by all threads, 16 bytes each, and staged in LDS;
    // the rotating waves fetch their 16 rows of R.
    const int nvec = HKW * (2 + R);
    const int rot_dblk = wave & 7;
    const bool rotating = wave < 8 * kRotGroups && (wave >> 3) * 16 < nvec;
    auto unit_vector = [&](int vc, int& kind, int& head) -> const half_t* {    // vc < nvec
        if (vc < HKW) {
            kind = 0; head = hg * HKW + vc;
            return f.k_src + (long long)g * f.kv_stride + (long long)head * kHeadDim;
        }
        if (vc < 2 * HKW) {
            kind = 1; head = hg * HKW + vc - HKW;
            return f.v_src + (long long)g * f.kv_stride + (long long)head * kHeadDim;
        }
        kind = 2; head = hg * HKW * R + (vc - 2 * HKW);
        return a.q + (long long)g * a.q_stride + (long long)head * kHeadDim;
    };
    uint4 stage = {0u, 0u, 0u, 0u};                    // piece tid % 16 of vector tid / 16
    if ((tid >> 4) < nvec) {
        int kind0, head0;
        stage = reinterpret_cast<const uint4*>(unit_vector(tid >> 4, kind0, head0))[tid & 15];
    }
    // R: wave w < 8 fetches rows 16w .. 16w + 15 (4 KB in a row, 4 fully used pieces per lane) and stages them
    // as an operand tile; the rotating waves read their operand from there
    uint4 rraw[4] = {};
    if (wave < 8) {
#pragma unroll
        for (int j = 0; j < 4; j++)
            rraw[j] = reinterpret_cast<const uint4*>(a.rotation + wave * 16 * kHeadDim)[j * kWave + lane];
    }

    // scaled centroid number lane % 16 (4 bit) or lane % 4 (2 bit), for the table build
    const float cent_lane = kAlpha * (BITS == 4 ? kCentroids4[lane & 15] : kCentroids2[lane & 3]);

    const int pos = uniform(a.positions[g]);
    const int n = pos + 1;
    // PAIR: wave = part * (HKW / 2) + pair; hk_local is the first head of the pair
    const int hk_local = PAIR ? 2 * (wave % (HKW >> 1)) : wave % HKW, part = PAIR ? wave / (HKW >> 1) : wave / HKW;
    const int h = hg * HKW + hk_local;                 // (first) KV head of this wave

    // producers' operands: the two weight vectors and the table rows of this sequence's position, 16 bytes per thread
    const bool normed = PROD && f.q_weight != nullptr, roped = PROD && f.cos_table != nullptr;
    uint4 prod = {0u, 0u, 0u, 0u};
    const int prod_row = tid >> 4, prod_piece = tid & 15;
    bool prod_live = false;
    if (PROD && tid < 64) {
        if (prod_row < 2 && normed) {
            prod = reinterpret_cast<const uint4*>(prod_row == 0 ? f.k_weight : f.q_weight)[prod_piece];
            prod_live = true;
        } else if (prod_row >= 2 && roped && prod_piece < (f.rope_dim >> 4)) {
            const half_t* tabrow = (prod_row == 2 ? f.cos_table : f.sin_table) + (long long)pos * (f.rope_dim >> 1);
            prod = reinterpret_cast<const uint4*>(tabrow)[prod_piece];
            prod_live = true;
        }
    }

    // ---- tiles of 32 tokens this wave scans.  They are dealt round by round: in round r part p takes tile
    // r * SPLIT + p, so that at any moment the workgroup -- and with it the other workgroups of the sequence,
    // which started together -- reads one window of consecutive rows (1.2 % faster at 8192 tokens than giving
    // every part one contiguous run).  The parts of the upper eight waves stop after `rounds` rounds (31/64 of
    // the tiles); what is left goes round the lower waves' parts.
    const int ntile_seq = (n + 31) >> 5;
    // SHARES: this workgroup's run of the sequence's tiles (even runs, the last one ends with the sequence)
    const int tile_lo = SHARES ? (int)((long long)share * ntile_seq / nshares) : 0;
    const int ntile = SHARES ? (int)((long long)(share + 1) * ntile_seq / nshares) - tile_lo : ntile_seq;
    const int halfparts = SPLIT >> 1;                      // SPLIT is 2, 4, 8 or 16
    const int lower = min(ntile, (int)((ntile * (PAIR ? kPairTileShare : kFusedShare) + 63u) / 64u));
    const int rounds = (ntile - lower) / halfparts;
    const int tail0 = rounds * SPLIT;                      // tail tiles tail0 + part + j * halfparts, lower parts only
    const int left = ntile - tail0 - part;
    const int ntiles = rounds + ((part < halfparts && left > 0) ? (left + halfparts - 1) / halfparts : 0);
    auto tile_at = [&](int i) -> int {                     // first token of this wave's i-th tile
        return 32 * (tile_lo + (i < rounds ? i * SPLIT + part : tail0 + part + (i - rounds) * halfparts));
    };
    const int first_tile = tile_at(0);

    // ---- scan set-up (as attention_mfma_kernel, contiguous layout)
    // Per-lane offsets and selectors.  They are derived after the rotations from a laundered copy of the lane
    // number: computed from the lane number itself they are hoisted to the top of the kernel, stay live across
    // the rotations, and the allocator spills some of them there and reloads them inside the scan loop, where a
    // reload waits for every load in flight.
    const char* tab_lane = reinterpret_cast<const char*>(tab_s);
    const uint32_t kvp = (uint32_t)Hk * kHeadBytes;
    const uint32_t nrow = (uint32_t)Hk * 2u;
    const uint32_t vstep = BITS == 4 ? kvp : 2u * kvp;  // V: dword i of a lane sits vstep bytes after dword 0 (one register for the four)
    const uint32_t sub_bytes = 16u * kvp;
    uint32_t lane_rep, koff, voff0, noff, sel_keep, sel_send;
    int ksrc, my_sub;
    bool odd, useful;
    half_t* p_w;
    const uint4* p_r;
    auto derive_lane = [&](int l) {
        const int ln_ = l & 15, kg_ = l >> 4;
        lane_rep = BITS == 4 ? (uint32_t)l * 4u : (uint32_t)(l & 31) * 8u;
        koff = (uint32_t)(l >> 2) * kvp + (kHeadBytes / 4) * (uint32_t)(l & 3);
        ksrc = 4 * (4 * ln_ + kg_);
        voff0 = BITS == 4 ? (uint32_t)(4 * kg_) * kvp + 4u * (uint32_t)ln_
                          : (uint32_t)(4 * kg_ + (ln_ & 1)) * kvp + 4u * (uint32_t)(ln_ >> 1);
        odd = (ln_ & 1) != 0;
        sel_keep = odd ? 0x07060302u : 0x05040100u;
        sel_send = odd ? 0x05040100u : 0x07060302u;
        my_sub = kg_ >> 1;
        useful = (kg_ & 1) == 0;
        noff = (uint32_t)ln_ * nrow + (uint32_t)my_sub * 16u * nrow;
        p_w = &p_s[wave][0][8 * (ln_ >> 2) + 4 * my_sub + (ln_ & 3)];
        p_r = reinterpret_cast<const uint4*>(&p_s[wave][ln_][8 * kg_]);
    };
    constexpr float kRaise = 5.0f;

    auto lut32 = [&](uint32_t addr) -> uint32_t { return *reinterpret_cast<const uint32_t*>(tab_lane + addr); };
    auto lut64 = [&](uint32_t addr) -> uint2 { return *reinterpret_cast<const uint2*>(tab_lane + addr); };

    const long long seq_row0 = (long long)g * a.seq_stride_rows;
    const char* kseq = reinterpret_cast<const char*>(a.k) + (long long)h * kHeadBytes;
    const char* vseq = reinterpret_cast<const char*>(a.v) + (long long)h * kHeadBytes;
    const char* knseq = reinterpret_cast<const char*>(a.k_norms) + (long long)h * 2;
    const char* vnseq = reinterpret_cast<const char*>(a.v_norms) + (long long)h * 2;

    auto load_k = [&](__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t (&dst)[KW]) {
        if constexpr (BITS == 4) {
            uint32x4_t q = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, 0);
            dst[0] = q[0]; dst[1] = q[1]; dst[2] = q[2]; dst[3] = q[3];
        } else {
            uint32x2_t q = __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0);
            dst[0] = q[0]; dst[1] = q[1];
        }
    };
    // Descriptors span the rows of the tile that exist (rows past the sequence's end read as zeros).
    auto issue_k = [&](uint32_t (&kreg)[2][KW], int tile) {
        __amdgpu_buffer_rsrc_t r = make_rsrc(kseq + (seq_row0 + tile) * kvp, max(min(n - tile, 32), 0) * (int)kvp);
        load_k(r, koff, kreg[0]);
        load_k(r, koff + sub_bytes, kreg[1]);
    };
    auto issue_v = [&](uint32_t (&vreg)[2][VW], int tile) {
        __amdgpu_buffer_rsrc_t r = make_rsrc(vseq + (seq_row0 + tile) * kvp, max(min(n - tile, 32), 0) * (int)kvp);
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
#pragma unroll
            for (int i = 0; i < VW; i++)
                vreg[sub][i] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)(voff0 + i * vstep + sub * sub_bytes), 0, 0);
        }
    };
    auto pick = [&](const uint32x4_t& q) -> uint32_t {
        const int dw = (h & 7) >> 1;
        uint32_t w = dw == 0 ? q[0] : dw == 1 ? q[1] : dw == 2 ? q[2] : q[3];
        return (h & 1) ? (w >> 16) : (w & 0xffffu);
    };
    auto issue_n = [&](int tile) -> uint32_t {        // fp16 bits of kn (low) and vn (high) of this lane's token
        const bool wide = (nrow & 15u) == 0;
        const uint32_t hgrp = (uint32_t)(h >> 3) * 16u;
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

    uint32_t kreg[2][KW];
    uint32_t vreg[2][VW];
    uint32_t nreg = 0;
    // (One head per wave: tiles are only requested after the rotations.  Asking for the first one up front, without the
    // row this workgroup is about to store, made launches 0.4 to 0.9 us slower at every context length, also with R
    // arriving in 4 coalesced pieces per lane, and no faster when only the waves without a rotation to do ask;
    // pulling further tiles towards the caches during the prologue cost 2 us per tile: what the prologue waits
    // for then queues behind them.)

    // ---- 1. rotations of the unit's vectors
    // early(): called once the staged vectors and R are in LDS, before the rotations -- where the scan asks for its
    // first tile when that tile lies wholly before the new token
    auto rotate_unit = [&](auto early) {
        const int i16 = ln, kk = kg;
        const int dblk = rot_dblk;
        // the centroid table while the loads are under way: entry e fills 256 bytes with replicas.  A thread writes
        // entries e0 + 4 NW k, k = 0, 1, ...: the low four bits of e are the thread's own in every round (their
        // centroids come out of a register by wave shuffle, once: lane c holds centroid c; indexing the constant array
        // with a per-lane index is a dependent memory load per look-up, several microseconds for this loop), the
        // upper four are the same for the whole wave (v_readlane).
        constexpr int kStep = NW * kWave * 4, kRounds = kTableWords / kStep;
        static_assert(kRounds * kStep == kTableWords && kStep % 1024 == 0, "a round advances e by a multiple of 16");
        const int e0 = tid >> 4, hi0 = uniform(tid >> 8);
        auto cent_of = [&](int c) -> float {                // c uniform over the wave
            return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cent_lane), c));
        };
        if constexpr (BITS == 4) {
            const half_t lo = (half_t)__shfl(cent_lane, e0 & 15, 64);
#pragma unroll
            for (int k = 0; k < kRounds; k++) {
                half2_t p = {lo, (half_t)cent_of(hi0 + (NW / 4) * k)};
                const uint32_t w = *reinterpret_cast<uint32_t*>(&p);
                *reinterpret_cast<uint4*>(&tab_s[tid * 4 + k * kStep]) = uint4{w, w, w, w};
            }
        } else {
            // a byte's four codes in the order 0, 2, 1, 3 (one head per wave: what its lane-pair exchange wants) or
            // in their own order (two heads per wave)
            const half_t c0 = (half_t)__shfl(cent_lane, e0 & 3, 64), c1 = (half_t)__shfl(cent_lane, (e0 >> 2) & 3, 64);
#pragma unroll
            for (int k = 0; k < kRounds; k++) {
                const int hi = hi0 + (NW / 4) * k;          // e >> 4
                const half_t c2 = (half_t)cent_of(hi & 3), c3 = (half_t)cent_of(hi >> 2);
                half2_t p0 = {c0, PAIR ? c1 : c2};
                half2_t p1 = {PAIR ? c2 : c1, c3};
                const uint32_t w0 = *reinterpret_cast<uint32_t*>(&p0), w1 = *reinterpret_cast<uint32_t*>(&p1);
                *reinterpret_cast<uint4*>(&tab_s[tid * 4 + k * kStep]) = uint4{w0, w1, w0, w1};
            }
        }

        // the staged vectors: rows of kStageStride bytes (16-byte aligned; a lane group's 2-byte reads below
        // fall into 32 different banks), in the space the merged outputs will use at the end
        char* x_s = reinterpret_cast<char*>(o_s);
        if ((tid >> 4) < nvec) *reinterpret_cast<uint4*>(x_s + (tid >> 4) * kStageStride + (tid & 15) * 16) = stage;
        if (PROD && prod_live) *reinterpret_cast<uint4*>(&prod_s[prod_row][8 * prod_piece]) = prod;
        if (wave < 8) stage_operand_tile(rot_s + wave * kOperandTileDwords, rraw, lane);
        lds_barrier();
        early();
        float rv[32];                                      // R[16 * rot_dblk + ln][4s + kg]
        if (rotating) read_operand_tile(rot_s + rot_dblk * kOperandTileDwords, lane, rv);
        if (PROD) {
            // optional producers on the staged K and query vectors, one vector per wave: per-head RMSNorm
            // (kernels.cu:880-923), then rotary embedding (927-961), each rounded to fp16 as the reference's
            // in-place kernels leave it; V vectors stay as they are
            for (int v = wave; v < nvec; v += NW) {
                int kind, head;
                (void)unit_vector(v, kind, head);
                if (kind == 1) continue;                           // uniform over the wave
                half_t* row = reinterpret_cast<half_t*>(x_s + v * kStageStride);
                float x0 = (float)row[lane], x1 = (float)row[lane + 64];
                HeadXform t;
                t.weight = normed ? &prod_s[0][0] + (kind == 0 ? 0 : kHeadDim) : nullptr;
                t.eps = f.eps;
                t.biased = f.biased;
                t.cos_row = roped ? prod_s[2] : nullptr;
                t.sin_row = prod_s[3];
                t.rope_dim = f.rope_dim;
                t.single_order = 0;
                xform_head(x0, x1, lane, t);
                row[lane] = (half_t)x0;                            // both are fp16 values already
                row[lane + 64] = (half_t)x1;
            }
            lds_barrier();
        }

        for (int vt = wave >> 3; rotating && vt * 16 < nvec; vt += kRotGroups) {  // uniform over the wave
            const int vi = vt * 16 + i16;
            const int vc = vi < nvec ? vi : nvec - 1;              // clamp reads, mask stores
            int kind, head;
            (void)unit_vector(vc, kind, head);
            const bool is_query = kind == 2;
            // B operand: coordinate 4s + kk of vector vc
            float xv[32];
            const half_t* xrow = reinterpret_cast<const half_t*>(x_s + vc * kStageStride) + kk;
#pragma unroll
            for (int s2 = 0; s2 < 32; s2++) xv[s2] = (float)xrow[4 * s2];
            const float n2 = rotation_tree_sum_sq(xv);                 // the reference's order, as rotate_kernel
            if (!is_query) {
                const float inv = 1.0f / sqrtf(n2 + 1e-12f);
#pragma unroll
                for (int s = 0; s < 32; s++) xv[s] *= inv;
            }
            float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 32; s++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(rv[s], xv[s], acc, 0, 0, 0);

            if (is_query && vi < nvec) {
                float4 o = {acc[0] * f.q_scale, acc[1] * f.q_scale, acc[2] * f.q_scale, acc[3] * f.q_scale};
                *reinterpret_cast<float4*>(&qrot_s[vc - 2 * HKW][dblk * 16 + 4 * kk]) = o;
            }
            uint32_t packed = 0;
#pragma unroll
            for (int r = 0; r < 4; r++) packed |= (uint32_t)turbo_quantize(acc[r], BITS) << (r * BITS);
            constexpr int PB = 4 * BITS;
            uint32_t p1 = (uint32_t)__shfl((int)packed, i16 + 16, 64);
            uint32_t p2 = (uint32_t)__shfl((int)packed, i16 + 32, 64);
            uint32_t p3 = (uint32_t)__shfl((int)packed, i16 + 48, 64);
            if (kk == 0 && vi < nvec && !is_query && appends) {
                constexpr int BPH = kHeadDim * BITS / 8;
                const long long crow = seq_row0 + pos;
                uint8_t* dst = (kind == 0 ? f.k_codes : f.v_codes) + (crow * Hk + head) * BPH + dblk * (2 * BITS);
                if (BITS == 4) {
                    uint2 o = {packed | (p1 << PB), p2 | (p3 << PB)};
                    *reinterpret_cast<uint2*>(dst) = o;
                } else {
                    *reinterpret_cast<uint32_t*>(dst) = packed | (p1 << PB) | (p2 << (2 * PB)) | (p3 << (3 * PB));
                }
                if (dblk == 0) (kind == 0 ? f.k_norms : f.v_norms)[crow * Hk + head] = (half_t)sqrtf(n2 + 1e-12f);
            }
        }
        __syncthreads();        // table, q_rot and the new cache row are in place; R has been read
        // the wave's slice of the probabilities starts at zero (no other wave touches it)
        *reinterpret_cast<uint4*>(&p_s[wave][0][0] + 8 * lane) = uint4{0u, 0u, 0u, 0u};
    };
    // ---- 3. the parts meet in LDS.  B operand of the rotate-back first (its loads run under the merge, and stay
    // hidden there: R brought in coalesced and passed through LDS instead was 0.25 us slower per launch):
    // R[32kk + s][16*dblk + i16], s = 0..31
    const int nv = HKW * R;                                  // output vectors of this unit
    const int dblk = wave & 7;
    const bool back = wave < 8 * kRotGroups && (wave >> 3) * 16 < nv;
    uint16_t rb[32];
    auto load_rb = [&]() {
    if (PAIR || back) {          // (PAIR: eight waves, every one of them rotates back)
        const uint16_t* rp = reinterpret_cast<const uint16_t*>(a.rotation) + (32 * kg) * kHeadDim + 16 * dblk + ln;
#pragma unroll
        for (int s = 0; s < 32; s++) rb[s] = rp[s * kHeadDim];
    }
    };
    if constexpr (PAIR) {
        // ---- 2 (PAIR). scan of this wave's part, two KV heads per wave (kv_pair_scan.hpp has the tile and why)
        int l2 = lane;
        asm volatile("" : "+v"(l2));
        PairLane<R, BITS> L;
        L.init(l2, p_s[wave], tab_s);
        const uint32_t kvp = (uint32_t)Hk * kHeadBytes;
        const uint32_t nrow = (uint32_t)Hk * 2u;
        const uint32_t koff = L.koff_rows * kvp + L.koff_bytes;
        const uint32_t voff = L.voff_rows * kvp + L.voff_bytes;
        const uint32_t noff = (uint32_t)L.tok0 * nrow;
        // the sequence's rows of this pair: a tile is one multiplication per array away
        const long long seq_row0 = (long long)g * a.seq_stride_rows;
        const char* kpair = reinterpret_cast<const char*>(a.k) + seq_row0 * kvp + (long long)h * kHeadBytes;
        const char* vpair = reinterpret_cast<const char*>(a.v) + seq_row0 * kvp + (long long)h * kHeadBytes;
        const char* knpair = reinterpret_cast<const char*>(a.k_norms) + seq_row0 * nrow + (long long)h * 2;
        const char* vnpair = reinterpret_cast<const char*>(a.v_norms) + seq_row0 * nrow + (long long)h * 2;
        // The tile whose loads are issued during the current one: first token and rows that exist.  (Loads of a tile
        // past the wave's last one get an empty extent: they return zeros without touching memory.)
        int next_tile = 0, next_rows = 0;
        auto set_next = [&](int i) {
            next_tile = tile_at(i);
            next_rows = i < ntiles ? max(min(n - next_tile, 32), 0) : 0;
        };
        // (4 bit: every load instruction covers whole lines, non-temporal; 2 bit: half lines, the ordinary policy)
        constexpr int kCodesAux = BITS == 4 ? kStreamCodes : 0;
        auto issue_k = [&](PairTileRegs<BITS>& t) {
            __amdgpu_buffer_rsrc_t r = make_rsrc(kpair + (long long)next_tile * kvp, next_rows * (int)kvp);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                if constexpr (BITS == 4) t.k[c] = __builtin_amdgcn_raw_buffer_load_b128(r, (int)(koff + (uint32_t)(8 * c) * kvp), 0, kCodesAux);
                else t.k[c] = __builtin_amdgcn_raw_buffer_load_b64(r, (int)(koff + (uint32_t)(8 * c) * kvp), 0, kCodesAux);
            }
        };
        auto issue_v = [&](PairTileRegs<BITS>& t) {
            __amdgpu_buffer_rsrc_t r = make_rsrc(vpair + (long long)next_tile * kvp, next_rows * (int)kvp);
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if constexpr (BITS == 4) t.v[sub][j] = __builtin_amdgcn_raw_buffer_load_b64(r, (int)(voff + (uint32_t)(16 * sub + j) * kvp), 0, kCodesAux);
                    else t.v[sub][j] = __builtin_amdgcn_raw_buffer_load_b32(r, (int)(voff + (uint32_t)(16 * sub + j) * kvp), 0, kCodesAux);
                }
            }
        };
        // (every lane asks, also those that own no token: they repeat a neighbour's address, which costs nothing, and
        // the loop has no branch here)
        auto issue_n = [&](PairTileRegs<BITS>& t) {
            __amdgpu_buffer_rsrc_t rk = make_rsrc(knpair + (long long)next_tile * nrow, next_rows * (int)nrow);
            __amdgpu_buffer_rsrc_t rv = make_rsrc(vnpair + (long long)next_tile * nrow, next_rows * (int)nrow);
            t.n[0][0] = __builtin_amdgcn_raw_buffer_load_b32(rk, (int)noff, 0, kStreamNorms);
            t.n[1][0] = __builtin_amdgcn_raw_buffer_load_b32(rk, (int)(noff + 16u * nrow), 0, kStreamNorms);
            t.n[0][1] = __builtin_amdgcn_raw_buffer_load_b32(rv, (int)noff, 0, kStreamNorms);
            t.n[1][1] = __builtin_amdgcn_raw_buffer_load_b32(rv, (int)(noff + 16u * nrow), 0, kStreamNorms);
        };

        PairState<R> S;
        S.reset();
        // One tile of loads in flight per wave.  (Tried: two tiles, 2 % slower; a second register set for K alone, whose
        // loads otherwise have only the softmax and P.V of one tile to arrive in, 6 % slower -- more requests in flight
        // make the memory slower here, not faster; the first tile asked for before the rotations, 0.4 us slower, as
        // with one head per wave; the scores of tile i + 1 placed beside the P.V of tile i for the scheduler to
        // interleave, 3 % slower.)
        PairTileRegs<BITS> t;
        // EARLY: a wave asks for its first tile in the middle of the prologue, behind the prologue's own loads
        // and ahead of the rotations, when all of its rows are older than the token this launch appends (the launch's
        // own row only exists after the barrier that ends the rotations).  Rollouts of a few hundred tokens gain
        // 4.5 % (128 sequences at 257..768 tokens: 21.6 against 22.6 us per launch); with 8 tiles per wave it makes no
        // difference, and with 16 and more the launch gets slower (64 x 4096 tokens: + 0.6 us, x 8192: + 2.2 us), as
        // with every other way of putting more requests in flight at the start that was tried.  (A second register set
        // in this short-context form, so that the tile after next is in flight too -- the memory is far from busy there:
        // 22.9 against 21.2 us per launch on the rollout, 24.7 against 23.5 at 64 x 1024 tokens, 8 % and 5 % slower; with
        // four query heads per KV head it does not fit the registers.  A wave's tile time at these sizes is the tile's
        // own chain of look-ups and matrix instructions, not the wait for its loads.)
        const bool first_early = EARLY && ntiles > 0 && tile_at(0) + 32 <= pos;      // uniform over the wave
        rotate_unit([&]() {
            if (first_early) { set_next(0); issue_k(t); issue_n(t); issue_v(t); }
        });
        if (!first_early) {
            set_next(0);
            issue_k(t);
            issue_n(t);
            issue_v(t);
        }
        load_rb();              // behind the first tile's loads; the registers are there, and the epilogue need not wait
        if (ntiles > 0) {
            S.load_query(L, [&](int i) -> const float* { return &qrot_s[hk_local * R + i][0]; });
            for (int it = 0; it < ntiles; it++) {
                const int tile = next_tile;
                set_next(it + 1);
                pair_scan_tile<R>(L, S, t, tile, n, [&]() { issue_k(t); }, [&]() { issue_n(t); }, [&]() { issue_v(t); });
            }
        }
        pair_scan_finish<R>(L, S, 1.0f / kAlpha, [&](int hd, int r, const float (&ov)[16]) {
            float* pr = &part_s[part * HKW + hk_local + hd][r][0];
#pragma unroll
            for (int j4 = 0; j4 < 4; j4++)
                *reinterpret_cast<float4*>(pr + 16 * (L.pn & 7) + 4 * j4) = float4{ov[4 * j4], ov[4 * j4 + 1], ov[4 * j4 + 2], ov[4 * j4 + 3]};
            if ((L.pn & 7) == 0) { pr[kHeadDim] = S.m_run[r]; pr[kHeadDim + 1] = S.l_run[r]; }
        });
    } else {
        rotate_unit([]() {});
        {
            int l2 = lane;
            asm volatile("" : "+v"(l2));
            derive_lane(l2);
        }

        // ---- 2. scan of this wave's part
        float4_t o[8];
    #pragma unroll
        for (int j = 0; j < 8; j++) o[j] = float4_t{0.f, 0.f, 0.f, 0.f};
        float m_run[R], l_run[R];
    #pragma unroll
        for (int r = 0; r < R; r++) { m_run[r] = kNegBig; l_run[r] = 0.0f; }

        if (ntiles > 0) {
            issue_k(kreg, first_tile);
            nreg = issue_n(first_tile);
            issue_v(vreg, first_tile);
            // A operand of the score MFMAs: q_rot[head][32kg + 8j + i], row m = fp16 value of head m, row m + 8
            // its rounding remainder; the 2-bit table returns the codes of a byte in the order 0,2,1,3
            half8_t aq[4];
            {
                const int hq = ln & 7;
                const bool lo_part = (ln & 8) != 0;
                const float* qr = &qrot_s[hk_local * R + (hq < R ? hq : 0)][32 * kg];
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

            for (int it = 0; it < ntiles; it++) {
                const int tile = tile_at(it);
                const int next_tile = tile_at(it + 1);
                const bool more = it + 1 < ntiles;

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

                // ---- online softmax (base 2): this lane owns token ln of sub-tile my_sub
                const float kn = h2f_bits(nreg & 0xffffu), vn = h2f_bits(nreg >> 16);
                if (more) nreg = issue_n(next_tile);
                const bool valid = useful && (tile + 16 * my_sub + ln < n);
                float raw[R], x[R];
                bool raise = false;
    #pragma unroll
                for (int r = 0; r < R; r++) {
                    uint32x2_t sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(s[0][r]), __float_as_uint(s[1][r]), false, false);
                    raw[r] = (__uint_as_float(sw[0]) + __uint_as_float(sw[1])) * kn;    // kernels.cu:1707
                    x[r] = valid ? raw[r] - m_run[r] : kNegBig;
                    raise = raise || (x[r] > kRaise);
                }
                if (__any(raise)) {
    #pragma unroll
                    for (int r = 0; r < R; r++) {
                        float m_new = fmaxf(m_run[r], wave_max(valid ? raw[r] : kNegBig));
                        float alpha = __builtin_amdgcn_exp2f(m_run[r] - m_new);
                        m_run[r] = m_new;
                        l_run[r] *= alpha;
                        x[r] = valid ? raw[r] - m_new : kNegBig;
    #pragma unroll
                        for (int j = 0; j < 8; j++) o[j][r] *= alpha;
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
                    uint32_t xe[4], xo[4];
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
                    for (int jp = 0; jp < 4; jp++) {
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
                    for (int q = 0; q < 4; q++) {
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
            }
        }

    load_rb();
    #pragma unroll
        for (int r = 0; r < R; r++) {
            l_run[r] = wave_sum(l_run[r]);
    #pragma unroll
            for (int j = 0; j < 8; j++) o[j][r] += __shfl_xor(o[j][r], 32, 64);   // row r + row r+8 (lo part of P)
        }
        if (kg == 0) {
    #pragma unroll
            for (int r = 0; r < R; r++) {
                float* pr = &part_s[wave][r][0];
                float4 lo4 = {o[0][r] * (1.0f / kAlpha), o[1][r] * (1.0f / kAlpha), o[2][r] * (1.0f / kAlpha), o[3][r] * (1.0f / kAlpha)};
                float4 hi4 = {o[4][r] * (1.0f / kAlpha), o[5][r] * (1.0f / kAlpha), o[6][r] * (1.0f / kAlpha), o[7][r] * (1.0f / kAlpha)};
                *reinterpret_cast<float4*>(pr + 8 * ln) = lo4;
                *reinterpret_cast<float4*>(pr + 8 * ln + 4) = hi4;
                if (ln == 0) { pr[kHeadDim] = m_run[r]; pr[kHeadDim + 1] = l_run[r]; }
            }
        }
    }
    lds_barrier();                 // the loads of R above stay in flight

    {   // merge: thread -> (vector tid / 32, coordinates 4 * (tid % 32) .. +3); vector = (local KV head, query head)
        const int vec = tid >> 5, k4 = (tid & 31) * 4;
        float4 o4 = {0.f, 0.f, 0.f, 0.f};
        float mg = kNegBig, lsum = 0.0f;
        float4 av = {0.f, 0.f, 0.f, 0.f};
        if (vec < nv) {
            const int hk_l = vec / R, r = vec - hk_l * R;
            for (int p = 0; p < SPLIT; p++) mg = fmaxf(mg, part_s[p * HKW + hk_l][r][kHeadDim]);
            for (int p = 0; p < SPLIT; p++) {
                const float* pr = &part_s[p * HKW + hk_l][r][0];
                const float fs = __builtin_amdgcn_exp2f(pr[kHeadDim] - mg);
                const float4 c = *reinterpret_cast<const float4*>(pr + k4);
                lsum = __builtin_fmaf(pr[kHeadDim + 1], fs, lsum);
                av.x = __builtin_fmaf(c.x, fs, av.x);
                av.y = __builtin_fmaf(c.y, fs, av.y);
                av.z = __builtin_fmaf(c.z, fs, av.z);
                av.w = __builtin_fmaf(c.w, fs, av.w);
            }
        }
        if constexpr (SHARES) {
            // this share's sums to memory (device scope: written through), then the ticket
            __shared__ unsigned last_s;
            const long long unit = (long long)g * nhg + hg;
            auto slot = [&](int sh) -> float* { return f.share_ws + ((unit * nshares + sh) * nv + vec) * kRowFloats; };
            auto put = [](float* p, float x) { __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
            auto get = [](const float* p) -> float { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
            if (vec < nv) {
                float* mine = slot(share);
                put(mine + k4, av.x); put(mine + k4 + 1, av.y); put(mine + k4 + 2, av.z); put(mine + k4 + 3, av.w);
                if (k4 == 0) { put(mine + kHeadDim, mg); put(mine + kHeadDim + 1, lsum); }
            }
            __builtin_amdgcn_s_waitcnt(0);          // every store of this wave has been acknowledged
            __syncthreads();
            if (tid == 0) {
                const unsigned old = __hip_atomic_fetch_add(f.tickets + unit, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                last_s = old == (unsigned)nshares - 1u ? 1u : 0u;
            }
            __syncthreads();
            if (!last_s) return;                    // uniform over the workgroup: the last share finishes the unit
            if (tid == 0) __hip_atomic_store(f.tickets + unit, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
            if (vec < nv) {
                float ms[kMaxShares], ls[kMaxShares];
                float4 as[kMaxShares];
                mg = kNegBig;
                for (int sh = 0; sh < nshares; sh++) {
                    const float* p = slot(sh);
                    as[sh] = float4{get(p + k4), get(p + k4 + 1), get(p + k4 + 2), get(p + k4 + 3)};
                    ms[sh] = get(p + kHeadDim);
                    ls[sh] = get(p + kHeadDim + 1);
                    mg = fmaxf(mg, ms[sh]);
                }
                lsum = 0.0f;
                av = float4{0.f, 0.f, 0.f, 0.f};
                for (int sh = 0; sh < nshares; sh++) {
                    const float fs = __builtin_amdgcn_exp2f(ms[sh] - mg);
                    lsum = __builtin_fmaf(ls[sh], fs, lsum);
                    av.x = __builtin_fmaf(as[sh].x, fs, av.x);
                    av.y = __builtin_fmaf(as[sh].y, fs, av.y);
                    av.z = __builtin_fmaf(as[sh].z, fs, av.z);
                    av.w = __builtin_fmaf(as[sh].w, fs, av.w);
                }
            }
        }
        if (vec < nv) {
            const float inv = 1.0f / (lsum + 1e-8f);             // kernels.cu:1746
            o4 = float4{av.x * inv, av.y * inv, av.z * inv, av.w * inv};
        }
        *reinterpret_cast<float4*>(&o_s[vec][k4]) = o4;
    }
    lds_barrier();

    // ---- out[vector][d] = sum_k o[vector][k] R[k][d]; lane group kk owns k in [32kk, 32kk+32).  On fp16 MFMAs: R is
    // exact in fp16, o enters as fp16 value + rounding remainder, every product is exact in the fp32 accumulator --
    // only the order of the additions differs from the reference's chain (kernels.cu:1769-1775), far inside what the
    // fp16 result resolves -- and the chain is 8 MFMAs instead of 32.
    for (int vt = wave >> 3; back && vt * 16 < nv; vt += kRotGroups) {
        float4_t acc = {0.f, 0.f, 0.f, 0.f};
        const float* orow = &o_s[vt * 16 + ln][32 * kg];
#pragma unroll
        for (int st = 0; st < 4; st++) {
            float4 oa = *reinterpret_cast<const float4*>(orow + 8 * st);
            float4 ob = *reinterpret_cast<const float4*>(orow + 8 * st + 4);
            const float ov[8] = {oa.x, oa.y, oa.z, oa.w, ob.x, ob.y, ob.z, ob.w};
            half8_t ahi, alo;
            union { uint16_t u[8]; half8_t h; } bm;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                ahi[i] = (half_t)ov[i];
                alo[i] = (half_t)(ov[i] - (float)ahi[i]);
                bm.u[i] = rb[8 * st + i];
            }
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bm.h, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bm.h, acc, 0, 0, 0);
        }
        // lane holds out[vector vt*16 + 4kk + r][d = 16*dblk + i16]
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int vec = vt * 16 + 4 * kg + r;
            if (vec < nv) {
                const int head = hg * HKW * R + vec;
                const long long col = (long long)head * kHeadDim + 16 * dblk + ln;
                half_t hv = (half_t)acc[r];
                if (a.gate) hv = gated(hv, a.gate[(long long)g * a.gate_stride + col]);
                a.out[(long long)g * a.q_stride + col] = hv;
            }
        }
    }
}

// Two KV heads per wave (PAIR) when the workgroup's heads come in pairs: eight waves, every cache line of the 4-bit
// cache fetched by one instruction.  The workgroup's HKW * (2 + R) vectors must fit its staging slots (a vector per
// 16 threads) and its HKW * R outputs its merge slots (one per 32 threads).
static bool pairs_fit(int bits, int R, int hkw) {
    return (bits == 4 || bits == 2) && (hkw & 1) == 0 && (2 * kPairWaves) % hkw == 0 && hkw * (2 + R) <= 4 * kPairWaves && hkw * R <= 2 * kPairWaves;
}
bool decode_fused_pairs(const AttnArgs& a, int hkw) { return pairs_fit(a.bits, a.num_heads / a.num_kv_heads, hkw); }

// The measured figures behind the estimates below.  MI355X: launches at batches 8 to 256 and contexts 1k to 8k
// reproduce within 5 %; hand-over costs from a probe in which all 512 workgroups of a streaming launch take part.
namespace {
constexpr PlanConstants kPlanTable[] = {
    {"gfx950", 12.0, {3.08, 2.72}, 2.45, {5.95, 4.68}, {7200.0, 5500.0}, {27.0, 25.0}, {7.2e6, 5.4e6}, {0.0, 3.7, 5.4, 8.7}},
};
}  // namespace
const PlanConstants& plan_constants() {
    static const PlanConstants* chosen = nullptr;
    if (!chosen) {
        const PlanConstants* pick = &kPlanTable[0];
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) {
            for (const PlanConstants& c : kPlanTable)
                if (strstr(prop.gcnArchName, c.device)) { pick = &c; break; }
        } else {
            (void)hipGetLastError();           // no device (a host-only process asking for the plan): the first entry
        }
        chosen = pick;
    }
    return *chosen;
}

// Microseconds one launch takes for G sequences of ctx tokens with hkw KV heads per workgroup, by a count fitted to
// measured launches (plan_constants): the workgroups run in rounds of one per CU; a round costs its fixed part and,
// per token of context, the cube-root sum of what one CU sustains for the workgroup's heads (a workgroup whose waves
// scan one head each moves its bytes at about half the rate of one whose waves scan two) and of the whole chip's rate
// for all the workgroups of the round.
double decode_fused_estimate_us(int G, int num_heads, int Hk, int bits, bool allow_pairs, int hkw, double ctx) {
    const PlanConstants& pc = plan_constants();
    const double cus = compute_units();
    const int R = Hk > 0 ? num_heads / Hk : 1;
    const int w = bits == 4 ? 0 : 1;
    const double bpt = bits == 4 ? 132.0 : 68.0;                  // bytes per token and KV head: K and V codes and norms
    const double units = (double)G * (Hk / hkw);
    const double rounds = std::ceil(units / cus), active = units < cus ? units : cus;
    const bool pair = allow_pairs && pairs_fit(bits, R, hkw);
    const double per_head_ns = pair ? (bits == 2 && hkw >= 4 ? pc.pair_wide2_ns : pc.pair_ns[w]) : pc.single_ns[w];
    const double k_cu = hkw * per_head_ns, k_bw = active * hkw * bpt / pc.one_bw[w];   // ns per token
    return rounds * (pc.one_fixed_us + ctx * 1e-3 * std::cbrt(k_cu * k_cu * k_cu + k_bw * k_bw * k_bw));
}

// Three launches (rotation, scan, merge) for the same step: their fixed cost and the scan at its rate.
double decode_three_estimate_us(int G, int Hk, int bits, double ctx) {
    const PlanConstants& pc = plan_constants();
    const int w = bits == 4 ? 0 : 1;
    const double bpt = bits == 4 ? 132.0 : 68.0;
    return pc.three_fixed_us[w] + (double)G * Hk * bpt * ctx / pc.three_bw[w];
}

// KV heads per workgroup (8, 4, 2 or 1): the choice with the smallest estimate at a context of 4096 tokens (the order
// hardly depends on the context); among equals the larger number, whose workgroups read longer contiguous pieces of a
// cache row.  (Batch 64 with 8 KV heads: 2, one round of 256 workgroups; batch 48: 2 again, 192 workgroups in one
// round, where two rounds of 384 single-head workgroups took 119 us against 85; batch 96: 4.)
int decode_fused_heads_per_workgroup(int G, int num_heads, int Hk, int bits, bool allow_pairs) {
    int best = 1;
    double best_us = 0.0;
    for (int c = 1; c <= 8; c <<= 1) {
        if (Hk % c != 0) continue;
        const double us = decode_fused_estimate_us(G, num_heads, Hk, bits, allow_pairs, c, 4096.0);
        if (c == 1 || us <= best_us) { best = c; best_us = us; }
    }
    return best;
}

// With shares: a launch of G * (Hk / hkw) * shares workgroups, each with 1 / shares of the context, plus what the
// hand-over costs at the end (plan_constants).  Shares are only taken while all workgroups fit the compute units in
// one round and a share still has a tile for every wave.
namespace {
std::atomic<int> g_force_hkw{0}, g_force_shares{0};
}  // namespace
void decode_fused_force_shape(int hkw, int shares) { g_force_hkw.store(hkw); g_force_shares.store(shares); }

FusedShape decode_fused_shape(int G, int num_heads, int Hk, int bits, bool allow_pairs, int max_shares, double ctx) {
    const bool can_share = max_shares >= 2;
    const int R = Hk > 0 ? num_heads / Hk : 1;
    const double cus = compute_units();
    FusedShape best{decode_fused_heads_per_workgroup(G, num_heads, Hk, bits, allow_pairs), 1, 0.0};
    best.us = decode_fused_estimate_us(G, num_heads, Hk, bits, allow_pairs, best.hkw, ctx);
    if (can_share) {
        for (int c = 1; c <= 8; c <<= 1) {
            if (Hk % c != 0) continue;
            const bool pair = allow_pairs && pairs_fit(bits, R, c);
            const int parts = (pair ? 2 * kPairWaves : kFusedWaves) / c;          // waves (parts of the context) per head
            for (int sh = 2, lg = 1; sh <= kMaxShares && sh <= max_shares; sh <<= 1, lg++) {
                if ((double)G * (Hk / c) * sh > cus) continue;
                if (ctx < 32.0 * parts * sh) continue;
                // every share is a launch of its own size: G * shares "sequences" of ctx / shares tokens
                const double us = decode_fused_estimate_us(G * sh, num_heads, Hk, bits, allow_pairs, c, ctx / sh) +
                                  plan_constants().handover_us[lg];
                if (us < best.us) best = FusedShape{c, sh, us};
            }
        }
    }
    const int fh = g_force_hkw.load(), fs = g_force_shares.load();
    if (fh > 0 && Hk % fh == 0) best.hkw = fh;
    if (fs > 0) best.shares = fs <= max_shares && fs <= kMaxShares ? fs : 1;
    return best;
}

bool decode_fused_usable(const AttnArgs& a, const FusedArgs& f) {
    const int R = a.num_kv_heads > 0 ? a.num_heads / a.num_kv_heads : 0;
    if (a.bits != 4 && a.bits != 2) return false;
    if (R != 1 && R != 2 && R != 4) return false;
    if (a.pos_mode != kPosArray || !a.positions || a.block_table || a.G <= 0) return false;
    if (a.seq_stride_rows <= 0) return false;
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    if (!al16(a.q) || !al16(f.k_src) || !al16(f.v_src) || !al16(a.rotation)) return false;
    if ((a.q_stride & 7) != 0 || (f.kv_stride & 7) != 0) return false;
    if (!al16(a.k) || !al16(a.v)) return false;
    if ((f.q_weight == nullptr) != (f.k_weight == nullptr) || (f.cos_table == nullptr) != (f.sin_table == nullptr)) return false;
    if (!al16(f.q_weight) || !al16(f.k_weight) || !al16(f.cos_table) || !al16(f.sin_table)) return false;
    if (f.cos_table && !(f.rope_dim == 128 || (f.rope_dim > 0 && f.rope_dim <= 64 && f.rope_dim % 16 == 0))) return false;
    // the scan addresses a tile through a 32-bit buffer offset from the tile's first row: always small
    return true;
}

void launch_decode_fused(const AttnArgs& a, const FusedArgs& f_in, hipStream_t s, bool allow_pairs) {
    FusedArgs f = f_in;
    const FusedShape shape = decode_fused_shape(a.G, a.num_heads, a.num_kv_heads, a.bits, allow_pairs,
                                                f.share_ws != nullptr && f.tickets != nullptr ? f.max_shares : 1,
                                                f.ctx_bound > 0 ? (double)f.ctx_bound : 4096.0);
    f.hkw = shape.hkw;
    f.shares = shape.shares;
    f.q_scale = attention_mfma_q_scale(a.bits);
    const int R = a.num_heads / a.num_kv_heads;
    const bool pair = allow_pairs && decode_fused_pairs(a, f.hkw);
    const dim3 g3((unsigned)(a.G * (a.num_kv_heads / f.hkw) * f.shares)), b3((pair ? kPairWaves : kFusedWaves) * kWave);
    const bool prod = f.q_weight != nullptr || f.cos_table != nullptr;
    // first tile in the middle of the prologue: when no wave gets more than 8 tiles of 32 tokens by the caller's bound
    // of the context (two heads per wave: 16 / hkw parts per head)
    const bool early = pair && f.shares == 1 && f.ctx_bound > 0 && f.ctx_bound <= 8 * 32 * (2 * kPairWaves / f.hkw);
    note_scan_kernel(pair ? (f.shares > 1 ? "decode_fused_kernel, two KV heads per wave, context shared by workgroups"
                                          : "decode_fused_kernel, two KV heads per wave")
                          : (f.shares > 1 ? "decode_fused_kernel, one KV head per wave, context shared by workgroups"
                                          : "decode_fused_kernel, one KV head per wave"));
#define TW_FUSED_E(RR, BB, PP, EE, SS) \
    do { if (prod) launch_scan_kernel(decode_fused_kernel<RR, BB, true, PP, EE, SS>, g3, b3, s, a, f); \
         else launch_scan_kernel(decode_fused_kernel<RR, BB, false, PP, EE, SS>, g3, b3, s, a, f); } while (0)
#define TW_FUSED(RR, BB, PP) do { if (f.shares > 1) TW_FUSED_E(RR, BB, PP, false, true); else if (PP && early) TW_FUSED_E(RR, BB, PP, PP, false); else TW_FUSED_E(RR, BB, PP, false, false); } while (0)
#define TW_FUSED_R(BB, PP) do { if (R == 1) TW_FUSED(1, BB, PP); else if (R == 2) TW_FUSED(2, BB, PP); else TW_FUSED(4, BB, PP); } while (0)
    if (a.bits == 4) { if (pair) TW_FUSED_R(4, true); else TW_FUSED_R(4, false); }
    else { if (pair) TW_FUSED_R(2, true); else TW_FUSED_R(2, false); }
#undef TW_FUSED_R
#undef TW_FUSED
#undef TW_FUSED_E
}

}  // namespace twkv
