// kv_attention_valu.hip -- GQA decode attention over the fp16 or the compressed
// cache, fp32 vector-ALU version, for gfx950.
//
// Replaces gqa_attention_{decode,batch}_kernel (kernels.cu:244-345, 981-1066),
// turbo_gqa_attention{,_batch}_kernel (kernels.cu:1641-1870) and, with
// pos = query index, the two causal prefill kernels (kernels.cu:1071-1158,
// 1874-1960).  The reference gives one 128-thread block per (sequence, query
// head), walks every K row byte by byte from a single thread and keeps the
// scores in an fp32 scratch array in memory.  Here:
//   - a workgroup owns (sequence, KV head, context chunk): the query heads of a
//     GQA group share every byte that is loaded, and long contexts are split
//     over workgroups (split-K) with a log-sum-exp merge;
//   - compressed cache: four adjacent lanes own one token: each loads 16 bytes (32 codes) of the
//     64-byte K row, so a wave reads 16 tokens per load instruction, dequantizes
//     in registers through a 16-entry LDS centroid table and reduces the dot
//     product over the quad with two cross-lane shuffles;
//   - fp16 cache: EIGHT adjacent lanes own one token and each load instruction takes 16 bytes
//     per lane, i.e. one whole 128-byte line of the head's 256-byte row per token: a line that one
//     instruction covers in full can be loaded non-temporally (every cache byte is read once per
//     launch; a plain read of the same bytes runs at 7.0 instead of 6.2 TB/s with the hint), while
//     a line that two instructions share would be fetched twice under it;
//   - softmax is online (running max / running sum per lane), so no score ever
//     goes to memory; V is accumulated in registers in the rotated basis and
//     rotated back once per (sequence, head) (kernels.cu:1769-1775).
// Arithmetic is fp32 throughout like the reference; only summation order differs.
// The file holds two scan kernels -- attention_valu_kernel, which the list above describes, and attention_rows_kernel
// for the fp16 cache with KV heads in eights (its waves read whole cache rows; described where it is defined) -- and
// attention_merge_kernel, the log-sum-exp merge of either one's partial results.

#include <algorithm>

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"

namespace twkv {

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / kWave;
// lanes that own one token, and the values of its head each of them holds
template <int MODE> struct LanesPerToken { static constexpr int value = MODE == 0 ? 8 : 4; };
// (kNegBig, the reference's max init of kernels.cu:1686, and seq_pos come from kv_mfma_util.hpp)

// Dimension owned by element e of lane c of a token's lanes.
template <int MODE>
__device__ __forceinline__ int lane_dim(int c, int e) {
    if (MODE == 0) return 64 * (e / 8) + 8 * c + (e % 8);  // two 16-byte pieces, one per 128-byte line
    return 32 * c + e;                                     // one contiguous piece of codes
}

// Load and dequantize the lane's values (16 of an fp16 row, 32 of a compressed one) of one cache row (one KV head).
// fresh: fp16 only, the head's 128 halves come from there instead (the row of the token being appended), or NULL.
template <int MODE>
__device__ __forceinline__ void load_vals(const void* __restrict__ base, long long row, int num_kv_heads,
                                          int h, int c, const float* __restrict__ cent_s, float* vals,
                                          const half_t* fresh = nullptr) {
    if (MODE == 0) {
        const half_t* p = reinterpret_cast<const half_t*>(base) + (row * num_kv_heads + h) * kHeadDim;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            half8_t h8 = *reinterpret_cast<const half8_t*>((fresh ? fresh : p) + 64 * j + 8 * c);
#pragma unroll
            for (int i = 0; i < 8; i++) vals[8 * j + i] = (float)h8[i];
        }
    } else if (MODE == 4) {
        const uint8_t* p = reinterpret_cast<const uint8_t*>(base) + (row * num_kv_heads + h) * 64 + 16 * c;
        uint4 w4 = *reinterpret_cast<const uint4*>(p);
        uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int i = 0; i < 8; i++) vals[8 * j + i] = cent_s[(w[j] >> (4 * i)) & 15u];
        }
    } else {
        const uint8_t* p = reinterpret_cast<const uint8_t*>(base) + (row * num_kv_heads + h) * 32 + 8 * c;
        uint2 w2 = *reinterpret_cast<const uint2*>(p);
        uint32_t w[2] = {w2.x, w2.y};
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
            for (int i = 0; i < 16; i++) vals[16 * j + i] = cent_s[(w[j] >> (2 * i)) & 3u];
        }
    }
}

// Normalise, rotate back (compressed cache) and store one head.
// o_s: 128 floats of LDS holding acc / (l + 1e-8).  Called by threads d < 128
// of a workgroup after a barrier that made o_s visible.
__device__ __forceinline__ void store_head(const AttnArgs& a, int g, int head, int d, const float* o_s) {
    float o;
    if (a.bits == 0) {
        o = o_s[d];
    } else {
        o = 0.0f;
        const half_t* rot = a.rotation;
#pragma unroll 8
        for (int k = 0; k < kHeadDim; k++) o = __builtin_fmaf((float)rot[k * kHeadDim + d], o_s[k], o);
    }
    half_t h = (half_t)o;
    if (a.gate) h = gated(h, a.gate[(long long)g * a.gate_stride + (long long)head * kHeadDim + d]);
    a.out[(long long)g * a.q_stride + (long long)head * kHeadDim + d] = h;
}

// APPEND (fp16 cache, batch decode): the token at positions[g] is not in the cache yet; its rows are a.k_new and
// a.v_new, read from there by whichever lane meets that token and stored into the cache by the workgroup whose
// chunk holds it (the one of the KV head's first query-head tile).
template <int MODE, int RT, bool APPEND>
__global__ void __launch_bounds__(kAttnThreads)
attention_valu_kernel(AttnArgs a) {
    __shared__ float q_s[RT][kHeadDim];
    __shared__ float red_s[kAttnWaves][RT][kHeadDim];
    __shared__ float ml_s[kAttnWaves][RT][2];
    __shared__ float cent_s[16];

    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    constexpr int LPT = LanesPerToken<MODE>::value;      // lanes per token
    constexpr int E = kHeadDim / LPT;                     // values of the head per lane
    constexpr int kTokensPerWave = kWave / LPT;
    constexpr int kTokensPerIter = kAttnWaves * kTokensPerWave;
    const int qd = lane / LPT, c = lane % LPT;
    const int chunk = blockIdx.x;
    const int g = blockIdx.z;
    const int group = a.num_heads / a.num_kv_heads;
    const int subs = group / RT;                // query-head tiles per KV head
    const int h = blockIdx.y / subs;
    const int head0 = h * group + (blockIdx.y % subs) * RT;

    const int n = seq_pos(a, g) + 1;
    int t0, t1;
    chunk_range(n, chunk, a.nsplit, t0, t1);
    if (t0 >= t1) return;                       // uniform for the workgroup

    // fp16 rows of a contiguous cache come in through buffer loads with the non-temporal hint (the eight lanes of a
    // token take one whole 128-byte line per instruction; written as an ordinary load beside the load of the appended
    // row the compiler folds the two into one load of a selected pointer and the hint is gone): a descriptor over
    // this sequence's rows of head h up to the chunk's end, 32-bit offsets inside it
    const uint32_t rowbytes = (uint32_t)a.num_kv_heads * kHeadDim * 2;
    const bool nt_rows = MODE == 0 && !a.block_table && (long long)t1 * rowbytes < (1LL << 31);
    __amdgpu_buffer_rsrc_t krs, vrs;
    if (MODE == 0) {
        const long long first = ((long long)g * a.seq_stride_rows * a.num_kv_heads + h) * kHeadDim * 2;
        krs = make_rsrc(reinterpret_cast<const char*>(a.k) + first, nt_rows ? t1 * (int)rowbytes : 0);
        vrs = make_rsrc(reinterpret_cast<const char*>(a.v) + first, nt_rows ? t1 * (int)rowbytes : 0);
    }
    auto load_row_nt = [&](__amdgpu_buffer_rsrc_t rs, int t, const half_t* fresh_row, float* vals) {
        const uint32_t off = (uint32_t)t * rowbytes + 16u * (uint32_t)c;
        uint32x4_t w[2];
        w[0] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, kStreamCodes);
        w[1] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(off + 128u), 0, kStreamCodes);
        if (fresh_row) {                               // the token being appended: its row is not in the cache yet
            w[0] = *reinterpret_cast<const uint32x4_t*>(fresh_row + 8 * c);
            w[1] = *reinterpret_cast<const uint32x4_t*>(fresh_row + 64 + 8 * c);
        }
#pragma unroll
        for (int j = 0; j < 2; j++) {
            union { uint32x4_t u; half8_t h; } cv;
            cv.u = w[j];
#pragma unroll
            for (int i = 0; i < 8; i++) vals[8 * j + i] = (float)cv.h[i];
        }
    };

    if (tid < 16) cent_s[tid] = (MODE == 2) ? kCentroids2[tid & 3] : kCentroids4[tid];
    const half_t* k_fresh = nullptr;
    const half_t* v_fresh = nullptr;
    if (APPEND) {
        k_fresh = a.k_new + (long long)g * a.kv_new_stride + (long long)h * kHeadDim;
        v_fresh = a.v_new + (long long)g * a.kv_new_stride + (long long)h * kHeadDim;
        if (t0 <= n - 1 && n - 1 < t1 && blockIdx.y % subs == 0 && tid < 32) {      // 16 pieces of 16 bytes each for K and V
            const long long row = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, g, n - 1);
            const half_t* src = (tid < 16 ? k_fresh : v_fresh) + 8 * (tid & 15);
            half_t* cache = reinterpret_cast<half_t*>(const_cast<void*>(tid < 16 ? a.k : a.v));
            half_t* dst = cache + (row * a.num_kv_heads + h) * kHeadDim + 8 * (tid & 15);
            *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
        }
    }

    // Query, rotated for the compressed cache: q_rot = R q (kernels.cu:1671-1681).
    for (int idx = tid; idx < RT * kHeadDim; idx += kAttnThreads) {
        int r = idx / kHeadDim, d = idx % kHeadDim;
        const half_t* qh = a.q + (long long)g * a.q_stride + (long long)(head0 + r) * kHeadDim;
        float val;
        if (MODE == 0) {
            val = (float)qh[d];
        } else {
            const half8_t* rot8 = reinterpret_cast<const half8_t*>(a.rotation + d * kHeadDim);
            const half8_t* q8 = reinterpret_cast<const half8_t*>(qh);
            val = 0.0f;
            for (int k8 = 0; k8 < kHeadDim / 8; k8++) {
                half8_t rr = rot8[k8], qq = q8[k8];
#pragma unroll
                for (int i = 0; i < 8; i++) val = __builtin_fmaf((float)rr[i], (float)qq[i], val);
            }
        }
        q_s[r][d] = val;
    }
    __syncthreads();

    float qreg[RT][E];
    float acc[RT][E];
    float m[RT], l[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) {
        m[r] = kNegBig;
        l[r] = 0.0f;
#pragma unroll
        for (int e = 0; e < E; e++) {
            qreg[r][e] = q_s[r][lane_dim<MODE>(c, e)];
            acc[r][e] = 0.0f;
        }
    }
    const float scale = 0.08838834764831845f;   // 1/sqrt(128)

    for (int tb = t0; tb < t1; tb += kTokensPerIter) {
        const int t = tb + wave * kTokensPerWave + qd;
        const bool valid = t < t1;
        const int tc = valid ? t : (t1 - 1);    // clamp: keep the shuffles among a token's lanes convergent
        const long long row = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, g, tc);
        float kn = 1.0f, vn = 1.0f;
        if (MODE != 0) {
            kn = (float)a.k_norms[row * a.num_kv_heads + h];
            vn = (float)a.v_norms[row * a.num_kv_heads + h];
        }
        float vals[E];
        const bool fresh = APPEND && tc == n - 1;
        if (MODE == 0 && nt_rows) load_row_nt(krs, tc, fresh ? k_fresh : nullptr, vals);
        else load_vals<MODE>(a.k, row, a.num_kv_heads, h, c, cent_s, vals, fresh ? k_fresh : nullptr);
        float s[RT];
#pragma unroll
        for (int r = 0; r < RT; r++) {
            float dot = 0.0f;
#pragma unroll
            for (int e = 0; e < E; e++) dot = __builtin_fmaf(qreg[r][e], vals[e], dot);
#pragma unroll
            for (int off = 1; off < LPT; off <<= 1) dot += __shfl_xor(dot, off, 64);
            s[r] = dot * (kn * scale);          // kernels.cu:1707
        }
        if (MODE == 0 && nt_rows) load_row_nt(vrs, tc, fresh ? v_fresh : nullptr, vals);
        else load_vals<MODE>(a.v, row, a.num_kv_heads, h, c, cent_s, vals, fresh ? v_fresh : nullptr);
        if (valid) {
#pragma unroll
            for (int r = 0; r < RT; r++) {
                if (s[r] > m[r]) {              // rare after the first tokens
                    float alpha = __expf(m[r] - s[r]);
                    l[r] *= alpha;
#pragma unroll
                    for (int e = 0; e < E; e++) acc[r][e] *= alpha;
                    m[r] = s[r];
                }
                float p = __expf(s[r] - m[r]);
                l[r] += p;
                float pv = p * vn;              // (s * vn) * centroid, kernels.cu:1765
#pragma unroll
                for (int e = 0; e < E; e++) acc[r][e] = __builtin_fmaf(pv, vals[e], acc[r][e]);
            }
        }
    }

    // ---- merge the token streams of the workgroup (64 / LPT per wave, 4 waves)
    float mw[RT];
#pragma unroll
    for (int r = 0; r < RT; r++) mw[r] = wave_max(m[r]);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < RT; r++) ml_s[wave][r][0] = mw[r];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < RT; r++) {
        float mg = ml_s[0][r][0];
#pragma unroll
        for (int w = 1; w < kAttnWaves; w++) mg = fmaxf(mg, ml_s[w][r][0]);
        float f = __expf(m[r] - mg);            // streams that saw no token: exp(-1e30 - mg) = 0
        m[r] = mg;
        l[r] *= f;
#pragma unroll
        for (int e = 0; e < E; e++) acc[r][e] *= f;
        // sum over the token streams of the wave (lanes with equal c)
#pragma unroll
        for (int off = LPT; off < 64; off <<= 1) {
            l[r] += __shfl_xor(l[r], off, 64);
#pragma unroll
            for (int e = 0; e < E; e++) acc[r][e] += __shfl_xor(acc[r][e], off, 64);
        }
    }
    if (qd == 0) {
#pragma unroll
        for (int r = 0; r < RT; r++) {
#pragma unroll
            for (int e = 0; e < E; e++) red_s[wave][r][lane_dim<MODE>(c, e)] = acc[r][e];
            if (c == 0) ml_s[wave][r][1] = l[r];
        }
    }
    __syncthreads();

    for (int idx = tid; idx < RT * kHeadDim; idx += kAttnThreads) {
        int r = idx / kHeadDim, d = idx % kHeadDim;
        float av = red_s[0][r][d], lv = ml_s[0][r][1], mg = ml_s[0][r][0];
#pragma unroll
        for (int w = 1; w < kAttnWaves; w++) {
            av += red_s[w][r][d];
            lv += ml_s[w][r][1];
            mg = fmaxf(mg, ml_s[w][r][0]);
        }
        if (a.nsplit > 1) {
            float* part = a.ws + ((long long)g * a.num_heads + head0 + r) * a.ws_stride +
                          (long long)chunk * kPartialFloats;
            part[d] = av;
            if (d == 0) {
                part[kHeadDim] = mg;
                part[kHeadDim + 1] = lv;
            }
        } else {
            q_s[r][d] = av * (1.0f / (lv + 1e-8f));   // kernels.cu:1746
        }
    }
    if (a.nsplit > 1) return;
    __syncthreads();
    for (int idx = tid; idx < RT * kHeadDim; idx += kAttnThreads) {
        int r = idx / kHeadDim, d = idx % kHeadDim;
        store_head(a, g, head0 + r, d, q_s[r]);
    }
}

// ---- fp16 cache, whole rows: a wave reads one token's row of eight KV heads per pair of load instructions.
// Lane = (KV head, one of eight 16-byte pieces of each of the head's two 128-byte lines), so every instruction takes
// eight whole lines of ONE 2-KB cache row; the eight waves of a workgroup take the tokens of a piece of context in
// turn.  The same bytes read as one head's 256-byte slices of eight different rows per instruction
// (attention_valu_kernel) come in at 6.5 instead of 7.0 TB/s.  Arithmetic per lane is attention_valu_kernel's: a
// lane's online-softmax stream is its head's tokens t0 + wave, t0 + wave + 8, ...; the workgroup's eight streams per
// head are merged through the LDS.
// The grid is at most two workgroups per CU (what fits at 128 VGPRs), so that all of them run at once, and the
// work is cut to match: every sequence's context into nsplit even chunks (units of 8 tokens), one item per
// (sequence, chunk, block of 8 KV heads); or, when the lengths differ by more than 1/8 or the items do not fit
// the grid in one go, the balanced walk: all 8-token units of all sequences form one list and every workgroup takes
// the same number of consecutive units, cut where a sequence ends (then the merge learns the number of partials of a
// sequence from the spare word of its partial 0).
constexpr int kRowWaves = 8;
constexpr int kRowThreads = kRowWaves * kWave;
constexpr int kRowHeads = 8;               // KV heads per workgroup = lanes / 8
constexpr int kRowUnit = 8;                // tokens: one per wave
union Half8Bits { uint32x4_t u; half8_t h; half2_t p[4]; };

// sum over the eight lanes of a token's head (the lanes 8i .. 8i+7 of a wave), in every one of them: lane ^ 1, lane ^ 2
// and the mirror image within the eight, as DPP operands of the additions
__device__ __forceinline__ float sum_8_lanes(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
    return v;
}

template <int RT, bool APPEND, bool DESC>
__global__ void __launch_bounds__(kRowThreads) __attribute__((amdgpu_waves_per_eu(RT == 4 ? 2 : 4, RT == 4 ? 2 : 4)))
attention_rows_kernel(AttnArgs a, int total_items, int hgroups) {
    __shared__ float red_s[2][RT][16][kWave];            // two waves' accumulators, [r][e][lane]: conflict-free
    __shared__ float l_s[2][RT][kWave];
    __shared__ float m_s[kRowWaves][RT][kRowHeads];
    __shared__ int pre_s[kMaxBalanceSeqs + 1];           // balanced walk: units of the sequences before g
    __shared__ int bal_s[2];                             // units per workgroup, units in all

    const int tid = threadIdx.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;
    const int hd = lane / 8, c = lane % 8;                // KV head within the workgroup's eight, piece
    const int group = a.num_heads / a.num_kv_heads;
    const int subs = group / RT;                          // query-head tiles per KV head
    const uint32_t rowbytes = (uint32_t)a.num_kv_heads * kHeadDim * 2;
    const uint32_t lane_off = 256u * (uint32_t)hd + 16u * (uint32_t)c;
    const float scale = 0.08838834764831845f;   // 1/sqrt(128)

    // ---- even chunks or balanced walk (uniform over the grid: every workgroup reads the same positions)
    bool balanced = false;
    if (a.balance) {
        int carry = 0, tmin = 0x7fffffff, tmax = 0;
        for (int base = 0; base < a.G; base += kWave) {
            const int gg = base + lane;
            const int tl = gg < a.G ? (seq_pos(a, gg) + kRowUnit) / kRowUnit : 0;     // units of n = pos + 1 tokens
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
        balanced = uniform(((tmax - tmin) * 8 > tmax || total_items > (int)gridDim.x) ? 1 : 0) != 0;
        if (wave == 0 && lane == 0) {
            pre_s[0] = 0;
            const int quota = (carry + (int)gridDim.x - 1) / (int)gridDim.x;
            const int by_slots = (tmax + a.max_slots - 2) / (a.max_slots - 1);   // a sequence gets <= max_slots pieces
            bal_s[0] = max(max(quota, by_slots), 1);
            bal_s[1] = carry;
        }
        __syncthreads();
    }

    // ---- the piece in hand (uniform over the workgroup)
    int chunk = 0, g = 0, hg = 0, n = 0, t0 = 0, t1 = 0, nseg = 0;
    int bal_cur = 0, bal_end = 0, bal_g = 0, bal_quota = 1;
    if (balanced) {
        bal_quota = bal_s[0];
        const long long first = (long long)blockIdx.x * bal_quota;
        bal_cur = (int)min(first, (long long)bal_s[1]);
        bal_end = (int)min(first + bal_quota, (long long)bal_s[1]);
        int lo = 0, hi = a.G;                                 // last sequence that starts at or before bal_cur
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (pre_s[mid] <= bal_cur) lo = mid; else hi = mid;
        }
        bal_g = lo;
    }
    auto next_piece = [&]() -> bool {
        if (bal_cur >= bal_end) return false;
        while (pre_s[bal_g + 1] <= bal_cur) bal_g++;
        g = bal_g;
        const int first = pre_s[g], last = pre_s[g + 1];
        const int stop = min(bal_end, last);
        n = uniform(seq_pos(a, g)) + 1;
        t0 = kRowUnit * (bal_cur - first);
        t1 = min(kRowUnit * (stop - first), n);
        chunk = (int)blockIdx.x - first / bal_quota;
        nseg = (last - 1) / bal_quota - first / bal_quota + 1;
        hg = 0;
        bal_cur = stop;
        return true;
    };
    auto decode = [&](int item) -> bool {                     // false: the chunk holds no token
        hg = item % hgroups;
        chunk = (item / hgroups) % a.nsplit;
        g = item / (hgroups * a.nsplit);
        n = uniform(seq_pos(a, g)) + 1;
        even_chunk_range(n, chunk, a.nsplit, t0, t1);
        return t0 < t1;
    };

    for (int item = (int)blockIdx.x;; item += (int)gridDim.x) {
        if (balanced) {
            if (!next_piece()) break;
        } else {
            if (item >= total_items) break;
            if (!decode(item)) continue;
        }
        const int sub = hg % subs;
        const int h0 = (hg / subs) * kRowHeads;               // first KV head of the piece
        const int h = h0 + hd;
        const int head0 = h * group + sub * RT;               // the lane's first query head

        // The token being appended is not in the cache yet: it is the last one of its sequence, hence of its wave's
        // stream, and is taken from its own rows after the loop over the cache.
        const int t_end = APPEND ? min(t1, n - 1) : t1;
        // DESC: the fp16 rows of a contiguous cache come in through buffer loads with the non-temporal hint: a
        // descriptor over this sequence's rows from KV head h0 on, up to the piece's end, 32-bit offsets inside it
        // (the host has checked that a sequence's rows stay below 2 GB); beyond the end it gives zeros and reads nothing
        const long long first = ((long long)g * a.seq_stride_rows * a.num_kv_heads + h0) * kHeadDim * 2;
        const __amdgpu_buffer_rsrc_t krs = make_rsrc(reinterpret_cast<const char*>(a.k) + first, DESC ? t_end * (int)rowbytes : 0);
        const __amdgpu_buffer_rsrc_t vrs = make_rsrc(reinterpret_cast<const char*>(a.v) + first, DESC ? t_end * (int)rowbytes : 0);
        auto issue_row = [&](const __amdgpu_buffer_rsrc_t& rs, const void* base, int t, Half8Bits* w) {
            if (DESC) {
                const uint32_t off = (uint32_t)t * rowbytes + lane_off;
                w[0].u = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, kStreamCodes);
                w[1].u = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(off + 128u), 0, kStreamCodes);
            } else if (t < t_end) {
                const long long row = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, g, t);
                const half_t* p = reinterpret_cast<const half_t*>(base) + (row * a.num_kv_heads + h) * kHeadDim + 8 * c;
                w[0].u = *reinterpret_cast<const uint32x4_t*>(p);
                w[1].u = *reinterpret_cast<const uint32x4_t*>(p + 64);
            }
        };
        // the first rows are requested before anything else of the piece
        Half8Bits kw[2] = {}, vw[2] = {};
        issue_row(krs, a.k, t0 + wave, kw);
        issue_row(vrs, a.v, t0 + wave, vw);

        if (APPEND && t0 <= n - 1 && n - 1 < t1 && sub == 0 && tid < 256) {   // 8 heads x 16 pieces of 16 bytes, K and V
            const long long row = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, g, n - 1);
            const int which = tid >> 7, piece = tid & 127;
            const half_t* src = (which ? a.v_new : a.k_new) + (long long)g * a.kv_new_stride + (long long)h0 * kHeadDim + 8 * piece;
            half_t* cache = reinterpret_cast<half_t*>(const_cast<void*>(which ? a.v : a.k));
            half_t* dst = cache + (row * a.num_kv_heads + h0) * kHeadDim + 8 * piece;
            *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
        }

        // The halves stay packed: the multiply-adds convert their fp16 operands on the way in (v_fma_mix_f32).
        Half8Bits qreg[RT][2];
        float acc[RT][16];
        float m[RT], l[RT];
#pragma unroll
        for (int r = 0; r < RT; r++) {
            m[r] = kNegBig;
            l[r] = 0.0f;
            const half_t* qh = a.q + (long long)g * a.q_stride + (long long)(head0 + r) * kHeadDim + 8 * c;
#pragma unroll
            for (int j = 0; j < 2; j++) qreg[r][j].u = *reinterpret_cast<const uint32x4_t*>(qh + 64 * j);
#pragma unroll
            for (int e = 0; e < 16; e++) acc[r][e] = 0.0f;
        }
        // one token of the lane's head: its 16 K values and 16 V values
        auto token = [&](const Half8Bits* kv, const Half8Bits* vv) {
#pragma unroll
            for (int r = 0; r < RT; r++) {
                float dot = 0.0f;             // two products per instruction, summed in fp32 (v_dot2_f32_f16)
#pragma unroll
                for (int e = 0; e < 8; e++) dot = __builtin_amdgcn_fdot2(qreg[r][e / 4].p[e % 4], kv[e / 4].p[e % 4], dot, false);
                const float sc = sum_8_lanes(dot) * scale;
                if (sc > m[r]) {                // rare after the first tokens
                    const float alpha = __expf(m[r] - sc);
                    l[r] *= alpha;
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[r][e] *= alpha;
                    m[r] = sc;
                }
                const float p = __expf(sc - m[r]);
                l[r] += p;
#pragma unroll
                for (int e = 0; e < 16; e++) acc[r][e] = __builtin_fmaf(p, (float)vv[e / 8].h[e % 8], acc[r][e]);
            }
        };

        // the next token's rows are requested before this one's arithmetic: two rows (8 KB) per wave in flight
        for (int t = t0 + wave; t < t_end; t += kRowWaves) {    // uniform for the wave
            Half8Bits kw_next[2] = {}, vw_next[2] = {};
            issue_row(krs, a.k, t + kRowWaves, kw_next);
            issue_row(vrs, a.v, t + kRowWaves, vw_next);
            token(kw, vw);
#pragma unroll
            for (int j = 0; j < 2; j++) { kw[j] = kw_next[j]; vw[j] = vw_next[j]; }
        }
        if (APPEND && t0 <= n - 1 && n - 1 < t1 && ((n - 1 - t0) & (kRowWaves - 1)) == wave) {
            const half_t* k_fresh = a.k_new + (long long)g * a.kv_new_stride + (long long)h * kHeadDim + 8 * c;
            const half_t* v_fresh = a.v_new + (long long)g * a.kv_new_stride + (long long)h * kHeadDim + 8 * c;
#pragma unroll
            for (int j = 0; j < 2; j++) {
                kw[j].u = *reinterpret_cast<const uint32x4_t*>(k_fresh + 64 * j);
                vw[j].u = *reinterpret_cast<const uint32x4_t*>(v_fresh + 64 * j);
            }
            token(kw, vw);
        }

        // ---- merge the eight waves' streams: common maximum per (head, r), then sums in a fixed order
        if (c == 0) {
#pragma unroll
            for (int r = 0; r < RT; r++) m_s[wave][r][hd] = m[r];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < RT; r++) {
            float mg = m_s[0][r][hd];
#pragma unroll
            for (int w = 1; w < kRowWaves; w++) mg = fmaxf(mg, m_s[w][r][hd]);
            const float f = __expf(m[r] - mg);      // a wave that saw no token: exp(-1e30 - mg) = 0
            m[r] = mg;
            l[r] *= f;
#pragma unroll
            for (int e = 0; e < 16; e++) acc[r][e] *= f;
        }
        // waves src..src+cnt-1 hand their sums to waves dst..dst+cnt-1: (4,5 -> 0,1) (6,7 -> 2,3) (2,3 -> 0,1) (1 -> 0);
        // the barrier that ends a round also frees m_s and the slots for the next piece
        auto hand_over = [&](int src, int dst, int cnt) {
            if (wave >= src && wave < src + cnt) {
#pragma unroll
                for (int r = 0; r < RT; r++) {
#pragma unroll
                    for (int e = 0; e < 16; e++) red_s[wave - src][r][e][lane] = acc[r][e];
                    l_s[wave - src][r][lane] = l[r];
                }
            }
            __syncthreads();
            if (wave >= dst && wave < dst + cnt) {
#pragma unroll
                for (int r = 0; r < RT; r++) {
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[r][e] += red_s[wave - dst][r][e][lane];
                    l[r] += l_s[wave - dst][r][lane];
                }
            }
            __syncthreads();
        };
        hand_over(4, 0, 2);
        hand_over(6, 2, 2);
        hand_over(2, 0, 2);
        hand_over(1, 0, 1);
        if (wave != 0) continue;

        const bool partials = a.nsplit > 1 || a.force_merge;
#pragma unroll
        for (int r = 0; r < RT; r++) {
            if (partials) {
                float* base = a.ws + ((long long)g * a.num_heads + head0 + r) * a.ws_stride;
                float* part = base + (long long)chunk * kPartialFloats;
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    float4 lo = {acc[r][8 * j + 0], acc[r][8 * j + 1], acc[r][8 * j + 2], acc[r][8 * j + 3]};
                    float4 hi = {acc[r][8 * j + 4], acc[r][8 * j + 5], acc[r][8 * j + 6], acc[r][8 * j + 7]};
                    *reinterpret_cast<float4*>(part + 64 * j + 8 * c) = lo;
                    *reinterpret_cast<float4*>(part + 64 * j + 8 * c + 4) = hi;
                }
                if (c == 0) {
                    part[kHeadDim] = m[r];
                    part[kHeadDim + 1] = l[r];
                    // whoever holds the sequence's first token tells the merge how many partials there are (0: even chunks)
                    if (t0 == 0) reinterpret_cast<int*>(base)[kHeadDim + 2] = balanced ? nseg : 0;
                }
            } else {
                const float inv = 1.0f / (l[r] + 1e-8f);                 // kernels.cu:1746
                const long long o = (long long)(head0 + r) * kHeadDim + 8 * c;
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    half8_t o8;
#pragma unroll
                    for (int i = 0; i < 8; i++) o8[i] = (half_t)(acc[r][8 * j + i] * inv);
                    if (a.gate) {
                        half8_t g8 = *reinterpret_cast<const half8_t*>(a.gate + (long long)g * a.gate_stride + o + 64 * j);
#pragma unroll
                        for (int i = 0; i < 8; i++) o8[i] = gated(o8[i], g8[i]);
                    }
                    *reinterpret_cast<half8_t*>(a.out + (long long)g * a.q_stride + o + 64 * j) = o8;
                }
            }
        }
    }
}

// Log-sum-exp merge of the split partials, normalisation, rotate-back, store.  Thread c first takes partial c's
// maximum and sum (at most kMergeSlots partials), so that the weights of all partials are known after one round trip
// to memory; the sums over the partials then run over loads that do not depend on each other.
constexpr int kMergeSlots = 64;
__global__ void __launch_bounds__(kHeadDim)
attention_merge_kernel(AttnArgs a) {
    __shared__ float o_s[kHeadDim];
    __shared__ float w_s[kMergeSlots];
    __shared__ float red_s[2][2];
    const int head = blockIdx.x, g = blockIdx.y, d = threadIdx.x;
    const int n = seq_pos(a, g) + 1;
    const float* part = a.ws + ((long long)g * a.num_heads + head) * a.ws_stride;
    // which slots were written: the first nseg (balanced walk) or the non-empty even chunks
    const int nseg = a.slots_from_ws ? reinterpret_cast<const int*>(part)[kHeadDim + 2] : 0;
    auto live = [&](int c) -> bool {
        if (nseg > 0) return c < nseg;
        return a.even_chunks ? even_chunk_nonempty(n, c, a.nsplit) : chunk_nonempty(n, c, a.nsplit);
    };
    const int nslots = min(nseg > 0 ? nseg : a.nsplit, kMergeSlots);
    const bool mine = d < nslots && live(d);                // no workgroup wrote the other slots
    float m_c = kNegBig, l_c = 0.0f;
    if (mine) {
        m_c = part[(long long)d * kPartialFloats + kHeadDim];
        l_c = part[(long long)d * kPartialFloats + kHeadDim + 1];
    }
    const float mw = wave_max(m_c);
    if ((d & 63) == 0) red_s[0][d >> 6] = mw;
    __syncthreads();
    const float mg = fmaxf(red_s[0][0], red_s[0][1]);
    const float w = mine ? (a.m_log2 ? __builtin_amdgcn_exp2f(m_c - mg) : __expf(m_c - mg)) : 0.0f;
    if (d < kMergeSlots) w_s[d] = w;
    const float lw = wave_sum(l_c * w);
    if ((d & 63) == 0) red_s[1][d >> 6] = lw;
    __syncthreads();
    const float lsum = red_s[1][0] + red_s[1][1];
    float av = 0.0f;
#pragma unroll 8
    for (int cidx = 0; cidx < nslots; cidx++) {
        const float wc = w_s[cidx];
        const float v = part[(long long)cidx * kPartialFloats + d];     // a slot nobody wrote: inside the block, not used
        av = wc != 0.0f ? __builtin_fmaf(v, wc, av) : av;
    }
    o_s[d] = av * (1.0f / (lsum + 1e-8f));
    __syncthreads();
    store_head(a, g, head, d, o_s);
}

template <int MODE>
static void launch_valu_mode(const AttnArgs& a, hipStream_t s) {
    const int group = a.num_heads / a.num_kv_heads;
    const int rt = (group % 4 == 0) ? 4 : (group % 2 == 0) ? 2 : 1;
    dim3 grid(a.nsplit, a.num_kv_heads * (group / rt), a.G);
    dim3 block(kAttnThreads);
    if (MODE == 0 && a.k_new) {
        if (rt == 4) launch_scan_kernel(attention_valu_kernel<0, 4, true>, grid, block, s, a);
        else if (rt == 2) launch_scan_kernel(attention_valu_kernel<0, 2, true>, grid, block, s, a);
        else launch_scan_kernel(attention_valu_kernel<0, 1, true>, grid, block, s, a);
        return;
    }
    if (rt == 4) launch_scan_kernel(attention_valu_kernel<MODE, 4, false>, grid, block, s, a);
    else if (rt == 2) launch_scan_kernel(attention_valu_kernel<MODE, 2, false>, grid, block, s, a);
    else launch_scan_kernel(attention_valu_kernel<MODE, 1, false>, grid, block, s, a);
}

// The whole-row kernel: fp16 cache, KV heads in blocks of eight, 16-byte aligned rows.  (Whether the batch is large
// enough for it is the split planner's question: it knows the bound of the context.)
bool attention_rows_usable(const AttnArgs& a) {
    if (a.bits != 0 || a.num_kv_heads <= 0 || a.num_kv_heads % kRowHeads != 0 || attention_variant() == 3) return false;
    auto al = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    if (!al(a.k) || !al(a.v) || !al(a.q) || !al(a.out) || (a.q_stride & 7) != 0) return false;
    if (a.gate && (!al(a.gate) || (a.gate_stride & 7) != 0)) return false;
    if (a.k_new && (!al(a.k_new) || !al(a.v_new) || (a.kv_new_stride & 7) != 0)) return false;
    if (a.ws && !al(a.ws)) return false;                         // 16-byte stores of the partials
    return true;
}

// blocks of 8 KV heads times tiles of query heads: the workgroups one chunk of one sequence takes
int attention_rows_groups(const AttnArgs& a) {
    const int group = a.num_heads / a.num_kv_heads;
    const int rt = (group % 4 == 0) ? 4 : (group % 2 == 0) ? 2 : 1;
    return (a.num_kv_heads / kRowHeads) * (group / rt);
}

// the balanced walk is for batches whose KV heads and query heads one workgroup covers
bool attention_rows_balances(const AttnArgs& a) {
    return attention_rows_groups(a) == 1 && a.G > 1 && a.G <= kMaxBalanceSeqs && a.ws && a.max_slots >= 3 &&
           (reinterpret_cast<uintptr_t>(a.ws) & 15u) == 0 && (a.ws_stride & 3) == 0;
}

static void launch_attention_rows(const AttnArgs& a, hipStream_t s) {
    const int group = a.num_heads / a.num_kv_heads;
    const int rt = (group % 4 == 0) ? 4 : (group % 2 == 0) ? 2 : 1;
    const int hgroups = attention_rows_groups(a);
    const long long items = (long long)a.G * a.nsplit * hgroups;
    const int grid = (int)std::min<long long>(items, (rt == 4 ? 1LL : 2LL) * compute_units());
    const dim3 g3(grid), b3(kRowThreads);
    // contiguous cache whose rows of one sequence stay below 2 GB: buffer loads with 32-bit offsets
    const long long seq_rows = a.seq_stride_rows > 0 ? a.seq_stride_rows
                               : a.pos_mode == kPosScalar ? (long long)a.pos_scalar + 1
                               : a.pos_mode == kPosIota ? (long long)a.G : (1LL << 40);
    const bool desc = !a.block_table && seq_rows * a.num_kv_heads * kHeadDim * 2 < (1LL << 31);
    note_scan_kernel("attention_rows_kernel");
#define TW_ROWS_D(RT_, AP_, D_) launch_scan_kernel(attention_rows_kernel<RT_, AP_, D_>, g3, b3, s, a, (int)items, hgroups)
#define TW_ROWS(RT_)                                                                                          \
    if (a.k_new) { if (desc) TW_ROWS_D(RT_, true, true); else TW_ROWS_D(RT_, true, false); }                  \
    else { if (desc) TW_ROWS_D(RT_, false, true); else TW_ROWS_D(RT_, false, false); }
    if (rt == 4) { TW_ROWS(4); }
    else if (rt == 2) { TW_ROWS(2); }
    else { TW_ROWS(1); }
#undef TW_ROWS
#undef TW_ROWS_D
}

void launch_attention_valu(const AttnArgs& a, hipStream_t s) {
    if (a.G <= 0) return;
    if (a.even_chunks) { launch_attention_rows(a, s); return; }     // the split planner chose the whole-row kernel
    note_scan_kernel("attention_valu_kernel");
    if (a.bits == 0) launch_valu_mode<0>(a, s);
    else if (a.bits == 4) launch_valu_mode<4>(a, s);
    else launch_valu_mode<2>(a, s);
}

void launch_attention_merge(const AttnArgs& a, hipStream_t s) {
    if (a.G <= 0 || (a.nsplit <= 1 && !a.force_merge)) return;
    hipLaunchKernelGGL(attention_merge_kernel, dim3(a.num_heads, a.G), dim3(kHeadDim), 0, s, a);
}

}  // namespace twkv
