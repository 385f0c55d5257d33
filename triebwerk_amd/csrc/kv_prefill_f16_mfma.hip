// kv_prefill_f16_mfma.hip -- causal prefill attention over the fp16 cache on the matrix cores (gfx950).
//
// Replaces gqa_prefill_attention_kernel (kernels.cu:1071-1158): query token t of every head attends
// cache rows 0..t of its KV head, out = softmax(q.K^T / sqrt(128)) V with the reference's
// `+ 1e-8` in the normalisation.  This is the one GEMM-shaped piece of the path, so both
// contractions run as v_mfma_f32_16x16x32_f16 with fp32 accumulation:
//
//   S^T[kv token][query] = K . Q^T   A = K rows from LDS, B = Q rows (registers, loaded once)
//   O[query][dim]       += P . V     A = P (the lane's own S^T values, no transposition),
//                                    B = V^T from LDS
//
// Computing S transposed leaves lane (query n, kg) with the scores of kv tokens 4kg..4kg+3 of both
// 16-token halves of a tile: exactly the 8 contraction slots the A operand of the second MFMA
// wants from that lane, once V^T is stored with its 32 token columns in the matching order
// (slot 8kg + 4s + i <-> token 16s + 4kg + i).  Softmax is online, base 2, with the running
// maximum raised only when a score exceeds it by 2^5 (then the accumulators are rescaled), so in
// the steady state a tile costs 16 MFMAs, 8 exponentials per lane and no shuffles.
//
// A workgroup of 4 waves takes one KV head and 64 NQ / R query tokens (R = GQA group: wave w serves
// query head w % R and 16 NQ tokens; with NQ = 2 the two 16-row blocks share every operand read),
// walks the kv tiles of 32 tokens up to its diagonal and shares each tile through LDS: K row-major
// (padded rows), V transposed on the way in (each thread interleaves the same 8 dims of two
// consecutive tokens and writes 8 dwords).  The loop is a pipeline, one barrier per tile, a tile
// taking five steps through it: global loads issued; written to LDS; K operands read into registers; score
// MFMAs (with the previous tile's exponentials between them) and maxima; exponentials and P.V MFMAs (with the
// next tile's maxima between them).  Two K buffers, four V buffers; the loop says which step does what.  For long prompts a workgroup does a token block and then its
// mirror image from the other end of the sequence, so causal rows cost every workgroup the same; short
// prompts take one block each, longest first.  The workgroups of a KV head run on one XCD, so the head's
// rows come out of one L2.

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"


namespace twkv {

namespace {

constexpr int kPfKRow = 2 * kHeadDim + 32;   // bytes per K row in LDS: with 288 the operand reads (16 rows x 4 column groups of 16 bytes) run at the LDS's full rate, with 272 at 53 % of it (measured)
constexpr int kPfVRow = 2 * 32 + 32;         // bytes per V^T row (32 token slots) in LDS: 96 at the full rate, 80 at 54 %

template <bool B> struct Flag { static constexpr bool value = B; };

// column of a tile's token in the V^T rows: the contraction slot order of the second MFMA
__device__ __forceinline__ int vt_slot(int token) { return 8 * ((token & 15) >> 2) + 4 * (token >> 4) + (token & 3); }

}  // namespace

// NQ: 16-row query blocks per wave (every K and V operand read feeds NQ MFMAs).  MIRROR: a workgroup does a
// token block and then its mirror image from the other end of the sequence.
// W: waves per workgroup, 4 (two workgroups per CU) or 8 (one: a tile is brought into LDS once for twice the queries).
template <int R, int NQ, bool MIRROR, int W>
__global__ void __launch_bounds__(W* kWave, W == 4 ? 2 : 1)  // two waves per SIMD either way (three would spill)
prefill_f16_mfma_kernel(AttnArgs a, int T) {
    static_assert(W == 4 || W == 8, "the staging maps are written for 256 and 512 threads");
    constexpr int TPW = 16 * NQ * W / R;                   // query tokens per workgroup pass
    __shared__ __attribute__((aligned(16))) char k_s[2][32 * kPfKRow];
    __shared__ __attribute__((aligned(16))) char v_s[4][kHeadDim * kPfVRow];

    const int tid = threadIdx.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;
    const int ln = lane & 15, kg = lane >> 4;
    const int nblk = (T + TPW - 1) / TPW;
    // Workgroups are dealt to the 8 XCDs in turn (linear id % 8), each with an L2 of its own.  The workgroups of a
    // KV head all walk the same K and V rows, so a head's workgroups go to one XCD (8, 16, ... heads) or to 8 / heads
    // of them (1, 2, 4 heads), and its rows are fetched from memory into one L2 instead of eight.
    int blk = blockIdx.x, kvh = blockIdx.y;
    {
        const int nbx = gridDim.x, nh = gridDim.y;
        const int lin = blockIdx.x + nbx * blockIdx.y, xcd = lin & 7, slot = lin >> 3;
        if ((nh & 7) == 0) {
            kvh = xcd + 8 * (slot / nbx); blk = slot % nbx;
        } else if ((nh == 1 || nh == 2 || nh == 4) && nbx % (8 / nh) == 0) {
            const int per = 8 / nh;                      // XCDs per head
            kvh = xcd % nh; blk = slot * per + xcd / nh;
        }
    }
    const int head = kvh * R + wave % R;
    const int kv_dim = a.num_kv_heads * kHeadDim;
    const half_t* kbase = reinterpret_cast<const half_t*>(a.k) + (long long)kvh * kHeadDim;
    const half_t* vbase = reinterpret_cast<const half_t*>(a.v) + (long long)kvh * kHeadDim;
    const float scale2 = kLog2e * kInvSqrtD;
    constexpr float kRaise = 5.0f;

    // ---- staging of a tile: thread (r = tid / 16, c = tid % 16) carries 16 bytes (dims 8c..8c+7) of
    // K rows r and r + 16 (512 threads: of row r alone); for V, thread (c = tid / 16, r = tid % 16) carries dims
    // 8c..8c+7 (512 threads: 4c..4c+3) of rows 2r and 2r + 1 (two consecutive tokens, interleaved on the way into the
    // transposed tile).
    const int sr = tid >> 4, sc = tid & 15;
    // V: 16 consecutive threads take the 16 token pairs of one dim octet, so that their dwords fill one V^T row
    // (64 contiguous bytes, all banks different); with the K mapping they would hit rows 8 apart, 8 to a bank
    const int vr_ = tid & 15, vc_ = tid >> 4;
    // Buffer loads: descriptor over the T rows of the cache (rows past the last token read as zeros and are
    // masked anyway), per-thread byte offsets fixed for the whole kernel, the tile's row offset in a scalar.
    const __amdgpu_buffer_rsrc_t krs = make_rsrc(reinterpret_cast<const char*>(kbase), T * kv_dim * 2 - kvh * kHeadDim * 2);
    const __amdgpu_buffer_rsrc_t vrs = make_rsrc(reinterpret_cast<const char*>(vbase), T * kv_dim * 2 - kvh * kHeadDim * 2);
    const int koff0 = (sr * kv_dim + 8 * sc) * 2, koff1 = koff0 + 16 * kv_dim * 2;
    const int voff0 = (2 * vr_ * kv_dim + (W == 4 ? 8 : 4) * vc_) * 2, voff1 = voff0 + kv_dim * 2;
    auto load_tile = [&](int tile, uint4 (&kr)[2], uint4 (&vr)[2]) {
        const int toff = tile * kv_dim * 2;
        const uint32x4_t k0 = __builtin_amdgcn_raw_buffer_load_b128(krs, koff0, toff, 0);
        kr[0] = uint4{k0[0], k0[1], k0[2], k0[3]};
        if constexpr (W == 4) {
            const uint32x4_t k1 = __builtin_amdgcn_raw_buffer_load_b128(krs, koff1, toff, 0);
            const uint32x4_t v0 = __builtin_amdgcn_raw_buffer_load_b128(vrs, voff0, toff, 0);
            const uint32x4_t v1 = __builtin_amdgcn_raw_buffer_load_b128(vrs, voff1, toff, 0);
            kr[1] = uint4{k1[0], k1[1], k1[2], k1[3]};
            vr[0] = uint4{v0[0], v0[1], v0[2], v0[3]};
            vr[1] = uint4{v1[0], v1[1], v1[2], v1[3]};
        } else {
            const uint32x2_t v0 = __builtin_amdgcn_raw_buffer_load_b64(vrs, voff0, toff, 0);
            const uint32x2_t v1 = __builtin_amdgcn_raw_buffer_load_b64(vrs, voff1, toff, 0);
            vr[0] = uint4{v0[0], v0[1], 0u, 0u};
            vr[1] = uint4{v1[0], v1[1], 0u, 0u};
        }
    };
    const int vcol = 2 * vt_slot(2 * vr_);                  // byte column of the token pair in a V^T row
    auto stash = [&](int buf, int vbuf, const uint4 (&kr)[2], const uint4 (&vr)[2]) {
        *reinterpret_cast<uint4*>(&k_s[buf][sr * kPfKRow + 16 * sc]) = kr[0];
        if constexpr (W == 4) *reinterpret_cast<uint4*>(&k_s[buf][(sr + 16) * kPfKRow + 16 * sc]) = kr[1];
        const uint32_t va[4] = {vr[0].x, vr[0].y, vr[0].z, vr[0].w};
        const uint32_t vb[4] = {vr[1].x, vr[1].y, vr[1].z, vr[1].w};
        char* dst = &v_s[vbuf][((W == 4 ? 8 : 4) * vc_) * kPfVRow + vcol];
#pragma unroll
        for (int i = 0; i < (W == 4 ? 4 : 2); i++) {       // dims 8c + 2i (low halves) and 8c + 2i + 1 (high halves); 512 threads: 4c + ...
            *reinterpret_cast<uint32_t*>(dst + (2 * i) * kPfVRow) = __builtin_amdgcn_perm(vb[i], va[i], 0x05040100u);
            *reinterpret_cast<uint32_t*>(dst + (2 * i + 1) * kPfVRow) = __builtin_amdgcn_perm(vb[i], va[i], 0x07060302u);
        }
    };

    // A workgroup takes token block blockIdx.x and its mirror image from the other end, one after the
    // other: with causal rows the two together cost the same for every workgroup.
    const int first = blk, second = nblk - 1 - blk;   // without MIRROR: longest blocks first
    for (int pass = 0; pass < (MIRROR ? 2 : 1); pass++) {
        if (pass == 1 && second == first) break;           // the middle block of an odd count
        const int tb = pass == 0 ? second : first;         // the long one first
        const int q0 = tb * TPW + 16 * NQ * (wave / R);    // this wave's 16 NQ query tokens
        const int wg_last = min(T, (tb + 1) * TPW) - 1;    // last query token of the pass
        const int ntiles = (wg_last >> 5) + 1;

        // ---- B operands of the first MFMA: Q[q0 + 16 nq + ln][32j + 8kg .. +7], j = 0..3
        half8_t qb[NQ][4];
#pragma unroll
        for (int nq = 0; nq < NQ; nq++) {
            const half_t* qrow = a.q + (long long)min(q0 + 16 * nq + ln, T - 1) * a.q_stride + (long long)head * kHeadDim + 8 * kg;
#pragma unroll
            for (int j = 0; j < 4; j++) qb[nq][j] = *reinterpret_cast<const half8_t*>(qrow + 32 * j);
        }
        float4_t o[NQ][8];
        float m_run[NQ], l_run[NQ];
#pragma unroll
        for (int nq = 0; nq < NQ; nq++) {
            m_run[nq] = kNegBig; l_run[nq] = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) o[nq][j] = float4_t{0.f, 0.f, 0.f, 0.f};
        }

        // ---- operand reads of a tile from LDS: K rows for the score MFMAs, V^T rows for the P.V MFMAs
        auto read_k = [&](int kbuf, half8_t (&kf)[8]) {
#pragma unroll
            for (int sub = 0; sub < 2; sub++) {
                const char* krow = &k_s[kbuf][(16 * sub + ln) * kPfKRow + 16 * kg];
#pragma unroll
                for (int j = 0; j < 4; j++) kf[4 * sub + j] = *reinterpret_cast<const half8_t*>(krow + 64 * j);
            }
        };
        auto read_v = [&](int vbuf, half8_t (&vf)[8]) {
            const char* vrow = &v_s[vbuf][ln * kPfVRow + 16 * kg];
#pragma unroll
            for (int j = 0; j < 8; j++) vf[j] = *reinterpret_cast<const half8_t*>(vrow + 16 * j * kPfVRow);
        };

        // The loop is a pipeline over tiles, one barrier per tile, in two phases that each pair 16 MFMAs with
        // vector arithmetic that does not depend on them.  Step t
        //   phase 1: score MFMAs of tile t + 1 (K operands read into registers by step t - 1)
        //            with the exponentials of tile t (scores from step t - 1) between them; V^T operands of tile t read;
        //   phase 2: P.V MFMAs of tile t with the maxima of tile t + 1 between them (and, rarely, a rescale after them);
        //            K operands of tile t + 2 read; tile t + 3 handed to LDS (its global loads were issued a step
        //            ago) and tile t + 4 asked for.
        // So no MFMA waits for an LDS read issued just before it, and a wave keeps the matrix cores and the
        // vector ALU busy at once.  Tiles live in LDS from three steps before their P.V product: two K buffers,
        // four V buffers.  Steps whose two tiles lie wholly below the wave's diagonal take a straight-line form;
        // the filling step t = -1 and those on the diagonal the general one.
        __syncthreads();                                   // a previous pass may still be reading its last V tile
        uint4 kr[2], vr[2];
        {
            uint4 kr1[2], vr1[2];                          // tiles 0, 1 and 2 are asked for together: one trip to memory, not three
            load_tile(0, kr, vr);
            if (ntiles > 1) load_tile(32, kr1, vr1);
            stash(0, 0, kr, vr);
            if (ntiles > 2) load_tile(64, kr, vr);
            if (ntiles > 1) stash(1, 1, kr1, vr1);
        }
        __syncthreads();
        half8_t kf[8];
        read_k(0, kf);
        __syncthreads();                                   // the first step overwrites the K buffer just read

        float x[NQ][8];                                    // raw scores of the tile whose exponentials come next
        bool have_x = false;
        const int n_below = q0 < T ? (q0 + 1) >> 5 : 0;    // tiles wholly below this wave's diagonal

        auto step = [&](auto steady_c, int t) {
            constexpr bool STEADY = decltype(steady_c)::value;
            const int tile1 = 32 * (t + 1);                // first token of tile t + 1
            const bool do_s = STEADY || (t + 1 < ntiles && tile1 <= q0 + 16 * NQ - 1 && q0 < T);   // tile t + 1 reaches this wave's queries
            const bool do_p = STEADY || have_x;
            // ---- phase 1 (the wave's priority falls through the step: of the two waves of a SIMD the one in its score
            // MFMAs goes first, 4 % at 8192 and 16384 tokens, whichever of the orders 1-0-0, 2-1-0, 3-1-0, 3-0-0)
            __builtin_amdgcn_s_setprio(2);
            half8_t vf[8];
            if (do_p) read_v(t & 3, vf);
            float4_t s[NQ][2];
            if (do_s) {
                // S^T[kv][query] for both 16-token halves and all query blocks
#pragma unroll
                for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                    for (int nq = 0; nq < NQ; nq++) s[nq][sub] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
#pragma unroll
                        for (int nq = 0; nq < NQ; nq++)
                            s[nq][sub] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[4 * sub + j], qb[nq][j], s[nq][sub], 0, 0, 0);
                    }
                }
            }
            half8_t pa[NQ];
            if (do_p) {
#pragma unroll
                for (int nq = 0; nq < NQ; nq++) {
                    half8_t pn;
#pragma unroll
                    for (int i = 0; i < 8; i++) pn[i] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf(x[nq][i], scale2, -m_run[nq]));
                    // the sum runs over the rounded values the matrix cores will see, two per instruction
                    const half2_t one2 = {(half_t)1.0f, (half_t)1.0f};
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        l_run[nq] = __builtin_amdgcn_fdot2(half2_t{pn[2 * i], pn[2 * i + 1]}, one2, l_run[nq], false);
                    pa[nq] = pn;
                }
            }
            if (STEADY) {
#pragma unroll
                for (int g = 0; g < 16; g++) {             // 16 MFMAs, 16 fma + 16 exp + 8 cvt + 8 dot2 between them
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                }
            }
            __builtin_amdgcn_s_setprio(1);
            // ---- phase 2: O[query][dim 16j + ln] += P . V of tile t
            if (do_p) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
#pragma unroll
                    for (int nq = 0; nq < NQ; nq++) o[nq][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa[nq], vf[j], o[nq][j], 0, 0, 0);
                }
            }
            if (STEADY || t + 2 < ntiles) read_k(t & 1, kf);                           // tile t + 2
            if (STEADY || t + 3 < ntiles) stash((t + 1) & 1, (t + 3) & 3, kr, vr);      // tile t + 3
            if (STEADY || t + 4 < ntiles) load_tile(32 * (t + 4), kr, vr);              // STEADY: rows past the cache read as zeros
            if (do_s) {
                // maxima of tile t + 1 per query: this lane holds kv tokens tile1 + 16 sub + 4kg + i
#pragma unroll
                for (int nq = 0; nq < NQ; nq++) {
                    const int tq = q0 + 16 * nq + ln;
#pragma unroll
                    for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                        for (int i = 0; i < 4; i++) x[nq][4 * sub + i] = s[nq][sub][i];     // raw: the scale goes into the exponent's fma
                    }
                    if (!STEADY && tile1 + 31 > q0 + 16 * nq) {   // the tile crosses this block's diagonal (uniform over the wave)
#pragma unroll
                        for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                if (tile1 + 16 * sub + 4 * kg + i > tq) x[nq][4 * sub + i] = kNegBig;
                            }
                        }
                    }
                    float mx = x[nq][0];
#pragma unroll
                    for (int i = 1; i < 8; i++) mx = fmaxf(mx, x[nq][i]);
                    mx *= scale2;
                    if (__any(mx > m_run[nq] + kRaise)) {  // rare after the first tiles
                        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));    // the query's maximum over the tile
                        const float m_new = fmaxf(m_run[nq], mx);
                        const float alpha = __builtin_amdgcn_exp2f(m_run[nq] - m_new);
                        m_run[nq] = m_new;
                        l_run[nq] *= alpha;
#pragma unroll
                        for (int i = 0; i < 4; i++) {      // accumulator register i belongs to query 4kg + i
                            const float ai = __shfl(alpha, 4 * kg + i, 64);
#pragma unroll
                            for (int j = 0; j < 8; j++) o[nq][j][i] *= ai;
                        }
                    }
                }
            }
            have_x = do_s;
            __builtin_amdgcn_s_setprio(0);
            __syncthreads();
        };
        step(Flag<false>{}, -1);
        int t = 0;
        const int n_steady = min(n_below - 1, ntiles - 3);      // steps with tiles t and t + 1 below the diagonal and tile t + 3 in range
#pragma clang loop unroll(disable)
        for (; t < n_steady; t++) step(Flag<true>{}, t);
#pragma clang loop unroll(disable)
        for (; t < ntiles; t++) step(Flag<false>{}, t);

        // ---- normalise (kernels.cu:1146: 1 / (sum + 1e-8)) and store; accumulator register i is query 4kg + i
#pragma unroll
        for (int nq = 0; nq < NQ; nq++) {
            float l = l_run[nq];
            l += __shfl_xor(l, 16, 64);
            l += __shfl_xor(l, 32, 64);
            const float inv = 1.0f / (l + 1e-8f);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float inv_i = __shfl(inv, 4 * kg + i, 64);
                const int t = q0 + 16 * nq + 4 * kg + i;
                if (t < T) {
                    const long long col = (long long)head * kHeadDim + ln;
                    half_t* orow = a.out + (long long)t * a.q_stride + col;
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        half_t h = (half_t)(o[nq][j][i] * inv_i);
                        if (a.gate) h = gated(h, a.gate[(long long)t * a.gate_stride + col + 16 * j]);
                        orow[16 * j] = h;
                    }
                }
            }
        }
    }
}

// fp16 cache, one sequence, query t attends rows 0..t, GQA group 1, 2 or 4, 16-byte aligned rows
bool prefill_f16_mfma_usable(const AttnArgs& a) {
    const int R = a.num_heads / a.num_kv_heads;
    if (a.bits != 0 || a.pos_mode != kPosIota || a.block_table || a.seq_stride_rows != 0) return false;
    if (R != 1 && R != 2 && R != 4) return false;
    if ((a.q_stride & 7) != 0) return false;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a.q) | reinterpret_cast<uintptr_t>(a.k) | reinterpret_cast<uintptr_t>(a.v);
    const long long cache_bytes = (long long)a.G * a.num_kv_heads * kHeadDim * 2;     // one buffer descriptor spans it
    return (bits & 15u) == 0 && a.G >= 1 && cache_bytes < (1LL << 31);
}

void launch_prefill_f16_mfma(const AttnArgs& a, hipStream_t s, int form) {
    const int R = a.num_heads / a.num_kv_heads;
    const int T = a.G;
    // Long prompts: eight waves per workgroup, two query blocks per wave and mirrored block pairs (a tile is brought
    // into LDS once for 256 query rows, every operand read feeds two MFMAs, equal work per workgroup).  Shorter ones
    // do not fill the GPU that way and take one query block per wave, then four waves, then unpaired workgroups.
    // Measured with 16 heads over 8 KV heads: the eight-wave forms win from three workgroups per four CUs upwards
    // (6144 tokens: 0.196 against 0.203 ms; 4096: 0.090 against 0.098; 3072: 0.065 against 0.072; at one per two CUs
    // they lose, 2048 tokens: 0.047 against 0.038), the four-wave ones from one per CU.
    const int cus = compute_units();
    auto pairs = [&](int waves, int nq) { const int tpw = 16 * nq * waves / R; return ((T + tpw - 1) / tpw + 1) / 2 * a.num_kv_heads; };
    int mode = 1;
    if (4 * pairs(8, 2) >= 3 * cus) mode = 6;
    else if (4 * pairs(8, 1) >= 3 * cus) mode = 5;
    else if (pairs(4, 1) >= cus) mode = 2;
    if ((form >= 1 && form <= 3) || form == 5 || form == 6) mode = form;    // forced by a test (4 is the compressed cache's other kernel)
    const int waves = mode >= 5 ? 8 : 4;
    const int nq = (mode == 3 || mode == 6) ? 2 : 1;
    const bool mirror = mode != 1;
    const int tpw = 16 * nq * waves / R;
    const int nblk = (T + tpw - 1) / tpw;
    const dim3 grid(mirror ? (nblk + 1) / 2 : nblk, a.num_kv_heads), block(waves * kWave);
    note_scan_kernel("prefill_f16_mfma_kernel");
#define TW_PF_LAUNCH(RR, NN, MM, WW) launch_scan_kernel(prefill_f16_mfma_kernel<RR, NN, MM, WW>, grid, block, s, a, T)
#define TW_PF_MODES(RR) \
    do { if (mode == 1) TW_PF_LAUNCH(RR, 1, false, 4); else if (mode == 2) TW_PF_LAUNCH(RR, 1, true, 4); \
         else if (mode == 3) TW_PF_LAUNCH(RR, 2, true, 4); else if (mode == 5) TW_PF_LAUNCH(RR, 1, true, 8); \
         else TW_PF_LAUNCH(RR, 2, true, 8); } while (0)
    if (R == 1) TW_PF_MODES(1); else if (R == 2) TW_PF_MODES(2); else TW_PF_MODES(4);
#undef TW_PF_MODES
#undef TW_PF_LAUNCH
}

}  // namespace twkv
