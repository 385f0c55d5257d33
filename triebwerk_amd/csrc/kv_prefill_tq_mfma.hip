// kv_prefill_tq_mfma.hip -- causal prefill attention over the TurboQuant-compressed cache on the matrix cores
// (gfx950), for prompts: the flash-attention kernel of kv_prefill_f16_mfma.hip (which documents the MFMA
// tiling, the transposed scores and the softmax) with one difference: a tile of K and V codes is expanded
// to fp16 centroids ONCE per workgroup on its way into LDS, instead of once per wave as in the decode
// scan's layout.  64 NQ / R query tokens of R heads then reuse it.
//
// Arithmetic (turbo_gqa_prefill_attention_kernel, kernels.cu:1874-1960, in the rotated space):
//   score[kv][q] = (sum_d c(K code[kv][d]) q_rot[q][d]) * k_norm[kv]          (kernels.cu:1707)
//   acc[q][d]   += (p * v_norm[kv]) * c(V code[kv][d])                        (kernels.cu:1765)
// with q_rot = R q pre-scaled by log2(e) / sqrt(128) / alpha (made in the kernel), centroids stored as
// fp16(alpha c) (alpha as in the decode scan: all magnitudes round with <= 1.1e-4 relative error), the
// norms applied in fp32.  A workgroup sees the whole context of its query tokens, so it also finishes them:
// normalisation (kernels.cu:1946) and the rotation back out of the rotated space (kernels.cu:1949-1957) on the
// matrix cores, the accumulator split into an fp16 value and its remainder; no partials, no merge launch.
// The accumulators are kept transposed (O^T[dim][query], the operands of the second MFMA swapped), which puts a
// query's running maximum, sum and accumulators in the same lanes and makes O^T the B operand of the rotation.

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_mfma_util.hpp"

namespace twkv {

namespace {

constexpr int kPtKRow = 2 * kHeadDim + 32;   // bytes per expanded K row in LDS (288: operand reads at the LDS's full rate, 272: 53 % of it)
constexpr int kPtVRow = 2 * 32 + 32;         // bytes per V^T row (32 token slots) in LDS (96: full rate, 80: 54 %)
constexpr int kPtVTile = kHeadDim * kPtVRow; // bytes of a V^T tile
constexpr int kPtVBytes = 3 * kPtVTile;      // 3 tiles, and room for the 128 x 128 fp16 rotation
static_assert(kPtVBytes >= 2 * kHeadDim * kHeadDim, "the rotation fits");

// column of a tile's token in the V^T rows: the contraction slot order of the second MFMA
__device__ __forceinline__ int vt_slot(int token) { return 8 * ((token & 15) >> 2) + 4 * (token >> 4) + (token & 3); }

}  // namespace

// NQ: 16-row query blocks per wave (every K and V operand read feeds NQ MFMAs).  MIRROR: a workgroup does a
// token block and then its mirror image from the other end of the sequence.
// W: waves per workgroup, 4 (two workgroups per CU) or 8 (one: a tile is expanded once for twice the queries).
template <int R, int BITS, int NQ, bool MIRROR, int W>
__global__ void __launch_bounds__(W* kWave, W == 4 ? 2 : 1)  // two waves per SIMD either way: at most 256 registers per lane
prefill_tq_mfma_kernel(AttnArgs a, int T) {
    static_assert(W == 4 || W == 8, "the staging maps are written for 256 and 512 threads");
    constexpr int TPW = 16 * NQ * W / R;                   // query tokens per workgroup pass
    constexpr float kAlpha = BITS == 4 ? kAlpha4 : kAlpha2;
    constexpr float kQScale = kLog2e * kInvSqrtD / kAlpha;   // score scale of kernels.cu:1707 in base 2, table scale undone
    constexpr int kHeadBytes = BITS * 16;                  // bytes of one head in a cache row
    constexpr int kEntryDwords = BITS == 4 ? 1 : 2;        // a byte holds 2 (4) codes -> 2 (4) halves
    constexpr int kPtReplicas = BITS == 4 ? 16 : 8;        // copies of the byte -> centroids table (16 KB either way): fewer bank conflicts in the expansion
    __shared__ __attribute__((aligned(16))) char k_s[2][32 * kPtKRow];
    __shared__ __attribute__((aligned(16))) char v_s[kPtVBytes];           // 3 V^T tiles; in the epilogue the rotation
    __shared__ __attribute__((aligned(16))) float n_s[3][2][32];          // [buffer][k | v][token]
    __shared__ __attribute__((aligned(8))) uint32_t tab_s[256 * kPtReplicas * kEntryDwords];

    const int tid = threadIdx.x;
    const int wave = uniform(tid / kWave), lane = tid % kWave;
    const int ln = lane & 15, kg = lane >> 4;
    const int nblk = (T + TPW - 1) / TPW;
    // Workgroups are dealt to the 8 XCDs in turn (linear id % 8), each with an L2 of its own.  The workgroups of a
    // KV head all walk the same rows, so a head's workgroups go to one XCD (8, 16, ... heads) or to 8 / heads of
    // them (1, 2, 4 heads), and its rows are fetched from memory into one L2 instead of eight.
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
    const int row_bytes = a.num_kv_heads * kHeadBytes;
    const char* kbase = reinterpret_cast<const char*>(a.k) + kvh * kHeadBytes;
    const char* vbase = reinterpret_cast<const char*>(a.v) + kvh * kHeadBytes;
    constexpr float kRaise = 5.0f;

    // ---- table: byte -> its codes' centroids (low field first) as fp16(alpha c), kPtReplicas copies
    for (int i = tid; i < 256 * kPtReplicas; i += W * kWave) {
        const int e = i / kPtReplicas;
        if constexpr (BITS == 4) {
            half2_t p = {(half_t)(kAlpha * kCentroids4[e & 15]), (half_t)(kAlpha * kCentroids4[e >> 4])};
            tab_s[i] = *reinterpret_cast<uint32_t*>(&p);
        } else {
            half2_t p0 = {(half_t)(kAlpha * kCentroids2[e & 3]), (half_t)(kAlpha * kCentroids2[(e >> 2) & 3])};
            half2_t p1 = {(half_t)(kAlpha * kCentroids2[(e >> 4) & 3]), (half_t)(kAlpha * kCentroids2[(e >> 6) & 3])};
            tab_s[2 * i] = *reinterpret_cast<uint32_t*>(&p0);
            tab_s[2 * i + 1] = *reinterpret_cast<uint32_t*>(&p1);
        }
    }
    const int rep = lane & (kPtReplicas - 1);
    // the 8 halves (4 dwords) of 8 consecutive coordinates from their packed codes (4 bytes at 4 bit, 2 at 2 bit)
    auto expand8 = [&](uint32_t codes, uint32_t (&out)[4]) {
        if constexpr (BITS == 4) {
#pragma unroll
            for (int b = 0; b < 4; b++) out[b] = tab_s[((codes >> (8 * b)) & 255u) * kPtReplicas + rep];
        } else {
#pragma unroll
            for (int b = 0; b < 2; b++) {
                const uint2 v = *reinterpret_cast<const uint2*>(&tab_s[2 * (((codes >> (8 * b)) & 255u) * kPtReplicas + rep)]);
                out[2 * b] = v.x; out[2 * b + 1] = v.y;
            }
        }
    };

    // the 4 halves (2 dwords) of 4 consecutive coordinates (2 bytes of codes at 4 bit, 1 at 2 bit)
    auto expand4 = [&](uint32_t codes, uint32_t (&out)[4]) {
        if constexpr (BITS == 4) {
#pragma unroll
            for (int b = 0; b < 2; b++) out[b] = tab_s[((codes >> (8 * b)) & 255u) * kPtReplicas + rep];
        } else {
            const uint2 v = *reinterpret_cast<const uint2*>(&tab_s[2 * ((codes & 255u) * kPtReplicas + rep)]);
            out[0] = v.x; out[1] = v.y;
        }
        out[2] = 0u; out[3] = 0u;
    };

    // ---- staging of a tile: thread (r = tid / 16, c = tid % 16) carries the codes of coordinates 8c..8c+7 of
    // K rows r and r + 16 (512 threads: of row r alone); for V, thread (c = tid / 16, r = tid % 16) carries those of
    // coordinates 8c..8c+7 (512 threads: 4c..4c+3) of rows 2r and 2r + 1 (two consecutive tokens, interleaved on the
    // way into the transposed tile); threads 0..63 also carry a norm.
    const int sr = tid >> 4, sc = tid & 15;
    // V: 16 consecutive threads take the 16 token pairs of one dim octet, so that their dwords fill one V^T row
    // (64 contiguous bytes, all banks different); with the K mapping they would hit rows 8 apart, 8 to a bank
    const int vr_ = tid & 15, vc_ = tid >> 4;
    constexpr int kPiece = BITS;                           // bytes of codes of 8 coordinates
    struct Staged { uint32_t k[2], v[2], nb; };            // codes, and the fp16 bits of a norm as loaded
    // Buffer loads: descriptors over the T rows of the cache (rows past the last token read as zeros and are
    // masked anyway), per-thread byte offsets fixed for the whole kernel, the tile's row offset in a scalar.
    const __amdgpu_buffer_rsrc_t krs = make_rsrc(kbase, T * row_bytes - kvh * kHeadBytes);
    const __amdgpu_buffer_rsrc_t vrs = make_rsrc(vbase, T * row_bytes - kvh * kHeadBytes);
    const int nrow_bytes = a.num_kv_heads * 2;
    const __amdgpu_buffer_rsrc_t knrs = make_rsrc(reinterpret_cast<const char*>(a.k_norms) + kvh * 2, T * nrow_bytes - kvh * 2);
    const __amdgpu_buffer_rsrc_t vnrs = make_rsrc(reinterpret_cast<const char*>(a.v_norms) + kvh * 2, T * nrow_bytes - kvh * 2);
    const int koff0 = sr * row_bytes + kPiece * sc, koff1 = koff0 + 16 * row_bytes;
    const int voff0 = 2 * vr_ * row_bytes + (W == 4 ? kPiece : kPiece / 2) * vc_, voff1 = voff0 + row_bytes;
    const int noff = (tid & 31) * nrow_bytes;
    const __amdgpu_buffer_rsrc_t nrs = (wave & 1) ? vnrs : knrs;     // wave-uniform: a scalar choice
    auto load_codes = [&](__amdgpu_buffer_rsrc_t rs, int voff, int soff) -> uint32_t {
        if constexpr (BITS == 4) return __builtin_amdgcn_raw_buffer_load_b32(rs, voff, soff, 0);
        else return __builtin_amdgcn_raw_buffer_load_b16(rs, voff, soff, 0);
    };
    auto load_half_codes = [&](__amdgpu_buffer_rsrc_t rs, int voff, int soff) -> uint32_t {     // 4 coordinates
        if constexpr (BITS == 4) return __builtin_amdgcn_raw_buffer_load_b16(rs, voff, soff, 0);
        else return __builtin_amdgcn_raw_buffer_load_b8(rs, voff, soff, 0);
    };
    auto load_tile = [&](int tile, Staged& st) {
        const int toff = tile * row_bytes;
        st.k[0] = load_codes(krs, koff0, toff);
        if constexpr (W == 4) {
            st.k[1] = load_codes(krs, koff1, toff);
            st.v[0] = load_codes(vrs, voff0, toff);
            st.v[1] = load_codes(vrs, voff1, toff);
        } else {
            st.v[0] = load_half_codes(vrs, voff0, toff);
            st.v[1] = load_half_codes(vrs, voff1, toff);
        }
        // Every thread asks for a norm of row tid % 32 -- even waves K's, odd waves V's; lanes 0..31 of waves 0 and 1
        // are the ones that keep it -- and holds the bits as they come: a load under a per-lane condition with a
        // descriptor that depends on the lane becomes a loop over the descriptors, and a value computed from a load
        // at the place of the load is a wait for every load in flight, here the tile that was just asked for.
        st.nb = __builtin_amdgcn_raw_buffer_load_b16(nrs, noff, tile * nrow_bytes, 0);
    };
    const int vcol = 2 * vt_slot(2 * vr_);                  // byte column of the token pair in a V^T row
    auto stash = [&](int buf, int vbuf, const Staged& st) {
        uint32_t e[4];
        expand8(st.k[0], e);
        *reinterpret_cast<uint4*>(&k_s[buf][sr * kPtKRow + 16 * sc]) = uint4{e[0], e[1], e[2], e[3]};
        if constexpr (W == 4) {
            expand8(st.k[1], e);
            *reinterpret_cast<uint4*>(&k_s[buf][(sr + 16) * kPtKRow + 16 * sc]) = uint4{e[0], e[1], e[2], e[3]};
        }
        uint32_t va[4], vb[4];
        if constexpr (W == 4) {
            expand8(st.v[0], va);
            expand8(st.v[1], vb);
        } else {
            expand4(st.v[0], va);
            expand4(st.v[1], vb);
        }
        char* dst = &v_s[vbuf * kPtVTile + ((W == 4 ? 8 : 4) * vc_) * kPtVRow + vcol];
#pragma unroll
        for (int i = 0; i < (W == 4 ? 4 : 2); i++) {       // dims 8c + 2i (low halves) and 8c + 2i + 1 (high halves); 512 threads: 4c + ...
            *reinterpret_cast<uint32_t*>(dst + (2 * i) * kPtVRow) = __builtin_amdgcn_perm(vb[i], va[i], 0x05040100u);
            *reinterpret_cast<uint32_t*>(dst + (2 * i + 1) * kPtVRow) = __builtin_amdgcn_perm(vb[i], va[i], 0x07060302u);
        }
        if (tid < 2 * kWave && (tid & 32) == 0) n_s[vbuf][tid >> 6][tid & 31] = h2f_bits(st.nb);
    };
    __syncthreads();                                       // the table is there

    // A workgroup takes token block blockIdx.x and its mirror image from the other end, one after the
    // other: with causal rows the two together cost the same for every workgroup.
    const int first = blk, second = nblk - 1 - blk;   // without MIRROR: longest blocks first
    for (int pass = 0; pass < (MIRROR ? 2 : 1); pass++) {
        if (pass == 1 && second == first) break;           // the middle block of an odd count
        const int tb = pass == 0 ? second : first;         // the long one first
        const int q0 = tb * TPW + 16 * NQ * (wave / R);    // this wave's 16 NQ query tokens
        const int wg_last = min(T, (tb + 1) * TPW) - 1;    // last query token of the pass
        const int ntiles = (wg_last >> 5) + 1;

        // ---- B operands of the first MFMA: q_rot[q0 + 16 nq + ln][32j + 8kg .. +7], j = 0..3, as an fp16 value
        // and what its rounding left over (scores reach tens of base-2 units on caches with outlier channels,
        // where a 2^-11 relative error of q alone would show in the output).  q_rot = R q (kernels.cu:1671-1681)
        // is made here, on the matrix cores: q_rot^T[d][query] = R[d][.] . q^T, 16 rows d at a time, the rows
        // picked so that the result lands where the operand wants it -- accumulator row 4kg + i of block (j, h)
        // is d = 32j + 8kg + 4h + i.  Both factors are exact in fp16 and the sum is kept in fp32.
        half8_t qb[NQ][4], ql[NQ][4];
        {
            half8_t qv[NQ][4];                             // q[query ln][32t + 8kg .. +7]
#pragma unroll
            for (int nq = 0; nq < NQ; nq++) {
                const half_t* qsrc = a.q + (long long)min(q0 + 16 * nq + ln, T - 1) * a.q_stride + head * kHeadDim + 8 * kg;
#pragma unroll
                for (int t = 0; t < 4; t++) qv[nq][t] = *reinterpret_cast<const half8_t*>(qsrc + 32 * t);
            }
            int rrow = 8 * (ln >> 2) + (ln & 3);           // row of R this lane feeds within a block, less 32j + 4h
            asm volatile("" : "+v"(rrow));                 // per pass: the 32 loads below are not kept across passes
            const half_t* rsrc = a.rotation + rrow * kHeadDim + 8 * kg;
#pragma unroll
            for (int j = 0; j < 4; j++) {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    float4_t y[NQ];
#pragma unroll
                    for (int nq = 0; nq < NQ; nq++) y[nq] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const half8_t ra = *reinterpret_cast<const half8_t*>(rsrc + (32 * j + 4 * h) * kHeadDim + 32 * t);
#pragma unroll
                        for (int nq = 0; nq < NQ; nq++) y[nq] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ra, qv[nq][t], y[nq], 0, 0, 0);
                    }
#pragma unroll
                    for (int nq = 0; nq < NQ; nq++) {
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float x = y[nq][i] * kQScale;
                            const half_t hi = (half_t)x;
                            qb[nq][j][4 * h + i] = hi;
                            ql[nq][j][4 * h + i] = (half_t)(x - (float)hi);
                        }
                    }
                }
            }
        }
        float4_t o[NQ][8];
        float m_run[NQ], l_run[NQ];
#pragma unroll
        for (int nq = 0; nq < NQ; nq++) {
            m_run[nq] = kNegBig; l_run[nq] = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) o[nq][j] = float4_t{0.f, 0.f, 0.f, 0.f};
        }

        // ---- O^T[dim 16j + 4kg + i][query ln] += V^T . P^T for one tile (value and remainder of p * v_norm)
        auto pv = [&](int vbuf, const half8_t (&pa)[NQ], const half8_t (&pl)[NQ]) {
            const char* vrow = &v_s[vbuf * kPtVTile + ln * kPtVRow + 16 * kg];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const half8_t vb = *reinterpret_cast<const half8_t*>(vrow + 16 * j * kPtVRow);
#pragma unroll
                for (int nq = 0; nq < NQ; nq++) {
                    o[nq][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vb, pa[nq], o[nq][j], 0, 0, 0);
                    o[nq][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vb, pl[nq], o[nq][j], 0, 0, 0);
                }
            }
        };

        // The loop is skewed by one tile: scores of tile t, then the P.V product of tile t - 1 (whose MFMAs do not
        // depend on tile t) ahead of the softmax arithmetic of tile t.  Three V (and norm) buffers, two K buffers.
        // (The fp16 kernel's deeper pipeline -- K operands a tile ahead in registers -- needs 64 registers more
        // than the 226 this kernel already uses with its second set of operands.)
        __syncthreads();                                   // a previous pass may still be reading its last V tile
        Staged st;
        load_tile(0, st);
        stash(0, 0, st);
        __syncthreads();

        half8_t pa_prev[NQ], pl_prev[NQ];
        bool have_prev = false;
        for (int it = 0; it < ntiles; it++) {
            const int buf = it & 1, nbuf = it % 3;
            const int tile = 32 * it;
            const bool more = it + 1 < ntiles;
            // the wave's priority falls through the tile (scores 3, P.V 2, softmax 1, hand-over 0): of the two waves of a
            // SIMD the one earlier in its tile goes first; 1.5 % at 8192 tokens, 3 % at 4096
            __builtin_amdgcn_s_setprio(3);
            if (more) load_tile(tile + 32, st);

            const bool active = tile <= q0 + 16 * NQ - 1 && q0 < T;      // the tile reaches this wave's queries (uniform over the wave)
            float4_t s[NQ][2];
            if (active) {
                // ---- S^T[kv][query] for both 16-token halves and all query blocks
#pragma unroll
                for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                    for (int nq = 0; nq < NQ; nq++) s[nq][sub] = float4_t{0.f, 0.f, 0.f, 0.f};
                    const char* krow = &k_s[buf][(16 * sub + ln) * kPtKRow + 16 * kg];
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const half8_t ka = *reinterpret_cast<const half8_t*>(krow + 64 * j);
#pragma unroll
                        for (int nq = 0; nq < NQ; nq++) {
                            s[nq][sub] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qb[nq][j], s[nq][sub], 0, 0, 0);
                            s[nq][sub] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, ql[nq][j], s[nq][sub], 0, 0, 0);
                        }
                    }
                }
            }
            __builtin_amdgcn_s_setprio(2);
            if (have_prev) pv((it + 2) % 3, pa_prev, pl_prev);           // tile it - 1 sits in V buffer (it - 1) % 3
            have_prev = active;
            __builtin_amdgcn_s_setprio(1);
            if (active) {
                // ---- online softmax per query: this lane holds kv tokens tile + 16 sub + 4kg + i
                float kn[8], vn[8];
#pragma unroll
                for (int sub = 0; sub < 2; sub++) {
                    const float4 k4 = *reinterpret_cast<const float4*>(&n_s[nbuf][0][16 * sub + 4 * kg]);
                    const float4 v4 = *reinterpret_cast<const float4*>(&n_s[nbuf][1][16 * sub + 4 * kg]);
                    kn[4 * sub] = k4.x; kn[4 * sub + 1] = k4.y; kn[4 * sub + 2] = k4.z; kn[4 * sub + 3] = k4.w;
                    vn[4 * sub] = v4.x; vn[4 * sub + 1] = v4.y; vn[4 * sub + 2] = v4.z; vn[4 * sub + 3] = v4.w;
                }
#pragma unroll
                for (int nq = 0; nq < NQ; nq++) {
                    const int tq = q0 + 16 * nq + ln;
                    float x[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) x[i] = s[nq][i >> 2][i & 3] * kn[i];              // kernels.cu:1707
                    if (tile + 31 > q0 + 16 * nq) {        // the tile crosses this block's diagonal (uniform over the wave)
#pragma unroll
                        for (int sub = 0; sub < 2; sub++) {
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                if (tile + 16 * sub + 4 * kg + i > tq) x[4 * sub + i] = kNegBig;
                            }
                        }
                    }
                    float mx = x[0];
#pragma unroll
                    for (int i = 1; i < 8; i++) mx = fmaxf(mx, x[i]);
                    if (__any(mx > m_run[nq] + kRaise)) {  // rare after the first tiles
                        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));    // the query's maximum over the tile
                        const float m_new = fmaxf(m_run[nq], mx);
                        const float alpha = __builtin_amdgcn_exp2f(m_run[nq] - m_new);
                        m_run[nq] = m_new;
                        l_run[nq] *= alpha;
#pragma unroll
                        for (int j = 0; j < 8; j++) {      // the lane's accumulators all belong to query ln
#pragma unroll
                            for (int i = 0; i < 4; i++) o[nq][j][i] *= alpha;
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const float p = __builtin_amdgcn_exp2f(x[i] - m_run[nq]);
                        l_run[nq] += p;
                        const float pvn = p * vn[i];                            // (s * vn) * centroid, kernels.cu:1765
                        const half_t hi = (half_t)pvn;
                        pa_prev[nq][i] = hi;
                        pl_prev[nq][i] = (half_t)(pvn - (float)hi);
                    }
                }
            }

            __builtin_amdgcn_s_setprio(0);
            if (more) stash(buf ^ 1, (it + 1) % 3, st);
            __syncthreads();
        }
        if (have_prev) pv((ntiles - 1) % 3, pa_prev, pl_prev);

        // ---- epilogue: out[q][d] = sum_k R[k][d] o[q][k] / (sum + 1e-8) (kernels.cu:1946-1957) as
        // out^T = R^T . O^T.  The rotation goes into the V buffers in operand order: 16-byte entry
        // (db * 4 + t) * 64 + lane holds R[k][16 db + ln] for the 8 k that lane (ln, kg) carries in step t,
        // k = 32t + 16 (e / 4) + 4kg + e % 4 -- the dims its accumulators o[.][2t + e / 4][e % 4] belong to.
        __syncthreads();                                   // every wave is done with the V tiles
        {
            // thread -> rows k = 16r + tid / 16, r = 0..7, columns 8c .. 8c + 7 with c = tid % 16; of k only r is
            // not fixed per thread, and r moves the destination by whole steps t = r / 2 and halves 4 (r % 2)
            const uint4* rsrc = reinterpret_cast<const uint4*>(a.rotation) + tid;
            const int krow = tid >> 4, c = tid & 15;       // 512 threads: rows k = 32r + tid / 16, r = 0..3
            char* dst0 = &v_s[(c >> 1) * 4096 + ((krow >> 2) & 3) * 256 + (c & 1) * 128 + 2 * (krow & 3) + (W == 8 ? 8 * (krow >> 4) : 0)];
#pragma unroll
            for (int r = 0; r < 32 / W; r++) {
                const uint4 rp = rsrc[r * (W * kWave)];
                const uint32_t w[4] = {rp.x, rp.y, rp.z, rp.w};
                const int step = W == 4 ? (r >> 1) * 1024 + (r & 1) * 8 : r * 1024;
#pragma unroll
                for (int x = 0; x < 8; x++)
                    *reinterpret_cast<uint16_t*>(dst0 + step + x * 16) = (uint16_t)(w[x >> 1] >> (16 * (x & 1)));
            }
        }
        __syncthreads();
        half8_t oh[NQ][4], ol[NQ][4];
#pragma unroll
        for (int nq = 0; nq < NQ; nq++) {
            float l = l_run[nq];
            l += __shfl_xor(l, 16, 64);
            l += __shfl_xor(l, 32, 64);
            const float inv = (1.0f / kAlpha) / (l + 1e-8f);
#pragma unroll
            for (int t = 0; t < 4; t++) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float x = o[nq][2 * t + (e >> 2)][e & 3] * inv;
                    const half_t hi = (half_t)x;
                    oh[nq][t][e] = hi;
                    ol[nq][t][e] = (half_t)(x - (float)hi);
                }
            }
        }
#pragma unroll
        for (int db = 0; db < 8; db++) {
            float4_t y[NQ];
#pragma unroll
            for (int nq = 0; nq < NQ; nq++) y[nq] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const half8_t ra = *reinterpret_cast<const half8_t*>(&v_s[((db * 4 + t) * 64 + lane) * 16]);
#pragma unroll
                for (int nq = 0; nq < NQ; nq++) {
                    y[nq] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ra, oh[nq][t], y[nq], 0, 0, 0);
                    y[nq] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ra, ol[nq][t], y[nq], 0, 0, 0);
                }
            }
            // lane holds out[tq][head][16 db + 4kg + i], i = 0..3, of its query token tq
#pragma unroll
            for (int nq = 0; nq < NQ; nq++) {
                const int tq = q0 + 16 * nq + ln;
                if (tq < T) {
                    const long long col = (long long)head * kHeadDim + 16 * db + 4 * kg;
                    half_t h[4] = {(half_t)y[nq][0], (half_t)y[nq][1], (half_t)y[nq][2], (half_t)y[nq][3]};
                    *reinterpret_cast<uint2*>(a.out + (long long)tq * a.q_stride + col) = *reinterpret_cast<const uint2*>(h);
                }
            }
        }
    }
}


// compressed cache, one sequence, query t attends rows 0..t, GQA group 1, 2 or 4
bool prefill_tq_mfma_usable(const AttnArgs& a) {
    const int R = a.num_heads / a.num_kv_heads;
    if ((a.bits != 4 && a.bits != 2) || a.pos_mode != kPosIota || a.block_table || a.seq_stride_rows != 0) return false;
    if (R != 1 && R != 2 && R != 4) return false;
    const long long cache_bytes = (long long)a.G * a.num_kv_heads * a.bits * 16;      // one buffer descriptor spans it
    // q and the rotation are read 16 bytes at a time, out is written 4 halves at a time
    return a.G >= 1 && (reinterpret_cast<uintptr_t>(a.q) & 15u) == 0 && (a.q_stride & 7) == 0 &&
           (reinterpret_cast<uintptr_t>(a.out) & 7u) == 0 && !a.gate &&        // (no caller gates a prompt's output)
           (reinterpret_cast<uintptr_t>(a.rotation) & 15u) == 0 && cache_bytes < (1LL << 31);
}

void launch_prefill_tq_mfma(const AttnArgs& a, hipStream_t s, int form) {
    const int R = a.num_heads / a.num_kv_heads;
    const int T = a.G;
    // forms as for the fp16 prefill kernel: long prompts take eight waves per workgroup, two query blocks per wave and
    // mirrored block pairs; shorter ones one query block per wave, then four waves, then unpaired workgroups
    const int cus = compute_units();
    auto pairs = [&](int waves, int nq) { const int tpw = 16 * nq * waves / R; return ((T + tpw - 1) / tpw + 1) / 2 * a.num_kv_heads; };
    int mode = 1;
    if (4 * pairs(8, 2) >= 3 * cus) mode = 6;
    else if (4 * pairs(8, 1) >= 3 * cus) mode = 5;
    else if (pairs(4, 1) >= cus) mode = 2;
    if ((form >= 1 && form <= 3) || form == 5 || form == 6) mode = form;    // forced by a test
    const int waves = mode >= 5 ? 8 : 4;
    const int nq = (mode == 3 || mode == 6) ? 2 : 1;
    const bool mirror = mode != 1;
    const int tpw = 16 * nq * waves / R;
    const int nblk = (T + tpw - 1) / tpw;
    const dim3 grid(mirror ? (nblk + 1) / 2 : nblk, a.num_kv_heads), block(waves * kWave);
    note_scan_kernel("prefill_tq_mfma_kernel");
#define TW_PT_LAUNCH(RR, BB, NN, MM, WW) launch_scan_kernel(prefill_tq_mfma_kernel<RR, BB, NN, MM, WW>, grid, block, s, a, T)
#define TW_PT_MODES(RR, BB) \
    do { if (mode == 1) TW_PT_LAUNCH(RR, BB, 1, false, 4); else if (mode == 2) TW_PT_LAUNCH(RR, BB, 1, true, 4); \
         else if (mode == 3) TW_PT_LAUNCH(RR, BB, 2, true, 4); else if (mode == 5) TW_PT_LAUNCH(RR, BB, 1, true, 8); \
         else TW_PT_LAUNCH(RR, BB, 2, true, 8); } while (0)
#define TW_PT_BITS(RR) do { if (a.bits == 4) TW_PT_MODES(RR, 4); else TW_PT_MODES(RR, 2); } while (0)
    if (R == 1) TW_PT_BITS(1); else if (R == 2) TW_PT_BITS(2); else TW_PT_BITS(4);
#undef TW_PT_BITS
#undef TW_PT_MODES
#undef TW_PT_LAUNCH
}

}  // namespace twkv
