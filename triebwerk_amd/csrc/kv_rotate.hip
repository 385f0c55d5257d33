// kv_rotate.hip -- the 128x128 rotation on the matrix cores (gfx950), for
//   - the TurboQuant compressed append: y = R (x / |x|), bin search, pack, norm
//     (turbo_kv_quantize{,_batch}_kernel, kernels.cu:1482-1636), K and V rows, and
//   - the query rotation q_rot = R q of the compressed attention (kernels.cu:1671-1681),
// all in one launch (any subset); optionally with the producers of q and k applied on the way in
// (per-head RMSNorm and rotary embedding, kernels.cu:880-961), which saves their two launches and
// the round trip of the rows through memory.
//
// Bit-exactness of the append.  The reference accumulates each output coordinate as
// one fp32 fused-multiply-add chain over k = 0..127.  v_mfma_f32_16x16x4_f32 chained
// over k-blocks of 4 produces the same bits: inside one instruction the four k of the
// block are accumulated in ascending order with fused multiply-adds, and blocks chain
// through the accumulator (checked on hardware against a host fmaf chain: 0 of 4096
// outputs differ).  The sum of squares keeps the reference's reduction tree
// (kernels.cu:1509-1520): offsets 16, 8 and 4 of the 32-lane shuffle tree only combine
// coordinates that are congruent mod 4, which one lane owns; offsets 2 and 1 and the
// combination of the four 32-coordinate groups, (s0+s2)+(s1+s3), are done across lanes.
//
// Mapping.  One wave = one work unit = (16 vectors) x (16 output coordinates):
//   A operand = R rows   : lane (i = lane%16, kk = lane/16) holds R[d0+i][4s+kk], s = 0..31
//   B operand = vectors  : the same lane holds u[v0+i][4s+kk]
//   D[16 x 16]           : lane holds y[d0 + 4*(lane/16) + r][v0 + lane%16], r = 0..3
// A wave needs nothing from any other wave, so a launch is ceil(vectors/16) * 8 independent single-wave
// workgroups that spread over the chip; that matters because the launches of a decode step are small (a few
// thousand vectors) and latency-bound.  The 8 waves that share a tile of vectors are numbered so that they land
// on one XCD (workgroup b runs on XCD b % 8), whose L2 then serves 7 of their 8 reads of it.
//
// Operand loads.  In the MFMA layout a lane wants every fourth half of a 256-byte row, and 16 lanes want 16
// different rows: asked for directly that is 16 loads per lane of which a quarter is used, each touching 16
// cache lines, and the address path of the CU becomes the limit of a big launch.  So a tile (16 rows, 4 KB)
// comes in as 4 fully used 16-byte pieces per lane, is written to LDS with the halves regrouped
// ([kk][row][s], kv_rotate_util.hpp), and each lane reads back its 32 halves as 4 x 16 bytes.

#include <algorithm>
#include <type_traits>

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_rotate_util.hpp"

namespace twkv {

namespace {

// Rotary embedding of a vector held as xv[s] = coordinate 4s + kk: coordinate d < HALF pairs with d + HALF
// (same lane, HALF4 = HALF / 4 registers further on); fp16 rounding as in rope_batch_kernel
// (kernels.cu:927-961).  The table rows hold HALF entries and arrive as 16-byte pieces.
template <int HALF4>
__device__ __forceinline__ void rope_registers(float (&xv)[32], const uint4 (&cp)[8], const uint4 (&sp)[8], int kk) {
#pragma clang fp contract(off)      // products rounded to fp32 first, as rope_batch_kernel's are
#pragma unroll
    for (int s = 0; s < HALF4; s++) {
        const float c = pick_half(cp[s >> 1], s & 1, kk), sn = pick_half(sp[s >> 1], s & 1, kk);
        const float x0 = xv[s], x1 = xv[s + HALF4];
        xv[s] = as_half_value(__builtin_fmaf(x0, c, -(x1 * sn)));
        xv[s + HALF4] = as_half_value(__builtin_fmaf(x0, sn, x1 * c));
    }
}

}  // namespace

// PROD: the producers of q and k may be switched on (their operands cost 64 registers and a third of the
// occupancy, which only the big launches of a prompt notice).
template <int BITS, bool PROD>
__global__ void __launch_bounds__(kWave)
rotate_kernel(RotArgs a) {
    __shared__ __attribute__((aligned(16))) uint32_t x_s[kOperandTileDwords];
    const int lane = threadIdx.x;
    const int i16 = lane & 15, kk = lane >> 4;

    // ---- which unit: (segment, group of a.nper vector tiles, block of 16 output coordinates)
    int unit = blockIdx.x;
    int seg = 0;
    while (seg < a.nseg - 1 && unit >= a.seg_units[seg]) { unit -= a.seg_units[seg]; seg++; }
    // Units of a segment in blocks of 64 = 8 tile groups x 8 coordinate blocks, the coordinate blocks of one
    // tile group 8 workgroups apart (same XCD; every segment starts at a multiple of 8); what is left over at the
    // end of the segment is numbered plainly.
    int dblk = unit & 7, vgroup = unit >> 3;
    if (unit < (a.seg_units[seg] >> 6) << 6) {
        vgroup = (unit >> 6) * 8 + (unit & 7);
        dblk = (unit >> 3) & 7;
    }
    const int nvec = a.seg_nvec[seg];
    const int heads = a.seg_heads[seg];                  // head vectors per source row
    const bool is_query = a.seg_kind[seg] != 0;
    const bool roped = PROD && a.seg_rope[seg] != 0;

    // ---- A operand, once per wave: R rows d0 .. d0 + 15 (4 KB in a row); requested now, staged after the
    // first tile of vectors has been requested too
    uint4 raw[4];
#pragma unroll
    for (int j = 0; j < 4; j++)
        raw[j] = reinterpret_cast<const uint4*>(a.rotation + dblk * 16 * kHeadDim)[j * kWave + lane];

    // 16-byte piece j * 64 + lane of a tile of vectors: piece lane % 16 of vector 4j + lane / 16
    const half_t* src = a.seg_src[seg];
    const long long stride = a.seg_stride[seg];
    auto request_tile = [&](int vtile, uint4 (&dst)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int vi = min(vtile * 16 + 4 * j + (lane >> 4), nvec - 1);
            const int ri = vi / heads, hi = vi - ri * heads;
            dst[j] = reinterpret_cast<const uint4*>(src + (long long)ri * stride + (long long)hi * kHeadDim)[lane & 15];
        }
    };
    const int vtile0 = vgroup * a.nper;
    if (vtile0 * 16 >= nvec) return;
    uint4 xraw[4];
    request_tile(vtile0, xraw);

    float rv[32];
    stage_operand_tile(x_s, raw, lane);
    lds_barrier();
    read_operand_tile(x_s, lane, rv);

    // Small launches (decode) give every wave one tile of 16 vectors; large ones (prompts) let a wave keep
    // its rows of R and walk a.nper tiles, the next tile requested while this one is worked on.
    for (int it = 0; it < a.nper; it++) {
    const int vtile = vtile0 + it;
    if (vtile * 16 >= nvec) break;
    const int v = vtile * 16 + i16;
    const int vc = v < nvec ? v : nvec - 1;              // clamp loads, mask stores
    const int row = vc / heads, head = vc - row * heads;

    // position of this vector's row: needed for the cache row and for the rotary table row, so it is asked for
    // early; everything that depends on it is requested before the operands are used
    const int pos_row = (!is_query || roped) ? a.positions[row] : 0;
    long long crow = 0;
    if (!is_query) {
        if (a.token_list) crow = pos_row;                                // sequence 0, kernels.cu:1499, 1553
        else crow = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, row, pos_row);
    }
    // ---- B operand: the tile's vectors through LDS
    lds_barrier();                                        // the reads of the previous tile (or of R) are done
    stage_operand_tile(x_s, xraw, lane);
    if (it + 1 < a.nper) request_tile(vtile + 1, xraw);   // clamped to the last vector: never out of bounds
    lds_barrier();
    float xv[32];
    read_operand_tile(x_s, lane, xv);

    // rotary table row of this position: rope_dim / 2 halves = rope_dim / 16 pieces
    uint4 cpiece[8], spiece[8];
    if (roped) {
        const int pieces = a.rope_dim >> 4;
        const uint4* cr = reinterpret_cast<const uint4*>(a.cos_table + (long long)pos_row * (a.rope_dim >> 1));
        const uint4* sr = reinterpret_cast<const uint4*>(a.sin_table + (long long)pos_row * (a.rope_dim >> 1));
#pragma unroll
        for (int q = 0; q < 8; q++) {
            if (q < pieces) { cpiece[q] = cr[q]; spiece[q] = sr[q]; }
        }
    }

    // ---- optional producers: per-head RMSNorm (kernels.cu:880-923), then rotary embedding (927-961),
    // each rounded to fp16 as the in-place kernels of the reference leave it
    if (PROD && a.seg_weight[seg]) {
#pragma clang fp contract(off)      // (x * rms) * w: two fp32 roundings, then the one to fp16
        const float rms = 1.0f / sqrtf(rotation_tree_sum_sq(xv) / (float)kHeadDim + a.eps);
        const uint4* wsrc = reinterpret_cast<const uint4*>(a.seg_weight[seg]);
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const uint4 wp = wsrc[q];
            float w0 = pick_half(wp, 0, kk), w1 = pick_half(wp, 1, kk);
            if (a.biased) { w0 += 1.0f; w1 += 1.0f; }
            xv[2 * q] = as_half_value((xv[2 * q] * rms) * w0);
            xv[2 * q + 1] = as_half_value((xv[2 * q + 1] * rms) * w1);
        }
    }
    if (roped) {
        switch (a.rope_dim >> 1) {                               // rope_dim: 128, or a multiple of 16 up to 64
            case 64: rope_registers<16>(xv, cpiece, spiece, kk); break;
            case 32: rope_registers<8>(xv, cpiece, spiece, kk); break;
            case 24: rope_registers<6>(xv, cpiece, spiece, kk); break;
            case 16: rope_registers<4>(xv, cpiece, spiece, kk); break;
            default: rope_registers<2>(xv, cpiece, spiece, kk); break;
        }
    }

    float n2 = 0.0f;
    if (!is_query) {
        n2 = rotation_tree_sum_sq(xv);
        const float inv = 1.0f / sqrtf(n2 + 1e-12f);
#pragma unroll
        for (int s = 0; s < 32; s++) xv[s] *= inv;
    }

    // ---- y[d][v] = sum_k R[d][k] u[v][k], k ascending
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 32; s++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(rv[s], xv[s], acc, 0, 0, 0);

    if (is_query) {
        if (v < nvec) {
            float* dst = a.qrot + (long long)v * a.qrot_stride + dblk * 16 + 4 * kk;
            float4 o = {acc[0] * a.q_scale, acc[1] * a.q_scale, acc[2] * a.q_scale, acc[3] * a.q_scale};
            *reinterpret_cast<float4*>(dst) = o;
        }
        continue;
    }

    // ---- quantize the lane's 4 consecutive coordinates d0 + 4kk .. +3 and pack (low field first)
    uint32_t packed = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) packed |= (uint32_t)turbo_quantize(acc[r], BITS) << (r * BITS);
    // gather the four lanes of a vector (kk = 0..3) into the kk == 0 lane
    constexpr int PB = 4 * BITS;                                  // bits per lane
    uint32_t p1 = (uint32_t)__shfl((int)packed, i16 + 16, 64);
    uint32_t p2 = (uint32_t)__shfl((int)packed, i16 + 32, 64);
    uint32_t p3 = (uint32_t)__shfl((int)packed, i16 + 48, 64);
    if (kk == 0 && v < nvec) {
        constexpr int BPH = kHeadDim * BITS / 8;                  // bytes per head: 64 or 32
        uint8_t* dst = a.seg_codes[seg] + (crow * a.num_kv_heads + head) * BPH + dblk * (2 * BITS);
        if (BITS == 4) {
            uint2 o = {packed | (p1 << PB), p2 | (p3 << PB)};
            *reinterpret_cast<uint2*>(dst) = o;                   // 16 codes = 8 bytes
        } else {
            *reinterpret_cast<uint32_t*>(dst) = packed | (p1 << PB) | (p2 << (2 * PB)) | (p3 << (3 * PB));
        }
        if (dblk == 0) a.seg_norms[seg][crow * a.num_kv_heads + head] = (half_t)sqrtf(n2 + 1e-12f);
    }
    }   // tiles of this wave
}

void launch_rotate(const RotArgs& args, int bits, hipStream_t s) {
    RotArgs a = args;
    // tiles of 16 vectors per wave: one while the launch is small, more once there are far more tiles than
    // the GPU holds waves
    long long tiles = 0;
    for (int i = 0; i < a.nseg; i++) tiles += (a.seg_nvec[i] + 15) / 16;
    constexpr long long kWantUnits = 16384;               // 64 single-wave workgroups per CU
    int nper = (int)((tiles * 8 + kWantUnits - 1) / kWantUnits);
    if (nper < 1) nper = 1;
    if (nper > 32) nper = 32;
    a.nper = nper;
    int units = 0;
    for (int i = 0; i < a.nseg; i++) {
        const int t = (a.seg_nvec[i] + 15) / 16;
        a.seg_units[i] = (t + nper - 1) / nper * 8;
        units += a.seg_units[i];
    }
    if (units <= 0) return;
    bool prod = false;
    for (int i = 0; i < a.nseg; i++) prod = prod || a.seg_weight[i] != nullptr || a.seg_rope[i] != 0;
    if (bits == 4) {
        if (prod) hipLaunchKernelGGL((rotate_kernel<4, true>), dim3(units), dim3(kWave), 0, s, a);
        else hipLaunchKernelGGL((rotate_kernel<4, false>), dim3(units), dim3(kWave), 0, s, a);
    } else {
        if (prod) hipLaunchKernelGGL((rotate_kernel<2, true>), dim3(units), dim3(kWave), 0, s, a);
        else hipLaunchKernelGGL((rotate_kernel<2, false>), dim3(units), dim3(kWave), 0, s, a);
    }
}

// ---------------------------------------------------------------- split merge + rotate-back
// out[g][head][d] = sum_k R[k][d] * o[k],  o = (sum_c f_c acc_c) / (sum_c f_c l_c + 1e-8),
// f_c = exp(m_c - max_c m_c): the log-sum-exp merge of the split partials, the
// normalisation of kernels.cu:1746 and the rotate-back of kernels.cu:1769-1775.
// A workgroup of 8 waves takes 16 (sequence, head) vectors: all threads merge into LDS,
// then wave w produces output coordinates [16w, 16w+16) with 32 fp32 MFMAs
// (v_mfma_f32_16x16x4_f32; A = merged vectors from LDS, B = a column block of R).
constexpr int kMergeVecs = 16;
constexpr int kMergeStride = kHeadDim + 4;     // floats per LDS row: conflict-free 16-byte reads

__global__ void __launch_bounds__(8 * kWave)
merge_rotate_kernel(AttnArgs a, int nper) {
    __shared__ __attribute__((aligned(16))) float o_s[kMergeVecs][kMergeStride];
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int i16 = lane & 15, kk = lane >> 4;
    const int total = a.G * a.num_heads;

    // B operand first (its loads overlap the merge): R[32kk + s][16*wave + i16], s = 0..31
    uint16_t rb[32];
    {
        const uint16_t* rp = reinterpret_cast<const uint16_t*>(a.rotation) + (32 * kk) * kHeadDim + 16 * wave + i16;
#pragma unroll
        for (int s = 0; s < 32; s++) rb[s] = rp[s * kHeadDim];
    }

    // A workgroup keeps its block of R and walks nper tiles of 16 vectors (1 in a decode step, more for a prompt).
    for (int it = 0; it < nper; it++) {
    const int v0 = (blockIdx.x * nper + it) * kMergeVecs;
    if (v0 >= total) break;
    if (it > 0) __syncthreads();                      // the previous tile's vectors have been read

    // ---- merge: thread -> (vector tid/32, coordinates 4*(tid%32) .. +3)
    {
        const int vl = tid >> 5, k4 = (tid & 31) * 4;
        const int vv = min(v0 + vl, total - 1);
        const int g = vv / a.num_heads;
        int n;
        if (a.pos_mode == kPosArray) n = a.positions[g] + 1;
        else if (a.pos_mode == kPosScalar) n = a.pos_scalar + 1;
        else n = g + 1;
        const float* part = a.ws + (long long)vv * a.ws_stride;
        const int nseg = a.slots_from_ws ? reinterpret_cast<const int*>(part)[kHeadDim + 2] : 0;
        // Slots in blocks with every load of a block issued before the first use, so a block costs one memory
        // latency rather than one per slot; the running maximum is carried across blocks as in an online softmax.
        float mg = -1e30f, lsum = 0.0f;
        float4 av = {0.f, 0.f, 0.f, 0.f};
        const int nslots = nseg > 0 ? nseg : a.nsplit;
        auto merge_block = [&](int c0, auto width) {
            constexpr int W = decltype(width)::value;
            float mc[W], lc[W];
            float4 pc4[W];
#pragma unroll
            for (int j = 0; j < W; j++) {
                const int c = c0 + j;
                // else: no workgroup wrote this slot.  With a fixed split (a decode step) the address does not wait
                // for that answer, which needs the position, a load of its own: every slot the workspace has room
                // for may be read, and what it holds is dropped below.
                const bool live = c < nslots && (nseg > 0 || chunk_nonempty(n, c, a.nsplit));
                const bool fetch = a.slots_from_ws ? live : c < a.max_slots;
                const float* pc = part + (long long)(fetch ? c : 0) * kPartialFloats;
                mc[j] = pc[kHeadDim];
                lc[j] = pc[kHeadDim + 1];
                pc4[j] = *reinterpret_cast<const float4*>(pc + k4);
                if (!live) { mc[j] = -1e30f; lc[j] = 0.0f; pc4[j] = float4{0.f, 0.f, 0.f, 0.f}; }
            }
            float mb = mg;
#pragma unroll
            for (int j = 0; j < W; j++) mb = fmaxf(mb, mc[j]);
            const float fo = a.m_log2 ? __builtin_amdgcn_exp2f(mg - mb) : __expf(mg - mb);
            lsum *= fo; av.x *= fo; av.y *= fo; av.z *= fo; av.w *= fo;
            mg = mb;
#pragma unroll
            for (int j = 0; j < W; j++) {
                float f = a.m_log2 ? __builtin_amdgcn_exp2f(mc[j] - mg) : __expf(mc[j] - mg);
                lsum = __builtin_fmaf(lc[j], f, lsum);
                av.x = __builtin_fmaf(pc4[j].x, f, av.x);
                av.y = __builtin_fmaf(pc4[j].y, f, av.y);
                av.z = __builtin_fmaf(pc4[j].z, f, av.z);
                av.w = __builtin_fmaf(pc4[j].w, f, av.w);
            }
        };
        // blocks of 8; a count of 1 or 2 (a prompt: the workspace says how many) is not padded to 8 loads
        if (nslots <= 2) {
            merge_block(0, std::integral_constant<int, 2>{});
        } else {
            for (int c0 = 0; c0 < nslots; c0 += 8) merge_block(c0, std::integral_constant<int, 8>{});
        }
        const float inv = 1.0f / (lsum + 1e-8f);
        float4 o4 = {av.x * inv, av.y * inv, av.z * inv, av.w * inv};
        *reinterpret_cast<float4*>(&o_s[vl][k4]) = o4;
    }
    __syncthreads();

    // ---- out[vector][d] = sum_k o[vector][k] R[k][d]; lane group kk owns k in [32kk, 32kk+32)
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    const float* orow = &o_s[i16][32 * kk];
#pragma unroll
    for (int s4 = 0; s4 < 8; s4++) {
        float4 o4 = *reinterpret_cast<const float4*>(orow + 4 * s4);
        const float ov[4] = {o4.x, o4.y, o4.z, o4.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            union { uint16_t u; half_t h; } cv;
            cv.u = rb[4 * s4 + j];
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ov[j], (float)cv.h, acc, 0, 0, 0);
        }
    }
    // lane holds out[vector 4kk + r][d = 16*wave + i16]
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int vv = v0 + 4 * kk + r;
        if (vv < total) {
            const int g = vv / a.num_heads, head = vv - g * a.num_heads;
            const long long col = (long long)head * kHeadDim + 16 * wave + i16;
            half_t h = (half_t)acc[r];
            if (a.gate) h = gated(h, a.gate[(long long)g * a.gate_stride + col]);
            a.out[(long long)g * a.q_stride + col] = h;
        }
    }
    }   // tiles of this workgroup
}

bool launch_merge_rotate(const AttnArgs& a, hipStream_t s) {
    if (a.bits == 0 || !a.ws) return false;
    if ((reinterpret_cast<uintptr_t>(a.ws) & 15u) != 0 || (a.ws_stride & 3) != 0) return false;
    const int total = a.G * a.num_heads;
    if (total <= 0) return true;
    // one tile per workgroup until there are 8 workgroups per CU, then up to 8
    const int tiles = (total + kMergeVecs - 1) / kMergeVecs;
    const int nper = std::max(1, std::min(8, tiles / 2048));
    hipLaunchKernelGGL(merge_rotate_kernel, dim3((tiles + nper - 1) / nper), dim3(8 * kWave), 0, s, a, nper);
    return true;
}

}  // namespace twkv
