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
// A wave needs nothing from any other wave (no LDS, no barrier), so a launch is
// ceil(vectors/16) * 8 independent single-wave workgroups that spread over the chip;
// that matters because these launches are small (a few thousand vectors) and
// latency-bound.

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

template <int BITS>
__global__ void __launch_bounds__(kWave)
rotate_kernel(RotArgs a) {
    const int lane = threadIdx.x;
    const int i16 = lane & 15, kk = lane >> 4;

    // ---- which unit: (segment, group of a.nper vector tiles, block of 16 output coordinates)
    int unit = blockIdx.x;
    int seg = 0;
    while (seg < a.nseg - 1 && unit >= a.seg_units[seg]) { unit -= a.seg_units[seg]; seg++; }
    const int dblk = unit & 7;
    const int vgroup = unit >> 3;
    const int nvec = a.seg_nvec[seg];
    const int heads = a.seg_heads[seg];                  // head vectors per source row
    const bool is_query = a.seg_kind[seg] != 0;
    const bool roped = a.seg_rope[seg] != 0;

    // ---- A operand, once per wave: R row d0 + i16 as 16 pieces of 8 halves
    const uint4* rsrc = reinterpret_cast<const uint4*>(a.rotation + (dblk * 16 + i16) * kHeadDim);
    float rv[32];
#pragma unroll
    for (int q = 0; q < 16; q++) {
        uint4 rp = rsrc[q];
        rv[2 * q] = pick_half(rp, 0, kk);
        rv[2 * q + 1] = pick_half(rp, 1, kk);
    }

    // Small launches (decode) give every wave one tile of 16 vectors; large ones (prompts) let a wave keep
    // its rows of R and walk a.nper tiles.
    for (int it = 0; it < a.nper; it++) {
    const int vtile = vgroup * a.nper + it;
    if (vtile * 16 >= nvec) break;
    const int v = vtile * 16 + i16;
    const int vc = v < nvec ? v : nvec - 1;              // clamp loads, mask stores
    const int row = vc / heads, head = vc - row * heads;

    // ---- B operand: source vector v as 16 pieces of 8 halves
    const uint4* xsrc = reinterpret_cast<const uint4*>(a.seg_src[seg] + (long long)row * a.seg_stride[seg] +
                                                       (long long)head * kHeadDim);
    // position of this vector's row: needed for the cache row and for the rotary table row, so it is the
    // first thing asked for; everything that depends on it is requested before the operands are used
    const int pos_row = (!is_query || roped) ? a.positions[row] : 0;
    long long crow = 0;
    if (!is_query) {
        if (a.token_list) crow = pos_row;                                // sequence 0, kernels.cu:1499, 1553
        else crow = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, row, pos_row);
    }
    float xv[32];
#pragma unroll
    for (int q = 0; q < 16; q++) {
        uint4 xp = xsrc[q];
        xv[2 * q] = pick_half(xp, 0, kk);
        xv[2 * q + 1] = pick_half(xp, 1, kk);
    }

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
    if (a.seg_weight[seg]) {
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
    if (bits == 4) hipLaunchKernelGGL(rotate_kernel<4>, dim3(units), dim3(kWave), 0, s, a);
    else hipLaunchKernelGGL(rotate_kernel<2>, dim3(units), dim3(kWave), 0, s, a);
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
merge_rotate_kernel(AttnArgs a) {
    __shared__ __attribute__((aligned(16))) float o_s[kMergeVecs][kMergeStride];
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int i16 = lane & 15, kk = lane >> 4;
    const int total = a.G * a.num_heads;
    const int v0 = blockIdx.x * kMergeVecs;

    // B operand first (its loads overlap the merge): R[32kk + s][16*wave + i16], s = 0..31
    uint16_t rb[32];
    {
        const uint16_t* rp = reinterpret_cast<const uint16_t*>(a.rotation) + (32 * kk) * kHeadDim + 16 * wave + i16;
#pragma unroll
        for (int s = 0; s < 32; s++) rb[s] = rp[s * kHeadDim];
    }

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
        // Chunks in blocks of 8 with every load of a block issued before the first use, so a
        // block costs one memory latency rather than one per chunk; the running maximum is
        // carried across blocks as in an online softmax.
        float mg = -1e30f, lsum = 0.0f;
        float4 av = {0.f, 0.f, 0.f, 0.f};
        const int nslots = nseg > 0 ? nseg : a.nsplit;
        for (int c0 = 0; c0 < nslots; c0 += 8) {
            float mc[8], lc[8];
            float4 pc4[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int c = c0 + j;
                // else: no workgroup wrote this slot.  The address does not wait for that answer (it needs the
                // partial count or the position, loads of their own): every slot the workspace has room for may be
                // read, whatever it holds is dropped below.
                const bool live = c < nslots && (nseg > 0 || chunk_nonempty(n, c, a.nsplit));
                const float* pc = part + (long long)(c < a.max_slots ? c : 0) * kPartialFloats;
                mc[j] = pc[kHeadDim];
                lc[j] = pc[kHeadDim + 1];
                pc4[j] = *reinterpret_cast<const float4*>(pc + k4);
                if (!live) { mc[j] = -1e30f; lc[j] = 0.0f; pc4[j] = float4{0.f, 0.f, 0.f, 0.f}; }
            }
            float mb = mg;
#pragma unroll
            for (int j = 0; j < 8; j++) mb = fmaxf(mb, mc[j]);
            const float fo = a.m_log2 ? __builtin_amdgcn_exp2f(mg - mb) : __expf(mg - mb);
            lsum *= fo; av.x *= fo; av.y *= fo; av.z *= fo; av.w *= fo;
            mg = mb;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float f = a.m_log2 ? __builtin_amdgcn_exp2f(mc[j] - mg) : __expf(mc[j] - mg);
                lsum = __builtin_fmaf(lc[j], f, lsum);
                av.x = __builtin_fmaf(pc4[j].x, f, av.x);
                av.y = __builtin_fmaf(pc4[j].y, f, av.y);
                av.z = __builtin_fmaf(pc4[j].z, f, av.z);
                av.w = __builtin_fmaf(pc4[j].w, f, av.w);
            }
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
}

bool launch_merge_rotate(const AttnArgs& a, hipStream_t s) {
    if (a.bits == 0 || !a.ws) return false;
    if ((reinterpret_cast<uintptr_t>(a.ws) & 15u) != 0 || (a.ws_stride & 3) != 0) return false;
    const int total = a.G * a.num_heads;
    if (total <= 0) return true;
    hipLaunchKernelGGL(merge_rotate_kernel, dim3((total + kMergeVecs - 1) / kMergeVecs), dim3(8 * kWave), 0, s, a);
    return true;
}

}  // namespace twkv
