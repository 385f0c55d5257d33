// kv_producer.hip -- the producers of q and k in front of the KV append, for gfx950:
// per-head RMSNorm (qk_norm_kernel, kernels.cu:137-186; qk_norm_batch_kernel, 880-923) and rotary
// position embedding (rope_kernel, 193-235; rope_batch_kernel, 927-961), as kernels of their own
// with the reference's in-place semantics, and fused with the fp16 append (one launch instead of
// qk_norm + rope + kv_cache_write).  The fusion into the compressed append lives in
// kv_rotate.hip, on that kernel's register layout.  Also here: the sigmoid gate of gated attention
// (sigmoid_gate_batch_kernel, kernels.cu:2987-2995), which the attention kernels can apply themselves.
//
// Bits.  Both steps round to fp16 in between, as the reference's in-place kernels do:
//   normed = half((float(x) * rms) * w),  rms = 1 / sqrt(sum / 128 + eps), w + 1 when `biased`;
//   out0 = half(fma(x0, c, -(x1 * s)));   out1 = half(fma(x0, s, x1 * c))   (batch kernel), or
//   out1 = half(fma(x1, c, x0 * s))   (single-sequence kernel, whose source has the other order).
// The sum of squares keeps the reference's reduction tree: a 32-lane shuffle-down tree per group of
// 32 coordinates, then (s0 + s2) + (s1 + s3).
//
// Mapping: one 64-lane wave owns a head vector, lane l holds coordinates l and l + 64, so the
// rotary pair (d, d + 64) of a full-width rotation sits in one lane; a partial rotation (rope_dim <
// 128) fetches the partner with a wave shuffle.  4 waves per workgroup.

#include "kv_common.hpp"
#include "kv_kernels.hpp"
#include "kv_producer_util.hpp"

// Every product below is rounded to fp32 before anything else happens to it, as in the reference's
// separate kernels: no fused multiply-add where the source has none, and no multiply fused into the
// conversion to fp16 (one rounding instead of two changes a result in a few hundred thousand).
#pragma clang fp contract(off)

namespace twkv {

namespace {

constexpr int kProdWaves = 4;

}  // namespace

// One head vector per wave.  Vector v = (row, head) with Q heads first, then K heads, then (write mode)
// V heads.  mode 0: transform Q and K in place.  mode 1: Q in place, K into its cache row, V copied
// into its cache row.
__global__ void __launch_bounds__(kProdWaves* kWave)
producer_kernel(ProducerArgs a) {
    const int lane = threadIdx.x % kWave;
    const long long v = (long long)blockIdx.x * kProdWaves + threadIdx.x / kWave;
    const int per_row = a.num_heads + a.num_kv_heads * (a.write_cache ? 2 : 1);
    if (v >= (long long)a.rows * per_row) return;
    const int row = (int)(v / per_row);
    int head = (int)(v - (long long)row * per_row);
    const int pos = a.positions ? a.positions[row] : a.pos_scalar;

    half_t* src;
    half_t* dst;
    const half_t* w;
    bool xform = true;
    if (head < a.num_heads) {
        src = a.q + (long long)row * a.q_stride + (long long)head * kHeadDim;
        dst = src;
        w = a.q_weight;
    } else {
        head -= a.num_heads;
        const bool is_v = head >= a.num_kv_heads;
        if (is_v) head -= a.num_kv_heads;
        half_t* base = is_v ? a.v : a.k;
        src = base + (long long)row * a.kv_stride + (long long)head * kHeadDim;
        dst = src;
        w = a.k_weight;
        xform = !is_v;
        if (a.write_cache) {
            const long long crow = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, row, pos);
            dst = (is_v ? a.cache_v : a.cache_k) + crow * a.kv_dim + (long long)head * kHeadDim;
        }
    }
    float x0 = (float)src[lane], x1 = (float)src[lane + 64];
    if (xform) {
        HeadXform t;
        t.weight = a.norm ? w : nullptr;
        t.eps = a.eps;
        t.biased = a.biased;
        t.cos_row = a.cos_table ? a.cos_table + (long long)pos * (a.rope_dim >> 1) : nullptr;
        t.sin_row = a.cos_table ? a.sin_table + (long long)pos * (a.rope_dim >> 1) : nullptr;
        t.rope_dim = a.rope_dim;
        t.single_order = a.single_order;
        xform_head(x0, x1, lane, t);
    }
    dst[lane] = (half_t)x0;
    dst[lane + 64] = (half_t)x1;
}

void launch_producer(const ProducerArgs& a, hipStream_t s) {
    const long long vecs = (long long)a.rows * (a.num_heads + a.num_kv_heads * (a.write_cache ? 2 : 1));
    if (vecs <= 0) return;
    const int blocks = (int)((vecs + kProdWaves - 1) / kProdWaves);
    hipLaunchKernelGGL(producer_kernel, dim3(blocks), dim3(kProdWaves * kWave), 0, s, a);
}

// ---------------------------------------------------------------- gated attention output
// sigmoid_gate_batch_kernel (kernels.cu:2987-2995) with row strides: 8 halves per lane
__global__ void __launch_bounds__(256)
sigmoid_gate_kernel(half_t* data, long long data_stride, const half_t* gate, long long gate_stride, int dim,
                    int rows, int vec_ok) {
    const int per_row = (dim + 7) / 8;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)rows * per_row) return;
    const int r = (int)(idx / per_row), c = (int)(idx - (long long)r * per_row) * 8;
    half_t* d = data + (long long)r * data_stride + c;
    const half_t* g = gate + (long long)r * gate_stride + c;
    if (vec_ok) {
        union { uint4 u; half_t h[8]; } dv, gv;
        dv.u = *reinterpret_cast<const uint4*>(d);
        gv.u = *reinterpret_cast<const uint4*>(g);
#pragma unroll
        for (int i = 0; i < 8; i++) dv.h[i] = gated(dv.h[i], gv.h[i]);
        *reinterpret_cast<uint4*>(d) = dv.u;
    } else {
        for (int i = 0; i < 8 && c + i < dim; i++) d[i] = gated(d[i], g[i]);
    }
}

void launch_sigmoid_gate(half_t* data, long long data_stride, const half_t* gate, long long gate_stride, int dim,
                         int rows, hipStream_t s) {
    if (rows <= 0 || dim <= 0) return;
    const int vec_ok = (dim % 8 == 0 && data_stride % 8 == 0 && gate_stride % 8 == 0 &&
                        ((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(gate)) & 15u) == 0) ? 1 : 0;
    const long long n = (long long)rows * ((dim + 7) / 8);
    hipLaunchKernelGGL(sigmoid_gate_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, data, data_stride, gate,
                       gate_stride, dim, rows, vec_ok);
}

}  // namespace twkv
