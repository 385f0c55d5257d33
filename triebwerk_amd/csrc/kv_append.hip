// kv_append.hip -- fp16 KV append and TurboQuant compressed append for gfx950.
//
// Replaces kv_cache_write_batch_kernel (kernels.cu:964-977) and
// turbo_kv_quantize{,_batch}_kernel (kernels.cu:1482-1636) of the reference.
//
// The compressed append must produce the reference's bytes, so its arithmetic
// keeps the reference's order where order matters:
//   - sum of squares: 32-lane shuffle-down tree per group of 32 coordinates,
//     then (s0+s2)+(s1+s3) over the four group sums (kernels.cu:1509-1520);
//   - 1/sqrt and sqrt correctly rounded;
//   - rotation: one fp32 fused multiply-add chain per output coordinate, k
//     ascending (kernels.cu:1528-1531);
//   - bin search with strict `<` (kernels.cu:1448-1473), low field first when
//     packing (1543-1552), norm stored as fp16 RNE (1557-1558).
// What changes is the mapping to the machine: one 64-lane wave owns a head
// vector (two coordinates per lane), the rotation matrix is staged once per
// workgroup in LDS as fp32 with a padded row stride so that the per-lane row
// walks are bank-conflict free, K and V rows go through one launch, and codes
// leave as 4-byte words.

#include "kv_common.hpp"
#include "kv_kernels.hpp"

namespace twkv {

// ---------------------------------------------------------------- fp16 append
__global__ void __launch_bounds__(256)
kv_write_kernel(half_t* __restrict__ ck, half_t* __restrict__ cv,
                const half_t* __restrict__ k, const half_t* __restrict__ v,
                const int* __restrict__ positions, const int* __restrict__ block_table,
                int bt_stride, long long seq_stride_rows, int G, int kv_dim, int vec_ok) {
    int g = blockIdx.x;
    if (g >= G) return;
    int pos = positions[g];
    long long row = cache_row(block_table, bt_stride, seq_stride_rows, g, pos);
    long long dst = row * kv_dim;
    long long src = (long long)g * kv_dim;
    if (vec_ok) {
        const uint4* k4 = reinterpret_cast<const uint4*>(k + src);
        const uint4* v4 = reinterpret_cast<const uint4*>(v + src);
        uint4* ck4 = reinterpret_cast<uint4*>(ck + dst);
        uint4* cv4 = reinterpret_cast<uint4*>(cv + dst);
        int n4 = kv_dim / 8;
        for (int i = threadIdx.x; i < n4; i += blockDim.x) {
            ck4[i] = k4[i];
            cv4[i] = v4[i];
        }
    } else {
        for (int d = threadIdx.x; d < kv_dim; d += blockDim.x) {
            ck[dst + d] = k[src + d];
            cv[dst + d] = v[src + d];
        }
    }
}

// ---------------------------------------------------------------- compressed append
constexpr int kRotStride = kHeadDim + 4;  // floats; 4*d + k spreads rows over the 32 LDS banks
constexpr int kQuantWaves = 4;

template <int BITS>
__global__ void __launch_bounds__(kQuantWaves * kWave)
turbo_quantize_kernel(QuantArgs a) {
    __shared__ float rot_s[kHeadDim * kRotStride];          // 67.6 KB
    __shared__ float u_s[kQuantWaves][kHeadDim];
    __shared__ uint8_t code_s[kQuantWaves][kHeadDim];

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid % kWave;

    // Stage R (fp16, row major) as fp32.  8 halves per load, coalesced.
    for (int i = tid; i < kHeadDim * kHeadDim / 8; i += blockDim.x) {
        half8_t r8 = reinterpret_cast<const half8_t*>(a.rotation)[i];
        int row = (i * 8) / kHeadDim, col = (i * 8) % kHeadDim;
        float* dst = &rot_s[row * kRotStride + col];
#pragma unroll
        for (int j = 0; j < 8; j++) dst[j] = (float)r8[j];
    }
    __syncthreads();

    constexpr int VPB = 8 / BITS;             // codes per byte
    constexpr int BPH = kHeadDim / VPB;       // bytes per head: 64 or 32
    const int nvec_stream = a.nrows * a.num_kv_heads;
    const int nvec = nvec_stream * a.nstreams;

    for (int base = blockIdx.x * kQuantWaves; base < nvec; base += gridDim.x * kQuantWaves) {
        const int vec = base + wave;
        const bool active = vec < nvec;
        int stream = 0, r = 0, h = 0;
        float n2 = 0.0f;
        if (active) {
            stream = vec / nvec_stream;
            int rem = vec - stream * nvec_stream;
            r = rem / a.num_kv_heads;
            h = rem - r * a.num_kv_heads;
            const half_t* src = a.src[stream] + (long long)r * a.kv_dim + (long long)h * kHeadDim;
            float x0 = (float)src[lane];
            float x1 = (float)src[lane + 64];
            // 32-lane shuffle-down trees over coordinates [0,32) [32,64) (first value)
            // and [64,96) [96,128) (second value).
            float t0 = x0 * x0, t1 = x1 * x1;
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) {
                t0 += __shfl_down(t0, off, 32);
                t1 += __shfl_down(t1, off, 32);
            }
            float s0 = __shfl(t0, 0, 64), s1 = __shfl(t0, 32, 64);
            float s2 = __shfl(t1, 0, 64), s3 = __shfl(t1, 32, 64);
            n2 = (s0 + s2) + (s1 + s3);
            float inv = 1.0f / sqrtf(n2 + 1e-12f);
            u_s[wave][lane] = x0 * inv;
            u_s[wave][lane + 64] = x1 * inv;
        }
        __syncthreads();
        if (active) {
            const float* ra = &rot_s[lane * kRotStride];
            const float* rb = &rot_s[(lane + 64) * kRotStride];
            const float* u = u_s[wave];
            float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll 8
            for (int k = 0; k < kHeadDim; k += 4) {
                float4 u4 = *reinterpret_cast<const float4*>(u + k);
                float4 a4 = *reinterpret_cast<const float4*>(ra + k);
                float4 b4 = *reinterpret_cast<const float4*>(rb + k);
                acc0 = __builtin_fmaf(a4.x, u4.x, acc0);
                acc1 = __builtin_fmaf(b4.x, u4.x, acc1);
                acc0 = __builtin_fmaf(a4.y, u4.y, acc0);
                acc1 = __builtin_fmaf(b4.y, u4.y, acc1);
                acc0 = __builtin_fmaf(a4.z, u4.z, acc0);
                acc1 = __builtin_fmaf(b4.z, u4.z, acc1);
                acc0 = __builtin_fmaf(a4.w, u4.w, acc0);
                acc1 = __builtin_fmaf(b4.w, u4.w, acc1);
            }
            code_s[wave][lane] = (uint8_t)turbo_quantize(acc0, BITS);
            code_s[wave][lane + 64] = (uint8_t)turbo_quantize(acc1, BITS);
        }
        __syncthreads();
        if (active) {
            long long row;
            if (a.token_list) {
                row = a.positions[r];  // sequence 0, kernels.cu:1499, 1553
            } else {
                row = cache_row(a.block_table, a.bt_stride, a.seq_stride_rows, r, a.positions[r]);
            }
            const long long kvp = (long long)a.num_kv_heads * BPH;
            if (lane < BPH / 4) {
                const uint8_t* c = &code_s[wave][lane * 4 * VPB];
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4 * VPB; j++) word |= (uint32_t)c[j] << (j * BITS);
                uint32_t* dst = reinterpret_cast<uint32_t*>(a.codes[stream] + row * kvp + (long long)h * BPH);
                dst[lane] = word;
            }
            if (lane == 0) {
                a.norms[stream][row * a.num_kv_heads + h] = (half_t)sqrtf(n2 + 1e-12f);
            }
        }
        // u_s / code_s are rewritten only after the next iteration's first barrier
        // has been passed by every wave, and every read above precedes it.
    }
}

void launch_kv_write(half_t* ck, half_t* cv, const half_t* k, const half_t* v,
                     const int* positions, const int* block_table, int bt_stride,
                     long long seq_stride_rows, int G, int kv_dim, hipStream_t s) {
    if (G <= 0) return;
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    int vec_ok = (kv_dim % 8 == 0) && al16(ck) && al16(cv) && al16(k) && al16(v);
    hipLaunchKernelGGL(kv_write_kernel, dim3(G), dim3(256), 0, s, ck, cv, k, v, positions,
                       block_table, bt_stride, seq_stride_rows, G, kv_dim, vec_ok);
}

void launch_turbo_quantize(const QuantArgs& a, int bits, hipStream_t s) {
    int nvec = a.nrows * a.num_kv_heads * a.nstreams;
    if (nvec <= 0) return;
    int blocks = (nvec + kQuantWaves - 1) / kQuantWaves;
    if (blocks > 2048) blocks = 2048;
    if (bits == 4) {
        hipLaunchKernelGGL(turbo_quantize_kernel<4>, dim3(blocks), dim3(kQuantWaves * kWave), 0, s, a);
    } else {
        hipLaunchKernelGGL(turbo_quantize_kernel<2>, dim3(blocks), dim3(kQuantWaves * kWave), 0, s, a);
    }
}

__global__ void increment_positions_kernel(int* positions, int G) {
    int g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g < G) positions[g]++;
}

void launch_increment(int* positions, int G, hipStream_t s) {
    if (G <= 0) return;
    hipLaunchKernelGGL(increment_positions_kernel, dim3((G + 255) / 256), dim3(256), 0, s, positions, G);
}

// ---------------------------------------------------------------- prefix broadcast
// The first T rows of one sequence's arrays copied to the same rows of other sequences: the
// reference's prefill-once-then-broadcast (engine.cpp:2173-2214) does it with one device-to-device
// copy per (layer, array, destination); here one launch takes up to four arrays and every destination.
// blockIdx.y = destination slot, blockIdx.z = array; the x blocks stride over the array's bytes.
template <typename W>
__global__ void __launch_bounds__(256)
broadcast_rows_kernel(BroadcastArgs a) {
    const int which = blockIdx.z;
    int g = a.dst_begin + blockIdx.y;
    if (a.src >= a.dst_begin && a.src < a.dst_end && g >= a.src) g++;   // destination slots skip the source
    const size_t n = a.bytes[which] / sizeof(W);
    const W* from = reinterpret_cast<const W*>(a.base[which] + (size_t)a.src * a.seq_bytes[which]);
    W* to = reinterpret_cast<W*>(a.base[which] + (size_t)g * a.seq_bytes[which]);
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) to[i] = from[i];
}

void launch_broadcast_rows(const BroadcastArgs& a, hipStream_t s) {
    int ndst = a.dst_end - a.dst_begin;
    if (a.src >= a.dst_begin && a.src < a.dst_end) ndst--;
    if (ndst <= 0 || a.narrays <= 0) return;
    size_t most = 0;
    unsigned align = 0;
    for (int w = 0; w < a.narrays; w++) {
        most = a.bytes[w] > most ? a.bytes[w] : most;
        align |= (unsigned)(reinterpret_cast<uintptr_t>(a.base[w]) | a.seq_bytes[w] | a.bytes[w]);
    }
    if (most == 0) return;
    const int width = (align & 15u) == 0 ? 16 : ((align & 3u) == 0 ? 4 : 2);    // rows are fp16 at least
    size_t blocks = (most / width + 255) / 256;
    if (blocks > 64) blocks = 64;                          // a block copies up to 4 KB per pass
    if (blocks < 1) blocks = 1;
    dim3 grid((unsigned)blocks, (unsigned)ndst, (unsigned)a.narrays);
    if (width == 16) hipLaunchKernelGGL(broadcast_rows_kernel<uint4>, grid, dim3(256), 0, s, a);
    else if (width == 4) hipLaunchKernelGGL(broadcast_rows_kernel<uint32_t>, grid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL(broadcast_rows_kernel<uint16_t>, grid, dim3(256), 0, s, a);
}

}  // namespace twkv
