// kv_oracle.cpp -- CPU restatement of the reference KV-cache kernels.
// TEST INFRASTRUCTURE ONLY: see kv_oracle.h for the rules and the parity pins.
//
// Build: oracle/Makefile (g++ -O2 -ffp-contract=off -mfma -fopenmp).
// -ffp-contract=off keeps the compiler from fusing anything on its own; every
// fused multiply-add below is an explicit fmaf() placed where nvcc contracts
// the reference's `acc += a * b`.

#include "kv_oracle.h"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr int kWarp = 32;       // CUDA warpSize the reference kernels assume
constexpr int kMaxBlock = 128;  // all hot-path kernels launch blockDim = 128

// ---------------------------------------------------------------- fp16 <-> fp32
float h2f_slow(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: normalise
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

struct H2FTable {
    float t[65536];
    H2FTable() { for (int i = 0; i < 65536; i++) t[i] = h2f_slow((uint16_t)i); }
};
const H2FTable& h2f_table() { static H2FTable tab; return tab; }
inline float h2f(uint16_t h) { return h2f_table().t[h]; }

uint16_t f2h(float f) {  // round to nearest even, like __float2half
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) {  // inf / nan
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
    }
    if (ax >= 0x477ff000u) {  // >= 65520 rounds to inf
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x33000001u) {  // <= 2^-25 rounds to zero (tie at exactly 2^-25 -> even = 0)
        return (uint16_t)sign;
    }
    int e = (int)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t hexp;
    if (e < -14) {  // subnormal half
        shift = 13 + (-14 - e);
        hexp = 0;
    } else {
        shift = 13;
        hexp = (uint32_t)(e + 15);
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    // mantissa overflow carries into the exponent, which is what we want
    return (uint16_t)(sign | ((hexp << 10) + q));
}

// ---------------------------------------------------------------- tables
// kernels.cu:1426-1445
const float CENTROIDS_2[4] = {-0.13351f, -0.04003f, 0.04003f, 0.13351f};
const float BOUNDS_2[3] = {-0.08677f, 0.0f, 0.08677f};
const float CENTROIDS_4[16] = {-0.24155f, -0.18293f, -0.14304f, -0.11099f,
                               -0.08330f, -0.05806f, -0.03432f, -0.01135f,
                               0.01135f,  0.03432f,  0.05806f,  0.08330f,
                               0.11099f,  0.14304f,  0.18293f,  0.24155f};
const float BOUNDS_4[15] = {-0.21224f, -0.16299f, -0.12701f, -0.09715f,
                            -0.07068f, -0.04619f, -0.02284f, 0.00000f,
                            0.02284f,  0.04619f,  0.07068f,  0.09715f,
                            0.12701f,  0.16299f,  0.21224f};

// kernels.cu:1448-1473.  Strict `<` in the 4-bit search: a value equal to a
// boundary lands in the upper bin; NaN fails every `<` and ends at 15.
// 2-bit: a count of `>=`; NaN fails all three and ends at 0.
inline int quantize(float val, int bits) {
    if (bits == 4) {
        const float* B = BOUNDS_4;
        int idx;
        if (val < B[7]) {
            if (val < B[3]) {
                if (val < B[1]) idx = val < B[0] ? 0 : 1;
                else idx = val < B[2] ? 2 : 3;
            } else {
                if (val < B[5]) idx = val < B[4] ? 4 : 5;
                else idx = val < B[6] ? 6 : 7;
            }
        } else {
            if (val < B[11]) {
                if (val < B[9]) idx = val < B[8] ? 8 : 9;
                else idx = val < B[10] ? 10 : 11;
            } else {
                if (val < B[13]) idx = val < B[12] ? 12 : 13;
                else idx = val < B[14] ? 14 : 15;
            }
        }
        return idx;
    }
    return (val >= BOUNDS_2[0]) + (val >= BOUNDS_2[1]) + (val >= BOUNDS_2[2]);
}

inline float centroid(int idx, int bits) {  // kernels.cu:1476-1478
    return bits == 4 ? CENTROIDS_4[idx] : CENTROIDS_2[idx];
}

inline float margin(float val, int bits) {
    const float* B = bits == 4 ? BOUNDS_4 : BOUNDS_2;
    int n = bits == 4 ? 15 : 3;
    float m = INFINITY;
    for (int i = 0; i < n; i++) m = fminf(m, fabsf(val - B[i]));
    return m;
}

// ---------------------------------------------------------------- block reductions
// __shfl_down_sync(full mask, v, off) on a 32-lane warp: lane i reads lane i+off,
// or keeps its own value when i+off falls outside the warp.
inline void warp_tree_sum(float* v) {
    for (int off = kWarp / 2; off > 0; off /= 2) {
        float nv[kWarp];
        for (int i = 0; i < kWarp; i++) nv[i] = v[i] + ((i + off < kWarp) ? v[i + off] : v[i]);
        memcpy(v, nv, sizeof(nv));
    }
}

// The sum every hot-path kernel uses (e.g. kernels.cu:1509-1520, 1734-1745):
// per-warp tree, lane 0 of each warp to shared memory, warp 0 reloads the
// partials (0.0f in lanes past the warp count) and runs the tree again.
float block_sum(const float* per_thread, int nthreads) {
    int nwarps = (nthreads + kWarp - 1) / kWarp;
    float partial[kWarp];
    for (int i = 0; i < kWarp; i++) partial[i] = 0.0f;
    for (int w = 0; w < nwarps; w++) {
        float lane[kWarp];
        for (int i = 0; i < kWarp; i++) {
            int t = w * kWarp + i;
            lane[i] = t < nthreads ? per_thread[t] : 0.0f;
        }
        warp_tree_sum(lane);
        partial[w] = lane[0];
    }
    warp_tree_sum(partial);
    return partial[0];
}

// ---------------------------------------------------------------- compressed append
// One (token-or-sequence, kv head) block of turbo_kv_quantize*_kernel
// (kernels.cu:1504-1559 / 1586-1635), head_dim threads.
void quantize_head(uint8_t* dst_codes, uint16_t* dst_norm, const uint16_t* src,
                   const uint16_t* rotation, int head_dim, int bits,
                   float* rotated_out, float* margin_out) {
    float head_vec[kMaxBlock];
    float sq[kMaxBlock];
    for (int d = 0; d < head_dim; d++) {
        float val = h2f(src[d]);
        head_vec[d] = val;
        sq[d] = val * val;
    }
    float norm_sq = block_sum(sq, head_dim);
    float inv_norm = 1.0f / sqrtf(norm_sq + 1e-12f);  // rsqrtf (1523/1605)
    for (int d = 0; d < head_dim; d++) head_vec[d] *= inv_norm;

    uint8_t quant_idx[kMaxBlock];
    for (int d = 0; d < head_dim; d++) {
        const uint16_t* rot_row = rotation + (size_t)d * head_dim;
        float rotated = 0.0f;
        for (int k = 0; k < head_dim; k++) rotated = fmaf(h2f(rot_row[k]), head_vec[k], rotated);
        quant_idx[d] = (uint8_t)quantize(rotated, bits);
        if (rotated_out) rotated_out[d] = rotated;
        if (margin_out) margin_out[d] = margin(rotated, bits);
    }
    int vals_per_byte = bits == 2 ? 4 : 2;
    int bytes_per_head = head_dim / vals_per_byte;
    for (int b = 0; b < bytes_per_head; b++) {  // pack, 1543-1552
        uint8_t packed;
        if (bits == 2) {
            int base = b * 4;
            packed = (uint8_t)(quant_idx[base] | (quant_idx[base + 1] << 2) |
                               (quant_idx[base + 2] << 4) | (quant_idx[base + 3] << 6));
        } else {
            int base = b * 2;
            packed = (uint8_t)(quant_idx[base] | (quant_idx[base + 1] << 4));
        }
        dst_codes[b] = packed;
    }
    *dst_norm = f2h(sqrtf(norm_sq + 1e-12f));  // 1557-1558
}

// ---------------------------------------------------------------- softmax shared by all four attention kernels
// scores[0..n) hold the scaled dot products; on return they hold the
// normalised weights.  Thread t owns positions t, t+nthreads, ...
void block_softmax(float* scores, int n, int nthreads) {
    float max_score = -1e30f;
    for (int p = 0; p < n; p++) max_score = fmaxf(max_score, scores[p]);
    float per_thread[kMaxBlock] = {0.0f};
    for (int t = 0; t < nthreads; t++) {
        float sum_exp = 0.0f;
        for (int p = t; p < n; p += nthreads) {
            float v = expf(scores[p] - max_score);
            scores[p] = v;
            sum_exp += v;
        }
        per_thread[t] = sum_exp;
    }
    float total = block_sum(per_thread, nthreads);
    float inv_sum = 1.0f / (total + 1e-8f);
    for (int p = 0; p < n; p++) scores[p] *= inv_sum;
}

// One (sequence, head) block of the fp16 attention kernels
// (kernels.cu:996-1065, 266-344, 1086-1157).  kbase/vbase point at position 0
// of this sequence; row stride is kv_dim halves.
void fp16_attention_head(uint16_t* out_head, const uint16_t* q_head,
                         const uint16_t* kbase, const uint16_t* vbase,
                         int n, int kv_dim, int kv_head, int head_dim, int nthreads,
                         float* scores) {
    float scale = 1.0f / sqrtf((float)head_dim);
    for (int p = 0; p < n; p++) {
        const uint16_t* kp = kbase + (size_t)p * kv_dim + (size_t)kv_head * head_dim;
        float dot = 0.0f;
        for (int d = 0; d < head_dim; d++) dot = fmaf(h2f(q_head[d]), h2f(kp[d]), dot);
        scores[p] = dot * scale;
    }
    block_softmax(scores, n, nthreads);
    for (int d2 = 0; d2 < head_dim / 2; d2++) {
        float val0 = 0.0f, val1 = 0.0f;
        for (int p = 0; p < n; p++) {
            const uint16_t* vp = vbase + (size_t)p * kv_dim + (size_t)kv_head * head_dim + 2 * d2;
            float s = scores[p];
            val0 = fmaf(s, h2f(vp[0]), val0);
            val1 = fmaf(s, h2f(vp[1]), val1);
        }
        out_head[2 * d2] = f2h(val0);
        out_head[2 * d2 + 1] = f2h(val1);
    }
}

// One (sequence, head) block of the compressed attention kernels
// (kernels.cu:1671-1775, 1805-1869, 1898-1959).  codes/norms point at
// position 0 of this sequence.
void turbo_attention_head(uint16_t* out_head, const uint16_t* q_head,
                          const uint8_t* kq, const uint8_t* vq,
                          const uint16_t* kn, const uint16_t* vn,
                          const uint16_t* rotation,
                          int n, int num_kv_heads, int kv_head, int head_dim, int bits,
                          float* scores) {
    const int vals_per_byte = bits == 2 ? 4 : 2;
    const int bytes_per_head = head_dim / vals_per_byte;
    const int kv_dim_packed = num_kv_heads * bytes_per_head;
    const float scale = 1.0f / sqrtf((float)head_dim);
    const int mask = bits == 4 ? 0xF : 3;
    const float* C = bits == 4 ? CENTROIDS_4 : CENTROIDS_2;

    // Phase 1: q_rot = R q
    float q_raw[kMaxBlock], q_rot[kMaxBlock];
    for (int d = 0; d < head_dim; d++) q_raw[d] = h2f(q_head[d]);
    for (int d = 0; d < head_dim; d++) {
        const uint16_t* rot_row = rotation + (size_t)d * head_dim;
        float r = 0.0f;
        for (int k = 0; k < head_dim; k++) r = fmaf(h2f(rot_row[k]), q_raw[k], r);
        q_rot[d] = r;
    }
    // Phase 2: scores
    for (int p = 0; p < n; p++) {
        float k_norm = h2f(kn[(size_t)p * num_kv_heads + kv_head]);
        const uint8_t* row = kq + (size_t)p * kv_dim_packed + (size_t)kv_head * bytes_per_head;
        float dot = 0.0f;
        for (int b = 0; b < bytes_per_head; b++) {
            uint8_t packed = row[b];
            for (int j = 0; j < vals_per_byte; j++)
                dot = fmaf(q_rot[b * vals_per_byte + j], C[(packed >> (j * bits)) & mask], dot);
        }
        dot *= k_norm * scale;
        scores[p] = dot;
    }
    block_softmax(scores, n, head_dim);
    // Phase 3: V weighted sum in the rotated basis
    float v_acc[kMaxBlock];
    for (int d = 0; d < head_dim; d++) {
        int sub = d % vals_per_byte, byte_in_head = d / vals_per_byte;
        int bit_shift = sub * bits;
        float acc = 0.0f;
        for (int p = 0; p < n; p++) {
            float s = scores[p];
            float vnorm = h2f(vn[(size_t)p * num_kv_heads + kv_head]);
            uint8_t packed = vq[(size_t)p * kv_dim_packed + (size_t)kv_head * bytes_per_head + byte_in_head];
            int idx = (packed >> bit_shift) & mask;
            acc = fmaf(s * vnorm, centroid(idx, bits), acc);
        }
        v_acc[d] = acc;
    }
    // Phase 4: out = R^T v_acc
    for (int d = 0; d < head_dim; d++) {
        float o = 0.0f;
        for (int k = 0; k < head_dim; k++) o = fmaf(h2f(rotation[(size_t)k * head_dim + d]), v_acc[k], o);
        out_head[d] = f2h(o);
    }
}


// ---------------------------------------------------------------- producers of q and k: per-head RMSNorm and RoPE
// One block of qk_norm_kernel (kernels.cu:137-186, 128 threads) or qk_norm_batch_kernel
// (kernels.cu:880-923, head_dim threads): thread t sums v*v over i = t, t + nthreads, ...
// (fused multiply-adds), block sum, rms = rsqrtf(sum / head_dim + eps), then
// data[i] = half((float(data[i]) * rms) * w[i]), w[i] + 1 first when `biased`.
void norm_head(uint16_t* data, const uint16_t* w, int head_dim, int nthreads, float eps, bool biased) {
    float per_thread[1024];
    if (nthreads > 1024) abort();
    for (int t = 0; t < nthreads; t++) {
        float sum_sq = 0.0f;
        for (int i = t; i < head_dim; i += nthreads) {
            float v = h2f(data[i]);
            sum_sq = fmaf(v, v, sum_sq);
        }
        per_thread[t] = sum_sq;
    }
    float total = block_sum(per_thread, nthreads);
    float rms = 1.0f / sqrtf(total / (float)head_dim + eps);   // rsqrtf (kernels.cu:179, 916)
    for (int i = 0; i < head_dim; i++) {
        float wv = h2f(w[i]);
        if (biased) wv += 1.0f;
        data[i] = f2h((h2f(data[i]) * rms) * wv);
    }
}

}  // namespace

extern "C" {

uint16_t tw_oracle_f32_to_f16(float x) { return f2h(x); }
float tw_oracle_f16_to_f32(uint16_t h) { return h2f(h); }
const float* tw_oracle_centroids(int bits) { return bits == 4 ? CENTROIDS_4 : CENTROIDS_2; }
const float* tw_oracle_bounds(int bits) { return bits == 4 ? BOUNDS_4 : BOUNDS_2; }
int tw_oracle_quantize(float val, int bits) { return quantize(val, bits); }
float tw_oracle_margin(float val, int bits) { return margin(val, bits); }

int tw_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
void tw_oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

// engine.cpp:366-392
void tw_oracle_make_rotation(uint16_t* out_f16, float* out_f32, int d, uint32_t seed) {
    std::mt19937 gen(seed);
    std::normal_distribution<float> dist(0.0f, 1.0f);
    std::vector<float> mat((size_t)d * d);
    for (int i = 0; i < d * d; i++) mat[i] = dist(gen);
    for (int i = 0; i < d; i++) {
        for (int j = 0; j < i; j++) {
            float dot = 0;
            for (int k = 0; k < d; k++) dot += mat[i * d + k] * mat[j * d + k];
            for (int k = 0; k < d; k++) mat[i * d + k] -= dot * mat[j * d + k];
        }
        float norm = 0;
        for (int k = 0; k < d; k++) norm += mat[i * d + k] * mat[i * d + k];
        norm = 1.0f / sqrtf(norm);
        for (int k = 0; k < d; k++) mat[i * d + k] *= norm;
    }
    for (int i = 0; i < d * d; i++) {
        out_f16[i] = f2h(mat[i]);
        if (out_f32) out_f32[i] = mat[i];
    }
}

void tw_oracle_kv_cache_write_batch(uint16_t* cache_k, uint16_t* cache_v,
                                    const uint16_t* k, const uint16_t* v,
                                    const int* positions, int max_seq_len, int G, int kv_dim) {
    for (int g = 0; g < G; g++) {
        int pos = positions[g];
        for (int d = 0; d < kv_dim; d++) {
            size_t src = (size_t)d + (size_t)g * kv_dim;
            size_t dst = ((size_t)g * max_seq_len + pos) * kv_dim + d;
            cache_k[dst] = k[src];
            cache_v[dst] = v[src];
        }
    }
}

void tw_oracle_turbo_kv_quantize(uint8_t* cache_q, uint16_t* cache_norms,
                                 const uint16_t* kv_buf, const uint16_t* rotation,
                                 const int* positions, int max_seq_len, int num_tokens,
                                 int num_kv_heads, int head_dim, int kv_dim, int bits,
                                 float* rotated_out, float* margin_out) {
    (void)max_seq_len;
    if (head_dim > kMaxBlock) abort();
    const int vpb = bits == 2 ? 4 : 2;
    const int bph = head_dim / vpb, kvp = kv_dim / vpb;
#pragma omp parallel for collapse(2) schedule(static)
    for (int tok = 0; tok < num_tokens; tok++) {
        for (int h = 0; h < num_kv_heads; h++) {
            int pos = positions[tok];
            size_t in = (size_t)tok * kv_dim + (size_t)h * head_dim;
            quantize_head(cache_q + (size_t)pos * kvp + (size_t)h * bph,
                          cache_norms + (size_t)pos * num_kv_heads + h,
                          kv_buf + in, rotation, head_dim, bits,
                          rotated_out ? rotated_out + in : nullptr,
                          margin_out ? margin_out + in : nullptr);
        }
    }
}

void tw_oracle_turbo_kv_quantize_batch(uint8_t* cache_q, uint16_t* cache_norms,
                                       const uint16_t* kv_buf, const uint16_t* rotation,
                                       const int* positions, int max_seq_len, int G,
                                       int num_kv_heads, int head_dim, int kv_dim, int bits,
                                       float* rotated_out, float* margin_out) {
    if (head_dim > kMaxBlock) abort();
    const int vpb = bits == 2 ? 4 : 2;
    const int bph = head_dim / vpb, kvp = kv_dim / vpb;
#pragma omp parallel for collapse(2) schedule(static)
    for (int g = 0; g < G; g++) {
        for (int h = 0; h < num_kv_heads; h++) {
            int pos = positions[g];
            size_t row = (size_t)g * max_seq_len + pos;
            size_t in = (size_t)g * kv_dim + (size_t)h * head_dim;
            quantize_head(cache_q + row * kvp + (size_t)h * bph,
                          cache_norms + row * num_kv_heads + h,
                          kv_buf + in, rotation, head_dim, bits,
                          rotated_out ? rotated_out + in : nullptr,
                          margin_out ? margin_out + in : nullptr);
        }
    }
}

void tw_oracle_gqa_attention(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                             uint16_t* output, int pos, int max_seq_len,
                             int num_heads, int num_kv_heads, int head_dim) {
    (void)max_seq_len;
    const int kv_dim = num_kv_heads * head_dim;
    const int groups = num_heads / num_kv_heads;
#pragma omp parallel for schedule(dynamic)
    for (int head = 0; head < num_heads; head++) {
        std::vector<float> scores((size_t)pos + 1);
        fp16_attention_head(output + (size_t)head * head_dim, q + (size_t)head * head_dim,
                            k_cache, v_cache, pos + 1, kv_dim, head / groups, head_dim,
                            /*blockDim=*/128, scores.data());
    }
}

void tw_oracle_gqa_attention_batch(uint16_t* out, const uint16_t* q,
                                   const uint16_t* cache_k, const uint16_t* cache_v,
                                   const int* positions, int max_seq_len, int G,
                                   int num_heads, int num_kv_heads, int head_dim,
                                   int q_dim, int kv_dim) {
    if (head_dim > kMaxBlock) abort();
    const int groups = num_heads / num_kv_heads;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int g = 0; g < G; g++) {
        for (int head = 0; head < num_heads; head++) {
            int pos = positions[g];
            std::vector<float> scores((size_t)pos + 1);
            size_t seq = (size_t)g * max_seq_len * kv_dim;
            fp16_attention_head(out + (size_t)g * q_dim + (size_t)head * head_dim,
                                q + (size_t)g * q_dim + (size_t)head * head_dim,
                                cache_k + seq, cache_v + seq, pos + 1, kv_dim, head / groups,
                                head_dim, /*blockDim=*/head_dim, scores.data());
        }
    }
}

void tw_oracle_gqa_prefill_attention(uint16_t* out, const uint16_t* q,
                                     const uint16_t* cache_k, const uint16_t* cache_v,
                                     int T, int max_seq_len,
                                     int num_heads, int num_kv_heads, int head_dim,
                                     int q_dim, int kv_dim) {
    (void)max_seq_len;
    if (head_dim > kMaxBlock) abort();
    const int groups = num_heads / num_kv_heads;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int tq = 0; tq < T; tq++) {
        for (int head = 0; head < num_heads; head++) {
            std::vector<float> scores((size_t)tq + 1);
            fp16_attention_head(out + (size_t)tq * q_dim + (size_t)head * head_dim,
                                q + (size_t)tq * q_dim + (size_t)head * head_dim,
                                cache_k, cache_v, tq + 1, kv_dim, head / groups,
                                head_dim, /*blockDim=*/head_dim, scores.data());
        }
    }
}

void tw_oracle_turbo_gqa_attention(const uint16_t* q,
                                   const uint8_t* ck_q, const uint8_t* cv_q,
                                   const uint16_t* k_norms, const uint16_t* v_norms,
                                   const uint16_t* rotation, uint16_t* output,
                                   int pos, int max_seq_len,
                                   int num_heads, int num_kv_heads, int head_dim, int bits) {
    (void)max_seq_len;
    if (head_dim > kMaxBlock) abort();
    const int groups = num_heads / num_kv_heads;
#pragma omp parallel for schedule(dynamic)
    for (int head = 0; head < num_heads; head++) {
        std::vector<float> scores((size_t)pos + 1);
        turbo_attention_head(output + (size_t)head * head_dim, q + (size_t)head * head_dim,
                             ck_q, cv_q, k_norms, v_norms, rotation, pos + 1,
                             num_kv_heads, head / groups, head_dim, bits, scores.data());
    }
}

void tw_oracle_turbo_gqa_attention_batch(uint16_t* out, const uint16_t* q,
                                         const uint8_t* ck_q, const uint8_t* cv_q,
                                         const uint16_t* k_norms, const uint16_t* v_norms,
                                         const uint16_t* rotation,
                                         const int* positions, int max_seq_len, int G,
                                         int num_heads, int num_kv_heads, int head_dim,
                                         int q_dim, int kv_dim, int bits) {
    if (head_dim > kMaxBlock) abort();
    const int groups = num_heads / num_kv_heads;
    const int vpb = bits == 2 ? 4 : 2;
    const size_t kvp = (size_t)kv_dim / vpb;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int g = 0; g < G; g++) {
        for (int head = 0; head < num_heads; head++) {
            int pos = positions[g];
            std::vector<float> scores((size_t)pos + 1);
            size_t seq = (size_t)g * max_seq_len;
            turbo_attention_head(out + (size_t)g * q_dim + (size_t)head * head_dim,
                                 q + (size_t)g * q_dim + (size_t)head * head_dim,
                                 ck_q + seq * kvp, cv_q + seq * kvp,
                                 k_norms + seq * num_kv_heads, v_norms + seq * num_kv_heads,
                                 rotation, pos + 1, num_kv_heads, head / groups, head_dim, bits,
                                 scores.data());
        }
    }
}

void tw_oracle_turbo_gqa_prefill_attention(uint16_t* out, const uint16_t* q,
                                           const uint8_t* ck_q, const uint8_t* cv_q,
                                           const uint16_t* k_norms, const uint16_t* v_norms,
                                           const uint16_t* rotation,
                                           int T, int max_seq_len,
                                           int num_heads, int num_kv_heads, int head_dim,
                                           int q_dim, int kv_dim, int bits) {
    (void)max_seq_len;
    (void)kv_dim;
    if (head_dim > kMaxBlock) abort();
    const int groups = num_heads / num_kv_heads;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int tq = 0; tq < T; tq++) {
        for (int head = 0; head < num_heads; head++) {
            std::vector<float> scores((size_t)tq + 1);
            turbo_attention_head(out + (size_t)tq * q_dim + (size_t)head * head_dim,
                                 q + (size_t)tq * q_dim + (size_t)head * head_dim,
                                 ck_q, cv_q, k_norms, v_norms, rotation, tq + 1,
                                 num_kv_heads, head / groups, head_dim, bits, scores.data());
        }
    }
}

void tw_oracle_increment_positions(int* positions, int G) {
    for (int g = 0; g < G; g++) positions[g]++;
}

void tw_oracle_qk_norm(uint16_t* q, uint16_t* k, const uint16_t* q_weight, const uint16_t* k_weight,
                       int num_q_heads, int num_kv_heads, int head_dim, float eps) {
    // launch_qk_norm (kernels.cu:706-717): one block of 128 threads per head, Q heads first
    for (int h = 0; h < num_q_heads; h++) norm_head(q + (size_t)h * head_dim, q_weight, head_dim, 128, eps, false);
    for (int h = 0; h < num_kv_heads; h++) norm_head(k + (size_t)h * head_dim, k_weight, head_dim, 128, eps, false);
}

void tw_oracle_qk_norm_batch(uint16_t* q, uint16_t* k, const uint16_t* q_weight, const uint16_t* k_weight,
                             int num_q, int num_kv, int head_dim, int G, float eps,
                             int q_dim, int kv_dim, int biased) {
    // launch_qk_norm_batch (kernels.cu:1345-1347): G * (num_q + num_kv) blocks of head_dim threads
    for (int g = 0; g < G; g++) {
        for (int h = 0; h < num_q; h++)
            norm_head(q + (size_t)g * q_dim + (size_t)h * head_dim, q_weight, head_dim, head_dim, eps, biased != 0);
        for (int h = 0; h < num_kv; h++)
            norm_head(k + (size_t)g * kv_dim + (size_t)h * head_dim, k_weight, head_dim, head_dim, eps, biased != 0);
    }
}

void tw_oracle_rope(uint16_t* q, uint16_t* k, const uint16_t* cos_table, const uint16_t* sin_table,
                    int pos, int max_seq_len, int num_heads, int num_kv_heads, int head_dim) {
    // launch_rope + rope_kernel (kernels.cu:719-735, 193-235): table row `pos` of head_dim/2 entries;
    // out0 = q0*c - q1*s, out1 = q1*c + q0*s, each one multiply and one fused multiply-add
    (void)max_seq_len;
    const int half = head_dim / 2;
    const uint16_t* ct = cos_table + (size_t)pos * half;
    const uint16_t* st = sin_table + (size_t)pos * half;
    for (int pass = 0; pass < 2; pass++) {
        uint16_t* x = pass ? k : q;
        const int heads = pass ? num_kv_heads : num_heads;
        for (int h = 0; h < heads; h++) {
            uint16_t* xh = x + (size_t)h * head_dim;
            for (int d = 0; d < half; d++) {
                float c = h2f(ct[d]), sn = h2f(st[d]);
                float x0 = h2f(xh[d]), x1 = h2f(xh[d + half]);
                xh[d] = f2h(fmaf(x0, c, -(x1 * sn)));
                xh[d + half] = f2h(fmaf(x1, c, x0 * sn));
            }
        }
    }
}

void tw_oracle_rope_batch(uint16_t* q, uint16_t* k, const uint16_t* cos_table, const uint16_t* sin_table,
                          const int* positions, int max_seq_len, int G, int num_heads, int num_kv_heads,
                          int head_dim, int q_dim, int kv_dim, int rope_dim) {
    // rope_batch_kernel (kernels.cu:927-961): table row positions[g] of rope_dim/2 entries; only the first
    // rope_dim coordinates of a head turn; out0 = q0*c - q1*s, out1 = q0*s + q1*c
    (void)max_seq_len;
    const int half = rope_dim / 2;
    for (int g = 0; g < G; g++) {
        const int pos = positions[g];
        const uint16_t* ct = cos_table + (size_t)pos * half;
        const uint16_t* st = sin_table + (size_t)pos * half;
        for (int pass = 0; pass < 2; pass++) {
            uint16_t* x = pass ? k + (size_t)g * kv_dim : q + (size_t)g * q_dim;
            const int heads = pass ? num_kv_heads : num_heads;
            for (int h = 0; h < heads; h++) {
                uint16_t* xh = x + (size_t)h * head_dim;
                for (int d = 0; d < half; d++) {
                    float c = h2f(ct[d]), sn = h2f(st[d]);
                    float x0 = h2f(xh[d]), x1 = h2f(xh[d + half]);
                    xh[d] = f2h(fmaf(x0, c, -(x1 * sn)));
                    xh[d + half] = f2h(fmaf(x0, sn, x1 * c));
                }
            }
        }
    }
}

void tw_oracle_rope_tables(uint16_t* cos_table, uint16_t* sin_table, int max_seq_len, int rope_dim, float theta) {
    // precompute_rope (engine.cpp:554-574); powf, cosf and sinf are this machine's libm
    const int half = rope_dim / 2;
    for (int pos = 0; pos < max_seq_len; pos++) {
        for (int d = 0; d < half; d++) {
            float freq = 1.0f / powf(theta, (float)(2 * d) / rope_dim);
            float angle = pos * freq;
            cos_table[(size_t)pos * half + d] = f2h(cosf(angle));
            sin_table[(size_t)pos * half + d] = f2h(sinf(angle));
        }
    }
}

void tw_oracle_sigmoid_gate_batch(uint16_t* data, const uint16_t* gate, int dim, int G) {
    // sigmoid_gate_batch_kernel (kernels.cu:2987-2995): data[i] = half(d / (1 + expf(-g))) over dim * G elements
    const long long total = (long long)dim * G;
    for (long long i = 0; i < total; i++) {
        float d = h2f(data[i]);
        float g = h2f(gate[i]);
        data[i] = f2h(d / (1.0f + expf(-g)));
    }
}

}  // extern "C"
