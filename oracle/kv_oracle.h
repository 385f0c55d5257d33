/*
 * kv_oracle.h -- CPU restatement of the triebwerk engine's KV-cache kernels.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the parity checker and the timed
 * CPU baseline.  Nothing in the shipped GPU path may call it: only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg load it.
 *
 * Every function follows one CUDA kernel (or host routine) of the reference
 * operation for operation: fp32 arithmetic, every `acc += a*b` of the source
 * is a fused multiply-add (nvcc contracts by default), loops run in the
 * source's order, and block reductions use the source's reduction tree
 * (32-lane shuffle-down tree, then a tree over the 4 warp sums).
 *
 * What the restatement cannot reproduce: the reference is built with
 * --use_fast_math (engine/CMakeLists.txt:13), so on an NVIDIA GPU rsqrtf,
 * expf, sqrtf and 1/x are approximate.  Here they are IEEE correctly rounded.
 *
 * Parity pins (all under tests/, none of them needs the reference to run):
 *   tables        : antisymmetry, boundaries = midpoints of centroids,
 *                   Lloyd-Max fixed point on N(0,1/128) re-derived numerically
 *   quantize      : brute force over every bin edge, NaN, +-inf, monotone
 *   pack          : exhaustive over all byte patterns, low field first
 *   rotation      : committed fixture (libstdc++ normal_distribution), R R^T = I
 *   append        : independent numpy restatement; reconstruction error equals
 *                   the Lloyd-Max distortion; zero rows
 *   fp16 attention: float64 softmax(QK^T/sqrt(D))V
 *   turbo attn    : float64 attention on the dequantized cache (identity)
 *   bookkeeping   : brute-force position model on tiny shapes
 *   qk norm, rope : float64 RMSNorm and complex rotation; position 0 and unit weights are
 *                   identities bit for bit; pair norms are kept; strides leave gaps untouched
 * The reference ships no golden vector, test or fixture for this path, so the
 * kernel source text is the only authority the restatement can be read against.
 * What stays unpinned: the fast-math last-ulp behaviour of the CUDA build.
 *
 * half is passed as uint16_t (IEEE binary16 bit pattern).
 */
#ifndef TW_KV_ORACLE_H
#define TW_KV_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* fp16 <-> fp32, round-to-nearest-even (CUDA __float2half / __half2float). */
uint16_t tw_oracle_f32_to_f16(float x);
float    tw_oracle_f16_to_f32(uint16_t h);

/* Lloyd-Max tables, kernels.cu:1426-1445.  bits in {2,4}. */
const float* tw_oracle_centroids(int bits);   /* 4 or 16 entries  */
const float* tw_oracle_bounds(int bits);      /* 3 or 15 entries  */
/* turbo_quantize, kernels.cu:1448-1473. */
int tw_oracle_quantize(float val, int bits);
/* distance of val to the nearest bin boundary of the `bits` table. */
float tw_oracle_margin(float val, int bits);

/* Rotation matrix, engine.cpp:366-392: mt19937(seed), normal_distribution<float>,
 * modified Gram-Schmidt over rows in fp32, then fp16 RNE.  d*d outputs.
 * out_f32 may be NULL. */
void tw_oracle_make_rotation(uint16_t* out_f16, float* out_f32, int d, uint32_t seed);

/* kv_cache_write_batch_kernel, kernels.cu:964-977. */
void tw_oracle_kv_cache_write_batch(uint16_t* cache_k, uint16_t* cache_v,
                                    const uint16_t* k, const uint16_t* v,
                                    const int* positions, int max_seq_len, int G, int kv_dim);

/* turbo_kv_quantize_kernel, kernels.cu:1482-1560 (token list, sequence 0).
 * rotated_out / margin_out (num_tokens*kv_dim floats each) may be NULL. */
void tw_oracle_turbo_kv_quantize(uint8_t* cache_q, uint16_t* cache_norms,
                                 const uint16_t* kv_buf, const uint16_t* rotation,
                                 const int* positions, int max_seq_len, int num_tokens,
                                 int num_kv_heads, int head_dim, int kv_dim, int bits,
                                 float* rotated_out, float* margin_out);

/* turbo_kv_quantize_batch_kernel, kernels.cu:1563-1636. */
void tw_oracle_turbo_kv_quantize_batch(uint8_t* cache_q, uint16_t* cache_norms,
                                       const uint16_t* kv_buf, const uint16_t* rotation,
                                       const int* positions, int max_seq_len, int G,
                                       int num_kv_heads, int head_dim, int kv_dim, int bits,
                                       float* rotated_out, float* margin_out);

/* gqa_attention_decode_kernel, kernels.cu:244-345 (single sequence, pos by value). */
void tw_oracle_gqa_attention(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                             uint16_t* output, int pos, int max_seq_len,
                             int num_heads, int num_kv_heads, int head_dim);

/* gqa_attention_batch_kernel, kernels.cu:981-1066. */
void tw_oracle_gqa_attention_batch(uint16_t* out, const uint16_t* q,
                                   const uint16_t* cache_k, const uint16_t* cache_v,
                                   const int* positions, int max_seq_len, int G,
                                   int num_heads, int num_kv_heads, int head_dim,
                                   int q_dim, int kv_dim);

/* gqa_prefill_attention_kernel, kernels.cu:1071-1158 (causal, sequence 0). */
void tw_oracle_gqa_prefill_attention(uint16_t* out, const uint16_t* q,
                                     const uint16_t* cache_k, const uint16_t* cache_v,
                                     int T, int max_seq_len,
                                     int num_heads, int num_kv_heads, int head_dim,
                                     int q_dim, int kv_dim);

/* turbo_gqa_attention_kernel, kernels.cu:1779-1870. */
void tw_oracle_turbo_gqa_attention(const uint16_t* q,
                                   const uint8_t* ck_q, const uint8_t* cv_q,
                                   const uint16_t* k_norms, const uint16_t* v_norms,
                                   const uint16_t* rotation, uint16_t* output,
                                   int pos, int max_seq_len,
                                   int num_heads, int num_kv_heads, int head_dim, int bits);

/* turbo_gqa_attention_batch_kernel, kernels.cu:1641-1776. */
void tw_oracle_turbo_gqa_attention_batch(uint16_t* out, const uint16_t* q,
                                         const uint8_t* ck_q, const uint8_t* cv_q,
                                         const uint16_t* k_norms, const uint16_t* v_norms,
                                         const uint16_t* rotation,
                                         const int* positions, int max_seq_len, int G,
                                         int num_heads, int num_kv_heads, int head_dim,
                                         int q_dim, int kv_dim, int bits);

/* turbo_gqa_prefill_attention_kernel, kernels.cu:1874-1960. */
void tw_oracle_turbo_gqa_prefill_attention(uint16_t* out, const uint16_t* q,
                                           const uint8_t* ck_q, const uint8_t* cv_q,
                                           const uint16_t* k_norms, const uint16_t* v_norms,
                                           const uint16_t* rotation,
                                           int T, int max_seq_len,
                                           int num_heads, int num_kv_heads, int head_dim,
                                           int q_dim, int kv_dim, int bits);

/* increment_positions_kernel, kernels.cu:1371-1374. */
void tw_oracle_increment_positions(int* positions, int G);

/* Producers of q and k, the step before the append (engine.cpp:1972-1977).
 * qk_norm_kernel (kernels.cu:137-186) / qk_norm_batch_kernel (880-923): per-head RMSNorm in place;
 * q_dim / kv_dim are row strides; biased adds 1 to the weights.
 * rope_kernel (193-235) / rope_batch_kernel (927-961): rotary embedding in place from fp16 tables
 * of rope_dim/2 entries per position (single sequence: rope_dim = head_dim).  The two differ in the
 * operand order of the second output (q1*c + q0*s against q0*s + q1*c).
 * `a*b - c*d` and `a*b + c*d` are restated as fma(a, b, -(c*d)) and fma(a, b, c*d): the first product
 * fused, the second rounded -- which product nvcc fuses is a last-ulp question only a run of the
 * CUDA build could settle (parity unpinned at that level, like the fast-math ulps). */
void tw_oracle_qk_norm(uint16_t* q, uint16_t* k, const uint16_t* q_weight, const uint16_t* k_weight,
                       int num_q_heads, int num_kv_heads, int head_dim, float eps);
void tw_oracle_qk_norm_batch(uint16_t* q, uint16_t* k, const uint16_t* q_weight, const uint16_t* k_weight,
                             int num_q, int num_kv, int head_dim, int G, float eps,
                             int q_dim, int kv_dim, int biased);
void tw_oracle_rope(uint16_t* q, uint16_t* k, const uint16_t* cos_table, const uint16_t* sin_table,
                    int pos, int max_seq_len, int num_heads, int num_kv_heads, int head_dim);
void tw_oracle_rope_batch(uint16_t* q, uint16_t* k, const uint16_t* cos_table, const uint16_t* sin_table,
                          const int* positions, int max_seq_len, int G, int num_heads, int num_kv_heads,
                          int head_dim, int q_dim, int kv_dim, int rope_dim);
/* precompute_rope, engine.cpp:554-574. */
void tw_oracle_rope_tables(uint16_t* cos_table, uint16_t* sin_table, int max_seq_len, int rope_dim, float theta);

/* sigmoid_gate_batch_kernel, kernels.cu:2987-3000: data *= sigmoid(gate), elementwise over dim*G
 * halves (gated attention, engine.cpp:2009-2012).  expf and the division are this machine's IEEE
 * ones; the reference's fast-math versions differ in the last bits (floating-point tolerance). */
void tw_oracle_sigmoid_gate_batch(uint16_t* data, const uint16_t* gate, int dim, int G);

/* Threads the OpenMP loops over (sequence, head) will use. */
int  tw_oracle_num_threads(void);
void tw_oracle_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
