/*
 * triebwerk_kv.h -- C ABI of the MI355X (gfx950) KV-cache hot path.
 *
 * Part 1 keeps the reference engine's own kernel-launcher boundary: the
 * `extern "C" void launch_*` functions that engine/engine.cpp declares at
 * lines 105-171 and engine/kernels.cu defines.  Names, parameter order and
 * parameter meaning are unchanged; `cudaStream_t` becomes `hipStream_t` and
 * `half*` is any pointer to IEEE binary16 storage.  A HIP build of the engine
 * links this library in place of the reference's `kernels` static library for
 * these entry points.
 *
 * Part 2 is what the reference does inline in engine.cpp for the same path
 * (cache sizing, arena carving, reset, rotation matrix, decode-step graph) plus
 * the paged-cache and fused-append entry points that have no counterpart there.
 *
 * Conventions (same as the reference, engine.cpp:105-171):
 *   - every pointer is a device pointer unless a comment says "host";
 *   - launchers are asynchronous on `stream`, allocate nothing, keep no pointer,
 *     and return void; a failed launch or a rejected argument is recorded and
 *     can be read with tw_kv_last_error() (the reference checks nothing);
 *   - activations are row-per-sequence: x[g * dim + i];
 *   - head_dim must be 128 (the reference kernels hard-size their shared
 *     arrays to 128, kernels.cu:1504, 1671);
 *   - attention covers cache positions 0..pos INCLUSIVE (kernels.cu:1688).
 */
#ifndef TRIEBWERK_KV_H
#define TRIEBWERK_KV_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifndef TW_HALF_T
#define TW_HALF_T uint16_t /* IEEE binary16 storage; `half` in the reference */
#endif
typedef TW_HALF_T tw_half;

#ifndef HIP_INCLUDE_HIP_HIP_RUNTIME_API_H
typedef struct ihipStream_t* hipStream_t;
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ Part 1
 * Reference launchers (drop-in).                                            */

/* engine.cpp:128, kernels.cu:1351 -- fp16 append of one K row and one V row
 * per sequence at cache row (g*msl + pos[g]). */
void launch_kv_cache_write_batch(tw_half* ck, tw_half* cv, const tw_half* k, const tw_half* v,
                                 const int* pos, int msl, int G, int kv_dim, hipStream_t s);

/* engine.cpp:136, kernels.cu:1963 -- compressed append of `num_tokens` rows of
 * sequence 0 at rows positions[tok] (prefill and single-sequence decode). */
void launch_turbo_kv_quantize(uint8_t* cache_q, tw_half* cache_norms, const tw_half* kv_buf,
                              const tw_half* rotation, const int* positions, int max_seq_len,
                              int num_tokens, int num_kv_heads, int head_dim, int kv_dim,
                              int bits, hipStream_t s);

/* engine.cpp:137, kernels.cu:1975 -- compressed append, one row per sequence at
 * row (g*max_seq_len + positions[g]).  Called once for K and once for V. */
void launch_turbo_kv_quantize_batch(uint8_t* cache_q, tw_half* cache_norms, const tw_half* kv_buf,
                                    const tw_half* rotation, const int* positions, int max_seq_len,
                                    int G, int num_kv_heads, int head_dim, int kv_dim,
                                    int bits, hipStream_t s);

/* engine.cpp:164, kernels.cu:737 -- fp16 decode attention, one sequence, `pos`
 * by value.  attn_scratch: num_heads*max_seq_len floats. */
void launch_gqa_attention(const tw_half* q, const tw_half* k_cache, const tw_half* v_cache,
                          tw_half* output, float* attn_scratch, int pos, int max_seq_len,
                          int num_heads, int num_kv_heads, int head_dim, hipStream_t stream);

/* engine.cpp:129, kernels.cu:1354 -- fp16 decode attention for G sequences,
 * positions read from device memory (graph-capturable).  q_dim is the row
 * stride of q and out.  as: G*num_heads*msl floats, used as split-K workspace. */
void launch_gqa_attention_batch(tw_half* out, const tw_half* q, const tw_half* ck,
                                const tw_half* cv, float* as, const int* pos, int msl, int G,
                                int num_heads, int num_kv_heads, int head_dim, int q_dim,
                                int kv_dim, hipStream_t s);

/* engine.cpp:139, kernels.cu:2001 -- compressed decode attention, one sequence. */
void launch_turbo_gqa_attention(const tw_half* q, const uint8_t* ck_q, const uint8_t* cv_q,
                                const tw_half* k_norms, const tw_half* v_norms,
                                const tw_half* rotation, tw_half* output, float* as, int pos,
                                int msl, int num_heads, int num_kv_heads, int head_dim, int bits,
                                hipStream_t s);

/* engine.cpp:138, kernels.cu:1986 -- compressed decode attention, G sequences. */
void launch_turbo_gqa_attention_batch(tw_half* out, const tw_half* q, const uint8_t* ck_q,
                                      const uint8_t* cv_q, const tw_half* k_norms,
                                      const tw_half* v_norms, const tw_half* rotation, float* as,
                                      const int* pos, int msl, int G, int num_heads,
                                      int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                      int bits, hipStream_t s);

/* engine.cpp:130, kernels.cu:1359 -- causal fp16 prefill attention over
 * sequence 0: query tq attends rows 0..tq.  as: T*num_heads*T floats. */
void launch_gqa_prefill_attention(tw_half* out, const tw_half* q, const tw_half* ck,
                                  const tw_half* cv, float* as, int T, int msl, int num_heads,
                                  int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                  hipStream_t s);

/* engine.cpp:140, kernels.cu:2015 -- causal compressed prefill attention. */
void launch_turbo_gqa_prefill_attention(tw_half* out, const tw_half* q, const uint8_t* ck_q,
                                        const uint8_t* cv_q, const tw_half* k_norms,
                                        const tw_half* v_norms, const tw_half* rotation, float* as,
                                        int T, int msl, int num_heads, int num_kv_heads,
                                        int head_dim, int q_dim, int kv_dim, int bits,
                                        hipStream_t s);

/* engine.cpp:133, kernels.cu:1376 -- positions[g] += 1 on the device. */
void launch_increment_positions(int* positions, int G, hipStream_t s);

/* The producers of q and k, the step in front of the append (forward_layer_batch step 3,
 * engine.cpp:1972-1977; single sequence engine.cpp:1060-1066).  In place, fp16 in and out.
 *
 * engine.cpp:126, kernels.cu:1345 -- per-head RMSNorm of the num_q heads of every q row and the
 * num_kv heads of every k row; q_dim and kv_dim are row strides (a gated q projection passes
 * 2*num_q*head_dim and the gate half stays untouched); `biased` adds 1 to the weights. */
void launch_qk_norm_batch(tw_half* q, tw_half* k, const tw_half* q_weight, const tw_half* k_weight,
                          int num_q, int num_kv, int head_dim, int G, float eps, int q_dim,
                          int kv_dim, hipStream_t s, bool biased);

/* engine.cpp:127, kernels.cu:1348 -- rotary embedding of the first rope_dim coordinates of every
 * head of q and k with the table row positions[g] (rope_dim/2 entries per position).  rope_dim:
 * 128, or a multiple of 16 up to 64. */
void launch_rope_batch(tw_half* q, tw_half* k, const tw_half* cos_table, const tw_half* sin_table,
                       const int* positions, int max_seq_len, int G, int num_heads,
                       int num_kv_heads, int head_dim, int q_dim, int kv_dim, int rope_dim,
                       hipStream_t s);

/* engine.cpp:162, kernels.cu:706 -- per-head RMSNorm, one sequence. */
void launch_qk_norm(tw_half* q, tw_half* k, const tw_half* q_weight, const tw_half* k_weight,
                    int num_q_heads, int num_kv_heads, int head_dim, float eps, hipStream_t stream);

/* engine.cpp:163, kernels.cu:719 -- rotary embedding, one sequence, `pos` by value, full width
 * (table rows of head_dim/2 entries). */
void launch_rope(tw_half* q, tw_half* k, const tw_half* cos_table, const tw_half* sin_table,
                 int pos, int max_seq_len, int num_heads, int num_kv_heads, int head_dim,
                 hipStream_t stream);

/* engine.cpp:158, kernels.cu:2997 -- gated attention: data[i] = data[i] * sigmoid(gate[i]) over
 * dim*G halves (forward_layer_batch step 6, engine.cpp:2009-2012). */
void launch_sigmoid_gate_batch(tw_half* data, const tw_half* gate, int dim, int G, hipStream_t s);

/* ------------------------------------------------------------------ Part 2
 * Error state, tuning and the entry points the reference has no twin for.   */

/* 0 = no error since the last call to tw_kv_clear_error().  Thread-local. */
int tw_kv_last_error(void);
const char* tw_kv_last_error_string(void);
void tw_kv_clear_error(void);

/* Library version / build info, for the loader to print. */
const char* tw_kv_build_info(void);

/* ---- Test and benchmark hooks (tw_kv_debug_*).  They force a kernel family, a split count or a kernel form so
 * that every path can be checked against the oracle and timed; production callers leave them alone.  All of them
 * are process-wide switches read at every launch and not synchronised with launches on other threads: set them
 * while no other thread is inside the library. */

/* Compressed-attention kernel family: 0 = automatic, 1 = fp32 vector-ALU kernels, 2 = MFMA kernels, 3 = MFMA kernels
 * with one KV head per wave also where the scan would give a wave two; 3 also keeps the fp16 cache on the kernel whose
 * workgroups scan one KV head where the one whose waves read whole rows of eight heads would run. */
void tw_kv_debug_set_attention_variant(int variant);
int tw_kv_debug_get_attention_variant(void);
/* Split count of decode attention (0 = automatic). */
void tw_kv_debug_set_num_splits(int nsplit);
/* Form of the matrix-core prefill kernels: 0 = chosen from the prompt length, 1 = one 16-row query block per wave,
 * 2 = the same with mirrored block pairs, 3 = two query blocks per wave with mirrored pairs, 4 = compressed cache
 * only: the kernel that expands tiles per wave, 5 and 6 = forms 2 and 3 with eight waves per
 * workgroup instead of four. */
void tw_kv_debug_set_prefill_form(int form);
/* tw_turbo_append_attention_batch and the calls built on it can run a layer's decode step as ONE kernel (append,
 * query rotation, scan, merge, rotate-back; a workgroup owns a sequence's heads) instead of three.  0 (default):
 * what tw_kv_decode_step_plan says; 1: one kernel whenever the shape allows it (contiguous compressed cache, GQA
 * group 1, 2 or 4); 2: never; 3: as 1, with one KV head per wave also where the 4-bit kernel would give a wave two. */
void tw_kv_debug_set_decode_fused(int mode);
/* Timing of the context-scanning attention kernel alone, with HIP events attached to that kernel's launches on
 * their stream.  Enable, run eager launches (not under stream capture; at most 4096 are kept), then read the
 * summed duration and the launch count.  Reading waits for the recorded launches and resets the counter. */
void tw_kv_debug_profile_attention(int enable);
int tw_kv_debug_profile_read(double* total_ms, int* launches);
/* Name of the kernel that the last attention call of this process launched (or recorded into a graph) for the
 * context: "attention_pair_kernel", "attention_mfma_kernel", "attention_rows_kernel", "attention_valu_kernel",
 * "decode_fused_kernel, two KV heads per wave", "decode_fused_kernel, one KV head per wave", a prefill kernel, or
 * "none".  A static string; lets a benchmark name the kernel its figures belong to. */
const char* tw_kv_debug_last_scan_kernel(void);

/* One launch or three for a layer's decode step over the compressed cache, as a pure function of what the host
 * knows (1 = one launch, 0 = three): G sequences,
 * cache width `bits`, max_seq_len, and the range of positions + 1 (ctx_max = 0: unknown).  One launch when every
 * wave gets at most 8 tiles of 32 tokens, or when the lengths are within 1/8 of each other and the one launch is the
 * cheaper of the two by estimates fitted to measured launches (one launch: rounds of one workgroup per CU, each the
 * time a workgroup needs for its heads of one sequence; three launches: their fixed cost plus the scan at its rate).
 * At 8 KV heads of 128 and a context of 8192 that is one launch for batches of about 40 to 64 sequences and again at
 * 128 (whole rounds of one workgroup per CU) at 4 bit, at batches 64 and 128 at 2 bit, and three for smaller ones,
 * which leave CUs idle, and for those in between; at 4096 tokens one launch up to batch 128 at both widths.
 * Alignment of the buffers, which the entry point also checks, is not part of it. */
int tw_kv_decode_step_plan(int G, int num_heads, int num_kv_heads, int bits, int max_seq_len, int ctx_min, int ctx_max);
/* The same for a caller that hands the step tickets (tw_layer_step_args::tickets; can_share != 0): the one launch may
 * then give a sequence's context to up to eight workgroups where the batch alone leaves compute units idle, which
 * makes it the choice for small batches of long sequences too (16 sequences of 4096 or 8192 tokens). */
int tw_kv_decode_step_plan2(int G, int num_heads, int num_kv_heads, int bits, int max_seq_len, int ctx_min, int ctx_max,
                            int can_share);
/* Test hook: KV heads per workgroup (0 = automatic; 1, 2, 4, 8) and workgroups per sequence and head group (0 =
 * automatic; 1, 2, 4 -- more than 1 only where the call has tickets) of the one-launch decode step. */
void tw_kv_debug_set_fused_shape(int hkw, int shares);
/* Layer steps that took the one-launch kernel since the library was loaded (launches issued or recorded into a
 * graph under capture): lets a benchmark say which kernel its figures belong to. */
long long tw_kv_decode_fused_launches(void);

/* No counterpart in the reference.  Rate (GB/s) at which this GPU streams `bytes` of device
 * memory through a plain contiguous 16-byte-per-lane read kernel, averaged over `iters`
 * launches and timed with HIP events on `s`; blocks until done.  The benchmark quotes it as
 * the practical ceiling beside the published HBM peak.  Returns 0 on error. */
double tw_kv_measure_read_bandwidth(const void* dev_buf, size_t bytes, int iters, hipStream_t s);

/* Prefix sharing without one copy per (array, destination): rows [0, T) of sequence `src` go to the same
 * rows of every sequence in [dst_begin, dst_end) (src itself skipped) for up to 4 arrays laid out
 * (sequence, row, ...), in one launch.  bases[i]: device pointer of array i, seq_bytes[i]: bytes per sequence
 * (rows per sequence * row bytes), bytes[i]: bytes to copy per sequence (T * row bytes).  Replaces the
 * cudaMemcpyAsync loop of engine.cpp:2173-2214.  Returns 0, or -1 on bad arguments. */
int tw_kv_broadcast_rows(void* const* bases, const size_t* seq_bytes, const size_t* bytes, int narrays,
                         int src, int dst_begin, int dst_end, hipStream_t s);

/* Floats of workspace the *_ws / paged attention entry points need for a
 * (G, num_heads, max_context) problem at the automatic split count.  The
 * reference-signature launchers instead fit their split count to the
 * G*num_heads*msl floats the engine already provides (engine.cpp:1371). */
size_t tw_attention_workspace_floats(int G, int num_heads, int max_context);

/* K and V compressed append in one launch: what engine.cpp:1985-1990 does with
 * two launches.  Same layout and arithmetic as launch_turbo_kv_quantize_batch. */
void tw_turbo_kv_append_batch(uint8_t* ck_q, tw_half* k_norms, uint8_t* cv_q, tw_half* v_norms,
                              const tw_half* k_buf, const tw_half* v_buf, const tw_half* rotation,
                              const int* positions, int max_seq_len, int G, int num_kv_heads,
                              int head_dim, int kv_dim, int bits, hipStream_t s);

/* The same for the T tokens of a prompt of one sequence (prefill_chunked's two launch_turbo_kv_quantize calls,
 * engine.cpp:2121-2131, in one launch): row t of k_buf / v_buf goes to cache row positions[t] of the sequence
 * whose arrays are passed.  Same layout and arithmetic as launch_turbo_kv_quantize. */
void tw_turbo_kv_append_tokens(uint8_t* ck_q, tw_half* k_norms, uint8_t* cv_q, tw_half* v_norms,
                               const tw_half* k_buf, const tw_half* v_buf, const tw_half* rotation,
                               const int* positions, int max_seq_len, int num_tokens, int num_kv_heads,
                               int head_dim, int kv_dim, int bits, hipStream_t s);

/* One decode step of one layer in a single call: append K and V at positions[g],
 * then attention over 0..positions[g] (forward_layer_batch steps 4-5,
 * engine.cpp:1979-2006).  Same results as tw_turbo_kv_append_batch followed by
 * launch_turbo_gqa_attention_batch; the rotation of the appended rows and of the
 * query share one launch. */
void tw_turbo_append_attention_batch(tw_half* out, const tw_half* q, const tw_half* k_buf,
                                     const tw_half* v_buf, uint8_t* ck_q, uint8_t* cv_q,
                                     tw_half* k_norms, tw_half* v_norms, const tw_half* rotation,
                                     float* as, const int* pos, int msl, int G, int num_heads,
                                     int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                     int bits, hipStream_t s);

/* The same for the fp16 cache: what engine.cpp:1979-2003 does with launch_kv_cache_write_batch and
 * launch_gqa_attention_batch, as one launch (plus the merge of the context chunks when there are several): the
 * attention kernel takes the new token's K and V rows from k_buf / v_buf and stores them into the cache itself.
 * Same cache bytes and outputs as the two calls.  (tw_kv_debug_set_decode_fused(2) keeps the two launches.) */
void tw_append_attention_batch(tw_half* out, const tw_half* q, const tw_half* k_buf, const tw_half* v_buf,
                               tw_half* ck, tw_half* cv, float* as, const int* pos, int msl, int G,
                               int num_heads, int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                               hipStream_t s);

/* Producers fused into the path (steps 3-5 of forward_layer_batch, engine.cpp:1972-2006, in one
 * call): per-head RMSNorm (q_weight / k_weight, `biased`) and rotary embedding (tables as for
 * launch_rope_batch) of q and k, append of K and V at positions[g], attention over
 * 0..positions[g].  Same cache bytes and, within the attention tolerance, the same output as
 * launch_qk_norm_batch + launch_rope_batch + the append + the attention.  q_weight == NULL skips
 * the normalisation, cos_table == NULL the rotation.
 *
 * Compressed cache: normalisation and rotation happen in the launch that rotates and quantizes the
 * rows, so q and k are only read (when that launch is not available for the shape, they are
 * transformed in place first: treat their contents after the call as unspecified). */
void tw_qk_norm_rope_turbo_append_attention_batch(
    tw_half* out, tw_half* q, tw_half* k_buf, const tw_half* v_buf, const tw_half* q_weight,
    const tw_half* k_weight, float eps, int biased, const tw_half* cos_table,
    const tw_half* sin_table, int rope_dim, uint8_t* ck_q, uint8_t* cv_q, tw_half* k_norms,
    tw_half* v_norms, const tw_half* rotation, float* as, const int* pos, int msl, int G,
    int num_heads, int num_kv_heads, int head_dim, int q_dim, int kv_dim, int bits, hipStream_t s);

/* fp16 cache: one launch transforms q in place and writes the transformed K rows and the V rows
 * to the cache (instead of qk_norm + rope + kv_cache_write), then the attention.  k_buf is only read. */
void tw_qk_norm_rope_append_attention_batch(
    tw_half* out, tw_half* q, const tw_half* k_buf, const tw_half* v_buf, const tw_half* q_weight,
    const tw_half* k_weight, float eps, int biased, const tw_half* cos_table,
    const tw_half* sin_table, int rope_dim, tw_half* ck, tw_half* cv, float* as, const int* pos,
    int msl, int G, int num_heads, int num_kv_heads, int head_dim, int q_dim, int kv_dim,
    hipStream_t s);

/* Steps 3-6 of forward_layer_batch (engine.cpp:1972-2012) for one layer in one call, every optional
 * part switched by a NULL pointer: producers of q and k (as tw_qk_norm_rope_*), append, attention, and
 * the sigmoid gate of gated attention applied by the kernel that writes `out`
 * (out = half(float(half(attention)) / (1 + exp(-gate))), the arithmetic of launch_sigmoid_gate_batch).
 * Forwards to the entry points above; their rules for q and k apply. */
typedef struct tw_layer_step_args {
    tw_half* out;              /* (G, q_dim) */
    tw_half* q;                /* (G, q_dim) */
    tw_half* k;                /* (G, kv_dim) */
    const tw_half* v;          /* (G, kv_dim) */
    int G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim;
    const int* positions;      /* device int32[G] */
    int max_seq_len;
    const tw_half* q_weight;   /* per-head RMSNorm weights (head_dim), NULL = none */
    const tw_half* k_weight;
    float eps;
    int biased;
    const tw_half* cos_table;  /* rotary tables (positions, rope_dim/2), NULL = none */
    const tw_half* sin_table;
    int rope_dim;
    int kv_bits;               /* 0 = fp16 cache, 2 or 4 = compressed */
    void* cache_k;             /* fp16 rows or packed codes, layout of the launchers above */
    void* cache_v;
    tw_half* k_norms;          /* compressed only */
    tw_half* v_norms;
    const tw_half* rotation;   /* compressed only */
    float* scratch;            /* G*num_heads*max_seq_len floats */
    const tw_half* gate;       /* row g at gate + g*gate_stride, laid out like a row of out; NULL = none */
    long long gate_stride;
    int ctx_min, ctx_max;      /* what the host knows of min and max over g of positions[g] + 1; 0, 0 = nothing.
                                * Only steers the choice between kernels (tw_kv_debug_set_decode_fused), never results. */
    unsigned* tickets;         /* NULL, or G*num_kv_heads device words that are ZERO before the first call and that
                                * only these calls touch (every call leaves them zero): with them, the one-launch step
                                * of a compressed layer may give a sequence's context to two, four or eight workgroups when
                                * the batch alone leaves compute units idle (their sums meet in `scratch`).  Calls that
                                * share tickets must not overlap.  Decode step only. */
} tw_layer_step_args;
void tw_layer_attention_step(const tw_layer_step_args* args, hipStream_t s);

/* The same for a prompt: steps 3-5b of a layer in prefill_chunked (engine.cpp:2097-2150: launch_qk_norm_batch,
 * launch_rope_batch, cudaMemcpyAsync x2 or launch_turbo_kv_quantize x2, launch_*_prefill_attention,
 * launch_sigmoid_gate_batch) in one call and at most four launches.  The struct is read with G = T, the number of
 * prompt tokens: row t of q / k / v / out / gate is token t, positions is device int32[T] and holds 0 .. T-1 (what
 * the engine puts there before prefill_chunked; the rotary table row and the cache row of token t are
 * positions[t]), the cache pointers are sequence 0's, scratch is sized as for the prefill launchers.  q (and with
 * the compressed cache k) come back normalised and rotated.  ctx_min / ctx_max are not used. */
void tw_layer_prompt_step(const tw_layer_step_args* args, hipStream_t s);

/* Paged cache.  A page holds TW_PAGE_TOKENS consecutive positions of one
 * sequence in the same row layout the contiguous cache uses, so
 *   row(g, p) = block_table[g*bt_stride + p/16]*16 + p%16
 * replaces the reference's row(g, p) = g*msl + p (kernels.cu:973, 1629, 1690)
 * and nothing else changes.  block_table is device int32. */
#define TW_PAGE_TOKENS 16

void tw_paged_kv_cache_write_batch(tw_half* ck, tw_half* cv, const tw_half* k, const tw_half* v,
                                   const int* positions, const int* block_table, int bt_stride,
                                   int G, int kv_dim, hipStream_t s);

void tw_paged_turbo_kv_append_batch(uint8_t* ck_q, tw_half* k_norms, uint8_t* cv_q,
                                    tw_half* v_norms, const tw_half* k_buf, const tw_half* v_buf,
                                    const tw_half* rotation, const int* positions,
                                    const int* block_table, int bt_stride, int G,
                                    int num_kv_heads, int head_dim, int kv_dim, int bits,
                                    hipStream_t s);

/* max_context bounds positions[g]+1 and fixes the launch grid (graph-safe).
 * ws: tw_attention_workspace_floats(G, num_heads, max_context) floats. */
void tw_paged_gqa_attention_batch(tw_half* out, const tw_half* q, const tw_half* ck,
                                  const tw_half* cv, float* ws, const int* positions,
                                  const int* block_table, int bt_stride, int max_context, int G,
                                  int num_heads, int num_kv_heads, int head_dim, int q_dim,
                                  int kv_dim, hipStream_t s);

void tw_paged_turbo_gqa_attention_batch(tw_half* out, const tw_half* q, const uint8_t* ck_q,
                                        const uint8_t* cv_q, const tw_half* k_norms,
                                        const tw_half* v_norms, const tw_half* rotation, float* ws,
                                        const int* positions, const int* block_table,
                                        int bt_stride, int max_context, int G, int num_heads,
                                        int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                        int bits, hipStream_t s);

/* One decode step of one layer over the paged compressed cache in a single call: append K and V at positions[g]
 * (into the page block_table names), then attention over 0..positions[g] -- tw_turbo_append_attention_batch with
 * the paged contract above.  The appended rows and the query are rotated in one launch, so the call is three
 * launches where tw_paged_turbo_kv_append_batch + tw_paged_turbo_gqa_attention_batch are four; same cache bytes,
 * same outputs.  ws and max_context as for tw_paged_turbo_gqa_attention_batch. */
void tw_paged_turbo_append_attention_batch(tw_half* out, const tw_half* q, const tw_half* k_buf, const tw_half* v_buf,
                                           uint8_t* ck_q, uint8_t* cv_q, tw_half* k_norms, tw_half* v_norms,
                                           const tw_half* rotation, float* ws, const int* positions,
                                           const int* block_table, int bt_stride, int max_context, int G,
                                           int num_heads, int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                           int bits, hipStream_t s);

/* No counterpart in the reference.  launch_turbo_gqa_attention_batch for callers that cannot allocate and have
 * no scratch to hand over (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * the same arguments without `as`, same kernels and results; the split workspace is a device array inside the
 * library, TW_NOALLOC_SCRATCH_BYTES per GPU, held from the first call on that GPU until the process ends.  The
 * call allocates and frees nothing (no hipMalloc / hipFree / event or stream creation); its first call on a GPU
 * looks the array's address up once and should not happen under stream capture.
 * Limit: G * num_heads <= TW_NOALLOC_MAX_HEAD_VECTORS, else nothing is launched and an error is returned.
 * All calls on one GPU share that GPU's array, which keeps the last call's contents (nothing in it needs to
 * start at zero: a call reads only what it wrote itself): calls that overlap on one GPU race -- run them on one
 * stream, or order them.  Returns 0, or non-zero with the message in tw_kv_last_error_string().  The return value
 * is this call's own outcome: an error an earlier call left uncleared on the thread does not make it fail (it is
 * still there afterwards when this call succeeds, and is replaced by this call's message when it fails). */
#define TW_NOALLOC_SCRATCH_BYTES (32u << 20)
#define TW_NOALLOC_MAX_HEAD_VECTORS 16384
int tw_turbo_gqa_attention_batch_noalloc(tw_half* out, const tw_half* q, const uint8_t* ck_q, const uint8_t* cv_q,
                                         const tw_half* k_norms, const tw_half* v_norms, const tw_half* rotation,
                                         const int* pos, int msl, int G, int num_heads, int num_kv_heads,
                                         int head_dim, int q_dim, int kv_dim, int bits, hipStream_t s);

/* Host: the rotation matrix of engine.cpp:366-392 (mt19937(42), N(0,1),
 * modified Gram-Schmidt over rows, fp16).  out: head_dim*head_dim halves, HOST. */
void tw_make_rotation_host(tw_half* out_host, int head_dim, unsigned seed);

/* ------------------------------------------------------------------ Engine
 * Host-side owner of the cache: the KV slice of InferenceEngine
 * (model.h:373-493).  Opaque; one host thread at a time, like the reference. */
typedef struct tw_engine tw_engine;

typedef struct tw_model_shape {
    int num_layers;
    int num_heads;
    int num_kv_heads;
    int head_dim;
} tw_model_shape;

/* InferenceEngine(max_seq_len, kv_bits), engine.cpp:300-317.  kv_bits outside
 * {0,2,4} prints the reference's warning and falls back to 0. */
tw_engine* tw_engine_create(int max_seq_len, int kv_bits);
void tw_engine_destroy(tw_engine* e);
int tw_engine_kv_bits(const tw_engine* e);      /* engine_py.cpp:25 */
int tw_engine_max_seq_len(const tw_engine* e);

/* load_config's share of the work: fix the model shape (engine.cpp:769). */
int tw_engine_set_shape(tw_engine* e, const tw_model_shape* shape);

/* alloc_batch, engine.cpp:1338-1560: one arena for G sequences of max_seq_len
 * rows, carved with 256-byte alignment in the reference's order (keys, values,
 * key norms, value norms per layer).  Returns 0 on success.  A call with the G and max_seq_len the engine
 * already has changes nothing; any other carves the caches anew and zeroes them -- inside the memory already
 * held when that is big enough -- so the steps below always work on exactly G rows (the reference keeps a
 * larger batch and its strides, engine.cpp:1339). */
int tw_engine_alloc_batch(tw_engine* e, int G, int max_seq_len);
/* set_arena, engine.cpp:1609-1620: carve out of caller-owned device memory. */
int tw_engine_set_arena(tw_engine* e, void* device_ptr, size_t bytes);
size_t tw_engine_arena_bytes_needed(const tw_engine* e, int G, int max_seq_len);

/* reset(), engine.cpp:893-916 / 2262-2283: zero every cache, positions to 0.
 * Stream order: reset, set_positions, alloc_batch, set_arena and sleep first wait for the stream the latest
 * step, prompt layer or prefix broadcast was issued on; reset returns when its own work is done.  Work that the
 * caller put on other streams is the caller's to order. */
int tw_engine_reset(tw_engine* e);

/* Device pointers into the arena (for tests and for callers that keep using
 * the launchers directly).  which: 0 keys, 1 values, 2 key norms, 3 value norms. */
void* tw_engine_cache_ptr(tw_engine* e, int layer, int which);
int* tw_engine_positions(tw_engine* e);          /* device int32[G] */
const tw_half* tw_engine_rotation(tw_engine* e); /* device, NULL when kv_bits==0 */
/* Host positions (each in [0, max_seq_len)) to the device array, engine.cpp:2364.  The engine keeps their range
 * on the host and advances it with every decode step: it picks the kernels from it, and refuses a step (-8,
 * nothing launched, cache and positions untouched) once a sequence has used its last row.  A caller that writes
 * the device array itself must keep positions[g] < max_seq_len on its own. */
int tw_engine_set_positions(tw_engine* e, const int* host_positions, int G);

/* Make the producers of q and k part of every step (forward_layer_batch step 3,
 * engine.cpp:1972-1977): per-head RMSNorm with the weights of the step's layer (q_norm, k_norm:
 * device, (num_layers, head_dim); NULL = none) and rotary embedding from the tables (device,
 * (positions, rope_dim/2); NULL = none).  mode 1 fuses them into the append (see
 * tw_qk_norm_rope_turbo_append_attention_batch), mode 2 runs the reference's two launches first,
 * mode 0 switches them off.  The pointers are kept, not copied.  With producers the q and k rows
 * handed to a step are scratch: they may come back transformed. */
int tw_engine_set_producers(tw_engine* e, int mode, const tw_half* q_norm, const tw_half* k_norm,
                            float eps, int biased, const tw_half* rope_cos, const tw_half* rope_sin,
                            int rope_dim);

/* One decode step of the path for `layer`: append K,V at positions[g], then
 * attention over 0..positions[g] (forward_layer_batch steps 4-5,
 * engine.cpp:1979-2006).  q/out: (G, num_heads*head_dim); k/v: (G, kv_dim). */
int tw_engine_layer_step(tw_engine* e, int layer, const tw_half* q, const tw_half* k,
                         const tw_half* v, tw_half* out, hipStream_t s);

/* The path of `layer` over a prompt of T tokens for sequence `seq` of the batch (prefill_chunked, engine.cpp:2097-2150,
 * which does it for sequence 0): the producers the engine was given, the T-token append into that sequence's cache
 * rows, causal attention.  q/out: (T, num_heads*head_dim); k/v: (T, kv_dim); token_positions: device int32[T] holding
 * 0 .. T-1.  The positions of the batch are the caller's to set afterwards (tw_engine_set_positions). */
int tw_engine_prompt_layer(tw_engine* e, int layer, int seq, const tw_half* q, const tw_half* k, const tw_half* v,
                           tw_half* out, const int* token_positions, int T, hipStream_t s);

/* All layers, then positions += 1.  q/out: (L, G, q_dim); k/v: (L, G, kv_dim).
 * With use_graph != 0 the step is captured once into a hipGraph and replayed
 * (engine.cpp:2369-2412, 2480); the capture is dropped when the arena, G or
 * the buffers change, and made again when the context lengths the host knows of have moved to where the other
 * choice of kernels (tw_kv_decode_step_plan) applies.  -8: a sequence has no row left (see
 * tw_engine_set_positions). */
int tw_engine_decode_step(tw_engine* e, const tw_half* q, const tw_half* k, const tw_half* v,
                          tw_half* out, int use_graph, hipStream_t s);
/* When the capture or the instantiation of the step's graph fails, the step is run without a graph, one line goes
 * to stderr, and so are all later steps with the same buffers (engine.cpp:2396-2410); the next change of buffers,
 * batch, arena or producers tries again.  graph_state tells what the latest decode step did: 0 run eagerly as asked,
 * 1 graph replayed, 2 run eagerly after a failed capture.  debug_fail_captures (test hook): the next n captures
 * are treated as failed after they have been recorded. */
int tw_engine_graph_state(const tw_engine* e);
void tw_engine_debug_fail_captures(tw_engine* e, int n);
/* roctx ranges (tw_engine_decode_step, tw_engine_prompt_layer, tw_engine_single_step) for a profiler's timeline,
 * where the reference prints std::chrono timings (engine.cpp:2305-2311, 2537-2544).  on != 0 looks the roctx
 * library up (dlopen; nothing is linked) and switches the ranges on: 0, or -1 when there is none.  Process-wide. */
int tw_kv_set_trace_ranges(int on);

/* Prefix sharing, engine.cpp:2173-2214: copy rows [0,T) of sequence `src` to
 * every sequence in [dst_begin, dst_end). */
int tw_engine_broadcast_prefix(tw_engine* e, int src, int dst_begin, int dst_end, int T,
                               hipStream_t s);

/* sleep() / wake(), engine.cpp:922-1022: sleep hands the cache memory back (frees an arena the engine
 * allocated, forgets one the caller owns, frees the single-sequence caches), drops the captured step and the
 * generation bookkeeping; wake re-allocates the single-sequence caches when the engine had them before the sleep
 * (zeroed, current_pos = 0); the batch state is re-created, zeroed, by the next tw_engine_alloc_batch (or
 * tw_engine_set_arena + tw_engine_alloc_batch), as in the reference. */
int tw_engine_sleep(tw_engine* e);
int tw_engine_wake(tw_engine* e);
int tw_engine_is_allocated(const tw_engine* e);

/* The single-sequence state of the reference's generate() / decode_token() path (model.h:195-204): per layer a key
 * and a value array of max_seq_len rows (compressed: codes and norms), each an allocation of its own as in
 * allocate_buffers (engine.cpp:322-331, 394-404), the attention scratch (num_heads * max_seq_len floats), the
 * rotation and current_pos.  alloc_single allocates and zeroes them for the shape and max_seq_len the engine has
 * (0 on success; a later tw_engine_set_shape frees them); tw_engine_reset zeroes them and sets current_pos to 0
 * (engine.cpp:893-916).  single_cache_ptr: which as in tw_engine_cache_ptr, rows (max_seq_len, ...). */
int tw_engine_alloc_single(tw_engine* e);
int tw_engine_single_is_allocated(const tw_engine* e);
void* tw_engine_single_cache_ptr(tw_engine* e, int layer, int which);
const tw_half* tw_engine_single_rotation(tw_engine* e);   /* device, NULL when kv_bits==0 */
int tw_engine_single_pos(const tw_engine* e);             /* state_.current_pos */
int tw_engine_single_set_pos(tw_engine* e, int pos);      /* 0 <= pos < max_seq_len; waits for the steps in flight */
/* forward_layer steps 4-5 for `layer` (engine.cpp:1069-1108): K and V of the token into row current_pos, attention
 * over rows 0 .. current_pos.  q/out: num_heads*head_dim halves, k/v: kv_dim halves, device.  Nothing is allocated
 * per call (the reference allocates and frees a device word per layer and token for the compressed append,
 * engine.cpp:1078-1092).  -8: current_pos has reached max_seq_len.  Stream 0 means the engine's own stream (the
 * reference runs this path on the legacy default stream). */
int tw_engine_single_step(tw_engine* e, int layer, const tw_half* q, const tw_half* k, const tw_half* v, tw_half* out,
                          hipStream_t s);
/* current_pos += 1 after the last layer of a token (decode_token), host and device, in stream order. */
int tw_engine_single_advance(tw_engine* e, hipStream_t s);

/* The tail of generate_batch's decode loop (engine.cpp:2350, 2496-2534), for the caller that owns the
 * sampling: begin_generation sizes a (max_new_tokens, G) token history on the device; record_tokens
 * copies a step's G tokens (device int32) into it without synchronising; check_stops does nothing on
 * most steps and, every 8th step and on the last one, waits for the stream, fetches positions and the
 * history rows not yet seen, extends the outputs of the sequences still running and marks those that
 * produced eos_token_id or the stop sequence.  It returns 1 when every sequence has finished, 0
 * otherwise, < 0 on error; *checked says whether the step was a checking one.  output() returns a
 * sequence's tokens so far (host memory owned by the engine) and whether it has finished. */
int tw_engine_begin_generation(tw_engine* e, int max_new_tokens, int eos_token_id,
                               const int* stop_ids_host, int n_stop);
int tw_engine_record_tokens(tw_engine* e, const int* d_tokens, int step, hipStream_t s);
int tw_engine_check_stops(tw_engine* e, int step, hipStream_t s, int* checked);
int tw_engine_output(tw_engine* e, int g, const int** tokens, int* n);
int tw_engine_host_position(const tw_engine* e, int g); /* positions as of the last check */

#ifdef __cplusplus
}
#endif
#endif /* TRIEBWERK_KV_H */
