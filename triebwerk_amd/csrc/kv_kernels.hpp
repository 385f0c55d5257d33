// kv_kernels.hpp -- internal launch interface between the C ABI (kv_capi.hip)
// and the kernel files.  Nothing here is exported.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "kv_common.hpp"

namespace twkv {

// ---------------------------------------------------------------- timing the context-scanning kernel
// When the profiler is on, kv_capi.hip hands the scan launch a pair of events; the launch attaches them
// to the kernel itself (start = the kernel begins, stop = it ends), so their distance is the kernel's
// duration without the gaps an event recorded before and after a launch would add.
extern thread_local hipEvent_t t_scan_start;
extern thread_local hipEvent_t t_scan_stop;
// Name of the kernel the last attention launch of this process used for the context (tw_kv_debug_last_scan_kernel):
// every launch function below records its own.
extern const char* volatile g_last_scan_kernel;
inline void note_scan_kernel(const char* name) { g_last_scan_kernel = name; }
template <typename... Args, typename F = void (*)(Args...)>
inline void launch_scan_kernel(F kernel, dim3 grid, dim3 block, hipStream_t s, Args... args) {
    if (t_scan_start) hipExtLaunchKernelGGL(kernel, grid, block, 0, s, t_scan_start, t_scan_stop, 0, args...);
    else hipLaunchKernelGGL(kernel, grid, block, 0, s, args...);
}

// ---------------------------------------------------------------- append
struct QuantArgs {
    // One or two streams (K, V) quantized by the same launch.
    uint8_t* codes[2];
    half_t* norms[2];
    const half_t* src[2];   // (nrows, kv_dim) fp16
    int nstreams;
    const half_t* rotation; // (128,128) fp16 row major
    const int* positions;   // device int32[nrows]
    const int* block_table; // NULL = contiguous cache
    int bt_stride;
    long long seq_stride_rows;  // max_seq_len for the contiguous batch layout
    int token_list;         // 1: row r goes to cache row positions[r] of sequence 0
    int nrows;              // G, or num_tokens
    int num_kv_heads;
    int kv_dim;
};

void launch_kv_write(half_t* ck, half_t* cv, const half_t* k, const half_t* v,
                     const int* positions, const int* block_table, int bt_stride,
                     long long seq_stride_rows, int G, int kv_dim, hipStream_t s);
void launch_turbo_quantize(const QuantArgs& a, int bits, hipStream_t s);
void launch_increment(int* positions, int G, hipStream_t s);

// Rows [0, T) of sequence `src` copied to sequences [dst_begin, dst_end) (src itself skipped) in up to four
// arrays that are laid out (sequence, row, ...): bytes = T * row bytes, seq_bytes = rows per sequence * row bytes.
struct BroadcastArgs {
    char* base[4];
    size_t seq_bytes[4];
    size_t bytes[4];
    int narrays;
    int src, dst_begin, dst_end;
};
void launch_broadcast_rows(const BroadcastArgs& a, hipStream_t s);

// ---------------------------------------------------------------- producers of q and k (kv_producer.hip)
struct ProducerArgs {
    half_t* q;               // (rows, q_stride), transformed in place
    half_t* k;               // (rows, kv_stride)
    half_t* v;               // write_cache only
    long long q_stride, kv_stride;
    int rows, num_heads, num_kv_heads;
    int norm;                // per-head RMSNorm with q_weight / k_weight
    const half_t* q_weight;  // (128)
    const half_t* k_weight;
    float eps;
    int biased;              // weight + 1
    const half_t* cos_table; // NULL: no rotation; (positions, rope_dim / 2)
    const half_t* sin_table;
    int rope_dim;
    int single_order;        // operand order of the single-sequence rope kernel
    const int* positions;    // device int32[rows], or NULL: pos_scalar
    int pos_scalar;
    int write_cache;         // K (transformed) and V rows go to their fp16 cache rows instead of back
    half_t* cache_k;
    half_t* cache_v;
    int kv_dim;              // halves per cache row
    const int* block_table;
    int bt_stride;
    long long seq_stride_rows;
};
void launch_producer(const ProducerArgs& a, hipStream_t s);
// data[r][i] = half(data[r][i] / (1 + exp(-gate[r][i]))), rows of `dim` halves with their own strides
void launch_sigmoid_gate(half_t* data, long long data_stride, const half_t* gate, long long gate_stride, int dim,
                         int rows, hipStream_t s);

// ---------------------------------------------------------------- rotation on the matrix cores
struct RotArgs {
    int nseg;                    // up to 3 segments: K rows, V rows (quantize), Q rows (rotate only)
    const half_t* seg_src[3];    // fp16 source, row r at src + r * stride
    long long seg_stride[3];     // halves per source row
    int seg_heads[3];            // head vectors per source row
    int seg_nvec[3];             // rows * heads
    int seg_units[3];            // work units = ceil(tiles / nper) * 8 (launch_rotate fills this in)
    int nper;                    // tiles of 16 vectors a wave walks (launch_rotate fills this in)
    int seg_kind[3];             // 0 = quantize into the cache, 1 = query rotation
    uint8_t* seg_codes[3];
    half_t* seg_norms[3];
    const half_t* rotation;
    const int* positions;
    const int* block_table;
    int bt_stride;
    long long seq_stride_rows;
    int token_list;              // 1: source row r goes to cache row positions[r] of sequence 0
    int num_kv_heads;
    float* qrot;                 // query output: vector v at qrot + v * qrot_stride (fp32)
    long long qrot_stride;
    float q_scale;
    // optional producers applied to a segment's vectors before anything else (kv_producer.hip has the rules)
    const half_t* seg_weight[3]; // per-head RMSNorm weight (128), NULL = none
    int seg_rope[3];             // rotate with the tables below at positions[row]
    float eps;
    int biased;
    const half_t* cos_table;     // (positions, rope_dim / 2)
    const half_t* sin_table;
    int rope_dim;                // multiple of 16
};

void launch_rotate(const RotArgs& a, int bits, hipStream_t s);

// ---------------------------------------------------------------- attention
enum PosMode { kPosArray = 0, kPosScalar = 1, kPosIota = 2 };

struct AttnArgs {
    const half_t* q;        // (G, q_stride)
    half_t* out;            // (G, q_stride)
    int q_stride;
    const void* k;          // fp16 rows (kv_bits 0) or packed codes
    const void* v;
    const half_t* k_norms;  // compressed only: (rows, num_kv_heads)
    const half_t* v_norms;
    const half_t* rotation; // compressed only
    const int* positions;   // kPosArray
    int pos_scalar;         // kPosScalar
    int pos_mode;           // kPosIota: sequence g attends rows 0..g (causal prefill)
    const int* block_table; // NULL = contiguous
    int bt_stride;
    long long seq_stride_rows;  // msl (batch), 0 (single sequence / prefill)
    int G, num_heads, num_kv_heads;
    int bits;               // 0, 2, 4
    float* ws;              // split workspace: per (g, head) block, nsplit partials then q_rot
    long long ws_stride;    // floats per (g, head) block
    float* qrot;            // ws + offset of q_rot inside a block (128 floats), or NULL
    int nsplit;             // >= 1; 1 = no workspace, one workgroup walks the sequence
    int force_merge;        // the scan kernel wrote partials even though nsplit == 1
    int m_log2;             // partial maxima are in base-2 units
    int balance;            // MFMA scan: may cut the batch by tiles instead of by sequence (ragged lengths)
    int max_slots;          // partials the workspace holds per (sequence, head): >= nsplit
    int slots_from_ws;      // merge: the spare word of partial 0 holds the number of partials (0: even chunks)
    int even_chunks;        // the chunks are the fp16 whole-row scan's (even_chunk_range), not chunk_range's
    // optional output gate (gated attention, kernels.cu:2987-2995): out = half(float(half(out)) * sigmoid(gate))
    const half_t* gate;     // row g at gate + g * gate_stride, laid out like a row of out; NULL = none
    long long gate_stride;
    // fp16 cache, batch decode: the K and V rows of the new token (position positions[g]).  The scan takes them
    // from here instead of the cache and one workgroup per (sequence, KV head) stores them there, which makes
    // the append part of the attention launch (kv_cache_write_batch_kernel, kernels.cu:964-977).  NULL = none.
    const half_t* k_new;    // (G, kv_new_stride)
    const half_t* v_new;
    long long kv_new_stride;
};

constexpr int kPartialFloats = kHeadDim + 4;  // acc[128], running max, running sum, 2 pad (16-byte rows)

void launch_attention_valu(const AttnArgs& a, hipStream_t s);
// fp16 cache: will launch_attention_valu run the kernel whose waves read whole rows (eight KV heads)?  Its workgroups
// have eight waves that share one chunk, so the split planner gives it more and smaller chunks.
bool attention_rows_usable(const AttnArgs& a);
int attention_rows_groups(const AttnArgs& a);      // workgroups per (sequence, chunk)
bool attention_rows_balances(const AttnArgs& a);   // may cut a ragged batch by tokens instead (needs max_slots set)
void launch_attention_merge(const AttnArgs& a, hipStream_t s);
bool launch_merge_rotate(const AttnArgs& a, hipStream_t s);   // MFMA merge + rotate-back; false = not applicable
// MFMA path, two steps so that the scan kernel can be timed alone:
// prepare = shape check + query rotation (false = shape not covered), then the scan.
bool prepare_attention_mfma(AttnArgs& a, hipStream_t s, bool rotate_query);
float attention_mfma_q_scale(int bits);
bool launch_attention_mfma_scan(const AttnArgs& a, hipStream_t s);   // true: the output is finished, no merge
// One decode step of a layer in one launch (kv_decode_fused.hip): append the new K and V rows, rotate the
// query, scan, merge and rotate back.  AttnArgs as for the batch decode over the contiguous compressed
// cache (positions array; no workspace needed), plus the rows to append and the cache as writable pointers.
struct FusedArgs {
    const half_t* k_src;    // (G, kv_stride) fp16 rows of the new token
    const half_t* v_src;
    long long kv_stride;
    uint8_t* k_codes;       // the arrays AttnArgs::k, v, k_norms, v_norms point at
    uint8_t* v_codes;
    half_t* k_norms;
    half_t* v_norms;
    int ctx_bound;          // in: upper bound of positions + 1 that the host knows (0: none)
    int hkw;                // KV heads per workgroup (launch_decode_fused fills this in)
    float q_scale;          // likewise
    // A unit's context shared by several workgroups, for batches whose units alone leave compute units idle:
    int shares;             // 1, 2, 4 or 8 (launch_decode_fused fills this in; > 1 only with the three below)
    int max_shares;         // as many shares as share_ws has room for (1: none)
    float* share_ws;        // G * num_heads * max_shares * (kHeadDim + 4) floats for the shares' unnormalised sums
    unsigned* tickets;      // one word per (sequence, KV head): zero before the first launch, left zero by every launch
    // optional producers of q and k applied on the way in, as RotArgs has them (V rows stay as they are)
    const half_t* q_weight; // per-head RMSNorm weights (128); both or neither
    const half_t* k_weight;
    float eps;
    int biased;
    const half_t* cos_table; // (positions, rope_dim / 2); both or neither
    const half_t* sin_table;
    int rope_dim;            // 128, or a multiple of 16 up to 64
};
// Everything the choice between the forms of a decode step rests on, in one place: rates and fixed costs measured on
// the device named, looked up once per process by the current device's name (plan_constants()).  A device that is
// not in the table gets the first entry's figures scaled by its own number of compute units only where the estimates
// use that number; tests/test_gpu_plan.py checks on the GPU at hand that the automatic choice is the faster form.
struct PlanConstants {
    const char* device;         // substring of hipDeviceProp_t::gcnArchName
    double one_fixed_us;        // one launch: prologue, first tile, epilogue, launch and drain
    double pair_ns[2];          // ns per token and KV head one compute unit sustains, waves with two heads: [4 bit, 2 bit]
    double pair_wide2_ns;       // the same at 2 bit with four or more heads per workgroup
    double single_ns[2];        // waves with one head each
    double one_bw[2];           // bytes per us the whole chip streams in the one-launch pattern
    double three_fixed_us[2];   // three launches: rotation, merge, launches and the scan's start and end
    double three_bw[2];         // bytes per us of the scan
    double handover_us[4];      // shares' sums through memory, by log2(shares)
};
const PlanConstants& plan_constants();
bool decode_fused_usable(const AttnArgs& a, const FusedArgs& f);
int decode_fused_heads_per_workgroup(int G, int num_heads, int num_kv_heads, int bits, bool allow_pairs);   // 8, 4, 2 or 1
// estimated microseconds of one launch with hkw KV heads per workgroup, all sequences at ctx tokens
double decode_fused_estimate_us(int G, int num_heads, int num_kv_heads, int bits, bool allow_pairs, int hkw, double ctx);
// estimated microseconds of the same step as three launches (rotation, scan, merge)
double decode_three_estimate_us(int G, int num_kv_heads, int bits, double ctx);
// The launch's shape when a unit's context may be shared by up to max_shares workgroups (1: the caller has no tickets
// or no room for the shares' sums): KV heads per workgroup, shares, and the estimate for sequences of ctx tokens.
struct FusedShape { int hkw, shares; double us; };
FusedShape decode_fused_shape(int G, int num_heads, int num_kv_heads, int bits, bool allow_pairs, int max_shares, double ctx);
// test hook (tw_kv_debug_set_fused_shape): force hkw and / or shares (0 = automatic)
void decode_fused_force_shape(int hkw, int shares);
// allow_pairs: the 4-bit kernel whose waves scan two KV heads each, where the shape admits it (false: one head per wave)
void launch_decode_fused(const AttnArgs& a, const FusedArgs& f, hipStream_t s, bool allow_pairs);
// causal prefill with blocks of query tokens per wave (kv_prefill_mfma.hip); same workspace and merge
bool prefill_mfma_usable(const AttnArgs& a);
void launch_prefill_mfma_scan(const AttnArgs& a, hipStream_t s);
// causal prefill over the fp16 cache on the matrix cores (kv_prefill_f16_mfma.hip); writes `out` directly
bool prefill_f16_mfma_usable(const AttnArgs& a);
// form: 0 = chosen from the prompt length; 1 one query block per wave, 2 the same with mirrored block pairs,
// 3 two query blocks per wave with mirrored pairs (1-3: four waves per workgroup); 5 and 6 = 2 and 3 with eight waves
void launch_prefill_f16_mfma(const AttnArgs& a, hipStream_t s, int form);
// causal prefill over the compressed cache with tiles expanded once per workgroup (kv_prefill_tq_mfma.hip);
// one launch, no workspace; forms as for launch_prefill_f16_mfma
bool prefill_tq_mfma_usable(const AttnArgs& a);
void launch_prefill_tq_mfma(const AttnArgs& a, hipStream_t s, int form);
// test hook (tw_kv_debug_set_prefill_form): 0 = automatic; 1-3, 5, 6 force a form of the flash prefill kernels; 4 = the
// compressed prefill kernel that expands tiles per wave
int prefill_form();
// 4-bit decode scan whose waves take two KV heads each and read whole cache lines (kv_attention_pair.hip); same
// workspace, partials and merge as attention_mfma_kernel
bool attention_pair_usable(const AttnArgs& a);
void launch_attention_pair_scan(const AttnArgs& a, hipStream_t s);
// test hook (tw_kv_debug_set_attention_variant): 0 automatic, 1 vector-ALU kernels, 2 MFMA kernels, 3 MFMA kernels
// with one KV head per wave also where the 4-bit scan would give a wave two
int attention_variant();

}  // namespace twkv
