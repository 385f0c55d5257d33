// kv_capi.hip -- the exported C ABI (include/triebwerk_kv.h): the reference's
// launcher entry points (engine.cpp:105-171) and the paged / fused additions.
// Argument checks and launch-geometry policy live here; kernels elsewhere.

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <random>
#include <vector>

#include "../../include/triebwerk_kv.h"
#include "kv_kernels.hpp"

using namespace twkv;

namespace twkv {
static std::atomic<long long> g_fused_launches{0};   // one-launch decode steps issued so far (tw_kv_decode_fused_launches)
static std::atomic<int> g_decode_fused{0};   // tw_kv_debug_set_decode_fused: 0 by context bound, 1 whenever possible, 2 never, 3 as 1 with one head per wave
static std::atomic<int> g_prefill_form{0};   // test hook, see prefill_form()
int prefill_form() { return g_prefill_form.load(); }
static std::atomic<int> g_attention_variant{0};   // tw_kv_debug_set_attention_variant, see attention_variant()
int attention_variant() { return g_attention_variant.load(); }
const char* volatile g_last_scan_kernel = "none";
thread_local hipEvent_t t_scan_start = nullptr;
thread_local hipEvent_t t_scan_stop = nullptr;
}  // namespace twkv

// ---------------------------------------------------------------- error state
namespace {
thread_local int g_err = 0;
thread_local char g_err_msg[256] = "";
std::atomic<int> g_variant{0};   // tw_kv_debug_set_attention_variant
std::atomic<int> g_nsplit_override{0};

constexpr int kMaxSplits = 64;
constexpr long long kPagedBlockFloats = 64 * (long long)kPartialFloats + 128 + 4;  // per (sequence, head): partials + rotated query
constexpr int kMinChunk = 128;       // tokens
constexpr int kTargetGroups = 2048;  // workgroups wanted per launch: 8 per CU on 256 CUs
constexpr int kMinRowChunk = 64;         // tokens: eight per wave
constexpr int kTargetItems = 512;    // (sequence, chunk) items wanted by the persistent MFMA scan: one per resident workgroup

void set_error(int code, const char* fmt, ...) {
    if (g_err != 0) return;  // keep the first one
    g_err = code;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err_msg, sizeof(g_err_msg), fmt, ap);
    va_end(ap);
}

void check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) set_error((int)e, "%s: %s", what, hipGetErrorString(e));
}

const half_t* H(const tw_half* p) { return reinterpret_cast<const half_t*>(p); }
half_t* H(tw_half* p) { return reinterpret_cast<half_t*>(p); }

bool check_shape(const char* fn, int num_heads, int num_kv_heads, int head_dim) {
    if (head_dim != kHeadDim) {
        set_error(1, "%s: head_dim=%d, only 128 is supported", fn, head_dim);
        return false;
    }
    if (num_kv_heads <= 0 || num_heads <= 0 || num_heads % num_kv_heads != 0) {
        set_error(1, "%s: num_heads=%d not a multiple of num_kv_heads=%d", fn, num_heads, num_kv_heads);
        return false;
    }
    return true;
}

bool check_bits(const char* fn, int bits) {
    if (bits != 2 && bits != 4) {
        set_error(1, "%s: bits=%d, expected 2 or 4", fn, bits);
        return false;
    }
    return true;
}

int compute_units_host();

// Split the context over workgroups.  ctx_bound: upper bound of positions+1
// known to the host (max_seq_len, or pos+1 for the by-value entry points).
// ws_floats_per_head: room per (sequence, head) in the caller's workspace.
void plan_splits(AttnArgs& a, int ctx_bound, long long ws_floats_per_head) {
    if (ctx_bound < 1) ctx_bound = 1;
    const bool mfma = a.bits != 0 && g_variant.load() != 1 && a.num_heads / a.num_kv_heads <= 4;
    // workgroups per split: the MFMA scan takes up to 8 KV heads per workgroup,
    // the vector-ALU kernel one (KV head, tile of query heads) each
    long long base_groups;
    // fp16 whole-row scan: 16 or more (sequence, head block) pairs, or fewer with a context long enough that its
    // chunks (at most kMaxSplits of at least kMinRowChunk tokens) still make 256 workgroups -- below that the kernel
    // with a workgroup per (sequence, KV head, chunk) has more of them in flight
    bool rows = !mfma && attention_rows_usable(a);
    if (rows) {
        const long long pairs = (long long)a.G * attention_rows_groups(a);
        const long long chunks = std::min<long long>(kMaxSplits, (ctx_bound + kMinRowChunk - 1) / kMinRowChunk);
        rows = pairs >= 16 || pairs * chunks >= 256;
    }
    if (mfma) {
        base_groups = (long long)a.G * ((a.num_kv_heads + 7) / 8);
    } else if (rows) {
        base_groups = (long long)a.G * attention_rows_groups(a);
    } else {
        const int group = a.num_heads / a.num_kv_heads;
        const int rt = (group % 4 == 0) ? 4 : (group % 2 == 0) ? 2 : 1;
        base_groups = (long long)a.G * a.num_kv_heads * (group / rt);
    }
    int want = g_nsplit_override.load();
    if (want <= 0) {
        // the whole-row fp16 scan runs two workgroups per CU at once and the MFMA scans kTargetItems items: as many
        // chunks as still fit in that one go (one more would leave a second round for a few items: batch 48 took
        // 112 us with 11 chunks per sequence, 528 items)
        if (rows) want = (int)std::max<long long>(1, 2LL * compute_units_host() / base_groups);
        else if (mfma) want = (int)std::max<long long>(1, kTargetItems / base_groups);
        else want = (int)((kTargetGroups + base_groups - 1) / base_groups);
    }
    const int min_chunk = rows ? kMinRowChunk : kMinChunk;
    int max_by_ctx = (ctx_bound + min_chunk - 1) / min_chunk;
    // a block holds nsplit partials, then (16-byte aligned) the rotated query
    int max_by_ws = a.ws ? (int)((ws_floats_per_head - kHeadDim - 3) / kPartialFloats) : 0;
    int nsplit = want;
    if (nsplit > max_by_ctx) nsplit = max_by_ctx;
    if (nsplit > kMaxSplits) nsplit = kMaxSplits;
    if (nsplit < 1) nsplit = 1;
    bool have_ws = max_by_ws >= 1;
    if (have_ws && nsplit > max_by_ws) nsplit = max_by_ws;
    if (!have_ws) nsplit = 1;
    a.nsplit = nsplit;
    // The MFMA scan may cut a ragged batch into up to max_slots pieces per sequence instead
    // (a long sequence among short ones takes several groups' worth of tiles).
    int slots = nsplit;
    if (have_ws && (mfma || rows) && a.pos_mode != kPosScalar) {
        slots = 4 * nsplit + 2;
        if (slots > max_by_ws) slots = max_by_ws;
        if (slots > kMaxSplits) slots = kMaxSplits;
        if (slots < nsplit) slots = nsplit;
    }
    a.max_slots = slots;
    if (have_ws) {
        long long qoff = ((long long)slots * kPartialFloats + 3) & ~3LL;
        a.ws_stride = qoff + kHeadDim;
        a.qrot = a.ws + qoff;
    } else {
        a.ws = nullptr;          // too small to hold anything: single pass, no workspace
        a.ws_stride = 0;
        a.qrot = nullptr;
    }
    if (rows) {
        a.even_chunks = 1;
        a.slots_from_ws = 1;
        // ragged batches: cut the work by tokens, not by sequence (decided on the device from the positions)
        a.balance = (a.pos_mode != kPosScalar && attention_rows_balances(a)) ? 1 : 0;
        a.force_merge = a.balance;
    }
}

// Optional timing of the dominant (context-scanning) kernel with HIP events on
// the launch stream; off by default, never active under stream capture.
constexpr int kProfSlots = 4096;
struct Profiler {
    std::atomic<int> enabled{0};
    hipEvent_t start[kProfSlots];
    hipEvent_t stop[kProfSlots];
    int created = 0;
    int used = 0;
} g_prof;

// query_done: q_rot is already in the workspace (the fused append + attention entry
// rotates the query together with the appended rows).
bool mfma_wanted(const AttnArgs& a) { return a.bits != 0 && g_variant.load() != 1; }

// When the profiler is on (and the stream is not capturing: events cannot ride on a launch that is only being
// recorded into a graph) the next scan launch on this thread carries a pair of its events (launch_scan_kernel).
void attach_profiler(hipStream_t s) {
    bool prof = g_prof.enabled.load() != 0 && g_prof.used < kProfSlots;
    if (prof) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &st) != hipSuccess || st != hipStreamCaptureStatusNone) prof = false;
    }
    if (prof) {
        while (g_prof.created <= g_prof.used) {
            if (hipEventCreate(&g_prof.start[g_prof.created]) != hipSuccess ||
                hipEventCreate(&g_prof.stop[g_prof.created]) != hipSuccess) { prof = false; break; }
            g_prof.created++;
        }
    }
    if (prof) { t_scan_start = g_prof.start[g_prof.used]; t_scan_stop = g_prof.stop[g_prof.used]; g_prof.used++; }
}

void run_attention(AttnArgs& a, hipStream_t s, const char* fn, bool query_done = false, bool may_profile = true) {
    if (may_profile) attach_profiler(s);   // creates events on first use: not for the entry point that allocates nothing
    if (a.bits == 0 && g_variant.load() != 1 && prefill_f16_mfma_usable(a)) {   // fp16 prefill: one MFMA kernel, no splits
        launch_prefill_f16_mfma(a, s, g_prefill_form.load());
        t_scan_start = t_scan_stop = nullptr;
        check_launch(fn);
        return;
    }
    const bool mfma = mfma_wanted(a) && prepare_attention_mfma(a, s, !query_done);   // (its query rotation is not a scan launch)
    bool finished = false;
    if (mfma) finished = launch_attention_mfma_scan(a, s);
    else launch_attention_valu(a, s);
    t_scan_start = t_scan_stop = nullptr;
    if (!finished && (a.nsplit > 1 || a.force_merge)) {
        if (!(g_variant.load() != 1 && launch_merge_rotate(a, s))) launch_attention_merge(a, s);
    }
    check_launch(fn);
}
int compute_units_host() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    return cus;
}
}  // namespace

extern "C" {

int tw_kv_last_error(void) { return g_err; }
const char* tw_kv_last_error_string(void) { return g_err_msg; }
void tw_kv_clear_error(void) { g_err = 0; g_err_msg[0] = 0; }
const char* tw_kv_build_info(void) { return "triebwerk_kv gfx950 " __DATE__ " " __TIME__; }
void tw_kv_debug_set_attention_variant(int v) { g_variant.store(v); twkv::g_attention_variant.store(v); }
int tw_kv_debug_get_attention_variant(void) { return g_variant.load(); }
void tw_kv_debug_set_num_splits(int n) { g_nsplit_override.store(n); }
void tw_kv_debug_set_prefill_form(int form) { g_prefill_form.store(form); }
void tw_kv_debug_set_decode_fused(int mode) { g_decode_fused.store(mode); }

// shares' sums that fit the attention scratch (max_seq_len floats per sequence and head): a power of two up to 8
static int shares_that_fit(int max_seq_len) {
    int n = 1;
    while (n < 8 && 2 * n * kPartialFloats <= max_seq_len) n *= 2;
    return n;
}

int tw_kv_decode_step_plan2(int G, int num_heads, int num_kv_heads, int bits, int max_seq_len, int ctx_min, int ctx_max,
                            int can_share) {
    if (G <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads != 0 || (bits != 2 && bits != 4)) return 0;
    const int group = num_heads / num_kv_heads;
    if (group != 1 && group != 2 && group != 4) return 0;
    const bool allow_pairs = g_decode_fused.load() != 3;
    const int hkw = decode_fused_heads_per_workgroup(G, num_heads, num_kv_heads, bits, allow_pairs);
    const int split = 16 / hkw;                                   // parts of the context per head: waves / heads
    const bool known = ctx_max > 0;
    const int bound = known ? ctx_max : max_seq_len;
    if (bound <= 256 * split) return 1;                           // at most 8 tiles of 32 tokens per wave
    if (!known || (long long)(ctx_max - ctx_min) * 8 > ctx_max) return 0;   // lengths unknown or ragged: the balanced walk
    // Equal lengths: the cheaper of the two by estimates fitted to measured launches (microseconds per layer; the
    // figures live in one table, plan_constants): one launch as decode_fused_shape counts it (with a sequence's context
    // shared by workgroups where the caller can hand over tickets and the batch alone leaves compute units idle), three
    // launches as decode_three_estimate_us does.
    const int max_shares = can_share != 0 ? shares_that_fit(max_seq_len) : 1;
    const double one = decode_fused_shape(G, num_heads, num_kv_heads, bits, allow_pairs, max_shares, ctx_max).us;
    const double three = decode_three_estimate_us(G, num_kv_heads, bits, ctx_max);
    return one <= three ? 1 : 0;
}
int tw_kv_decode_step_plan(int G, int num_heads, int num_kv_heads, int bits, int max_seq_len, int ctx_min, int ctx_max) {
    return tw_kv_decode_step_plan2(G, num_heads, num_kv_heads, bits, max_seq_len, ctx_min, ctx_max, 0);
}
void tw_kv_debug_set_fused_shape(int hkw, int shares) { decode_fused_force_shape(hkw, shares); }
long long tw_kv_decode_fused_launches(void) { return g_fused_launches.load(); }
const char* tw_kv_debug_last_scan_kernel(void) { return twkv::g_last_scan_kernel; }

void tw_kv_debug_profile_attention(int enable) {
    g_prof.enabled.store(enable);
    if (enable) g_prof.used = 0;
}

int tw_kv_debug_profile_read(double* total_ms, int* launches) {
    double sum = 0.0;
    for (int i = 0; i < g_prof.used; i++) {
        if (hipEventSynchronize(g_prof.stop[i]) != hipSuccess) return -1;
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, g_prof.start[i], g_prof.stop[i]) != hipSuccess) return -1;
        sum += ms;
    }
    if (total_ms) *total_ms = sum;
    if (launches) *launches = g_prof.used;
    g_prof.used = 0;
    return 0;
}

// A plain streaming read of [buf, buf + bytes): 16 bytes per lane, eight loads in flight,
// grid-stride.  What this GPU delivers for the friendliest possible access pattern; the
// benchmark quotes it next to the scan's rate.
__device__ unsigned g_stream_read_sink;
__global__ void __launch_bounds__(512) stream_read_kernel(const uint4* __restrict__ src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned acc = 0;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = src[i + j * stride];
#pragma unroll
        for (int j = 0; j < 8; j++) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
    }
    for (; i < n16; i += stride) { uint4 v = src[i]; acc ^= v.x ^ v.y ^ v.z ^ v.w; }
    if (acc == 0x9e3779b9u) g_stream_read_sink = acc;   // keeps the loads alive; practically never taken
}

double tw_kv_measure_read_bandwidth(const void* dev_buf, size_t bytes, int iters, hipStream_t s) {
    if (!dev_buf || bytes < 16 || iters < 1 || (reinterpret_cast<uintptr_t>(dev_buf) & 15u) != 0) {
        set_error(1, "tw_kv_measure_read_bandwidth: needs a 16-byte aligned device buffer and iters >= 1");
        return 0.0;
    }
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return 0.0;
    const size_t n16 = bytes / 16;
    const int bpc = 4, thr = 512;                 // the best of several shapes tried on MI355X
    const int grid = compute_units_host() * bpc;
    hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(thr), 0, s, reinterpret_cast<const uint4*>(dev_buf), n16);
    hipEventRecord(e0, s);
    for (int i = 0; i < iters; i++)
        hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(thr), 0, s, reinterpret_cast<const uint4*>(dev_buf), n16);
    hipEventRecord(e1, s);
    float ms = 0.0f;
    double gbps = 0.0;
    if (hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess && ms > 0.0f)
        gbps = (double)n16 * 16.0 * iters / (ms * 1e-3) * 1e-9;
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    check_launch("tw_kv_measure_read_bandwidth");
    return gbps;
}

int tw_kv_broadcast_rows(void* const* bases, const size_t* seq_bytes, const size_t* bytes, int narrays,
                         int src, int dst_begin, int dst_end, hipStream_t s) {
    if (!bases || !seq_bytes || !bytes || narrays < 0 || narrays > 4 || src < 0 || dst_begin < 0 || dst_end < dst_begin) {
        set_error(1, "tw_kv_broadcast_rows: bad arguments");
        return -1;
    }
    BroadcastArgs b{};
    b.src = src; b.dst_begin = dst_begin; b.dst_end = dst_end;
    for (int i = 0; i < narrays; i++) {
        if (!bases[i] || bytes[i] > seq_bytes[i] || ((reinterpret_cast<uintptr_t>(bases[i]) | seq_bytes[i] | bytes[i]) & 1u)) {
            set_error(1, "tw_kv_broadcast_rows: arrays must be fp16-aligned and T rows must fit a sequence");
            return -1;
        }
        if (bytes[i] == 0) continue;
        b.base[b.narrays] = static_cast<char*>(bases[i]);
        b.seq_bytes[b.narrays] = seq_bytes[i];
        b.bytes[b.narrays] = bytes[i];
        b.narrays++;
    }
    launch_broadcast_rows(b, s);
    check_launch("tw_kv_broadcast_rows");
    return 0;
}

size_t tw_attention_workspace_floats(int G, int num_heads, int max_context) {
    (void)max_context;
    return (size_t)G * num_heads * kPagedBlockFloats;
}

// ---------------------------------------------------------------- append
void launch_kv_cache_write_batch(tw_half* ck, tw_half* cv, const tw_half* k, const tw_half* v,
                                 const int* pos, int msl, int G, int kv_dim, hipStream_t s) {
    launch_kv_write(H(ck), H(cv), H(k), H(v), pos, nullptr, 0, msl, G, kv_dim, s);
    check_launch("launch_kv_cache_write_batch");
}

void tw_paged_kv_cache_write_batch(tw_half* ck, tw_half* cv, const tw_half* k, const tw_half* v,
                                   const int* positions, const int* block_table, int bt_stride,
                                   int G, int kv_dim, hipStream_t s) {
    if (!block_table) { set_error(1, "tw_paged_kv_cache_write_batch: block_table is NULL"); return; }
    launch_kv_write(H(ck), H(cv), H(k), H(v), positions, block_table, bt_stride, 0, G, kv_dim, s);
    check_launch("tw_paged_kv_cache_write_batch");
}

static void fill_quant_segments(RotArgs& r, uint8_t* c0, tw_half* n0, const tw_half* s0, uint8_t* c1,
                                tw_half* n1, const tw_half* s1, int nstreams, int nrows,
                                int num_kv_heads, int kv_dim) {
    uint8_t* c[2] = {c0, c1};
    tw_half* n[2] = {n0, n1};
    const tw_half* src[2] = {s0, s1};
    for (int i = 0; i < nstreams; i++) {
        int k = r.nseg++;
        r.seg_src[k] = H(src[i]);
        r.seg_stride[k] = kv_dim;
        r.seg_heads[k] = num_kv_heads;
        r.seg_nvec[k] = nrows * num_kv_heads;
        r.seg_units[k] = (r.seg_nvec[k] + 15) / 16 * 8;
        r.seg_kind[k] = 0;
        r.seg_codes[k] = c[i];
        r.seg_norms[k] = H(n[i]);
    }
}

static void quantize_common(const char* fn, uint8_t* c0, tw_half* n0, const tw_half* s0,
                            uint8_t* c1, tw_half* n1, const tw_half* s1, int nstreams,
                            const tw_half* rotation, const int* positions, const int* block_table,
                            int bt_stride, long long seq_stride_rows, int token_list, int nrows,
                            int num_kv_heads, int head_dim, int kv_dim, int bits, hipStream_t s) {
    if (!check_shape(fn, num_kv_heads, num_kv_heads, head_dim) || !check_bits(fn, bits)) return;
    if (kv_dim < num_kv_heads * head_dim) {
        set_error(1, "%s: kv_dim=%d smaller than num_kv_heads*head_dim", fn, kv_dim);
        return;
    }
    if (g_variant.load() == 1) {   // vector-ALU kernel, kept for cross-checks
        QuantArgs a;
        memset(&a, 0, sizeof(a));
        a.codes[0] = c0; a.norms[0] = H(n0); a.src[0] = H(s0);
        a.codes[1] = c1; a.norms[1] = H(n1); a.src[1] = H(s1);
        a.nstreams = nstreams;
        a.rotation = H(rotation);
        a.positions = positions;
        a.block_table = block_table;
        a.bt_stride = bt_stride;
        a.seq_stride_rows = seq_stride_rows;
        a.token_list = token_list;
        a.nrows = nrows;
        a.num_kv_heads = num_kv_heads;
        a.kv_dim = kv_dim;
        launch_turbo_quantize(a, bits, s);
        check_launch(fn);
        return;
    }
    RotArgs r;
    memset(&r, 0, sizeof(r));
    fill_quant_segments(r, c0, n0, s0, c1, n1, s1, nstreams, nrows, num_kv_heads, kv_dim);
    r.rotation = H(rotation);
    r.positions = positions;
    r.block_table = block_table;
    r.bt_stride = bt_stride;
    r.seq_stride_rows = seq_stride_rows;
    r.token_list = token_list;
    r.num_kv_heads = num_kv_heads;
    launch_rotate(r, bits, s);
    check_launch(fn);
}

void launch_turbo_kv_quantize(uint8_t* cache_q, tw_half* cache_norms, const tw_half* kv_buf,
                              const tw_half* rotation, const int* positions, int max_seq_len,
                              int num_tokens, int num_kv_heads, int head_dim, int kv_dim,
                              int bits, hipStream_t s) {
    quantize_common("launch_turbo_kv_quantize", cache_q, cache_norms, kv_buf, nullptr, nullptr,
                    nullptr, 1, rotation, positions, nullptr, 0, max_seq_len, 1, num_tokens,
                    num_kv_heads, head_dim, kv_dim, bits, s);
}

void launch_turbo_kv_quantize_batch(uint8_t* cache_q, tw_half* cache_norms, const tw_half* kv_buf,
                                    const tw_half* rotation, const int* positions, int max_seq_len,
                                    int G, int num_kv_heads, int head_dim, int kv_dim,
                                    int bits, hipStream_t s) {
    quantize_common("launch_turbo_kv_quantize_batch", cache_q, cache_norms, kv_buf, nullptr,
                    nullptr, nullptr, 1, rotation, positions, nullptr, 0, max_seq_len, 0, G,
                    num_kv_heads, head_dim, kv_dim, bits, s);
}

void tw_turbo_kv_append_batch(uint8_t* ck_q, tw_half* k_norms, uint8_t* cv_q, tw_half* v_norms,
                              const tw_half* k_buf, const tw_half* v_buf, const tw_half* rotation,
                              const int* positions, int max_seq_len, int G, int num_kv_heads,
                              int head_dim, int kv_dim, int bits, hipStream_t s) {
    quantize_common("tw_turbo_kv_append_batch", ck_q, k_norms, k_buf, cv_q, v_norms, v_buf, 2,
                    rotation, positions, nullptr, 0, max_seq_len, 0, G, num_kv_heads, head_dim,
                    kv_dim, bits, s);
}

void tw_turbo_kv_append_tokens(uint8_t* ck_q, tw_half* k_norms, uint8_t* cv_q, tw_half* v_norms,
                               const tw_half* k_buf, const tw_half* v_buf, const tw_half* rotation,
                               const int* positions, int max_seq_len, int num_tokens, int num_kv_heads,
                               int head_dim, int kv_dim, int bits, hipStream_t s) {
    quantize_common("tw_turbo_kv_append_tokens", ck_q, k_norms, k_buf, cv_q, v_norms, v_buf, 2,
                    rotation, positions, nullptr, 0, max_seq_len, 1, num_tokens, num_kv_heads, head_dim,
                    kv_dim, bits, s);
}

void tw_paged_turbo_kv_append_batch(uint8_t* ck_q, tw_half* k_norms, uint8_t* cv_q,
                                    tw_half* v_norms, const tw_half* k_buf, const tw_half* v_buf,
                                    const tw_half* rotation, const int* positions,
                                    const int* block_table, int bt_stride, int G,
                                    int num_kv_heads, int head_dim, int kv_dim, int bits,
                                    hipStream_t s) {
    if (!block_table) { set_error(1, "tw_paged_turbo_kv_append_batch: block_table is NULL"); return; }
    quantize_common("tw_paged_turbo_kv_append_batch", ck_q, k_norms, k_buf, cv_q, v_norms, v_buf,
                    2, rotation, positions, block_table, bt_stride, 0, 0, G, num_kv_heads,
                    head_dim, kv_dim, bits, s);
}

void launch_increment_positions(int* positions, int G, hipStream_t s) {
    launch_increment(positions, G, s);
    check_launch("launch_increment_positions");
}

// ---------------------------------------------------------------- attention
// Output gate of the attention call being set up on this thread (tw_layer_attention_step sets it around
// the entry point it forwards to).
static thread_local const tw_half* t_gate = nullptr;
static thread_local long long t_gate_stride = 0;

static void fill_common(AttnArgs& a, tw_half* out, const tw_half* q, int q_stride, const void* k,
                        const void* v, const tw_half* kn, const tw_half* vn, const tw_half* rot,
                        int G, int num_heads, int num_kv_heads, int bits, float* ws) {
    memset(&a, 0, sizeof(a));
    a.q = H(q); a.out = H(out); a.q_stride = q_stride;
    a.k = k; a.v = v; a.k_norms = H(kn); a.v_norms = H(vn); a.rotation = H(rot);
    a.G = G; a.num_heads = num_heads; a.num_kv_heads = num_kv_heads; a.bits = bits;
    a.ws = ws;
    a.gate = H(t_gate); a.gate_stride = t_gate_stride;
}

void launch_gqa_attention(const tw_half* q, const tw_half* k_cache, const tw_half* v_cache,
                          tw_half* output, float* attn_scratch, int pos, int max_seq_len,
                          int num_heads, int num_kv_heads, int head_dim, hipStream_t stream) {
    if (!check_shape("launch_gqa_attention", num_heads, num_kv_heads, head_dim)) return;
    if (pos < 0) { set_error(1, "launch_gqa_attention: pos=%d", pos); return; }
    AttnArgs a;
    fill_common(a, output, q, num_heads * head_dim, k_cache, v_cache, nullptr, nullptr, nullptr, 1,
                num_heads, num_kv_heads, 0, attn_scratch);
    a.pos_mode = kPosScalar; a.pos_scalar = pos; a.seq_stride_rows = 0;
    plan_splits(a, pos + 1, max_seq_len);
    run_attention(a, stream, "launch_gqa_attention");
}

void launch_gqa_attention_batch(tw_half* out, const tw_half* q, const tw_half* ck,
                                const tw_half* cv, float* as, const int* pos, int msl, int G,
                                int num_heads, int num_kv_heads, int head_dim, int q_dim,
                                int kv_dim, hipStream_t s) {
    if (!check_shape("launch_gqa_attention_batch", num_heads, num_kv_heads, head_dim)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "launch_gqa_attention_batch: kv_dim=%d != num_kv_heads*head_dim", kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck, cv, nullptr, nullptr, nullptr, G, num_heads, num_kv_heads, 0, as);
    a.pos_mode = kPosArray; a.positions = pos; a.seq_stride_rows = msl;
    plan_splits(a, msl, msl);
    run_attention(a, s, "launch_gqa_attention_batch");
}

void tw_append_attention_batch(tw_half* out, const tw_half* q, const tw_half* k_buf, const tw_half* v_buf,
                               tw_half* ck, tw_half* cv, float* as, const int* pos, int msl, int G, int num_heads,
                               int num_kv_heads, int head_dim, int q_dim, int kv_dim, hipStream_t s) {
    const char* fn = "tw_append_attention_batch";
    if (!check_shape(fn, num_heads, num_kv_heads, head_dim)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "%s: kv_dim=%d != num_kv_heads*head_dim", fn, kv_dim);
        return;
    }
    const bool aligned = ((reinterpret_cast<uintptr_t>(k_buf) | reinterpret_cast<uintptr_t>(v_buf) |
                           reinterpret_cast<uintptr_t>(ck) | reinterpret_cast<uintptr_t>(cv)) & 15u) == 0;
    if (!aligned || g_decode_fused.load() == 2) {       // the two launches of the reference
        launch_kv_cache_write_batch(ck, cv, k_buf, v_buf, pos, msl, G, kv_dim, s);
        launch_gqa_attention_batch(out, q, ck, cv, as, pos, msl, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, s);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck, cv, nullptr, nullptr, nullptr, G, num_heads, num_kv_heads, 0, as);
    a.pos_mode = kPosArray; a.positions = pos; a.seq_stride_rows = msl;
    a.k_new = H(k_buf); a.v_new = H(v_buf); a.kv_new_stride = kv_dim;
    plan_splits(a, msl, msl);
    run_attention(a, s, fn);
}

void launch_gqa_prefill_attention(tw_half* out, const tw_half* q, const tw_half* ck,
                                  const tw_half* cv, float* as, int T, int msl, int num_heads,
                                  int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                  hipStream_t s) {
    (void)msl;
    if (!check_shape("launch_gqa_prefill_attention", num_heads, num_kv_heads, head_dim)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "launch_gqa_prefill_attention: kv_dim=%d != num_kv_heads*head_dim", kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck, cv, nullptr, nullptr, nullptr, T, num_heads, num_kv_heads, 0, as);
    a.pos_mode = kPosIota; a.seq_stride_rows = 0;
    plan_splits(a, T, T);   // scratch is T floats per (query, head), kernels.cu:1088
    run_attention(a, s, "launch_gqa_prefill_attention");
}

void launch_turbo_gqa_attention(const tw_half* q, const uint8_t* ck_q, const uint8_t* cv_q,
                                const tw_half* k_norms, const tw_half* v_norms,
                                const tw_half* rotation, tw_half* output, float* as, int pos,
                                int msl, int num_heads, int num_kv_heads, int head_dim, int bits,
                                hipStream_t s) {
    if (!check_shape("launch_turbo_gqa_attention", num_heads, num_kv_heads, head_dim) ||
        !check_bits("launch_turbo_gqa_attention", bits)) return;
    if (pos < 0) { set_error(1, "launch_turbo_gqa_attention: pos=%d", pos); return; }
    AttnArgs a;
    fill_common(a, output, q, num_heads * head_dim, ck_q, cv_q, k_norms, v_norms, rotation, 1,
                num_heads, num_kv_heads, bits, as);
    a.pos_mode = kPosScalar; a.pos_scalar = pos; a.seq_stride_rows = 0;
    plan_splits(a, pos + 1, msl);
    run_attention(a, s, "launch_turbo_gqa_attention");
}

void launch_turbo_gqa_attention_batch(tw_half* out, const tw_half* q, const uint8_t* ck_q,
                                      const uint8_t* cv_q, const tw_half* k_norms,
                                      const tw_half* v_norms, const tw_half* rotation, float* as,
                                      const int* pos, int msl, int G, int num_heads,
                                      int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                      int bits, hipStream_t s) {
    if (!check_shape("launch_turbo_gqa_attention_batch", num_heads, num_kv_heads, head_dim) ||
        !check_bits("launch_turbo_gqa_attention_batch", bits)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "launch_turbo_gqa_attention_batch: kv_dim=%d != num_kv_heads*head_dim", kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck_q, cv_q, k_norms, v_norms, rotation, G, num_heads,
                num_kv_heads, bits, as);
    a.pos_mode = kPosArray; a.positions = pos; a.seq_stride_rows = msl;
    plan_splits(a, msl, msl);
    run_attention(a, s, "launch_turbo_gqa_attention_batch");
}

// Range of positions + 1 over the batch as far as the caller of tw_layer_attention_step knows it on the host
// (0, 0 = unknown), for the call being set up on this thread.
static thread_local int t_ctx_min = 0;
static thread_local int t_ctx_max = 0;
// Its tickets (tw_layer_step_args::tickets): with them the one-launch step may share a sequence's context between
// workgroups; the shares' sums go to the attention scratch.
static thread_local unsigned* t_tickets = nullptr;

// The whole step in one launch (kv_decode_fused.hip)?  There one workgroup owns a sequence's heads from the first
// token to the last: it saves two launches and the scan's ramp (~10 us of a layer) and loses to the three-kernel
// path where that one's balanced walk or its row-wise loads matter.  Taken when
//   - every wave gets at most 8 tiles (launch-bound whatever the spread of the lengths), or
//   - the lengths are known to be within 1/8 of each other and the batch gives at least half the CUs a workgroup,
//     up to the size where the three-kernel path's better streaming rate has made up for its start-up
//     (measured on MI355X: 4 bit ~1M tokens per launch; 2 bit with 8 KV heads, where the three-kernel path
//     loads whole rows cooperatively, ~256k).
// false = not taken.
static FusedArgs fused_args(const tw_half* k_buf, const tw_half* v_buf, int kv_dim, uint8_t* ck_q, uint8_t* cv_q,
                            tw_half* k_norms, tw_half* v_norms) {
    FusedArgs f;
    memset(&f, 0, sizeof(f));
    f.k_src = H(k_buf); f.v_src = H(v_buf); f.kv_stride = kv_dim;
    f.k_codes = ck_q; f.v_codes = cv_q; f.k_norms = H(k_norms); f.v_norms = H(v_norms);
    return f;
}

static bool try_decode_fused(const AttnArgs& a, const FusedArgs& f_in, int msl, hipStream_t s, const char* fn) {
    const int mode = g_decode_fused.load();
    FusedArgs f = f_in;
    f.ctx_bound = t_ctx_max > 0 ? (t_ctx_max < msl ? t_ctx_max : msl) : msl;
    if (mode == 2 || g_variant.load() == 1) return false;
    if (!decode_fused_usable(a, f)) return false;
    // shares: the caller's tickets, and the attention scratch (G * num_heads * msl floats) for up to four shares' sums
    const bool can_share = t_tickets != nullptr && a.ws != nullptr && shares_that_fit(msl) >= 2 &&
                           (reinterpret_cast<uintptr_t>(a.ws) & 3u) == 0;
    f.max_shares = 1;
    if (can_share) { f.tickets = t_tickets; f.share_ws = a.ws; f.max_shares = shares_that_fit(msl); }
    if (mode != 1 && mode != 3 &&
        !tw_kv_decode_step_plan2(a.G, a.num_heads, a.num_kv_heads, a.bits, msl, t_ctx_min, t_ctx_max, can_share ? 1 : 0)) return false;
    attach_profiler(s);
    g_fused_launches.fetch_add(1);
    launch_decode_fused(a, f, s, /*allow_pairs=*/mode != 3);
    t_scan_start = t_scan_stop = nullptr;
    check_launch(fn);
    return true;
}

void tw_turbo_append_attention_batch(tw_half* out, const tw_half* q, const tw_half* k_buf,
                                     const tw_half* v_buf, uint8_t* ck_q, uint8_t* cv_q,
                                     tw_half* k_norms, tw_half* v_norms, const tw_half* rotation,
                                     float* as, const int* pos, int msl, int G, int num_heads,
                                     int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                     int bits, hipStream_t s) {
    const char* fn = "tw_turbo_append_attention_batch";
    if (!check_shape(fn, num_heads, num_kv_heads, head_dim) || !check_bits(fn, bits)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "%s: kv_dim=%d != num_kv_heads*head_dim", fn, kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck_q, cv_q, k_norms, v_norms, rotation, G, num_heads,
                num_kv_heads, bits, as);
    a.pos_mode = kPosArray; a.positions = pos; a.seq_stride_rows = msl;
    if (try_decode_fused(a, fused_args(k_buf, v_buf, kv_dim, ck_q, cv_q, k_norms, v_norms), msl, s, fn)) return;
    plan_splits(a, msl, msl);
    // one rotation launch for the appended K and V rows and, when the MFMA scan will run,
    // for the query as well
    const int R = num_heads / num_kv_heads;
    const bool fuse_q = mfma_wanted(a) && a.qrot && (R == 1 || R == 2 || R == 4) &&
                        (reinterpret_cast<uintptr_t>(a.qrot) & 15u) == 0;
    if (g_variant.load() == 1 || !fuse_q) {
        tw_turbo_kv_append_batch(ck_q, k_norms, cv_q, v_norms, k_buf, v_buf, rotation, pos, msl, G,
                                 num_kv_heads, head_dim, kv_dim, bits, s);
        run_attention(a, s, fn);
        return;
    }
    RotArgs r;
    memset(&r, 0, sizeof(r));
    fill_quant_segments(r, ck_q, k_norms, k_buf, cv_q, v_norms, v_buf, 2, G, num_kv_heads, kv_dim);
    int k = r.nseg++;
    r.seg_src[k] = H(q);
    r.seg_stride[k] = q_dim;
    r.seg_heads[k] = num_heads;
    r.seg_nvec[k] = G * num_heads;
    r.seg_units[k] = (r.seg_nvec[k] + 15) / 16 * 8;
    r.seg_kind[k] = 1;
    r.rotation = H(rotation);
    r.positions = pos;
    r.seq_stride_rows = msl;
    r.num_kv_heads = num_kv_heads;
    r.qrot = a.qrot;
    r.qrot_stride = a.ws_stride;
    r.q_scale = attention_mfma_q_scale(bits);
    launch_rotate(r, bits, s);
    run_attention(a, s, fn, /*query_done=*/true);
}

// ---------------------------------------------------------------- producers of q and k
static bool check_rope_dim(const char* fn, int rope_dim) {
    if (rope_dim == kHeadDim || (rope_dim >= 16 && rope_dim <= 64 && rope_dim % 16 == 0)) return true;
    set_error(1, "%s: rope_dim=%d, expected 128 or a multiple of 16 up to 64", fn, rope_dim);
    return false;
}

static void fill_producer(ProducerArgs& p, tw_half* q, tw_half* k, int rows, int num_heads,
                          int num_kv_heads, long long q_stride, long long kv_stride) {
    memset(&p, 0, sizeof(p));
    p.q = reinterpret_cast<half_t*>(q);
    p.k = reinterpret_cast<half_t*>(k);
    p.rows = rows;
    p.num_heads = num_heads;
    p.num_kv_heads = num_kv_heads;
    p.q_stride = q_stride;
    p.kv_stride = kv_stride;
}

void launch_qk_norm_batch(tw_half* q, tw_half* k, const tw_half* q_weight, const tw_half* k_weight,
                          int num_q, int num_kv, int head_dim, int G, float eps, int q_dim,
                          int kv_dim, hipStream_t s, bool biased) {
    const char* fn = "launch_qk_norm_batch";
    if (head_dim != kHeadDim) { set_error(1, "%s: head_dim=%d, only 128 is supported", fn, head_dim); return; }
    ProducerArgs p;
    fill_producer(p, q, k, G, num_q, num_kv, q_dim, kv_dim);
    p.norm = 1; p.q_weight = H(q_weight); p.k_weight = H(k_weight); p.eps = eps; p.biased = biased ? 1 : 0;
    launch_producer(p, s);
    check_launch(fn);
}

void launch_rope_batch(tw_half* q, tw_half* k, const tw_half* cos_table, const tw_half* sin_table,
                       const int* positions, int max_seq_len, int G, int num_heads,
                       int num_kv_heads, int head_dim, int q_dim, int kv_dim, int rope_dim,
                       hipStream_t s) {
    (void)max_seq_len;
    const char* fn = "launch_rope_batch";
    if (head_dim != kHeadDim) { set_error(1, "%s: head_dim=%d, only 128 is supported", fn, head_dim); return; }
    if (!check_rope_dim(fn, rope_dim)) return;
    ProducerArgs p;
    fill_producer(p, q, k, G, num_heads, num_kv_heads, q_dim, kv_dim);
    p.cos_table = H(cos_table); p.sin_table = H(sin_table); p.rope_dim = rope_dim; p.positions = positions;
    launch_producer(p, s);
    check_launch(fn);
}

void launch_qk_norm(tw_half* q, tw_half* k, const tw_half* q_weight, const tw_half* k_weight,
                    int num_q_heads, int num_kv_heads, int head_dim, float eps, hipStream_t stream) {
    const char* fn = "launch_qk_norm";
    if (head_dim != kHeadDim) { set_error(1, "%s: head_dim=%d, only 128 is supported", fn, head_dim); return; }
    ProducerArgs p;
    fill_producer(p, q, k, 1, num_q_heads, num_kv_heads, 0, 0);
    p.norm = 1; p.q_weight = H(q_weight); p.k_weight = H(k_weight); p.eps = eps;
    launch_producer(p, stream);
    check_launch(fn);
}

void launch_rope(tw_half* q, tw_half* k, const tw_half* cos_table, const tw_half* sin_table,
                 int pos, int max_seq_len, int num_heads, int num_kv_heads, int head_dim,
                 hipStream_t stream) {
    (void)max_seq_len;
    const char* fn = "launch_rope";
    if (head_dim != kHeadDim) { set_error(1, "%s: head_dim=%d, only 128 is supported", fn, head_dim); return; }
    ProducerArgs p;
    fill_producer(p, q, k, 1, num_heads, num_kv_heads, 0, 0);
    p.cos_table = H(cos_table); p.sin_table = H(sin_table); p.rope_dim = head_dim;
    p.pos_scalar = pos; p.single_order = 1;
    launch_producer(p, stream);
    check_launch(fn);
}

void tw_qk_norm_rope_turbo_append_attention_batch(
    tw_half* out, tw_half* q, tw_half* k_buf, const tw_half* v_buf, const tw_half* q_weight,
    const tw_half* k_weight, float eps, int biased, const tw_half* cos_table,
    const tw_half* sin_table, int rope_dim, uint8_t* ck_q, uint8_t* cv_q, tw_half* k_norms,
    tw_half* v_norms, const tw_half* rotation, float* as, const int* pos, int msl, int G,
    int num_heads, int num_kv_heads, int head_dim, int q_dim, int kv_dim, int bits, hipStream_t s) {
    const char* fn = "tw_qk_norm_rope_turbo_append_attention_batch";
    if (!check_shape(fn, num_heads, num_kv_heads, head_dim) || !check_bits(fn, bits)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "%s: kv_dim=%d != num_kv_heads*head_dim", fn, kv_dim);
        return;
    }
    if (cos_table && !check_rope_dim(fn, rope_dim)) return;
    if ((q_weight == nullptr) != (k_weight == nullptr) || (cos_table == nullptr) != (sin_table == nullptr)) {
        set_error(1, "%s: q_weight/k_weight and cos_table/sin_table come in pairs", fn);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck_q, cv_q, k_norms, v_norms, rotation, G, num_heads,
                num_kv_heads, bits, as);
    a.pos_mode = kPosArray; a.positions = pos; a.seq_stride_rows = msl;
    {
        FusedArgs f = fused_args(k_buf, v_buf, kv_dim, ck_q, cv_q, k_norms, v_norms);
        f.q_weight = H(q_weight); f.k_weight = H(k_weight); f.eps = eps; f.biased = biased ? 1 : 0;
        f.cos_table = H(cos_table); f.sin_table = H(sin_table); f.rope_dim = rope_dim;
        if (try_decode_fused(a, f, msl, s, fn)) return;
    }
    plan_splits(a, msl, msl);
    const int R = num_heads / num_kv_heads;
    const bool aligned = ((reinterpret_cast<uintptr_t>(q_weight) | reinterpret_cast<uintptr_t>(k_weight) |
                           reinterpret_cast<uintptr_t>(cos_table) | reinterpret_cast<uintptr_t>(sin_table)) & 15u) == 0;
    const bool fuse = g_variant.load() != 1 && mfma_wanted(a) && a.qrot && (R == 1 || R == 2 || R == 4) &&
                      (reinterpret_cast<uintptr_t>(a.qrot) & 15u) == 0 && aligned;
    if (!fuse) {   // the kernels of their own, in place, then the plain fused step
        if (q_weight) launch_qk_norm_batch(q, k_buf, q_weight, k_weight, num_heads, num_kv_heads, head_dim, G, eps,
                                           q_dim, kv_dim, s, biased != 0);
        if (cos_table) launch_rope_batch(q, k_buf, cos_table, sin_table, pos, msl, G, num_heads, num_kv_heads,
                                         head_dim, q_dim, kv_dim, rope_dim, s);
        tw_turbo_append_attention_batch(out, q, k_buf, v_buf, ck_q, cv_q, k_norms, v_norms, rotation, as, pos, msl,
                                        G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits, s);
        return;
    }
    RotArgs r;
    memset(&r, 0, sizeof(r));
    fill_quant_segments(r, ck_q, k_norms, k_buf, cv_q, v_norms, v_buf, 2, G, num_kv_heads, kv_dim);
    int k = r.nseg++;
    r.seg_src[k] = H(q);
    r.seg_stride[k] = q_dim;
    r.seg_heads[k] = num_heads;
    r.seg_nvec[k] = G * num_heads;
    r.seg_units[k] = (r.seg_nvec[k] + 15) / 16 * 8;
    r.seg_kind[k] = 1;
    r.rotation = H(rotation);
    r.positions = pos;
    r.seq_stride_rows = msl;
    r.num_kv_heads = num_kv_heads;
    r.qrot = a.qrot;
    r.qrot_stride = a.ws_stride;
    r.q_scale = attention_mfma_q_scale(bits);
    // segment 0 = K rows, 1 = V rows (left as they are), 2 = Q rows
    r.seg_weight[0] = H(k_weight);
    r.seg_weight[2] = H(q_weight);
    r.seg_rope[0] = r.seg_rope[2] = cos_table ? 1 : 0;
    r.eps = eps;
    r.biased = biased ? 1 : 0;
    r.cos_table = H(cos_table);
    r.sin_table = H(sin_table);
    r.rope_dim = rope_dim;
    launch_rotate(r, bits, s);
    run_attention(a, s, fn, /*query_done=*/true);
}

void tw_qk_norm_rope_append_attention_batch(
    tw_half* out, tw_half* q, const tw_half* k_buf, const tw_half* v_buf, const tw_half* q_weight,
    const tw_half* k_weight, float eps, int biased, const tw_half* cos_table,
    const tw_half* sin_table, int rope_dim, tw_half* ck, tw_half* cv, float* as, const int* pos,
    int msl, int G, int num_heads, int num_kv_heads, int head_dim, int q_dim, int kv_dim,
    hipStream_t s) {
    const char* fn = "tw_qk_norm_rope_append_attention_batch";
    if (!check_shape(fn, num_heads, num_kv_heads, head_dim)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "%s: kv_dim=%d != num_kv_heads*head_dim", fn, kv_dim);
        return;
    }
    if (cos_table && !check_rope_dim(fn, rope_dim)) return;
    if ((q_weight == nullptr) != (k_weight == nullptr) || (cos_table == nullptr) != (sin_table == nullptr)) {
        set_error(1, "%s: q_weight/k_weight and cos_table/sin_table come in pairs", fn);
        return;
    }
    ProducerArgs p;
    fill_producer(p, q, const_cast<tw_half*>(k_buf), G, num_heads, num_kv_heads, q_dim, kv_dim);
    p.v = reinterpret_cast<half_t*>(const_cast<tw_half*>(v_buf));
    p.norm = q_weight ? 1 : 0; p.q_weight = H(q_weight); p.k_weight = H(k_weight); p.eps = eps; p.biased = biased ? 1 : 0;
    p.cos_table = H(cos_table); p.sin_table = H(sin_table); p.rope_dim = rope_dim; p.positions = pos;
    p.write_cache = 1;
    p.cache_k = reinterpret_cast<half_t*>(ck);
    p.cache_v = reinterpret_cast<half_t*>(cv);
    p.kv_dim = kv_dim;
    p.seq_stride_rows = msl;
    launch_producer(p, s);
    check_launch(fn);
    launch_gqa_attention_batch(out, q, ck, cv, as, pos, msl, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, s);
}

void launch_sigmoid_gate_batch(tw_half* data, const tw_half* gate, int dim, int G, hipStream_t s) {
    launch_sigmoid_gate(reinterpret_cast<half_t*>(data), dim, H(gate), dim, dim, G, s);
    check_launch("launch_sigmoid_gate_batch");
}

void tw_layer_attention_step(const tw_layer_step_args* p, hipStream_t s) {
    const char* fn = "tw_layer_attention_step";
    if (!p) { set_error(1, "%s: NULL arguments", fn); return; }
    if (p->kv_bits != 0 && !check_bits(fn, p->kv_bits)) return;
    const bool producers = p->q_weight || p->cos_table;
    t_gate = p->gate;
    t_gate_stride = p->gate ? p->gate_stride : 0;
    t_ctx_min = p->ctx_max > 0 ? p->ctx_min : 0;
    t_ctx_max = p->ctx_max > 0 ? p->ctx_max : 0;
    t_tickets = p->tickets;
    if (p->kv_bits == 0) {
        if (producers) {
            tw_qk_norm_rope_append_attention_batch(p->out, p->q, p->k, p->v, p->q_weight, p->k_weight, p->eps, p->biased,
                                                   p->cos_table, p->sin_table, p->rope_dim, (tw_half*)p->cache_k,
                                                   (tw_half*)p->cache_v, p->scratch, p->positions, p->max_seq_len, p->G,
                                                   p->num_heads, p->num_kv_heads, p->head_dim, p->q_dim, p->kv_dim, s);
        } else {
            tw_append_attention_batch(p->out, p->q, p->k, p->v, (tw_half*)p->cache_k, (tw_half*)p->cache_v, p->scratch,
                                      p->positions, p->max_seq_len, p->G, p->num_heads, p->num_kv_heads, p->head_dim,
                                      p->q_dim, p->kv_dim, s);
        }
    } else if (producers) {
        tw_qk_norm_rope_turbo_append_attention_batch(
            p->out, p->q, p->k, p->v, p->q_weight, p->k_weight, p->eps, p->biased, p->cos_table, p->sin_table,
            p->rope_dim, (uint8_t*)p->cache_k, (uint8_t*)p->cache_v, p->k_norms, p->v_norms, p->rotation, p->scratch,
            p->positions, p->max_seq_len, p->G, p->num_heads, p->num_kv_heads, p->head_dim, p->q_dim, p->kv_dim,
            p->kv_bits, s);
    } else {
        tw_turbo_append_attention_batch(p->out, p->q, p->k, p->v, (uint8_t*)p->cache_k, (uint8_t*)p->cache_v, p->k_norms,
                                        p->v_norms, p->rotation, p->scratch, p->positions, p->max_seq_len, p->G,
                                        p->num_heads, p->num_kv_heads, p->head_dim, p->q_dim, p->kv_dim, p->kv_bits, s);
    }
    t_gate = nullptr;
    t_gate_stride = 0;
    t_ctx_min = t_ctx_max = 0;
    t_tickets = nullptr;
}

// Steps 3-5b of a layer over a prompt (prefill_chunked, engine.cpp:2097-2150): rows are the prompt's tokens,
// the cache rows are sequence 0's.
void tw_layer_prompt_step(const tw_layer_step_args* p, hipStream_t s) {
    const char* fn = "tw_layer_prompt_step";
    if (!p) { set_error(1, "%s: NULL arguments", fn); return; }
    if (p->kv_bits != 0 && !check_bits(fn, p->kv_bits)) return;
    if (!check_shape(fn, p->num_heads, p->num_kv_heads, p->head_dim)) return;
    if (p->kv_dim != p->num_kv_heads * p->head_dim) {
        set_error(1, "%s: kv_dim=%d != num_kv_heads*head_dim", fn, p->kv_dim);
        return;
    }
    if (p->cos_table && !check_rope_dim(fn, p->rope_dim)) return;
    if ((p->q_weight == nullptr) != (p->k_weight == nullptr) || (p->cos_table == nullptr) != (p->sin_table == nullptr)) {
        set_error(1, "%s: q_weight/k_weight and cos_table/sin_table come in pairs", fn);
        return;
    }
    const int T = p->G;
    if (T <= 0) return;
    const bool producers = p->q_weight || p->cos_table;
    ProducerArgs pr;
    fill_producer(pr, p->q, p->k, T, p->num_heads, p->num_kv_heads, p->q_dim, p->kv_dim);
    pr.norm = p->q_weight ? 1 : 0; pr.q_weight = H(p->q_weight); pr.k_weight = H(p->k_weight);
    pr.eps = p->eps; pr.biased = p->biased ? 1 : 0;
    pr.cos_table = H(p->cos_table); pr.sin_table = H(p->sin_table); pr.rope_dim = p->rope_dim; pr.positions = p->positions;
    if (p->kv_bits == 0) {
        tw_half* ck = (tw_half*)p->cache_k;
        tw_half* cv = (tw_half*)p->cache_v;
        if (producers) {               // q in place; K (transformed) and V straight to rows positions[t] of sequence 0
            pr.v = reinterpret_cast<half_t*>(const_cast<tw_half*>(p->v));
            pr.write_cache = 1;
            pr.cache_k = reinterpret_cast<half_t*>(ck);
            pr.cache_v = reinterpret_cast<half_t*>(cv);
            pr.kv_dim = p->kv_dim;
            pr.seq_stride_rows = 0;
            launch_producer(pr, s);
        } else {
            launch_kv_write(reinterpret_cast<half_t*>(ck), reinterpret_cast<half_t*>(cv), H(p->k), H(p->v), p->positions,
                            nullptr, 0, 0, T, p->kv_dim, s);
        }
        check_launch(fn);
        launch_gqa_prefill_attention(p->out, p->q, ck, cv, p->scratch, T, p->max_seq_len, p->num_heads, p->num_kv_heads,
                                     p->head_dim, p->q_dim, p->kv_dim, s);
    } else {
        if (producers) {               // q and k in place
            launch_producer(pr, s);
            check_launch(fn);
        }
        quantize_common(fn, (uint8_t*)p->cache_k, p->k_norms, p->k, (uint8_t*)p->cache_v, p->v_norms, p->v, 2, p->rotation,
                        p->positions, nullptr, 0, p->max_seq_len, 1, T, p->num_kv_heads, p->head_dim, p->kv_dim,
                        p->kv_bits, s);
        launch_turbo_gqa_prefill_attention(p->out, p->q, (const uint8_t*)p->cache_k, (const uint8_t*)p->cache_v, p->k_norms,
                                           p->v_norms, p->rotation, p->scratch, T, p->max_seq_len, p->num_heads,
                                           p->num_kv_heads, p->head_dim, p->q_dim, p->kv_dim, p->kv_bits, s);
    }
    if (p->gate) {
        launch_sigmoid_gate(reinterpret_cast<half_t*>(p->out), p->q_dim, H(p->gate), p->gate_stride,
                            p->num_heads * p->head_dim, T, s);
        check_launch(fn);
    }
}

void launch_turbo_gqa_prefill_attention(tw_half* out, const tw_half* q, const uint8_t* ck_q,
                                        const uint8_t* cv_q, const tw_half* k_norms,
                                        const tw_half* v_norms, const tw_half* rotation, float* as,
                                        int T, int msl, int num_heads, int num_kv_heads,
                                        int head_dim, int q_dim, int kv_dim, int bits,
                                        hipStream_t s) {
    (void)msl;
    if (!check_shape("launch_turbo_gqa_prefill_attention", num_heads, num_kv_heads, head_dim) ||
        !check_bits("launch_turbo_gqa_prefill_attention", bits)) return;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "launch_turbo_gqa_prefill_attention: kv_dim=%d != num_kv_heads*head_dim", kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck_q, cv_q, k_norms, v_norms, rotation, T, num_heads,
                num_kv_heads, bits, as);
    a.pos_mode = kPosIota; a.seq_stride_rows = 0;
    plan_splits(a, T, T);
    run_attention(a, s, "launch_turbo_gqa_prefill_attention");
}

// ---------------------------------------------------------------- attention without any allocation
}  // extern "C"

// The split workspace of launch_turbo_gqa_attention_batch as a device array of the library itself, for callers
// that can neither allocate nor hand over scratch memory.  In host code the array's name only stands for the
// symbol: its address on a device comes from hipGetSymbolAddress with that device current (every device has its
// own copy), is looked up once per device and is what the kernels get.
static __device__ __align__(256) float scratch[TW_NOALLOC_SCRATCH_BYTES / sizeof(float)];

namespace {
constexpr int kNoallocMaxDevices = 64;
float* g_scratch_ptr[kNoallocMaxDevices];   // per device, nullptr = not looked up yet
std::mutex g_scratch_mutex;

float* static_scratch_on_current_device(const char* fn) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kNoallocMaxDevices) {
        set_error(e != hipSuccess ? (int)e : 1, "%s: no usable current device (%d)", fn, dev);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_error(e != hipSuccess ? (int)e : 1, "%s: hipGetSymbolAddress(scratch): %s", fn, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = static_cast<float*>(p);
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" {

int tw_turbo_gqa_attention_batch_noalloc(tw_half* out, const tw_half* q, const uint8_t* ck_q, const uint8_t* cv_q,
                                         const tw_half* k_norms, const tw_half* v_norms, const tw_half* rotation,
                                         const int* pos, int msl, int G, int num_heads, int num_kv_heads, int head_dim,
                                         int q_dim, int kv_dim, int bits, hipStream_t s) {
    const char* fn = "tw_turbo_gqa_attention_batch_noalloc";
    // The return value is this call's own outcome, whatever an earlier call left in the thread's sticky error: that
    // one is set aside while the call runs and put back when the call succeeds; when the call fails, its own message
    // is the one tw_kv_last_error_string() returns afterwards.
    struct StickyAside {
        int code; char msg[sizeof(g_err_msg)];
        StickyAside() : code(g_err) { memcpy(msg, g_err_msg, sizeof(msg)); g_err = 0; g_err_msg[0] = 0; }
        ~StickyAside() { if (g_err == 0 && code != 0) { g_err = code; memcpy(g_err_msg, msg, sizeof(msg)); } }
    } aside;
    if (!check_shape(fn, num_heads, num_kv_heads, head_dim) || !check_bits(fn, bits)) return 1;
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "%s: kv_dim=%d != num_kv_heads*head_dim", fn, kv_dim);
        return 1;
    }
    if (G <= 0 || msl <= 0) { set_error(1, "%s: G=%d, msl=%d", fn, G, msl); return 1; }
    if ((long long)G * num_heads > TW_NOALLOC_MAX_HEAD_VECTORS) {
        set_error(1, "%s: G*num_heads=%lld exceeds the %d (sequence, head) pairs the library's %d MiB of scratch serve",
                  fn, (long long)G * num_heads, TW_NOALLOC_MAX_HEAD_VECTORS, (int)(TW_NOALLOC_SCRATCH_BYTES >> 20));
        return 1;
    }
    float* ws = static_scratch_on_current_device(fn);
    if (!ws) return 2;
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck_q, cv_q, k_norms, v_norms, rotation, G, num_heads, num_kv_heads, bits, ws);
    a.pos_mode = kPosArray; a.positions = pos; a.seq_stride_rows = msl;
    // the room per (sequence, head) the reference-signature launcher has (msl floats) when the array gives that much:
    // then both make the same plan and the same bits
    const long long room = (long long)(TW_NOALLOC_SCRATCH_BYTES / sizeof(float)) / ((long long)G * num_heads);
    plan_splits(a, msl, room < msl ? room : msl);
    run_attention(a, s, fn, /*query_done=*/false, /*may_profile=*/false);
    return g_err != 0 ? 3 : 0;
}

void tw_paged_gqa_attention_batch(tw_half* out, const tw_half* q, const tw_half* ck,
                                  const tw_half* cv, float* ws, const int* positions,
                                  const int* block_table, int bt_stride, int max_context, int G,
                                  int num_heads, int num_kv_heads, int head_dim, int q_dim,
                                  int kv_dim, hipStream_t s) {
    if (!check_shape("tw_paged_gqa_attention_batch", num_heads, num_kv_heads, head_dim)) return;
    if (!block_table) { set_error(1, "tw_paged_gqa_attention_batch: block_table is NULL"); return; }
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "tw_paged_gqa_attention_batch: kv_dim=%d != num_kv_heads*head_dim", kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck, cv, nullptr, nullptr, nullptr, G, num_heads, num_kv_heads, 0, ws);
    a.pos_mode = kPosArray; a.positions = positions;
    a.block_table = block_table; a.bt_stride = bt_stride;
    plan_splits(a, max_context, kPagedBlockFloats);
    run_attention(a, s, "tw_paged_gqa_attention_batch");
}

void tw_paged_turbo_gqa_attention_batch(tw_half* out, const tw_half* q, const uint8_t* ck_q,
                                        const uint8_t* cv_q, const tw_half* k_norms,
                                        const tw_half* v_norms, const tw_half* rotation, float* ws,
                                        const int* positions, const int* block_table,
                                        int bt_stride, int max_context, int G, int num_heads,
                                        int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                        int bits, hipStream_t s) {
    if (!check_shape("tw_paged_turbo_gqa_attention_batch", num_heads, num_kv_heads, head_dim) ||
        !check_bits("tw_paged_turbo_gqa_attention_batch", bits)) return;
    if (!block_table) { set_error(1, "tw_paged_turbo_gqa_attention_batch: block_table is NULL"); return; }
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "tw_paged_turbo_gqa_attention_batch: kv_dim=%d != num_kv_heads*head_dim", kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck_q, cv_q, k_norms, v_norms, rotation, G, num_heads,
                num_kv_heads, bits, ws);
    a.pos_mode = kPosArray; a.positions = positions;
    a.block_table = block_table; a.bt_stride = bt_stride;
    plan_splits(a, max_context, kPagedBlockFloats);
    run_attention(a, s, "tw_paged_turbo_gqa_attention_batch");
}

// One decode step of a layer over the paged cache: the K and V rows of the new token and the query are rotated in
// one launch (the appended rows quantized into their pages), then the scan over the pages and the merge -- three
// launches where tw_paged_turbo_kv_append_batch + tw_paged_turbo_gqa_attention_batch take four.
void tw_paged_turbo_append_attention_batch(tw_half* out, const tw_half* q, const tw_half* k_buf, const tw_half* v_buf,
                                           uint8_t* ck_q, uint8_t* cv_q, tw_half* k_norms, tw_half* v_norms,
                                           const tw_half* rotation, float* ws, const int* positions,
                                           const int* block_table, int bt_stride, int max_context, int G,
                                           int num_heads, int num_kv_heads, int head_dim, int q_dim, int kv_dim,
                                           int bits, hipStream_t s) {
    const char* fn = "tw_paged_turbo_append_attention_batch";
    if (!check_shape(fn, num_heads, num_kv_heads, head_dim) || !check_bits(fn, bits)) return;
    if (!block_table) { set_error(1, "%s: block_table is NULL", fn); return; }
    if (kv_dim != num_kv_heads * head_dim) {
        set_error(1, "%s: kv_dim=%d != num_kv_heads*head_dim", fn, kv_dim);
        return;
    }
    AttnArgs a;
    fill_common(a, out, q, q_dim, ck_q, cv_q, k_norms, v_norms, rotation, G, num_heads, num_kv_heads, bits, ws);
    a.pos_mode = kPosArray; a.positions = positions;
    a.block_table = block_table; a.bt_stride = bt_stride;
    plan_splits(a, max_context, kPagedBlockFloats);
    const int R = num_heads / num_kv_heads;
    const bool fuse_q = mfma_wanted(a) && a.qrot && (R == 1 || R == 2 || R == 4) &&
                        (reinterpret_cast<uintptr_t>(a.qrot) & 15u) == 0;
    if (!fuse_q) {                 // shapes the MFMA kernels do not take: the two calls
        tw_paged_turbo_kv_append_batch(ck_q, k_norms, cv_q, v_norms, k_buf, v_buf, rotation, positions, block_table,
                                       bt_stride, G, num_kv_heads, head_dim, kv_dim, bits, s);
        run_attention(a, s, fn);
        return;
    }
    RotArgs r;
    memset(&r, 0, sizeof(r));
    fill_quant_segments(r, ck_q, k_norms, k_buf, cv_q, v_norms, v_buf, 2, G, num_kv_heads, kv_dim);
    int k = r.nseg++;
    r.seg_src[k] = H(q);
    r.seg_stride[k] = q_dim;
    r.seg_heads[k] = num_heads;
    r.seg_nvec[k] = G * num_heads;
    r.seg_units[k] = (r.seg_nvec[k] + 15) / 16 * 8;
    r.seg_kind[k] = 1;
    r.rotation = H(rotation);
    r.positions = positions;
    r.block_table = block_table;
    r.bt_stride = bt_stride;
    r.num_kv_heads = num_kv_heads;
    r.qrot = a.qrot;
    r.qrot_stride = a.ws_stride;
    r.q_scale = attention_mfma_q_scale(bits);
    launch_rotate(r, bits, s);
    run_attention(a, s, fn, /*query_done=*/true);
}

// ---------------------------------------------------------------- rotation (host)
// engine.cpp:366-392, same recipe and same library calls so that the matrix is
// the one the reference engine uploads.
void tw_make_rotation_host(tw_half* out_host, int n, unsigned seed) {
    // The recipe fixes every rounding: N(0,1) entries drawn row-major from mt19937(seed) through libstdc++'s
    // normal_distribution<float>, then modified Gram-Schmidt over the rows in fp32 -- each earlier row's component
    // is removed in turn (the projection is taken from the row as updated so far), each sum runs over the columns
    // in ascending order with separate multiply and add, and the row is scaled by 1 / sqrtf(sum of squares).
    std::mt19937 engine(seed);
    std::normal_distribution<float> gauss(0.0f, 1.0f);
    std::vector<float> rows((size_t)n * n);
    for (float& x : rows) x = gauss(engine);
    for (int r = 0; r < n; r++) {
        float* row = &rows[(size_t)r * n];
        for (int e = 0; e < r; e++) {
            const float* earlier = &rows[(size_t)e * n];
            float proj = 0.0f;
            for (int c = 0; c < n; c++) proj += row[c] * earlier[c];
            for (int c = 0; c < n; c++) row[c] -= proj * earlier[c];
        }
        float sq = 0.0f;
        for (int c = 0; c < n; c++) sq += row[c] * row[c];
        const float scale = 1.0f / sqrtf(sq);
        for (int c = 0; c < n; c++) row[c] *= scale;
    }
    for (size_t i = 0; i < rows.size(); i++) {
        const _Float16 h = (_Float16)rows[i];      // round to nearest even, as __float2half
        memcpy(&out_host[i], &h, sizeof(h));
    }
}

}  // extern "C"
