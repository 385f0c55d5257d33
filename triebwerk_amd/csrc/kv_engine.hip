// kv_engine.hip -- host-side owner of the KV cache: the slice of the reference's
// InferenceEngine (model.h:373-493, engine.cpp) that the KV-cache path needs.
//
//   constructor / kv_bits switch ....... engine.cpp:300-317
//   rotation matrix .................... engine.cpp:366-392
//   batch arena, 256-byte bump carve ... engine.cpp:1338-1560, model.h:264-279
//   external arena ..................... engine.cpp:1609-1620
//   reset / zero-fill .................. engine.cpp:893-916, 2262-2283
//   append -> attention per layer ...... engine.cpp:1979-2006
//   decode-step graph .................. engine.cpp:2369-2412, 2472-2480
//   prefix broadcast ................... engine.cpp:2173-2214
//   single-sequence caches ............. engine.cpp:322-331, 394-404 (allocation), 893-916 (reset),
//                                        922-1022 (sleep / wake), 1069-1108 (append -> attention of a layer)
//
// Everything else the reference engine owns (weights, GEMMs, sampling) is not
// part of this library.

#include <hip/hip_runtime.h>
#include <dlfcn.h>

#include <cstdio>
#include <cstring>
#include <new>
#include <vector>

#include "../../include/triebwerk_kv.h"

namespace {
constexpr int kMaxLayers = 128;  // model.h:9

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }  // GpuArena::alloc, model.h:270-275
}  // namespace

struct tw_engine {
    int max_seq_len = 1024;
    int kv_bits = 0;
    tw_model_shape shape{28, 16, 8, 128};  // ModelConfig::qwen3_0_6b(), model.h:66-74

    // batch state (BatchState, model.h:283-330)
    int G = 0;
    int batch_msl = 0;
    char* arena = nullptr;
    size_t arena_cap = 0;
    bool arena_owned = false;
    void* cache[kMaxLayers][4] = {};  // keys, values, key norms, value norms
    float* attn_scores = nullptr;     // G * num_heads * msl floats, engine.cpp:1371
    int* d_positions = nullptr;
    tw_half* d_rotation = nullptr;
    unsigned* d_tickets = nullptr;    // G * num_kv_heads words for the one-launch step's shared contexts: zero between steps

    hipStream_t stream = nullptr;     // engine_stream_, engine.cpp:309

    // single-sequence state (InferenceState / KVCache, model.h:195-204): per-layer caches of max_seq_len rows, each
    // an allocation of its own as in allocate_buffers (engine.cpp:322-331, 394-404), the attention scratch of
    // num_heads * max_seq_len floats, the rotation, and current_pos -- on the host and, for the launchers that take
    // positions from device memory, in one device word that lives as long as the caches (the reference allocates and
    // frees such a word per layer and token, engine.cpp:1078-1092)
    void* single[kMaxLayers][4] = {};
    float* single_scores = nullptr;
    tw_half* single_rotation = nullptr;
    int* single_d_pos = nullptr;
    unsigned* single_tickets = nullptr;   // num_kv_heads words, zero between steps (tw_layer_step_args::tickets)
    int single_pos = 0;
    bool single_allocated = false;
    bool single_wanted = false;       // wake() re-allocates what sleep() freed (engine.cpp:985-1022)

    // producers of q and k run with the step (forward_layer_batch step 3, engine.cpp:1972-1977);
    // caller-owned device memory: weights (num_layers, head_dim), tables (positions, rope_dim / 2)
    int producers = 0;                // 0 none, 1 fused into the append, 2 as launches of their own
    const tw_half* q_norm = nullptr;
    const tw_half* k_norm = nullptr;
    float norm_eps = 1e-6f;
    int norm_biased = 0;
    const tw_half* rope_cos = nullptr;
    const tw_half* rope_sin = nullptr;
    int rope_dim = 0;

    // captured decode step
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    const void* graph_key[4] = {};
    int graph_G = 0;
    int graph_plan = 0;               // tw_kv_decode_step_plan's answer the captured launches were chosen under
    // generate_batch goes on without a graph when capture or instantiation fails (engine.cpp:2396-2410): so does
    // tw_engine_decode_step, until the buffers, the batch or the producers change
    bool graph_failed = false;
    const void* graph_failed_key[4] = {};
    int graph_state = 0;              // of the latest decode step: 0 eager as asked, 1 graph replayed, 2 eager after a failed capture
    int fail_next_captures = 0;       // test hook: treat this many coming captures as failed

    // The stream of the latest step: reset, set_positions and everything that lets go of the arena wait for it
    // first (a caller's stream has no implicit order with the engine's own stream or with the null stream).
    hipStream_t last_stream = nullptr;
    bool steps_in_flight = false;
    void note_step(hipStream_t s) { last_stream = s; steps_in_flight = true; }
    void wait_for_steps() {
        if (steps_in_flight) (void)hipStreamSynchronize(last_stream);
        steps_in_flight = false;
    }

    // generation bookkeeping (generate_batch, engine.cpp:2350, 2496-2534)
    int* d_token_history = nullptr;   // (max_new_tokens, G) device
    std::vector<int> h_token_history;
    std::vector<int> h_positions;
    // range of the device positions as far as the host has seen them (set_positions, reset, + 1 per decode
    // step); a caller that writes the device array itself makes it stale, which only costs kernel choice
    bool pos_known = false;
    int pos_min = 0, pos_max = 0;
    std::vector<char> h_finished;
    std::vector<std::vector<int>> outputs;
    std::vector<int> stop_ids;
    int eos_token = -1;
    int max_new_tokens = 0;
    int last_checked = -1;

    void drop_generation() {
        if (d_token_history) { hipFree(d_token_history); d_token_history = nullptr; }
        h_token_history.clear(); h_positions.clear(); h_finished.clear(); outputs.clear(); stop_ids.clear();
        max_new_tokens = 0; last_checked = -1;
    }

    int kv_dim() const { return shape.num_kv_heads * shape.head_dim; }
    int q_dim() const { return shape.num_heads * shape.head_dim; }
    // KV_DIM_PACKED, engine.cpp:294
    size_t kv_dim_packed() const { return kv_bits == 4 ? kv_dim() / 2 : kv_dim() / 4; }

    void drop_graph() {
        if (graph_exec) { hipGraphExecDestroy(graph_exec); graph_exec = nullptr; }
        if (graph) { hipGraphDestroy(graph); graph = nullptr; }
        graph_G = 0;
    }
    void drop_arena() {
        // the arena may be freed below: wait for everything on the device, not only for the stream of the latest step
        // (steps issued earlier on other streams may still be reading it)
        if (arena) (void)hipDeviceSynchronize();
        steps_in_flight = false;
        graph_failed = false;
        drop_graph();  // the capture holds arena addresses, engine.cpp:1440-1442
        drop_generation();
        if (arena && arena_owned) hipFree(arena);
        arena = nullptr; arena_cap = 0; arena_owned = false;
        G = 0; batch_msl = 0;
        memset(cache, 0, sizeof(cache));
        attn_scores = nullptr; d_positions = nullptr; d_rotation = nullptr; d_tickets = nullptr;
    }
};

namespace {

size_t arena_need(const tw_engine* e, int G, int msl) {
    size_t need = 0;
    auto add = [&](size_t bytes) { need = align256(need); need += bytes; };
    add((size_t)G * e->shape.num_heads * msl * sizeof(float));  // attn_scores
    for (int i = 0; i < e->shape.num_layers; i++) {
        if (e->kv_bits == 0) {
            add((size_t)G * msl * e->kv_dim() * 2);
            add((size_t)G * msl * e->kv_dim() * 2);
        } else {
            add((size_t)G * msl * e->kv_dim_packed());
            add((size_t)G * msl * e->kv_dim_packed());
            add((size_t)G * msl * e->shape.num_kv_heads * 2);
            add((size_t)G * msl * e->shape.num_kv_heads * 2);
        }
    }
    add((size_t)G * sizeof(int));                                                    // positions
    add((size_t)e->shape.head_dim * e->shape.head_dim * 2);                          // rotation
    add((size_t)G * e->shape.num_kv_heads * sizeof(unsigned));                       // tickets
    return align256(need);
}

int carve(tw_engine* e, int G, int msl) {
    size_t off = 0;
    auto take = [&](size_t bytes) { off = align256(off); void* p = e->arena + off; off += bytes; return p; };
    e->attn_scores = (float*)take((size_t)G * e->shape.num_heads * msl * sizeof(float));
    for (int i = 0; i < e->shape.num_layers; i++) {
        if (e->kv_bits == 0) {
            e->cache[i][0] = take((size_t)G * msl * e->kv_dim() * 2);
            e->cache[i][1] = take((size_t)G * msl * e->kv_dim() * 2);
            e->cache[i][2] = e->cache[i][3] = nullptr;
        } else {  // keys_q, values_q, keys_norms, values_norms: engine.cpp:1503-1506
            e->cache[i][0] = take((size_t)G * msl * e->kv_dim_packed());
            e->cache[i][1] = take((size_t)G * msl * e->kv_dim_packed());
            e->cache[i][2] = take((size_t)G * msl * e->shape.num_kv_heads * 2);
            e->cache[i][3] = take((size_t)G * msl * e->shape.num_kv_heads * 2);
        }
    }
    e->d_positions = (int*)take((size_t)G * sizeof(int));
    e->d_rotation = (tw_half*)take((size_t)e->shape.head_dim * e->shape.head_dim * 2);
    e->d_tickets = (unsigned*)take((size_t)G * e->shape.num_kv_heads * sizeof(unsigned));
    if (off > e->arena_cap) return -1;
    e->G = G;
    e->batch_msl = msl;
    e->pos_known = false;        // until reset or set_positions
    if (e->kv_bits > 0) {
        std::vector<tw_half> rot((size_t)e->shape.head_dim * e->shape.head_dim);
        tw_make_rotation_host(rot.data(), e->shape.head_dim, 42u);
        if (hipMemcpy(e->d_rotation, rot.data(), rot.size() * 2, hipMemcpyHostToDevice) != hipSuccess) return -2;
    }
    return 0;
}

hipStream_t pick(tw_engine* e, hipStream_t s) { return s ? s : e->stream; }

// ---- trace ranges (the reference prints std::chrono timings around these phases, engine.cpp:2305-2311, 2537-2544;
// here they are roctx ranges a profiler can show).  Off until tw_kv_set_trace_ranges(1) finds the roctx library.
typedef int (*roctx_push_fn)(const char*);
typedef int (*roctx_pop_fn)();
roctx_push_fn g_range_push = nullptr;
roctx_pop_fn g_range_pop = nullptr;
bool g_ranges_on = false;
struct TraceRange {
    bool on;
    explicit TraceRange(const char* name) : on(g_ranges_on && g_range_push && g_range_pop) { if (on) g_range_push(name); }
    ~TraceRange() { if (on) g_range_pop(); }
};

// per-array row bytes of a cache: keys, values, key norms, value norms (0: the array does not exist)
size_t cache_row_bytes(const tw_engine* e, int which) {
    if (e->kv_bits == 0) return which < 2 ? (size_t)e->kv_dim() * 2 : 0;
    return which < 2 ? e->kv_dim_packed() : (size_t)e->shape.num_kv_heads * 2;
}

void free_single(tw_engine* e) {
    if (!e->single_allocated) return;
    (void)hipDeviceSynchronize();
    for (int i = 0; i < kMaxLayers; i++)
        for (int w = 0; w < 4; w++)
            if (e->single[i][w]) { hipFree(e->single[i][w]); e->single[i][w] = nullptr; }
    if (e->single_scores) { hipFree(e->single_scores); e->single_scores = nullptr; }
    if (e->single_rotation) { hipFree(e->single_rotation); e->single_rotation = nullptr; }
    if (e->single_d_pos) { hipFree(e->single_d_pos); e->single_d_pos = nullptr; }
    if (e->single_tickets) { hipFree(e->single_tickets); e->single_tickets = nullptr; }
    e->single_allocated = false;
}

int zero_single(tw_engine* e) {
    const size_t rows = (size_t)e->max_seq_len;
    for (int i = 0; i < e->shape.num_layers; i++)
        for (int w = 0; w < 4; w++)
            if (e->single[i][w] && hipMemset(e->single[i][w], 0, rows * cache_row_bytes(e, w)) != hipSuccess) return -1;
    if (hipMemset(e->single_d_pos, 0, sizeof(int)) != hipSuccess) return -1;
    if (hipMemset(e->single_tickets, 0, (size_t)e->shape.num_kv_heads * sizeof(unsigned)) != hipSuccess) return -1;
    e->single_pos = 0;
    return 0;
}

// A step appends at positions[g]: once the furthest sequence the host knows of has used its last row there is no
// row left, and the append would land in the next sequence's rows (or past the array).
bool cache_full(const tw_engine* e) { return e->pos_known && e->pos_max >= e->batch_msl; }

// What tw_layer_attention_step will choose for the compressed cache from the host's view of the positions
// (one launch per layer or three); the captured graph holds the launches of one such choice.
int step_plan(const tw_engine* e) {
    if (e->kv_bits == 0) return 0;
    return tw_kv_decode_step_plan2(e->G, e->shape.num_heads, e->shape.num_kv_heads, e->kv_bits, e->batch_msl,
                                   e->pos_known ? e->pos_min + 1 : 0, e->pos_known ? e->pos_max + 1 : 0,
                                   e->d_tickets != nullptr);
}

// forward_layer_batch steps 4-5 (with producers: 3-5), engine.cpp:1972-2006.
void layer_step(tw_engine* e, int layer, const tw_half* q, const tw_half* k, const tw_half* v,
                tw_half* out, hipStream_t s) {
    const tw_model_shape& m = e->shape;
    tw_half* qm = const_cast<tw_half*>(q);      // with producers q and k are the caller's scratch rows
    tw_half* km = const_cast<tw_half*>(k);
    const tw_half* qw = e->q_norm ? e->q_norm + (size_t)layer * m.head_dim : nullptr;
    const tw_half* kw = e->k_norm ? e->k_norm + (size_t)layer * m.head_dim : nullptr;
    if (e->producers == 2) {                    // the reference's sequence of launches
        if (qw) launch_qk_norm_batch(qm, km, qw, kw, m.num_heads, m.num_kv_heads, m.head_dim, e->G, e->norm_eps,
                                     e->q_dim(), e->kv_dim(), s, e->norm_biased != 0);
        if (e->rope_cos) launch_rope_batch(qm, km, e->rope_cos, e->rope_sin, e->d_positions, e->batch_msl, e->G,
                                           m.num_heads, m.num_kv_heads, m.head_dim, e->q_dim(), e->kv_dim(),
                                           e->rope_dim, s);
    }
    const bool fused = e->producers == 1;
    tw_layer_step_args p;
    memset(&p, 0, sizeof(p));
    p.out = out; p.q = qm; p.k = km; p.v = v;
    p.G = e->G; p.num_heads = m.num_heads; p.num_kv_heads = m.num_kv_heads; p.head_dim = m.head_dim;
    p.q_dim = e->q_dim(); p.kv_dim = e->kv_dim();
    p.positions = e->d_positions; p.max_seq_len = e->batch_msl;
    if (fused) {
        p.q_weight = qw; p.k_weight = kw; p.eps = e->norm_eps; p.biased = e->norm_biased;
        p.cos_table = e->rope_cos; p.sin_table = e->rope_sin; p.rope_dim = e->rope_dim;
    }
    p.kv_bits = e->kv_bits;
    p.cache_k = e->cache[layer][0]; p.cache_v = e->cache[layer][1];
    p.k_norms = (tw_half*)e->cache[layer][2]; p.v_norms = (tw_half*)e->cache[layer][3];
    p.rotation = e->d_rotation; p.scratch = e->attn_scores;
    // what the host knows of the context lengths (positions + 1, the appended token included)
    if (e->pos_known) { p.ctx_min = e->pos_min + 1; p.ctx_max = e->pos_max + 1; }
    p.tickets = e->d_tickets;
    tw_layer_attention_step(&p, s);
}

void all_layers(tw_engine* e, const tw_half* q, const tw_half* k, const tw_half* v, tw_half* out,
                hipStream_t s) {
    const size_t qs = (size_t)e->G * e->q_dim(), ks = (size_t)e->G * e->kv_dim();
    for (int l = 0; l < e->shape.num_layers; l++)
        layer_step(e, l, q + l * qs, k + l * ks, v + l * ks, out + l * qs, s);
    launch_increment_positions(e->d_positions, e->G, s);  // engine.cpp:2394
}

}  // namespace

extern "C" {

tw_engine* tw_engine_create(int max_seq_len, int kv_bits) {
    tw_engine* e = new (std::nothrow) tw_engine();
    if (!e) return nullptr;
    e->max_seq_len = max_seq_len;
    e->kv_bits = kv_bits;
    if (kv_bits != 0 && kv_bits != 2 && kv_bits != 4) {  // engine.cpp:310-313
        fprintf(stderr, "WARNING: kv_bits=%d not supported, using 0 (fp16)\n", kv_bits);
        e->kv_bits = 0;
    }
    return e;
}

void tw_engine_destroy(tw_engine* e) {
    if (!e) return;
    e->drop_arena();
    free_single(e);
    if (e->stream) hipStreamDestroy(e->stream);
    delete e;
}

int tw_engine_kv_bits(const tw_engine* e) { return e->kv_bits; }
int tw_engine_max_seq_len(const tw_engine* e) { return e->max_seq_len; }

int tw_engine_set_shape(tw_engine* e, const tw_model_shape* shape) {
    if (!shape || shape->num_layers < 1 || shape->num_layers > kMaxLayers || shape->head_dim != 128 ||
        shape->num_kv_heads < 1 || shape->num_heads % shape->num_kv_heads != 0)
        return -1;
    e->drop_arena();
    free_single(e);                   // sized by the shape; tw_engine_alloc_single makes them anew
    e->shape = *shape;
    return 0;
}

size_t tw_engine_arena_bytes_needed(const tw_engine* e, int G, int max_seq_len) {
    return arena_need(e, G, max_seq_len);
}

int tw_engine_alloc_batch(tw_engine* e, int G, int max_seq_len) {
    if (G < 1 || max_seq_len < 1) return -1;
    if (!e->stream && hipStreamCreate(&e->stream) != hipSuccess) return -3;
    // engine.cpp:1339 keeps a batch that is already large enough and goes on striding with its G and max_seq_len.
    // Here the steps take their row counts and strides from the batch as allocated, so only an identical batch
    // is kept as it is; a different one is carved anew (and zeroed), inside the memory already held when that
    // is big enough.
    if (e->arena && e->G == G && e->batch_msl == max_seq_len) return 0;
    size_t need = arena_need(e, G, max_seq_len);
    if (!(e->arena && e->arena_cap >= need)) {
        e->drop_arena();
        void* p = nullptr;
        if (hipMalloc(&p, need) != hipSuccess) return -2;
        e->arena = (char*)p;
        e->arena_cap = need;
        e->arena_owned = true;
    } else {
        // the rows are about to be re-carved and zeroed: as in drop_arena, wait for the whole device
        (void)hipDeviceSynchronize();
        e->steps_in_flight = false;
        e->graph_failed = false;
        e->drop_graph();
        e->drop_generation();
    }
    int rc = carve(e, G, max_seq_len);
    if (rc != 0) return rc;
    return tw_engine_reset(e);
}

int tw_engine_set_arena(tw_engine* e, void* device_ptr, size_t bytes) {
    if (!device_ptr || (reinterpret_cast<uintptr_t>(device_ptr) & 255u)) return -1;
    e->drop_arena();
    e->arena = (char*)device_ptr;
    e->arena_cap = bytes;
    e->arena_owned = false;
    return 0;
}

int tw_engine_reset(tw_engine* e) {
    if (e->single_allocated) {                 // reset(), engine.cpp:893-916: the single-sequence caches, current_pos = 0
        e->wait_for_steps();
        if (zero_single(e) != 0) return -1;
    }
    if (!e->arena || e->G == 0) return 0;
    e->wait_for_steps();
    hipStream_t s = e->stream;
    const size_t rows = (size_t)e->G * e->batch_msl;
    for (int i = 0; i < e->shape.num_layers; i++)
        for (int w = 0; w < 4; w++)
            if (e->cache[i][w]) hipMemsetAsync(e->cache[i][w], 0, rows * cache_row_bytes(e, w), s);
    hipMemsetAsync(e->d_positions, 0, (size_t)e->G * sizeof(int), s);
    hipMemsetAsync(e->d_tickets, 0, (size_t)e->G * e->shape.num_kv_heads * sizeof(unsigned), s);
    e->pos_known = true;
    e->pos_min = e->pos_max = 0;
    return hipStreamSynchronize(s) == hipSuccess ? 0 : -1;
}

void* tw_engine_cache_ptr(tw_engine* e, int layer, int which) {
    if (layer < 0 || layer >= e->shape.num_layers || which < 0 || which > 3) return nullptr;
    return e->cache[layer][which];
}
int* tw_engine_positions(tw_engine* e) { return e->d_positions; }
const tw_half* tw_engine_rotation(tw_engine* e) { return e->kv_bits > 0 ? e->d_rotation : nullptr; }

int tw_engine_set_positions(tw_engine* e, const int* host_positions, int G) {
    if (!e->d_positions || G > e->G) return -1;
    for (int g = 0; g < G; g++)
        if (host_positions[g] < 0 || host_positions[g] >= e->batch_msl) return -2;
    e->wait_for_steps();
    // engine.cpp:2364
    if (hipMemcpy(e->d_positions, host_positions, (size_t)G * sizeof(int), hipMemcpyHostToDevice) != hipSuccess) return -3;
    e->pos_known = G == e->G && G > 0;
    if (e->pos_known) {
        e->pos_min = e->pos_max = host_positions[0];
        for (int g = 1; g < G; g++) {
            e->pos_min = host_positions[g] < e->pos_min ? host_positions[g] : e->pos_min;
            e->pos_max = host_positions[g] > e->pos_max ? host_positions[g] : e->pos_max;
        }
    }
    return 0;
}

int tw_engine_set_producers(tw_engine* e, int mode, const tw_half* q_norm, const tw_half* k_norm, float eps,
                            int biased, const tw_half* rope_cos, const tw_half* rope_sin, int rope_dim) {
    if (mode < 0 || mode > 2) return -1;
    if ((q_norm == nullptr) != (k_norm == nullptr) || (rope_cos == nullptr) != (rope_sin == nullptr)) return -1;
    if (rope_cos && !(rope_dim == 128 || (rope_dim >= 16 && rope_dim <= 64 && rope_dim % 16 == 0))) return -1;
    e->drop_graph();                  // a captured step holds the old sequence of launches
    e->graph_failed = false;
    e->producers = (q_norm || rope_cos) ? mode : 0;
    e->q_norm = q_norm; e->k_norm = k_norm; e->norm_eps = eps; e->norm_biased = biased ? 1 : 0;
    e->rope_cos = rope_cos; e->rope_sin = rope_sin; e->rope_dim = rope_dim;
    return 0;
}

// sleep(), engine.cpp:922-983: give the device memory back -- the arena when the engine allocated it (a caller's
// arena is only forgotten) and the single-sequence caches -- and drop everything that points into it.
// wake(), engine.cpp:985-1022: re-allocate the single-sequence caches that sleep freed (zeroed, current_pos = 0:
// the reference leaves them as cudaMalloc returns them and relies on the reset() in front of every generate);
// the batch state comes back with the next alloc_batch, as in the reference.
int tw_engine_sleep(tw_engine* e) {
    if (e->stream) hipStreamSynchronize(e->stream);
    e->drop_arena();
    free_single(e);
    return 0;
}

int tw_engine_wake(tw_engine* e) {
    if (e->single_wanted && !e->single_allocated) return tw_engine_alloc_single(e);
    return 0;
}

// allocate_buffers' share for this path, engine.cpp:322-331 (fp16) and 394-404 (compressed): per layer a key and a
// value array of max_seq_len rows (and the two norm arrays), each an allocation of its own.
int tw_engine_alloc_single(tw_engine* e) {
    e->single_wanted = true;
    if (e->single_allocated) return 0;
    if (!e->stream && hipStreamCreate(&e->stream) != hipSuccess) return -3;
    const size_t rows = (size_t)e->max_seq_len;
    if (rows < 1) return -1;
    bool ok = true;
    e->single_allocated = true;               // from here on free_single lets go of whatever was obtained
    for (int i = 0; i < e->shape.num_layers && ok; i++)
        for (int w = 0; w < 4 && ok; w++) {
            const size_t rb = cache_row_bytes(e, w);
            if (rb) ok = hipMalloc(&e->single[i][w], rows * rb) == hipSuccess;
        }
    ok = ok && hipMalloc((void**)&e->single_scores, (size_t)e->shape.num_heads * rows * sizeof(float)) == hipSuccess;
    ok = ok && hipMalloc((void**)&e->single_d_pos, sizeof(int)) == hipSuccess;
    ok = ok && hipMalloc((void**)&e->single_tickets, (size_t)e->shape.num_kv_heads * sizeof(unsigned)) == hipSuccess;
    if (ok && e->kv_bits > 0) {
        const size_t n = (size_t)e->shape.head_dim * e->shape.head_dim;
        ok = hipMalloc((void**)&e->single_rotation, n * 2) == hipSuccess;
        if (ok) {
            std::vector<tw_half> rot(n);
            tw_make_rotation_host(rot.data(), e->shape.head_dim, 42u);
            ok = hipMemcpy(e->single_rotation, rot.data(), n * 2, hipMemcpyHostToDevice) == hipSuccess;
        }
    }
    if (ok) ok = zero_single(e) == 0;
    if (!ok) { (void)hipGetLastError(); free_single(e); return -2; }
    return 0;
}

int tw_engine_single_is_allocated(const tw_engine* e) { return e->single_allocated ? 1 : 0; }
int tw_engine_single_pos(const tw_engine* e) { return e->single_pos; }
void* tw_engine_single_cache_ptr(tw_engine* e, int layer, int which) {
    if (layer < 0 || layer >= e->shape.num_layers || which < 0 || which > 3) return nullptr;
    return e->single[layer][which];
}
const tw_half* tw_engine_single_rotation(tw_engine* e) { return e->kv_bits > 0 ? e->single_rotation : nullptr; }

int tw_engine_single_set_pos(tw_engine* e, int pos) {
    if (!e->single_allocated) return -1;
    if (pos < 0 || pos >= e->max_seq_len) return -2;
    e->wait_for_steps();
    if (hipMemcpy(e->single_d_pos, &pos, sizeof(int), hipMemcpyHostToDevice) != hipSuccess) return -3;
    e->single_pos = pos;
    return 0;
}

// forward_layer steps 4-5 (engine.cpp:1069-1108) at current_pos: K and V of the token into row current_pos of the
// layer's cache, attention over rows 0 .. current_pos.  One call of the layer step of the batch path with a batch
// of one, so the single sequence gets the same kernels (the append inside the attention launch for the fp16 cache,
// the whole step in one launch for the compressed one); nothing is allocated per token.
int tw_engine_single_step(tw_engine* e, int layer, const tw_half* q, const tw_half* k, const tw_half* v, tw_half* out,
                          hipStream_t s) {
    if (!e->single_allocated || layer < 0 || layer >= e->shape.num_layers) return -1;
    if (e->single_pos >= e->max_seq_len) return -8;
    TraceRange range("tw_engine_single_step");
    s = pick(e, s);
    e->note_step(s);
    tw_kv_clear_error();
    const tw_model_shape& m = e->shape;
    tw_layer_step_args p;
    memset(&p, 0, sizeof(p));
    p.out = out; p.q = const_cast<tw_half*>(q); p.k = const_cast<tw_half*>(k); p.v = v;
    p.G = 1; p.num_heads = m.num_heads; p.num_kv_heads = m.num_kv_heads; p.head_dim = m.head_dim;
    p.q_dim = e->q_dim(); p.kv_dim = e->kv_dim();
    p.positions = e->single_d_pos; p.max_seq_len = e->max_seq_len;
    p.kv_bits = e->kv_bits;
    p.cache_k = e->single[layer][0]; p.cache_v = e->single[layer][1];
    p.k_norms = (tw_half*)e->single[layer][2]; p.v_norms = (tw_half*)e->single[layer][3];
    p.rotation = e->single_rotation; p.scratch = e->single_scores;
    p.ctx_min = p.ctx_max = e->single_pos + 1;
    p.tickets = e->single_tickets;          // one sequence leaves most compute units idle: its context may be shared
    tw_layer_attention_step(&p, s);
    return tw_kv_last_error();
}

// decode_token's `state_.current_pos++` after the last layer: host and device word, in stream order
int tw_engine_single_advance(tw_engine* e, hipStream_t s) {
    if (!e->single_allocated) return -1;
    if (e->single_pos >= e->max_seq_len) return -8;
    s = pick(e, s);
    e->note_step(s);
    tw_kv_clear_error();
    launch_increment_positions(e->single_d_pos, 1, s);
    e->single_pos++;
    return tw_kv_last_error();
}

int tw_engine_is_allocated(const tw_engine* e) { return e->arena != nullptr && e->G > 0; }

int tw_engine_begin_generation(tw_engine* e, int max_new_tokens, int eos_token_id, const int* stop_ids_host,
                               int n_stop) {
    if (!e->arena || e->G == 0 || max_new_tokens < 1 || n_stop < 0) return -1;
    e->drop_generation();
    if (hipMalloc((void**)&e->d_token_history, (size_t)max_new_tokens * e->G * sizeof(int)) != hipSuccess) return -2;
    e->h_token_history.assign((size_t)max_new_tokens * e->G, 0);
    e->h_positions.assign(e->G, 0);
    e->h_finished.assign(e->G, 0);
    e->outputs.assign(e->G, std::vector<int>());
    e->stop_ids.assign(stop_ids_host, stop_ids_host + n_stop);
    e->eos_token = eos_token_id;
    e->max_new_tokens = max_new_tokens;
    e->last_checked = -1;
    return 0;
}

// engine.cpp:2496-2498: the step's tokens go into the history on the device, no synchronisation
int tw_engine_record_tokens(tw_engine* e, const int* d_tokens, int step, hipStream_t s) {
    if (!e->d_token_history || step < 0 || step >= e->max_new_tokens) return -1;
    s = pick(e, s);
    return hipMemcpyAsync(e->d_token_history + (size_t)step * e->G, d_tokens, (size_t)e->G * sizeof(int),
                          hipMemcpyDeviceToDevice, s) == hipSuccess ? 0 : -2;
}

// engine.cpp:2499-2534: every 8th step and on the last one, wait for the stream, fetch positions and the
// history rows not yet seen, extend the outputs of the sequences still running and mark those that
// produced the end token or the stop sequence.  Returns 1 when all have finished, 0 otherwise.
int tw_engine_check_stops(tw_engine* e, int step, hipStream_t s, int* checked) {
    constexpr int kCheckInterval = 8;      // engine.cpp:2350
    if (!e->d_token_history || step < 0 || step >= e->max_new_tokens) return -1;
    const bool should_check = ((step + 1) % kCheckInterval == 0) || (step + 1 == e->max_new_tokens);
    if (checked) *checked = should_check ? 1 : 0;
    if (!should_check) return 0;
    s = pick(e, s);
    const int G = e->G;
    if (hipStreamSynchronize(s) != hipSuccess) return -2;
    if (hipMemcpy(e->h_positions.data(), e->d_positions, (size_t)G * sizeof(int), hipMemcpyDeviceToHost) != hipSuccess)
        return -2;
    const int check_start = e->last_checked + 1;
    const size_t count = (size_t)(step + 1 - check_start) * G;
    if (hipMemcpy(e->h_token_history.data() + (size_t)check_start * G, e->d_token_history + (size_t)check_start * G,
                  count * sizeof(int), hipMemcpyDeviceToHost) != hipSuccess)
        return -2;
    bool all_done = true;
    const int stop_len = (int)e->stop_ids.size();
    for (int st = check_start; st <= step; st++) {
        for (int g = 0; g < G; g++) {
            if (e->h_finished[g]) continue;
            const int tok = e->h_token_history[(size_t)st * G + g];
            std::vector<int>& out = e->outputs[g];
            out.push_back(tok);
            if (tok == e->eos_token) {
                e->h_finished[g] = 1;
            } else if (stop_len > 0 && (int)out.size() >= stop_len) {
                bool match = true;
                for (int j = 0; j < stop_len; j++) {
                    if (out[out.size() - stop_len + j] != e->stop_ids[j]) { match = false; break; }
                }
                if (match) e->h_finished[g] = 1;
            }
            if (!e->h_finished[g]) all_done = false;
        }
    }
    e->last_checked = step;
    return all_done ? 1 : 0;
}

int tw_engine_output(tw_engine* e, int g, const int** tokens, int* n) {
    if (g < 0 || g >= (int)e->outputs.size() || !tokens || !n) return -1;
    *tokens = e->outputs[g].data();
    *n = (int)e->outputs[g].size();
    return e->h_finished[g] ? 1 : 0;
}

int tw_engine_host_position(const tw_engine* e, int g) {
    return (g >= 0 && g < (int)e->h_positions.size()) ? e->h_positions[g] : -1;
}

int tw_engine_layer_step(tw_engine* e, int layer, const tw_half* q, const tw_half* k,
                         const tw_half* v, tw_half* out, hipStream_t s) {
    if (!e->arena || layer < 0 || layer >= e->shape.num_layers) return -1;
    if (cache_full(e)) return -8;
    tw_kv_clear_error();
    s = pick(e, s);
    e->note_step(s);
    layer_step(e, layer, q, k, v, out, s);
    return tw_kv_last_error();
}

int tw_engine_prompt_layer(tw_engine* e, int layer, int seq, const tw_half* q, const tw_half* k, const tw_half* v,
                           tw_half* out, const int* token_positions, int T, hipStream_t s) {
    if (!e->arena || layer < 0 || layer >= e->shape.num_layers || seq < 0 || seq >= e->G || T < 0 || T > e->batch_msl ||
        !token_positions)
        return -1;
    if (T == 0) return 0;
    TraceRange range("tw_engine_prompt_layer");
    s = pick(e, s);
    e->note_step(s);
    tw_kv_clear_error();
    const tw_model_shape& m = e->shape;
    tw_half* qm = const_cast<tw_half*>(q);      // with producers q and k are the caller's scratch rows
    tw_half* km = const_cast<tw_half*>(k);
    const tw_half* qw = e->q_norm ? e->q_norm + (size_t)layer * m.head_dim : nullptr;
    const tw_half* kw = e->k_norm ? e->k_norm + (size_t)layer * m.head_dim : nullptr;
    if (e->producers == 2) {                    // the reference's sequence of launches (engine.cpp:2103-2108)
        if (qw) launch_qk_norm_batch(qm, km, qw, kw, m.num_heads, m.num_kv_heads, m.head_dim, T, e->norm_eps,
                                     e->q_dim(), e->kv_dim(), s, e->norm_biased != 0);
        if (e->rope_cos) launch_rope_batch(qm, km, e->rope_cos, e->rope_sin, token_positions, e->batch_msl, T,
                                           m.num_heads, m.num_kv_heads, m.head_dim, e->q_dim(), e->kv_dim(),
                                           e->rope_dim, s);
    }
    tw_layer_step_args p;
    memset(&p, 0, sizeof(p));
    p.out = out; p.q = qm; p.k = km; p.v = v;
    p.G = T; p.num_heads = m.num_heads; p.num_kv_heads = m.num_kv_heads; p.head_dim = m.head_dim;
    p.q_dim = e->q_dim(); p.kv_dim = e->kv_dim();
    p.positions = token_positions; p.max_seq_len = e->batch_msl;
    if (e->producers == 1) {
        p.q_weight = qw; p.k_weight = kw; p.eps = e->norm_eps; p.biased = e->norm_biased;
        p.cos_table = e->rope_cos; p.sin_table = e->rope_sin; p.rope_dim = e->rope_dim;
    }
    p.kv_bits = e->kv_bits;
    const size_t msl = (size_t)e->batch_msl;
    const size_t row = e->kv_bits == 0 ? (size_t)e->kv_dim() * 2 : e->kv_dim_packed();
    const size_t nrow = (size_t)m.num_kv_heads * 2;
    p.cache_k = (char*)e->cache[layer][0] + seq * msl * row;
    p.cache_v = (char*)e->cache[layer][1] + seq * msl * row;
    if (e->kv_bits != 0) {
        p.k_norms = (tw_half*)((char*)e->cache[layer][2] + seq * msl * nrow);
        p.v_norms = (tw_half*)((char*)e->cache[layer][3] + seq * msl * nrow);
    }
    p.rotation = e->d_rotation;
    // the batch's attention scratch holds G * num_heads * max_seq_len floats (engine.cpp:1371); the prefill
    // launchers count on T floats per (token, head) and do without a workspace when there is none
    p.scratch = ((size_t)T * T <= (size_t)e->G * msl) ? e->attn_scores : nullptr;
    tw_layer_prompt_step(&p, s);
    return tw_kv_last_error();
}

int tw_engine_decode_step(tw_engine* e, const tw_half* q, const tw_half* k, const tw_half* v,
                          tw_half* out, int use_graph, hipStream_t s) {
    if (!e->arena) return -1;
    if (cache_full(e)) return -8;          // before any launch or replay: cache and positions stay as they are
    TraceRange range("tw_engine_decode_step");
    s = pick(e, s);
    e->note_step(s);
    tw_kv_clear_error();
    const void* key[4] = {q, k, v, out};
    auto eager = [&](int state) -> int {
        all_layers(e, q, k, v, out, s);
        if (e->pos_known) { e->pos_min++; e->pos_max++; }
        e->graph_state = state;
        return tw_kv_last_error();
    };
    if (!use_graph) return eager(0);
    // a capture that failed for these buffers is not tried again step after step (engine.cpp:2396-2410 tries once
    // per generate_batch and decodes eagerly when it fails)
    if (e->graph_failed && memcmp(key, e->graph_failed_key, sizeof(key)) == 0) return eager(2);
    // The launches in a captured step were chosen from the context lengths at capture; when the lengths have
    // grown (or spread) to where the other kernels are the better choice, the step is captured again.
    const int plan = step_plan(e);
    if (!e->graph_exec || e->graph_G != e->G || e->graph_plan != plan || memcmp(key, e->graph_key, sizeof(key)) != 0) {
        e->drop_graph();
        // Capture records the launches without running them, so unlike the
        // reference (engine.cpp:2414-2444) nothing has to be re-prefilled.
        int why = 0;                       // -4 begin, -5 end of capture or a launcher's error, -6 instantiation
        hipGraph_t g = nullptr;
        hipError_t err = hipStreamBeginCapture(s, hipStreamCaptureModeRelaxed);
        if (err != hipSuccess) {
            why = -4;
        } else {
            all_layers(e, q, k, v, out, s);
            err = hipStreamEndCapture(s, &g);
            if (err != hipSuccess || !g || tw_kv_last_error() != 0) why = -5;
            else if (e->fail_next_captures > 0) { e->fail_next_captures--; why = -6; err = hipErrorUnknown; }
            else if ((err = hipGraphInstantiate(&e->graph_exec, g, nullptr, nullptr, 0)) != hipSuccess) why = -6;
        }
        if (why != 0) {
            if (g) hipGraphDestroy(g);
            e->graph_exec = nullptr;
            (void)hipGetLastError();
            fprintf(stderr, "  hipGraph capture FAILED (step %d, err=%d): decoding without a graph\n", why, (int)err);
            tw_kv_clear_error();
            e->graph_failed = true;
            memcpy(e->graph_failed_key, key, sizeof(key));
            return eager(2);               // the recorded launches never ran: run the step now
        }
        e->graph = g;
        e->graph_G = e->G;
        e->graph_plan = plan;
        memcpy(e->graph_key, key, sizeof(key));
    }
    if (hipGraphLaunch(e->graph_exec, s) != hipSuccess) return -7;
    if (e->pos_known) { e->pos_min++; e->pos_max++; }
    e->graph_state = 1;
    return 0;
}

int tw_engine_graph_state(const tw_engine* e) { return e->graph_state; }
void tw_engine_debug_fail_captures(tw_engine* e, int n) { e->fail_next_captures = n > 0 ? n : 0; }

int tw_kv_set_trace_ranges(int on) {
    if (!on) { g_ranges_on = false; return 0; }
    if (!g_range_push || !g_range_pop) {
        for (const char* name : {"librocprofiler-sdk-roctx.so.1", "librocprofiler-sdk-roctx.so", "libroctx64.so.4", "libroctx64.so"}) {
            void* h = dlopen(name, RTLD_NOW | RTLD_GLOBAL);
            if (!h) continue;
            g_range_push = reinterpret_cast<roctx_push_fn>(dlsym(h, "roctxRangePushA"));
            g_range_pop = reinterpret_cast<roctx_pop_fn>(dlsym(h, "roctxRangePop"));
            if (g_range_push && g_range_pop) break;
            g_range_push = nullptr; g_range_pop = nullptr;
        }
    }
    g_ranges_on = g_range_push && g_range_pop;
    return g_ranges_on ? 0 : -1;
}

int tw_engine_broadcast_prefix(tw_engine* e, int src, int dst_begin, int dst_end, int T, hipStream_t s) {
    if (!e->arena || src < 0 || src >= e->G || dst_begin < 0 || dst_end > e->G || T < 0 || T > e->batch_msl)
        return -1;
    s = pick(e, s);
    e->note_step(s);
    const size_t msl = (size_t)e->batch_msl;
    for (int l = 0; l < e->shape.num_layers; l++) {
        void* bases[4];
        size_t seq_bytes[4], bytes[4];
        int n = 0;
        for (int which = 0; which < 4; which++) {
            if (!e->cache[l][which]) continue;
            size_t row_bytes;
            if (e->kv_bits == 0) row_bytes = (size_t)e->kv_dim() * 2;
            else row_bytes = which < 2 ? e->kv_dim_packed() : (size_t)e->shape.num_kv_heads * 2;
            bases[n] = e->cache[l][which];
            seq_bytes[n] = msl * row_bytes;
            bytes[n] = (size_t)T * row_bytes;
            n++;
        }
        // one launch per layer: every array, every destination
        if (tw_kv_broadcast_rows(bases, seq_bytes, bytes, n, src, dst_begin, dst_end, s) != 0) return -2;
    }
    return 0;
}

}  // extern "C"
