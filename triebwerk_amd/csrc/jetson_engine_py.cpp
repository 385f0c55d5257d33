// jetson_engine_py.cpp -- the pybind11 module `jetson_engine` with the part of the reference's `Engine` class that
// belongs to the KV-cache path (engine/engine_py.cpp:18-26, 44-45): the constructor
// Engine(max_seq_len=1024, kv_bits=0), kv_bits() and reset(), under the reference's own module and class names, so
// that `jetson_engine.Engine(1024, kv_bits)` (triebwerk/engine.py:23) constructs this library's engine object.
// Everything else of that class needs weights and is not part of this library; instead the cache calls are exposed
// on raw device pointers (tensor.data_ptr()), the way the reference's share_* methods take them
// (engine_py.cpp:48-75).  Host code only: it links against libtriebwerk_kv.so and is compiled without hipcc.

#include <pybind11/pybind11.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "../../include/triebwerk_kv.h"

namespace py = pybind11;

namespace {

template <typename T> T* ptr(size_t p) { return reinterpret_cast<T*>(p); }

// Errors become std::runtime_error, RuntimeError in Python, as the reference's CUDA_CHECK does (engine.cpp:21-28).
void check(int rc, const char* what) {
    if (rc == 0) return;
    std::string msg = std::string(what) + " failed (" + std::to_string(rc) + ")";
    if (tw_kv_last_error() != 0) {
        msg += std::string(": ") + tw_kv_last_error_string();
        tw_kv_clear_error();
    }
    throw std::runtime_error(msg);
}

class Engine {
public:
    Engine(int max_seq_len, int kv_bits) : e_(tw_engine_create(max_seq_len, kv_bits)) {
        if (!e_) throw std::runtime_error("tw_engine_create failed");
    }
    ~Engine() { tw_engine_destroy(e_); }
    Engine(const Engine&) = delete;
    Engine& operator=(const Engine&) = delete;

    int kv_bits() const { return tw_engine_kv_bits(e_); }
    int max_seq_len() const { return tw_engine_max_seq_len(e_); }
    void reset() { check(tw_engine_reset(e_), "reset"); }

    void set_shape(int layers, int heads, int kv_heads, int head_dim) {
        tw_model_shape s{layers, heads, kv_heads, head_dim};
        check(tw_engine_set_shape(e_, &s), "set_shape");
    }
    size_t arena_bytes_needed(int G, int max_seq_len) const { return tw_engine_arena_bytes_needed(e_, G, max_seq_len); }
    void set_arena(size_t data_ptr, size_t bytes) { check(tw_engine_set_arena(e_, ptr<void>(data_ptr), bytes), "set_arena"); }
    void alloc_batch(int G, int max_seq_len) { check(tw_engine_alloc_batch(e_, G, max_seq_len), "alloc_batch"); }
    void sleep() { check(tw_engine_sleep(e_), "sleep"); }
    void wake() { check(tw_engine_wake(e_), "wake"); }
    bool is_allocated() const { return tw_engine_is_allocated(e_) != 0; }
    size_t cache_ptr(int layer, int which) { return reinterpret_cast<size_t>(tw_engine_cache_ptr(e_, layer, which)); }
    size_t positions_ptr() { return reinterpret_cast<size_t>(tw_engine_positions(e_)); }
    size_t rotation_ptr() { return reinterpret_cast<size_t>(tw_engine_rotation(e_)); }
    void set_positions(const py::list& positions) {
        std::vector<int> p;
        for (auto h : positions) p.push_back(h.cast<int>());
        check(tw_engine_set_positions(e_, p.data(), (int)p.size()), "set_positions");
    }
    void layer_step(int layer, size_t q, size_t k, size_t v, size_t out, size_t stream) {
        check(tw_engine_layer_step(e_, layer, ptr<const tw_half>(q), ptr<const tw_half>(k), ptr<const tw_half>(v),
                                   ptr<tw_half>(out), ptr<ihipStream_t>(stream)), "layer_step");
    }
    void decode_step(size_t q, size_t k, size_t v, size_t out, bool use_graph, size_t stream) {
        check(tw_engine_decode_step(e_, ptr<const tw_half>(q), ptr<const tw_half>(k), ptr<const tw_half>(v), ptr<tw_half>(out),
                                    use_graph ? 1 : 0, ptr<ihipStream_t>(stream)), "decode_step");
    }
    void broadcast_prefix(int src, int dst_begin, int dst_end, int T, size_t stream) {
        check(tw_engine_broadcast_prefix(e_, src, dst_begin, dst_end, T, ptr<ihipStream_t>(stream)), "broadcast_prefix");
    }

private:
    tw_engine* e_;
};

}  // namespace

PYBIND11_MODULE(jetson_engine, m) {
    m.doc() = "KV-cache path of the triebwerk inference engine on MI355X (libtriebwerk_kv)";
    m.def("build_info", []() { return std::string(tw_kv_build_info()); });

    py::class_<Engine>(m, "Engine")
        // engine_py.cpp:22-26
        .def(py::init<int, int>(), py::arg("max_seq_len") = 1024, py::arg("kv_bits") = 0,
             "Create the engine's KV-cache object. kv_bits=0: fp16 KV cache, 4 or 2: TurboQuant codes; "
             "any other value falls back to 0 with a warning")
        .def("kv_bits", &Engine::kv_bits, "KV cache quantization bits (0 = fp16, 4 or 2 = TurboQuant)")
        // engine_py.cpp:44-45
        .def("reset", &Engine::reset, "Reset KV cache for new generation")
        // the cache calls the reference reaches only through generate*(): on raw device pointers
        .def("max_seq_len", &Engine::max_seq_len)
        .def("set_shape", &Engine::set_shape, py::arg("num_layers"), py::arg("num_heads"), py::arg("num_kv_heads"),
             py::arg("head_dim") = 128)
        .def("arena_bytes_needed", &Engine::arena_bytes_needed, py::arg("G"), py::arg("max_seq_len"))
        .def("set_arena", &Engine::set_arena, py::arg("data_ptr"), py::arg("bytes"),
             "Carve the caches out of caller-owned device memory (pass tensor.data_ptr(), 256-byte aligned)")
        .def("alloc_batch", &Engine::alloc_batch, py::arg("G"), py::arg("max_seq_len"))
        .def("sleep", &Engine::sleep)
        .def("wake", &Engine::wake)
        .def("is_allocated", &Engine::is_allocated)
        .def("cache_ptr", &Engine::cache_ptr, py::arg("layer"), py::arg("which"),
             "Device address of a layer's array: 0 keys, 1 values, 2 key norms, 3 value norms")
        .def("positions_ptr", &Engine::positions_ptr)
        .def("rotation_ptr", &Engine::rotation_ptr)
        .def("set_positions", &Engine::set_positions, py::arg("positions"))
        .def("layer_step", &Engine::layer_step, py::arg("layer"), py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"),
             py::arg("stream") = 0, "Append K, V at positions[g], then attention, for one layer (device pointers)")
        .def("decode_step", &Engine::decode_step, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("out"),
             py::arg("use_graph") = false, py::arg("stream") = 0,
             "All layers, then positions += 1; q/out (L, G, H*D), k/v (L, G, Hk*D) device pointers")
        .def("broadcast_prefix", &Engine::broadcast_prefix, py::arg("src"), py::arg("dst_begin"), py::arg("dst_end"),
             py::arg("T"), py::arg("stream") = 0);
}
