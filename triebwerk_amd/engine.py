"""``Engine(max_seq_len, kv_bits)``: the KV-cache face of the reference's
``jetson_engine.Engine`` (engine/engine_py.cpp:21-45), backed by the C++ engine
object behind the C ABI (``tw_engine_*`` in include/triebwerk_kv.h).

The reference class reaches append and attention only through ``generate*``;
weights, GEMMs and sampling are not part of this library, so the cache calls
are exposed directly instead: ``alloc_batch``, ``layer_step``, ``decode_step``.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from .kvcache import _ptr, _stream


class Engine:
    def __init__(self, max_seq_len: int = 1024, kv_bits: int = 0):
        # engine_py.cpp:22: py::init<int,int>(), max_seq_len=1024, kv_bits=0
        self._lib = _lib.load()
        self._h = self._lib.tw_engine_create(int(max_seq_len), int(kv_bits))
        if not self._h:
            raise RuntimeError("tw_engine_create failed")
        self._arena = None
        self._shape = (28, 16, 8, 128)
        self._G = 0
        self._msl = 0

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.tw_engine_destroy(h)

    # ---- the reference's surface for this path
    def kv_bits(self) -> int:  # engine_py.cpp:25
        return self._lib.tw_engine_kv_bits(self._h)

    def reset(self) -> None:  # engine_py.cpp:44
        rc = self._lib.tw_engine_reset(self._h)
        if rc != 0:
            raise RuntimeError(f"reset failed ({rc})")

    # ---- cache management the reference does inside load_config / generate_batch
    def max_seq_len(self) -> int:
        return self._lib.tw_engine_max_seq_len(self._h)

    def set_shape(self, num_layers: int, num_heads: int, num_kv_heads: int, head_dim: int = 128) -> None:
        shape = _lib.ModelShape(num_layers, num_heads, num_kv_heads, head_dim)
        if self._lib.tw_engine_set_shape(self._h, C.byref(shape)) != 0:
            raise ValueError("unsupported model shape (head_dim must be 128, heads a multiple of kv heads)")
        self._shape = (num_layers, num_heads, num_kv_heads, head_dim)
        self._arena = None

    def alloc_batch(self, G: int, max_seq_len: int, device="cuda") -> None:
        """Carve the caches for G sequences out of one torch-owned arena
        (the reference's set_arena + alloc_batch, engine.cpp:1609-1620, 1338)."""
        need = self._lib.tw_engine_arena_bytes_needed(self._h, G, max_seq_len)
        if self._arena is None or self._arena.numel() < need + 256:
            arena = torch.empty(need + 256, dtype=torch.uint8, device=device)
            base = (arena.data_ptr() + 255) & ~255
            # set_arena waits for the stream of the latest step before it lets go of the old memory,
            # which torch frees when the last reference below goes
            rc = self._lib.tw_engine_set_arena(self._h, base, arena.numel() - (base - arena.data_ptr()))
            if rc != 0:
                raise RuntimeError(f"set_arena failed ({rc})")
            self._arena = arena
        # a batch that fits the memory already held is carved anew inside it (and zeroed)
        rc = self._lib.tw_engine_alloc_batch(self._h, G, max_seq_len)
        if rc != 0:
            raise RuntimeError(f"alloc_batch failed ({rc})")
        self._G, self._msl = G, max_seq_len

    def _view(self, ptr: int, nbytes: int, dtype, shape):
        off = ptr - self._arena.data_ptr()
        return self._arena[off:off + nbytes].view(dtype).view(shape)

    def cache(self, layer: int):
        """Torch views of one layer's cache: (keys, values, key_norms, value_norms)."""
        L, H, Hk, D = self._shape
        G, msl = self._G, self._msl
        bits = self.kv_bits()
        ptrs = [self._lib.tw_engine_cache_ptr(self._h, layer, w) for w in range(4)]
        if bits == 0:
            n = G * msl * Hk * D * 2
            return (self._view(ptrs[0], n, torch.float16, (G, msl, Hk * D)),
                    self._view(ptrs[1], n, torch.float16, (G, msl, Hk * D)), None, None)
        kvp = Hk * D * bits // 8
        return (self._view(ptrs[0], G * msl * kvp, torch.uint8, (G, msl, kvp)),
                self._view(ptrs[1], G * msl * kvp, torch.uint8, (G, msl, kvp)),
                self._view(ptrs[2], G * msl * Hk * 2, torch.float16, (G, msl, Hk)),
                self._view(ptrs[3], G * msl * Hk * 2, torch.float16, (G, msl, Hk)))

    def positions(self) -> torch.Tensor:
        return self._view(self._lib.tw_engine_positions(self._h), self._G * 4, torch.int32, (self._G,))

    def rotation(self):
        p = self._lib.tw_engine_rotation(self._h)
        if not p:
            return None
        D = self._shape[3]
        return self._view(p, D * D * 2, torch.float16, (D, D))

    def set_positions(self, positions) -> None:
        arr = (C.c_int * len(positions))(*[int(x) for x in positions])
        rc = self._lib.tw_engine_set_positions(self._h, arr, len(positions))
        if rc != 0:
            raise ValueError(f"set_positions failed ({rc})")

    def set_producers(self, mode, q_norm=None, k_norm=None, eps=1e-6, biased=False, rope_cos=None, rope_sin=None,
                      rope_dim=0) -> None:
        """Run the per-head RMSNorm (weights (L, D) per layer) and the rotary embedding (tables
        (positions, rope_dim/2)) of q and k with every step: mode 1 fused into the append, mode 2 as the
        reference's two launches, 0 off.  The tensors must stay alive while they are set."""
        rc = self._lib.tw_engine_set_producers(self._h, int(mode), _ptr(q_norm, "f16", "q_norm"),
                                               _ptr(k_norm, "f16", "k_norm"), float(eps), int(biased),
                                               _ptr(rope_cos, "f16", "rope_cos"), _ptr(rope_sin, "f16", "rope_sin"),
                                               int(rope_dim))
        if rc != 0:
            raise ValueError(f"set_producers failed ({rc})")
        self._producers = (q_norm, k_norm, rope_cos, rope_sin)

    def _check_rows(self, q, k, v, out, lead) -> None:
        """The C side takes the row counts from the batch as allocated: the buffers must have exactly that shape."""
        if self._G == 0:
            return                      # nothing allocated: the call itself reports that
        L, H, Hk, D = self._shape
        want_q, want_kv = (*lead, self._G, H * D), (*lead, self._G, Hk * D)
        for name, t, want in (("q", q, want_q), ("out", out, want_q), ("k", k, want_kv), ("v", v, want_kv)):
            if tuple(t.shape) != want:
                raise ValueError(f"{name}: shape {tuple(t.shape)}, the allocated batch needs {want}")

    def layer_step(self, layer, q, k, v, out, stream=None) -> None:
        self._check_rows(q, k, v, out, ())
        rc = self._lib.tw_engine_layer_step(self._h, layer, _ptr(q, "f16", "q"), _ptr(k, "f16", "k"),
                                            _ptr(v, "f16", "v"), _ptr(out, "f16", "out"), _stream(stream))
        if rc != 0:
            _lib.check(self._lib)
            raise RuntimeError(f"layer_step failed ({rc})")

    def prompt_layer(self, layer, seq, q, k, v, out, token_positions, stream=None) -> None:
        """The path of one layer over a prompt (rows of q/k/v/out = its tokens, token_positions = 0 .. T-1) for
        sequence `seq`: producers, T-token append, causal attention (prefill_chunked, engine.cpp:2097-2150)."""
        rc = self._lib.tw_engine_prompt_layer(self._h, layer, seq, _ptr(q, "f16", "q"), _ptr(k, "f16", "k"),
                                              _ptr(v, "f16", "v"), _ptr(out, "f16", "out"),
                                              _ptr(token_positions, "i32", "token_positions"), int(q.shape[0]),
                                              _stream(stream))
        if rc != 0:
            _lib.check(self._lib)
            raise RuntimeError(f"prompt_layer failed ({rc})")

    def decode_step(self, q, k, v, out, use_graph: bool = False, stream=None) -> None:
        """Append + attention for every layer, then positions += 1.
        q/out: (L, G, H*D); k/v: (L, G, Hk*D)."""
        self._check_rows(q, k, v, out, (self._shape[0],))
        rc = self._lib.tw_engine_decode_step(self._h, _ptr(q, "f16", "q"), _ptr(k, "f16", "k"),
                                             _ptr(v, "f16", "v"), _ptr(out, "f16", "out"),
                                             1 if use_graph else 0, _stream(stream))
        if rc != 0:
            _lib.check(self._lib)
            raise RuntimeError(f"decode_step failed ({rc})")

    def broadcast_prefix(self, src: int, dst_begin: int, dst_end: int, T: int, stream=None) -> None:
        rc = self._lib.tw_engine_broadcast_prefix(self._h, src, dst_begin, dst_end, T, _stream(stream))
        if rc != 0:
            raise RuntimeError(f"broadcast_prefix failed ({rc})")

    def graph_state(self) -> int:
        """What the latest decode_step did: 0 eager as asked, 1 graph replayed, 2 eager after a failed capture
        (generate_batch decodes without a graph when the capture fails, engine.cpp:2396-2410)."""
        return self._lib.tw_engine_graph_state(self._h)

    # ---- the single-sequence state of generate() / decode_token() (engine.cpp:322-331, 394-404, 1069-1108)
    def alloc_single(self) -> None:
        """Per-layer caches of max_seq_len rows for one sequence, each an allocation of its own as in the reference."""
        rc = self._lib.tw_engine_alloc_single(self._h)
        if rc != 0:
            raise RuntimeError(f"alloc_single failed ({rc})")

    def single_is_allocated(self) -> bool:
        return bool(self._lib.tw_engine_single_is_allocated(self._h))

    def single_pos(self) -> int:
        return self._lib.tw_engine_single_pos(self._h)

    def single_set_pos(self, pos: int) -> None:
        rc = self._lib.tw_engine_single_set_pos(self._h, int(pos))
        if rc != 0:
            raise ValueError(f"single_set_pos failed ({rc})")

    @staticmethod
    def _wrap(ptr: int, nbytes: int, dtype, shape):
        """A torch view of device memory the engine owns (valid until the engine frees it)."""
        class _Mem:
            __cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (int(ptr), False), "version": 2}
        return torch.as_tensor(_Mem(), device="cuda").view(dtype).view(shape)

    def single_cache(self, layer: int):
        """Torch views of one layer's single-sequence cache: (keys, values, key_norms, value_norms), rows
        (max_seq_len, ...); valid until sleep, set_shape or the engine's end."""
        L, H, Hk, D = self._shape
        msl, bits = self.max_seq_len(), self.kv_bits()
        ptrs = [self._lib.tw_engine_single_cache_ptr(self._h, layer, w) for w in range(4)]
        if not ptrs[0]:
            raise RuntimeError("single-sequence caches are not allocated")
        if bits == 0:
            n = msl * Hk * D * 2
            return (self._wrap(ptrs[0], n, torch.float16, (msl, Hk * D)),
                    self._wrap(ptrs[1], n, torch.float16, (msl, Hk * D)), None, None)
        kvp = Hk * D * bits // 8
        return (self._wrap(ptrs[0], msl * kvp, torch.uint8, (msl, kvp)), self._wrap(ptrs[1], msl * kvp, torch.uint8, (msl, kvp)),
                self._wrap(ptrs[2], msl * Hk * 2, torch.float16, (msl, Hk)), self._wrap(ptrs[3], msl * Hk * 2, torch.float16, (msl, Hk)))

    def single_rotation(self):
        p = self._lib.tw_engine_single_rotation(self._h)
        if not p:
            return None
        D = self._shape[3]
        return self._wrap(p, D * D * 2, torch.float16, (D, D))

    def single_step(self, layer, q, k, v, out, stream=None) -> None:
        """forward_layer's append + attention for `layer` at current_pos (engine.cpp:1069-1108).
        q/out: (H*D,), k/v: (Hk*D,)."""
        L, H, Hk, D = self._shape
        for name, t, n in (("q", q, H * D), ("out", out, H * D), ("k", k, Hk * D), ("v", v, Hk * D)):
            if t.numel() != n:
                raise ValueError(f"{name}: {t.numel()} elements, expected {n}")
        rc = self._lib.tw_engine_single_step(self._h, layer, _ptr(q, "f16", "q"), _ptr(k, "f16", "k"), _ptr(v, "f16", "v"),
                                             _ptr(out, "f16", "out"), _stream(stream))
        if rc != 0:
            _lib.check(self._lib)
            raise RuntimeError(f"single_step failed ({rc})")

    def single_advance(self, stream=None) -> None:
        """current_pos += 1 (decode_token, after the last layer)."""
        rc = self._lib.tw_engine_single_advance(self._h, _stream(stream))
        if rc != 0:
            _lib.check(self._lib)
            raise RuntimeError(f"single_advance failed ({rc})")

    # ---- memory lifecycle (engine.cpp:922-1022)
    def sleep(self) -> None:
        """Give the cache memory back (the torch arena is released, the single-sequence caches are freed) and drop
        the captured step."""
        self._lib.tw_engine_sleep(self._h)
        self._arena = None
        self._G = self._msl = 0

    def wake(self) -> None:
        """Re-allocate the single-sequence caches if the engine had them before sleep (engine.cpp:985-1022); the
        batch comes back with the next alloc_batch."""
        rc = self._lib.tw_engine_wake(self._h)
        if rc != 0:
            raise RuntimeError(f"wake failed ({rc})")

    def is_allocated(self) -> bool:
        return bool(self._lib.tw_engine_is_allocated(self._h))

    # ---- tail of the decode loop (engine.cpp:2350, 2496-2534)
    def begin_generation(self, max_new_tokens: int, eos_token_id: int, stop_token_ids=()) -> None:
        ids = (C.c_int * max(len(stop_token_ids), 1))(*[int(x) for x in stop_token_ids])
        rc = self._lib.tw_engine_begin_generation(self._h, int(max_new_tokens), int(eos_token_id), ids, len(stop_token_ids))
        if rc != 0:
            raise RuntimeError(f"begin_generation failed ({rc})")

    def record_tokens(self, tokens, step: int, stream=None) -> None:
        rc = self._lib.tw_engine_record_tokens(self._h, _ptr(tokens, "i32", "tokens"), int(step), _stream(stream))
        if rc != 0:
            raise RuntimeError(f"record_tokens failed ({rc})")

    def check_stops(self, step: int, stream=None):
        """-> (all_done, checked)"""
        checked = C.c_int(0)
        rc = self._lib.tw_engine_check_stops(self._h, int(step), _stream(stream), C.byref(checked))
        if rc < 0:
            raise RuntimeError(f"check_stops failed ({rc})")
        return bool(rc), bool(checked.value)

    def output(self, g: int):
        """-> (tokens so far, finished)"""
        ptr, n = C.POINTER(C.c_int)(), C.c_int(0)
        rc = self._lib.tw_engine_output(self._h, int(g), C.byref(ptr), C.byref(n))
        if rc < 0:
            raise IndexError(g)
        return [ptr[i] for i in range(n.value)], bool(rc)
