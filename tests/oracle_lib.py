"""ctypes wrapper of oracle/libkv_oracle.so for the tests (numpy in, numpy out).

The oracle is the parity checker; the GPU library never sees it.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
LIB = ROOT / "oracle" / "libkv_oracle.so"

P, I = C.c_void_p, C.c_int


def _p(a, dtype):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.dtype == dtype and a.flags["C_CONTIGUOUS"], (a.dtype, dtype)
    return a.ctypes.data


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        lib.tw_oracle_f32_to_f16.restype = C.c_uint16
        lib.tw_oracle_f32_to_f16.argtypes = [C.c_float]
        lib.tw_oracle_f16_to_f32.restype = C.c_float
        lib.tw_oracle_f16_to_f32.argtypes = [C.c_uint16]
        lib.tw_oracle_centroids.restype = C.POINTER(C.c_float)
        lib.tw_oracle_centroids.argtypes = [I]
        lib.tw_oracle_bounds.restype = C.POINTER(C.c_float)
        lib.tw_oracle_bounds.argtypes = [I]
        lib.tw_oracle_quantize.restype = I
        lib.tw_oracle_quantize.argtypes = [C.c_float, I]
        lib.tw_oracle_margin.restype = C.c_float
        lib.tw_oracle_margin.argtypes = [C.c_float, I]
        lib.tw_oracle_make_rotation.argtypes = [P, P, I, C.c_uint32]
        lib.tw_oracle_kv_cache_write_batch.argtypes = [P, P, P, P, P, I, I, I]
        lib.tw_oracle_turbo_kv_quantize.argtypes = [P, P, P, P, P, I, I, I, I, I, I, P, P]
        lib.tw_oracle_turbo_kv_quantize_batch.argtypes = [P, P, P, P, P, I, I, I, I, I, I, P, P]
        lib.tw_oracle_gqa_attention.argtypes = [P, P, P, P, I, I, I, I, I]
        lib.tw_oracle_gqa_attention_batch.argtypes = [P, P, P, P, P, I, I, I, I, I, I, I]
        lib.tw_oracle_gqa_prefill_attention.argtypes = [P, P, P, P, I, I, I, I, I, I, I]
        lib.tw_oracle_turbo_gqa_attention.argtypes = [P, P, P, P, P, P, P, I, I, I, I, I, I]
        lib.tw_oracle_turbo_gqa_attention_batch.argtypes = [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I]
        lib.tw_oracle_turbo_gqa_prefill_attention.argtypes = [P, P, P, P, P, P, P, I, I, I, I, I, I, I, I]
        lib.tw_oracle_increment_positions.argtypes = [P, I]
        lib.tw_oracle_qk_norm.argtypes = [P, P, P, P, I, I, I, C.c_float]
        lib.tw_oracle_qk_norm_batch.argtypes = [P, P, P, P, I, I, I, I, C.c_float, I, I, I]
        lib.tw_oracle_rope.argtypes = [P, P, P, P, I, I, I, I, I]
        lib.tw_oracle_rope_batch.argtypes = [P, P, P, P, P, I, I, I, I, I, I, I, I]
        lib.tw_oracle_rope_tables.argtypes = [P, P, I, I, C.c_float]
        lib.tw_oracle_sigmoid_gate_batch.argtypes = [P, P, I, I]
        lib.tw_oracle_num_threads.restype = I
        lib.tw_oracle_set_num_threads.argtypes = [I]

    # ---- scalars / tables
    def centroids(self, bits):
        n = 16 if bits == 4 else 4
        return np.array([self.lib.tw_oracle_centroids(bits)[i] for i in range(n)], dtype=np.float32)

    def bounds(self, bits):
        n = 15 if bits == 4 else 3
        return np.array([self.lib.tw_oracle_bounds(bits)[i] for i in range(n)], dtype=np.float32)

    def quantize(self, val, bits):
        return self.lib.tw_oracle_quantize(float(val), bits)

    def make_rotation(self, d=128, seed=42):
        f16 = np.empty((d, d), dtype=np.float16)
        f32 = np.empty((d, d), dtype=np.float32)
        self.lib.tw_oracle_make_rotation(f16.ctypes.data, f32.ctypes.data, d, seed)
        return f16, f32

    # ---- kernels (arrays are modified in place, like the device buffers)
    def kv_cache_write_batch(self, ck, cv, k, v, pos, msl, G, kv_dim):
        self.lib.tw_oracle_kv_cache_write_batch(_p(ck, np.float16), _p(cv, np.float16), _p(k, np.float16),
                                                _p(v, np.float16), _p(pos, np.int32), msl, G, kv_dim)

    def turbo_kv_quantize(self, cache_q, cache_norms, kv_buf, rotation, positions, msl, num_tokens,
                          Hk, D, kv_dim, bits, rotated=None, margin=None):
        self.lib.tw_oracle_turbo_kv_quantize(_p(cache_q, np.uint8), _p(cache_norms, np.float16),
                                             _p(kv_buf, np.float16), _p(rotation, np.float16),
                                             _p(positions, np.int32), msl, num_tokens, Hk, D, kv_dim, bits,
                                             _p(rotated, np.float32), _p(margin, np.float32))

    def turbo_kv_quantize_batch(self, cache_q, cache_norms, kv_buf, rotation, positions, msl, G,
                                Hk, D, kv_dim, bits, rotated=None, margin=None):
        self.lib.tw_oracle_turbo_kv_quantize_batch(_p(cache_q, np.uint8), _p(cache_norms, np.float16),
                                                   _p(kv_buf, np.float16), _p(rotation, np.float16),
                                                   _p(positions, np.int32), msl, G, Hk, D, kv_dim, bits,
                                                   _p(rotated, np.float32), _p(margin, np.float32))

    def gqa_attention(self, q, kc, vc, out, pos, msl, H, Hk, D):
        self.lib.tw_oracle_gqa_attention(_p(q, np.float16), _p(kc, np.float16), _p(vc, np.float16),
                                         _p(out, np.float16), pos, msl, H, Hk, D)

    def gqa_attention_batch(self, out, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim):
        self.lib.tw_oracle_gqa_attention_batch(_p(out, np.float16), _p(q, np.float16), _p(ck, np.float16),
                                               _p(cv, np.float16), _p(pos, np.int32), msl, G, H, Hk, D,
                                               q_dim, kv_dim)

    def gqa_prefill_attention(self, out, q, ck, cv, T, msl, H, Hk, D, q_dim, kv_dim):
        self.lib.tw_oracle_gqa_prefill_attention(_p(out, np.float16), _p(q, np.float16), _p(ck, np.float16),
                                                 _p(cv, np.float16), T, msl, H, Hk, D, q_dim, kv_dim)

    def turbo_gqa_attention(self, q, ckq, cvq, kn, vn, rot, out, pos, msl, H, Hk, D, bits):
        self.lib.tw_oracle_turbo_gqa_attention(_p(q, np.float16), _p(ckq, np.uint8), _p(cvq, np.uint8),
                                               _p(kn, np.float16), _p(vn, np.float16), _p(rot, np.float16),
                                               _p(out, np.float16), pos, msl, H, Hk, D, bits)

    def turbo_gqa_attention_batch(self, out, q, ckq, cvq, kn, vn, rot, pos, msl, G, H, Hk, D, q_dim,
                                  kv_dim, bits):
        self.lib.tw_oracle_turbo_gqa_attention_batch(_p(out, np.float16), _p(q, np.float16),
                                                     _p(ckq, np.uint8), _p(cvq, np.uint8),
                                                     _p(kn, np.float16), _p(vn, np.float16),
                                                     _p(rot, np.float16), _p(pos, np.int32), msl, G, H,
                                                     Hk, D, q_dim, kv_dim, bits)

    def turbo_gqa_prefill_attention(self, out, q, ckq, cvq, kn, vn, rot, T, msl, H, Hk, D, q_dim,
                                    kv_dim, bits):
        self.lib.tw_oracle_turbo_gqa_prefill_attention(_p(out, np.float16), _p(q, np.float16),
                                                       _p(ckq, np.uint8), _p(cvq, np.uint8),
                                                       _p(kn, np.float16), _p(vn, np.float16),
                                                       _p(rot, np.float16), T, msl, H, Hk, D, q_dim,
                                                       kv_dim, bits)

    def increment_positions(self, pos, G):
        self.lib.tw_oracle_increment_positions(_p(pos, np.int32), G)

    def qk_norm(self, q, k, qw, kw, H, Hk, D, eps):
        self.lib.tw_oracle_qk_norm(_p(q, np.float16), _p(k, np.float16), _p(qw, np.float16), _p(kw, np.float16),
                                   H, Hk, D, eps)

    def qk_norm_batch(self, q, k, qw, kw, H, Hk, D, G, eps, q_dim, kv_dim, biased=False):
        self.lib.tw_oracle_qk_norm_batch(_p(q, np.float16), _p(k, np.float16), _p(qw, np.float16),
                                         _p(kw, np.float16), H, Hk, D, G, eps, q_dim, kv_dim, int(biased))

    def rope(self, q, k, ct, st, pos, msl, H, Hk, D):
        self.lib.tw_oracle_rope(_p(q, np.float16), _p(k, np.float16), _p(ct, np.float16), _p(st, np.float16),
                                pos, msl, H, Hk, D)

    def rope_batch(self, q, k, ct, st, positions, msl, G, H, Hk, D, q_dim, kv_dim, rope_dim):
        self.lib.tw_oracle_rope_batch(_p(q, np.float16), _p(k, np.float16), _p(ct, np.float16), _p(st, np.float16),
                                      _p(positions, np.int32), msl, G, H, Hk, D, q_dim, kv_dim, rope_dim)

    def rope_tables(self, msl, rope_dim, theta):
        ct = np.empty((msl, rope_dim // 2), np.float16)
        st = np.empty((msl, rope_dim // 2), np.float16)
        self.lib.tw_oracle_rope_tables(ct.ctypes.data, st.ctypes.data, msl, rope_dim, theta)
        return ct, st

    def sigmoid_gate_batch(self, data, gate, dim, G):
        self.lib.tw_oracle_sigmoid_gate_batch(_p(data, np.float16), _p(gate, np.float16), dim, G)

    def num_threads(self):
        return self.lib.tw_oracle_num_threads()

    def set_num_threads(self, n):
        self.lib.tw_oracle_set_num_threads(n)


_cached = None


LIB_O3 = ROOT / "oracle" / "libkv_oracle_o3.so"
_cached_o3 = None


def load() -> Oracle:
    global _cached
    if _cached is None:
        if not LIB.exists():
            subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
        _cached = Oracle(C.CDLL(str(LIB)))
    return _cached


def load_o3() -> Oracle:
    """The -O3 build of the same source (oracle/Makefile): what the benchmark times as the CPU baseline."""
    global _cached_o3
    if _cached_o3 is None:
        if not LIB_O3.exists():
            subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
        _cached_o3 = Oracle(C.CDLL(str(LIB_O3)))
    return _cached_o3
