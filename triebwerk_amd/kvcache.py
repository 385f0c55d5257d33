"""Python entry points over the C ABI, one per launcher of ``include/triebwerk_kv.h``.

Argument order and meaning are the launchers' own (reference: engine.cpp:105-171);
tensors replace raw device pointers and the HIP stream defaults to torch's
current stream.  torch is used for device memory and streams only.
"""
from __future__ import annotations

import torch

from . import _lib

_DT = {"f16": torch.float16, "u8": torch.uint8, "i32": torch.int32, "f32": torch.float32}


def _ptr(t, kind: str, name: str):
    if t is None:
        return None
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name}: expected a CUDA/HIP tensor")
    if t.dtype != _DT[kind]:
        raise TypeError(f"{name}: expected dtype {_DT[kind]}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: tensor must be contiguous")
    return t.data_ptr()


def _stream(stream):
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return int(stream)


def _done(lib):
    _lib.check(lib)


def launch_kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim, stream=None):
    lib = _lib.load()
    lib.launch_kv_cache_write_batch(_ptr(ck, "f16", "ck"), _ptr(cv, "f16", "cv"), _ptr(k, "f16", "k"),
                                    _ptr(v, "f16", "v"), _ptr(pos, "i32", "pos"), msl, G, kv_dim,
                                    _stream(stream))
    _done(lib)


def launch_turbo_kv_quantize(cache_q, cache_norms, kv_buf, rotation, positions, max_seq_len,
                             num_tokens, num_kv_heads, head_dim, kv_dim, bits, stream=None):
    lib = _lib.load()
    lib.launch_turbo_kv_quantize(_ptr(cache_q, "u8", "cache_q"), _ptr(cache_norms, "f16", "cache_norms"),
                                 _ptr(kv_buf, "f16", "kv_buf"), _ptr(rotation, "f16", "rotation"),
                                 _ptr(positions, "i32", "positions"), max_seq_len, num_tokens,
                                 num_kv_heads, head_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def launch_turbo_kv_quantize_batch(cache_q, cache_norms, kv_buf, rotation, positions, max_seq_len,
                                   G, num_kv_heads, head_dim, kv_dim, bits, stream=None):
    lib = _lib.load()
    lib.launch_turbo_kv_quantize_batch(_ptr(cache_q, "u8", "cache_q"), _ptr(cache_norms, "f16", "cache_norms"),
                                       _ptr(kv_buf, "f16", "kv_buf"), _ptr(rotation, "f16", "rotation"),
                                       _ptr(positions, "i32", "positions"), max_seq_len, G,
                                       num_kv_heads, head_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def launch_gqa_attention(q, k_cache, v_cache, output, attn_scratch, pos, max_seq_len, num_heads,
                         num_kv_heads, head_dim, stream=None):
    lib = _lib.load()
    lib.launch_gqa_attention(_ptr(q, "f16", "q"), _ptr(k_cache, "f16", "k_cache"),
                             _ptr(v_cache, "f16", "v_cache"), _ptr(output, "f16", "output"),
                             _ptr(attn_scratch, "f32", "attn_scratch"), pos, max_seq_len, num_heads,
                             num_kv_heads, head_dim, _stream(stream))
    _done(lib)


def launch_gqa_attention_batch(out, q, ck, cv, scratch, pos, msl, G, num_heads, num_kv_heads,
                               head_dim, q_dim, kv_dim, stream=None):
    lib = _lib.load()
    lib.launch_gqa_attention_batch(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(ck, "f16", "ck"),
                                   _ptr(cv, "f16", "cv"), _ptr(scratch, "f32", "as"),
                                   _ptr(pos, "i32", "pos"), msl, G, num_heads, num_kv_heads, head_dim,
                                   q_dim, kv_dim, _stream(stream))
    _done(lib)


def launch_gqa_prefill_attention(out, q, ck, cv, scratch, T, msl, num_heads, num_kv_heads, head_dim,
                                 q_dim, kv_dim, stream=None):
    lib = _lib.load()
    lib.launch_gqa_prefill_attention(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(ck, "f16", "ck"),
                                     _ptr(cv, "f16", "cv"), _ptr(scratch, "f32", "as"), T, msl,
                                     num_heads, num_kv_heads, head_dim, q_dim, kv_dim, _stream(stream))
    _done(lib)


def launch_turbo_gqa_attention(q, ck_q, cv_q, k_norms, v_norms, rotation, output, scratch, pos, msl,
                               num_heads, num_kv_heads, head_dim, bits, stream=None):
    lib = _lib.load()
    lib.launch_turbo_gqa_attention(_ptr(q, "f16", "q"), _ptr(ck_q, "u8", "ck_q"), _ptr(cv_q, "u8", "cv_q"),
                                   _ptr(k_norms, "f16", "k_norms"), _ptr(v_norms, "f16", "v_norms"),
                                   _ptr(rotation, "f16", "rotation"), _ptr(output, "f16", "output"),
                                   _ptr(scratch, "f32", "as"), pos, msl, num_heads, num_kv_heads,
                                   head_dim, bits, _stream(stream))
    _done(lib)


def launch_turbo_gqa_attention_batch(out, q, ck_q, cv_q, k_norms, v_norms, rotation, scratch, pos,
                                     msl, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits,
                                     stream=None):
    lib = _lib.load()
    lib.launch_turbo_gqa_attention_batch(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"),
                                         _ptr(ck_q, "u8", "ck_q"), _ptr(cv_q, "u8", "cv_q"),
                                         _ptr(k_norms, "f16", "k_norms"), _ptr(v_norms, "f16", "v_norms"),
                                         _ptr(rotation, "f16", "rotation"), _ptr(scratch, "f32", "as"),
                                         _ptr(pos, "i32", "pos"), msl, G, num_heads, num_kv_heads,
                                         head_dim, q_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def tw_turbo_gqa_attention_batch_noalloc(out, q, ck_q, cv_q, k_norms, v_norms, rotation, pos, msl, G, num_heads,
                                         num_kv_heads, head_dim, q_dim, kv_dim, bits, stream=None):
    """launch_turbo_gqa_attention_batch without the scratch argument: the library's own device array is the
    workspace and the call allocates nothing."""
    lib = _lib.load()
    rc = lib.tw_turbo_gqa_attention_batch_noalloc(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"),
                                                  _ptr(ck_q, "u8", "ck_q"), _ptr(cv_q, "u8", "cv_q"),
                                                  _ptr(k_norms, "f16", "k_norms"), _ptr(v_norms, "f16", "v_norms"),
                                                  _ptr(rotation, "f16", "rotation"), _ptr(pos, "i32", "pos"), msl, G,
                                                  num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits,
                                                  _stream(stream))
    _done(lib)
    if rc != 0:
        raise RuntimeError(f"tw_turbo_gqa_attention_batch_noalloc returned {rc}")


def launch_turbo_gqa_prefill_attention(out, q, ck_q, cv_q, k_norms, v_norms, rotation, scratch, T,
                                       msl, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits,
                                       stream=None):
    lib = _lib.load()
    lib.launch_turbo_gqa_prefill_attention(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"),
                                           _ptr(ck_q, "u8", "ck_q"), _ptr(cv_q, "u8", "cv_q"),
                                           _ptr(k_norms, "f16", "k_norms"), _ptr(v_norms, "f16", "v_norms"),
                                           _ptr(rotation, "f16", "rotation"), _ptr(scratch, "f32", "as"),
                                           T, msl, num_heads, num_kv_heads, head_dim, q_dim, kv_dim,
                                           bits, _stream(stream))
    _done(lib)


def launch_increment_positions(positions, G, stream=None):
    lib = _lib.load()
    lib.launch_increment_positions(_ptr(positions, "i32", "positions"), G, _stream(stream))
    _done(lib)


def tw_turbo_kv_append_batch(ck_q, k_norms, cv_q, v_norms, k_buf, v_buf, rotation, positions,
                             max_seq_len, G, num_kv_heads, head_dim, kv_dim, bits, stream=None):
    lib = _lib.load()
    lib.tw_turbo_kv_append_batch(_ptr(ck_q, "u8", "ck_q"), _ptr(k_norms, "f16", "k_norms"),
                                 _ptr(cv_q, "u8", "cv_q"), _ptr(v_norms, "f16", "v_norms"),
                                 _ptr(k_buf, "f16", "k_buf"), _ptr(v_buf, "f16", "v_buf"),
                                 _ptr(rotation, "f16", "rotation"), _ptr(positions, "i32", "positions"),
                                 max_seq_len, G, num_kv_heads, head_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def tw_turbo_kv_append_tokens(ck_q, k_norms, cv_q, v_norms, k_buf, v_buf, rotation, positions,
                              max_seq_len, num_tokens, num_kv_heads, head_dim, kv_dim, bits, stream=None):
    """K and V rows of a prompt's tokens into one sequence's cache, one launch (engine.cpp:2121-2131)."""
    lib = _lib.load()
    lib.tw_turbo_kv_append_tokens(_ptr(ck_q, "u8", "ck_q"), _ptr(k_norms, "f16", "k_norms"),
                                  _ptr(cv_q, "u8", "cv_q"), _ptr(v_norms, "f16", "v_norms"),
                                  _ptr(k_buf, "f16", "k_buf"), _ptr(v_buf, "f16", "v_buf"),
                                  _ptr(rotation, "f16", "rotation"), _ptr(positions, "i32", "positions"),
                                  max_seq_len, num_tokens, num_kv_heads, head_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def tw_turbo_append_attention_batch(out, q, k_buf, v_buf, ck_q, cv_q, k_norms, v_norms, rotation, scratch,
                                    pos, msl, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits,
                                    stream=None):
    lib = _lib.load()
    lib.tw_turbo_append_attention_batch(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(k_buf, "f16", "k_buf"),
                                        _ptr(v_buf, "f16", "v_buf"), _ptr(ck_q, "u8", "ck_q"),
                                        _ptr(cv_q, "u8", "cv_q"), _ptr(k_norms, "f16", "k_norms"),
                                        _ptr(v_norms, "f16", "v_norms"), _ptr(rotation, "f16", "rotation"),
                                        _ptr(scratch, "f32", "as"), _ptr(pos, "i32", "pos"), msl, G,
                                        num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits,
                                        _stream(stream))
    _done(lib)


def tw_paged_kv_cache_write_batch(ck, cv, k, v, positions, block_table, bt_stride, G, kv_dim,
                                  stream=None):
    lib = _lib.load()
    lib.tw_paged_kv_cache_write_batch(_ptr(ck, "f16", "ck"), _ptr(cv, "f16", "cv"), _ptr(k, "f16", "k"),
                                      _ptr(v, "f16", "v"), _ptr(positions, "i32", "positions"),
                                      _ptr(block_table, "i32", "block_table"), bt_stride, G, kv_dim,
                                      _stream(stream))
    _done(lib)


def tw_paged_turbo_kv_append_batch(ck_q, k_norms, cv_q, v_norms, k_buf, v_buf, rotation, positions,
                                   block_table, bt_stride, G, num_kv_heads, head_dim, kv_dim, bits,
                                   stream=None):
    lib = _lib.load()
    lib.tw_paged_turbo_kv_append_batch(_ptr(ck_q, "u8", "ck_q"), _ptr(k_norms, "f16", "k_norms"),
                                       _ptr(cv_q, "u8", "cv_q"), _ptr(v_norms, "f16", "v_norms"),
                                       _ptr(k_buf, "f16", "k_buf"), _ptr(v_buf, "f16", "v_buf"),
                                       _ptr(rotation, "f16", "rotation"),
                                       _ptr(positions, "i32", "positions"),
                                       _ptr(block_table, "i32", "block_table"), bt_stride, G,
                                       num_kv_heads, head_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def tw_paged_gqa_attention_batch(out, q, ck, cv, ws, positions, block_table, bt_stride, max_context,
                                 G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, stream=None):
    lib = _lib.load()
    lib.tw_paged_gqa_attention_batch(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(ck, "f16", "ck"),
                                     _ptr(cv, "f16", "cv"), _ptr(ws, "f32", "ws"),
                                     _ptr(positions, "i32", "positions"),
                                     _ptr(block_table, "i32", "block_table"), bt_stride, max_context,
                                     G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim,
                                     _stream(stream))
    _done(lib)


def tw_paged_turbo_gqa_attention_batch(out, q, ck_q, cv_q, k_norms, v_norms, rotation, ws, positions,
                                       block_table, bt_stride, max_context, G, num_heads,
                                       num_kv_heads, head_dim, q_dim, kv_dim, bits, stream=None):
    lib = _lib.load()
    lib.tw_paged_turbo_gqa_attention_batch(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"),
                                           _ptr(ck_q, "u8", "ck_q"), _ptr(cv_q, "u8", "cv_q"),
                                           _ptr(k_norms, "f16", "k_norms"), _ptr(v_norms, "f16", "v_norms"),
                                           _ptr(rotation, "f16", "rotation"), _ptr(ws, "f32", "ws"),
                                           _ptr(positions, "i32", "positions"),
                                           _ptr(block_table, "i32", "block_table"), bt_stride,
                                           max_context, G, num_heads, num_kv_heads, head_dim, q_dim,
                                           kv_dim, bits, _stream(stream))
    _done(lib)


def tw_paged_turbo_append_attention_batch(out, q, k_buf, v_buf, ck_q, cv_q, k_norms, v_norms, rotation, ws, positions,
                                          block_table, bt_stride, max_context, G, num_heads, num_kv_heads, head_dim,
                                          q_dim, kv_dim, bits, stream=None):
    lib = _lib.load()
    lib.tw_paged_turbo_append_attention_batch(_ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(k_buf, "f16", "k_buf"),
                                              _ptr(v_buf, "f16", "v_buf"), _ptr(ck_q, "u8", "ck_q"),
                                              _ptr(cv_q, "u8", "cv_q"), _ptr(k_norms, "f16", "k_norms"),
                                              _ptr(v_norms, "f16", "v_norms"), _ptr(rotation, "f16", "rotation"),
                                              _ptr(ws, "f32", "ws"), _ptr(positions, "i32", "positions"),
                                              _ptr(block_table, "i32", "block_table"), bt_stride, max_context, G,
                                              num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def attention_workspace_floats(G, num_heads, max_context) -> int:
    return int(_lib.load().tw_attention_workspace_floats(G, num_heads, max_context))


def make_rotation(head_dim: int = 128, seed: int = 42) -> torch.Tensor:
    """The engine's rotation matrix (engine.cpp:366-392) as a CPU fp16 tensor."""
    out = torch.empty((head_dim, head_dim), dtype=torch.float16)
    _lib.load().tw_make_rotation_host(out.data_ptr(), head_dim, seed)
    return out


def set_attention_variant(variant: int) -> None:
    _lib.load().tw_kv_debug_set_attention_variant(int(variant))


def set_prefill_form(form: int) -> None:
    _lib.load().tw_kv_debug_set_prefill_form(int(form))


def set_decode_fused(mode: int) -> None:
    """tw_kv_debug_set_decode_fused: 0 the library's own choice, 1 one launch whenever the shape allows it, 2 never,
    3 as 1 but with one KV head per wave also where the 4-bit kernel would give a wave two."""
    _lib.load().tw_kv_debug_set_decode_fused(int(mode))


def set_fused_shape(hkw: int = 0, shares: int = 0) -> None:
    """tw_kv_debug_set_fused_shape: KV heads per workgroup and workgroups per (sequence, head group) of the one-launch
    decode step; 0 = the library's own choice."""
    _lib.load().tw_kv_debug_set_fused_shape(int(hkw), int(shares))


def last_scan_kernel() -> str:
    """Name of the kernel that the last decode-attention call launched for the context scan (a test hook)."""
    return _lib.load().tw_kv_debug_last_scan_kernel().decode()


def set_num_splits(nsplit: int) -> None:
    _lib.load().tw_kv_debug_set_num_splits(int(nsplit))


# ---- producers of q and k (engine.cpp:126-127, 162-163), in place
def launch_qk_norm_batch(q, k, q_weight, k_weight, num_q, num_kv, head_dim, G, eps, q_dim, kv_dim,
                         stream=None, biased=False):
    lib = _lib.load()
    lib.launch_qk_norm_batch(_ptr(q, "f16", "q"), _ptr(k, "f16", "k"), _ptr(q_weight, "f16", "q_weight"),
                             _ptr(k_weight, "f16", "k_weight"), num_q, num_kv, head_dim, G, eps, q_dim, kv_dim,
                             _stream(stream), bool(biased))
    _done(lib)


def launch_rope_batch(q, k, cos_table, sin_table, positions, max_seq_len, G, num_heads, num_kv_heads,
                      head_dim, q_dim, kv_dim, rope_dim, stream=None):
    lib = _lib.load()
    lib.launch_rope_batch(_ptr(q, "f16", "q"), _ptr(k, "f16", "k"), _ptr(cos_table, "f16", "cos_table"),
                          _ptr(sin_table, "f16", "sin_table"), _ptr(positions, "i32", "positions"), max_seq_len,
                          G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, rope_dim, _stream(stream))
    _done(lib)


def launch_qk_norm(q, k, q_weight, k_weight, num_q_heads, num_kv_heads, head_dim, eps, stream=None):
    lib = _lib.load()
    lib.launch_qk_norm(_ptr(q, "f16", "q"), _ptr(k, "f16", "k"), _ptr(q_weight, "f16", "q_weight"),
                       _ptr(k_weight, "f16", "k_weight"), num_q_heads, num_kv_heads, head_dim, eps,
                       _stream(stream))
    _done(lib)


def launch_rope(q, k, cos_table, sin_table, pos, max_seq_len, num_heads, num_kv_heads, head_dim, stream=None):
    lib = _lib.load()
    lib.launch_rope(_ptr(q, "f16", "q"), _ptr(k, "f16", "k"), _ptr(cos_table, "f16", "cos_table"),
                    _ptr(sin_table, "f16", "sin_table"), pos, max_seq_len, num_heads, num_kv_heads, head_dim,
                    _stream(stream))
    _done(lib)


def tw_append_attention_batch(out, q, k_buf, v_buf, ck, cv, scratch, pos, msl, G, num_heads, num_kv_heads, head_dim,
                              q_dim, kv_dim, stream=None):
    """fp16 cache: append at pos[g] and attend 0..pos[g] in one launch (engine.cpp:1979-2003)."""
    lib = _lib.load()
    lib.tw_append_attention_batch(
        _ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(k_buf, "f16", "k_buf"), _ptr(v_buf, "f16", "v_buf"),
        _ptr(ck, "f16", "ck"), _ptr(cv, "f16", "cv"), _ptr(scratch, "f32", "scratch"), _ptr(pos, "i32", "pos"),
        msl, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, _stream(stream))
    _done(lib)


def tw_qk_norm_rope_turbo_append_attention_batch(out, q, k_buf, v_buf, q_weight, k_weight, eps, biased, cos_table,
                                                 sin_table, rope_dim, ck_q, cv_q, k_norms, v_norms, rotation,
                                                 scratch, pos, msl, G, num_heads, num_kv_heads, head_dim, q_dim,
                                                 kv_dim, bits, stream=None):
    lib = _lib.load()
    lib.tw_qk_norm_rope_turbo_append_attention_batch(
        _ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(k_buf, "f16", "k_buf"), _ptr(v_buf, "f16", "v_buf"),
        _ptr(q_weight, "f16", "q_weight"), _ptr(k_weight, "f16", "k_weight"), eps, int(biased),
        _ptr(cos_table, "f16", "cos_table"), _ptr(sin_table, "f16", "sin_table"), rope_dim,
        _ptr(ck_q, "u8", "ck_q"), _ptr(cv_q, "u8", "cv_q"), _ptr(k_norms, "f16", "k_norms"),
        _ptr(v_norms, "f16", "v_norms"), _ptr(rotation, "f16", "rotation"), _ptr(scratch, "f32", "scratch"),
        _ptr(pos, "i32", "pos"), msl, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, bits, _stream(stream))
    _done(lib)


def tw_qk_norm_rope_append_attention_batch(out, q, k_buf, v_buf, q_weight, k_weight, eps, biased, cos_table,
                                           sin_table, rope_dim, ck, cv, scratch, pos, msl, G, num_heads,
                                           num_kv_heads, head_dim, q_dim, kv_dim, stream=None):
    lib = _lib.load()
    lib.tw_qk_norm_rope_append_attention_batch(
        _ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(k_buf, "f16", "k_buf"), _ptr(v_buf, "f16", "v_buf"),
        _ptr(q_weight, "f16", "q_weight"), _ptr(k_weight, "f16", "k_weight"), eps, int(biased),
        _ptr(cos_table, "f16", "cos_table"), _ptr(sin_table, "f16", "sin_table"), rope_dim,
        _ptr(ck, "f16", "ck"), _ptr(cv, "f16", "cv"), _ptr(scratch, "f32", "scratch"), _ptr(pos, "i32", "pos"),
        msl, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim, _stream(stream))
    _done(lib)


def launch_sigmoid_gate_batch(data, gate, dim, G, stream=None):
    lib = _lib.load()
    lib.launch_sigmoid_gate_batch(_ptr(data, "f16", "data"), _ptr(gate, "f16", "gate"), dim, G, _stream(stream))
    _done(lib)


def tw_layer_attention_step(out, q, k, v, positions, max_seq_len, G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim,
                            cache_k, cache_v, scratch, kv_bits=0, k_norms=None, v_norms=None, rotation=None,
                            q_weight=None, k_weight=None, eps=1e-6, biased=False, cos_table=None, sin_table=None,
                            rope_dim=0, gate=None, gate_stride=0, gate_offset=0, ctx_min=0, ctx_max=0, stream=None,
                            prompt=False, tickets=None):
    """Steps 3-6 of a layer (producers, append, attention, gate) through tw_layer_attention_step.
    `gate` may be the q tensor itself with gate_offset = num_heads*head_dim (gated q projection).
    prompt=True: the rows are the G = T tokens of a prompt of sequence 0 (tw_layer_prompt_step)."""
    lib = _lib.load()
    a = _lib.LayerStepArgs()
    a.out, a.q, a.k, a.v = _ptr(out, "f16", "out"), _ptr(q, "f16", "q"), _ptr(k, "f16", "k"), _ptr(v, "f16", "v")
    a.G, a.num_heads, a.num_kv_heads, a.head_dim, a.q_dim, a.kv_dim = G, num_heads, num_kv_heads, head_dim, q_dim, kv_dim
    a.positions, a.max_seq_len = _ptr(positions, "i32", "positions"), max_seq_len
    a.q_weight, a.k_weight = _ptr(q_weight, "f16", "q_weight"), _ptr(k_weight, "f16", "k_weight")
    a.eps, a.biased = eps, int(biased)
    a.cos_table, a.sin_table, a.rope_dim = _ptr(cos_table, "f16", "cos_table"), _ptr(sin_table, "f16", "sin_table"), rope_dim
    a.kv_bits = kv_bits
    a.cache_k = _ptr(cache_k, "u8" if kv_bits else "f16", "cache_k")
    a.cache_v = _ptr(cache_v, "u8" if kv_bits else "f16", "cache_v")
    a.k_norms, a.v_norms = _ptr(k_norms, "f16", "k_norms"), _ptr(v_norms, "f16", "v_norms")
    a.rotation, a.scratch = _ptr(rotation, "f16", "rotation"), _ptr(scratch, "f32", "scratch")
    gp = _ptr(gate, "f16", "gate")
    a.gate = (gp + 2 * gate_offset) if gp is not None else None
    a.gate_stride = gate_stride
    a.ctx_min, a.ctx_max = int(ctx_min), int(ctx_max)       # host knowledge of positions + 1; 0, 0 = none
    # G * num_kv_heads zeroed int32 words: lets the one-launch step share a sequence's context between workgroups
    a.tickets = _ptr(tickets, "i32", "tickets")
    (lib.tw_layer_prompt_step if prompt else lib.tw_layer_attention_step)(_lib.C.byref(a), _stream(stream))
    _done(lib)


def tw_layer_prompt_step(out, q, k, v, positions, max_seq_len, T, *args, **kwargs):
    """Steps 3-5b of a layer over a prompt of T tokens (prefill_chunked, engine.cpp:2097-2150); arguments as
    tw_layer_attention_step with T in the place of G, positions = 0 .. T-1, the caches of sequence 0."""
    tw_layer_attention_step(out, q, k, v, positions, max_seq_len, T, *args, prompt=True, **kwargs)
