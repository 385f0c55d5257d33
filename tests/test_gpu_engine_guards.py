"""The engine object's guards: a smaller batch after a larger one, a step on a full cache, and the captured
step following the choice of kernels as the contexts grow.  All through the C ABI (ctypes mirror)."""
import numpy as np
import pytest

import gen
from test_gpu_parity import D, TOL, assert_bytes_equal, dev, host, rel_err

pytestmark = pytest.mark.gpu


def _oracle_step(oracle, caches, q, k, v, rot, pos, msl, G, H, Hk, bits):
    kv_dim, q_dim = Hk * D, H * D
    ok, ov, okn, ovn = caches
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_kv_quantize_batch(ok, okn, k, rot, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(ov, ovn, v, rot, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_gqa_attention_batch(want, q, ok, ov, okn, ovn, rot, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    return want


def _zero_caches(G, msl, Hk, bits):
    kvp = Hk * D * bits // 8
    return (np.zeros((G, msl, kvp), np.uint8), np.zeros((G, msl, kvp), np.uint8),
            np.zeros((G, msl, Hk), np.float16), np.zeros((G, msl, Hk), np.float16))


def test_engine_smaller_batch_after_larger(oracle):
    """alloc_batch(8) then alloc_batch(4) inside the same memory: the steps work on 4 rows with 4-row strides
    (every layer reads its own rows), caches start zeroed, a (L, 8, .) buffer is refused."""
    import torch
    from triebwerk_amd import Engine
    r = gen.rng(8801)
    L, H, Hk, msl, bits = 3, 16, 8, 40, 4
    kv_dim, q_dim = Hk * D, H * D
    eng = Engine(kv_bits=bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(8, msl)
    arena_before = eng._arena.data_ptr()
    big = [dev(gen.normal_f16(r, (L, 8, n))) for n in (q_dim, kv_dim, kv_dim)]
    out8 = torch.zeros((L, 8, q_dim), dtype=torch.float16, device="cuda")
    eng.decode_step(big[0], big[1], big[2], out8)
    torch.cuda.synchronize()
    G = 4
    eng.alloc_batch(G, msl)
    assert eng._arena.data_ptr() == arena_before, "the memory already held is big enough"
    assert not host(eng.cache(L - 1)[0]).any() and not host(eng.positions()).any()
    with pytest.raises(ValueError):
        eng.decode_step(big[0], big[1], big[2], out8)
    rot = host(eng.rotation())
    caches = [_zero_caches(G, msl, Hk, bits) for _ in range(L)]
    pos = np.zeros(G, np.int32)
    for step in range(3):
        q = gen.normal_f16(r, (L, G, q_dim)); k = gen.normal_f16(r, (L, G, kv_dim)); v = gen.normal_f16(r, (L, G, kv_dim))
        out = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
        eng.decode_step(dev(q), dev(k), dev(v), out, use_graph=(step > 0))
        got = host(out)
        for l in range(L):
            want = _oracle_step(oracle, caches[l], q[l], k[l], v[l], rot, pos, msl, G, H, Hk, bits)
            assert rel_err(got[l], want) <= TOL, f"step {step} layer {l}"
        pos += 1
    for l in range(L):
        c = eng.cache(l)
        for i, what in enumerate(("K codes", "V codes", "K norms", "V norms")):
            assert_bytes_equal(host(c[i]), caches[l][i], f"layer {l} {what}")
    assert np.array_equal(host(eng.positions()), pos)


@pytest.mark.parametrize("kv_bits", [0, 4])
@pytest.mark.parametrize("use_graph", [False, True])
def test_engine_refuses_a_step_on_a_full_cache(kv_bits, use_graph):
    """Positions at the last row: that step runs; the next one returns an error before anything is launched
    and leaves cache and positions as they were (it would write row max_seq_len = the next sequence's row 0)."""
    import torch
    from triebwerk_amd import Engine
    r = gen.rng(8802 + kv_bits)
    L, H, Hk, G, msl = 2, 16, 8, 3, 16
    kv_dim, q_dim = Hk * D, H * D
    eng = Engine(kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    eng.set_positions([msl - 1, 2, msl - 2])
    d = [dev(gen.normal_f16(r, (L, G, n))) for n in (q_dim, kv_dim, kv_dim)]
    out = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
    eng.decode_step(d[0], d[1], d[2], out, use_graph=use_graph)
    torch.cuda.synchronize()
    before = [[None if t is None else host(t).copy() for t in eng.cache(l)] for l in range(L)]
    pos_before = host(eng.positions()).copy()
    assert pos_before.tolist() == [msl, 3, msl - 1]
    out_before = host(out).copy()
    with pytest.raises(RuntimeError, match="-8"):
        eng.decode_step(d[0], d[1], d[2], out, use_graph=use_graph)
    with pytest.raises(RuntimeError, match="-8"):
        eng.layer_step(0, d[0][0], d[1][0], d[2][0], out[0])
    torch.cuda.synchronize()
    assert np.array_equal(host(eng.positions()), pos_before)
    assert_bytes_equal(host(out), out_before, "output buffer")
    for l in range(L):
        for i, t in enumerate(eng.cache(l)):
            if t is not None:
                assert_bytes_equal(host(t), before[l][i], f"layer {l} array {i}")


def test_engine_captured_step_follows_the_plan(oracle):
    """A step captured at short contexts holds the one-launch kernel; when the contexts the host knows of move
    to where the three-kernel path is the choice (and back), the step is captured again with that choice, and
    the results stay the oracle's."""
    import torch
    from triebwerk_amd import Engine, _lib
    lib = _lib.load()
    r = gen.rng(8803)
    # (the engine hands the step its tickets, so small batches of long sequences stay on the one launch with their
    # contexts shared by workgroups: a batch that fills the compute units by itself is what changes over)
    L, H, Hk, G, msl, bits = 2, 16, 8, 72, 4352, 4
    kv_dim, q_dim = Hk * D, H * D
    assert lib.tw_kv_decode_step_plan2(G, H, Hk, bits, msl, 11, 11, 1) == 1
    assert lib.tw_kv_decode_step_plan2(G, H, Hk, bits, msl, 4201, 4201, 1) == 0
    eng = Engine(kv_bits=bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    rot = host(eng.rotation())
    caches = [_zero_caches(G, msl, Hk, bits) for _ in range(L)]
    d_q = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
    d_k = torch.zeros((L, G, kv_dim), dtype=torch.float16, device="cuda")
    d_v = torch.zeros((L, G, kv_dim), dtype=torch.float16, device="cuda")
    d_out = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
    fused_recorded = []
    for start in (10, 4200, 20):
        pos = np.full(G, start, np.int32)
        eng.set_positions(pos)
        for step in range(2):
            q = gen.normal_f16(r, (L, G, q_dim)); k = gen.normal_f16(r, (L, G, kv_dim)); v = gen.normal_f16(r, (L, G, kv_dim))
            d_q.copy_(dev(q)); d_k.copy_(dev(k)); d_v.copy_(dev(v))
            torch.cuda.synchronize()
            n0 = lib.tw_kv_decode_fused_launches()
            eng.decode_step(d_q, d_k, d_v, d_out, use_graph=True)
            fused_recorded.append(lib.tw_kv_decode_fused_launches() - n0)
            got = host(d_out)
            for l in range(L):
                want = _oracle_step(oracle, caches[l], q[l], k[l], v[l], rot, pos, msl, G, H, Hk, bits)
                assert rel_err(got[l], want) <= TOL, f"start {start} step {step} layer {l}"
            pos += 1
    # capture with the one-launch kernel, replay, capture with three kernels, replay, capture with one again, replay
    assert fused_recorded == [L, 0, 0, 0, L, 0]
    for l in range(L):
        c = eng.cache(l)
        for i, what in enumerate(("K codes", "V codes", "K norms", "V norms")):
            assert_bytes_equal(host(c[i]), caches[l][i], f"layer {l} {what}")
