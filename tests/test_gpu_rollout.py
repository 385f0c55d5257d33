"""The GRPO rollout as a loop (generate_batch, engine.cpp:2173-2214, 2369-2412, 2472-2497): a shared prompt prefix
goes through the prompt call into the first sequence of every group, the prefix broadcast copies it to the
group's other members, and then decode steps are replayed from one captured graph -- steps that READ the rows the
broadcast wrote.  Through the engine object of the C ABI.

  reduced size, against the CPU oracle step by step: every cache byte and position bit for bit, outputs within 2e-3
  (per head vector, ||gpu - oracle||_inf / ||oracle||_inf);
  full size (128 sequences, 28 layers, 256-token prefix), by properties the oracle need not be run for.
"""
import numpy as np
import pytest

import gen
from test_gpu_parity import D, TOL, assert_bytes_equal, dev, host, rel_err

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kv_bits", [0, 4])
def test_rollout_loop_against_the_oracle(oracle, kv_bits):
    import torch
    from triebwerk_amd import Engine
    L, H, Hk, groups, members, T, steps = 2, 16, 8, 4, 4, 32, 40
    G, msl = groups * members, T + steps + 8
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(7700 + kv_bits)
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    rot = host(eng.rotation()) if kv_bits else None

    # oracle-side caches, one set per layer
    if kv_bits:
        kvp = kv_dim * kv_bits // 8
        o_k = [np.zeros((G, msl, kvp), np.uint8) for _ in range(L)]; o_v = [np.zeros((G, msl, kvp), np.uint8) for _ in range(L)]
        o_kn = [np.zeros((G, msl, Hk), np.float16) for _ in range(L)]; o_vn = [np.zeros((G, msl, Hk), np.float16) for _ in range(L)]
    else:
        o_k = [np.zeros((G, msl, kv_dim), np.float16) for _ in range(L)]; o_v = [np.zeros((G, msl, kv_dim), np.float16) for _ in range(L)]

    # ---- the prompt: every group's own prefix into its first sequence, layer by layer, then the broadcast
    tok = np.arange(T, dtype=np.int32)
    for l in range(L):
        for gr in range(groups):
            g0 = gr * members
            q = gen.normal_f16(r, (T, q_dim)); k = gen.kv_rows_with_outliers(r, (T, kv_dim), kv_dim)[0]; v = gen.normal_f16(r, (T, kv_dim))
            out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
            eng.prompt_layer(l, g0, dev(q), dev(k), dev(v), out, dev(tok))
            want = np.zeros((T, q_dim), np.float16)
            if kv_bits:
                oracle.turbo_kv_quantize(o_k[l][g0], o_kn[l][g0], k, rot, tok, msl, T, Hk, D, kv_dim, kv_bits)
                oracle.turbo_kv_quantize(o_v[l][g0], o_vn[l][g0], v, rot, tok, msl, T, Hk, D, kv_dim, kv_bits)
                oracle.turbo_gqa_prefill_attention(want, q, o_k[l][g0], o_v[l][g0], o_kn[l][g0], o_vn[l][g0], rot, T, msl, H, Hk,
                                                   D, q_dim, kv_dim, kv_bits)
            else:
                o_k[l][g0, :T] = k; o_v[l][g0, :T] = v
                oracle.gqa_prefill_attention(want, q, o_k[l][g0], o_v[l][g0], T, msl, H, Hk, D, q_dim, kv_dim)
            assert rel_err(host(out), want) <= TOL, f"prompt, layer {l}, group {gr}"
    for gr in range(groups):
        g0 = gr * members
        eng.broadcast_prefix(g0, g0 + 1, g0 + members, T)
        arrays = (o_k, o_v, o_kn, o_vn) if kv_bits else (o_k, o_v)
        for arr in arrays:
            for l in range(L):
                arr[l][g0 + 1:g0 + members, :T] = arr[l][g0, :T]
    pos = np.full(G, T, np.int32)
    eng.set_positions(pos)

    # ---- decode: one graph, replayed; fresh inputs are copied into its buffers before every step
    d_q = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
    d_k = torch.zeros((L, G, kv_dim), dtype=torch.float16, device="cuda")
    d_v = torch.zeros((L, G, kv_dim), dtype=torch.float16, device="cuda")
    d_out = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
    stream = torch.cuda.Stream()
    for step in range(steps):
        q = gen.normal_f16(r, (L, G, q_dim)); k = gen.normal_f16(r, (L, G, kv_dim)); v = gen.normal_f16(r, (L, G, kv_dim))
        d_q.copy_(dev(q)); d_k.copy_(dev(k)); d_v.copy_(dev(v))
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            eng.decode_step(d_q, d_k, d_v, d_out, use_graph=True, stream=stream)
        stream.synchronize()
        got = host(d_out)
        for l in range(L):
            want = np.zeros((G, q_dim), np.float16)
            if kv_bits:
                oracle.turbo_kv_quantize_batch(o_k[l], o_kn[l], k[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_kv_quantize_batch(o_v[l], o_vn[l], v[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_gqa_attention_batch(want, q[l], o_k[l], o_v[l], o_kn[l], o_vn[l], rot, pos, msl, G, H, Hk, D, q_dim,
                                                 kv_dim, kv_bits)
            else:
                oracle.kv_cache_write_batch(o_k[l], o_v[l], k[l], v[l], pos, msl, G, kv_dim)
                oracle.gqa_attention_batch(want, q[l], o_k[l], o_v[l], pos, msl, G, H, Hk, D, q_dim, kv_dim)
            err = rel_err(got[l], want)
            assert err <= TOL, f"decode step {step}, layer {l}: {err}"
        oracle.increment_positions(pos, G)
        assert np.array_equal(host(eng.positions()), pos), f"positions after step {step}"
    for l in range(L):
        c = eng.cache(l)
        assert_bytes_equal(host(c[0]), o_k[l], f"layer {l} K cache")
        assert_bytes_equal(host(c[1]), o_v[l], f"layer {l} V cache")
        if kv_bits:
            assert_bytes_equal(host(c[2]), o_kn[l], f"layer {l} K norms")
            assert_bytes_equal(host(c[3]), o_vn[l], f"layer {l} V norms")


@pytest.mark.parametrize("kv_bits", [0, 4])
def test_rollout_loop_full_size_by_properties(kv_bits):
    """BASELINE config 5 as it is: 16 prompts x 8 = 128 sequences, 28 layers, a 256-token prefix per group, all 512
    graph-replayed decode steps (contexts 257 .. 768, max_seq_len 776).  Without the oracle: positions = 768 at the
    end; the prefix rows of every group member equal its source's bytes, before and after the steps (decode never
    touches them); outputs finite; two members of a group that are fed the same q, k and v rows produce the same
    output bits and the same appended cache bytes, members fed different rows do not; the step after a reset of the
    positions reproduces the first step's output bit for bit.  (The choice of kernels does not change inside this
    rollout: tw_kv_decode_step_plan answers "one launch" for 128 sequences up to contexts of several thousand tokens;
    test_gpu_engine_single.py crosses a change of plan at BASELINE config 4's size.)"""
    import torch
    from triebwerk_amd import Engine, _lib
    L, H, Hk, groups, members, T, steps = 28, 16, 8, 16, 8, 256, 512
    G, msl = groups * members, 776
    kv_dim, q_dim = Hk * D, H * D
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    gt = torch.Generator(device="cuda"); gt.manual_seed(31 + kv_bits)
    tok = torch.arange(T, dtype=torch.int32, device="cuda")
    for l in range(L):
        for gr in range(groups):
            q = torch.randn((T, q_dim), generator=gt, device="cuda", dtype=torch.float16)
            k = torch.randn((T, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
            v = torch.randn((T, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
            out = torch.empty((T, q_dim), dtype=torch.float16, device="cuda")
            eng.prompt_layer(l, gr * members, q, k, v, out, tok)
        assert torch.isfinite(out.float()).all()
    for gr in range(groups):
        eng.broadcast_prefix(gr * members, gr * members + 1, (gr + 1) * members, T)
    eng.set_positions([T] * G)
    torch.cuda.synchronize()

    def prefix_equal_to_source():
        for l in (0, L // 2, L - 1):
            for arr in eng.cache(l):
                if arr is None:
                    continue
                a = arr[:, :T].reshape(groups, members, -1)
                assert torch.equal(a, a[:, :1].expand_as(a)), f"layer {l}: a member's prefix differs from its source's"
                assert arr[:, :T].view(torch.uint8).any()
    prefix_equal_to_source()

    # members 0 and 1 of every group get the same rows, the others their own
    q = torch.randn((L, G, q_dim), generator=gt, device="cuda", dtype=torch.float16)
    k = torch.randn((L, G, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
    v = torch.randn((L, G, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
    for t in (q, k, v):
        tv = t.view(L, groups, members, -1)
        tv[:, :, 1] = tv[:, :, 0]
    out = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
    stream = torch.cuda.Stream()
    first = None
    lib = _lib.load()
    plans = set()
    with torch.cuda.stream(stream):
        for step in range(steps):
            if kv_bits:
                plans.add(lib.tw_kv_decode_step_plan(G, H, Hk, kv_bits, msl, T + step + 1, T + step + 1))
            eng.decode_step(q, k, v, out, use_graph=True, stream=stream)
            assert eng.graph_state() == 1
            if step == 0:
                stream.synchronize()
                first = out.clone()
            if step % 64 == 63:
                print(f"rollout kv_bits={kv_bits}: step {step + 1} of {steps}", flush=True)
    stream.synchronize()
    assert T + steps == 768 and host(eng.positions()).tolist() == [768] * G
    assert plans <= {1}, "the plan changed inside the rollout: say so in the docstring"
    assert torch.isfinite(out.float()).all()
    ov = out.view(L, groups, members, -1)
    assert torch.equal(ov[:, :, 0], ov[:, :, 1]), "same prefix, same inputs: different output bits"
    assert not torch.equal(ov[:, :, 0], ov[:, :, 2])
    for l in (0, L - 1):
        for arr in eng.cache(l):
            if arr is None:
                continue
            a = arr[:, T:T + steps].reshape(groups, members, -1)
            assert torch.equal(a[:, 0], a[:, 1]) and not torch.equal(a[:, 0], a[:, 2])
            assert not arr[:, T + steps:].view(torch.uint8).any(), "rows past the positions were written"
    prefix_equal_to_source()
    # back to the end of the prefix: the same graph, the same first step
    eng.set_positions([T] * G)
    with torch.cuda.stream(stream):
        eng.decode_step(q, k, v, out, use_graph=True, stream=stream)
    stream.synchronize()
    assert torch.equal(out, first), "replaying from the prefix does not reproduce the first step"
