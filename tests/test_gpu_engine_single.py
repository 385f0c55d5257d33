"""The engine object's single-sequence state (generate() / decode_token(): engine.cpp:322-331, 394-404 allocation,
893-916 reset, 922-1022 sleep / wake, 1069-1108 append -> attention of a layer), the decode step that goes on without a
graph when the capture fails (engine.cpp:2396-2410), and the trace ranges.  All through the C ABI (ctypes mirror),
against the CPU oracle's single-sequence functions: cache bytes bit for bit, outputs within 2e-3 per head vector.
"""
import numpy as np
import pytest

import gen
from test_gpu_parity import D, TOL, assert_bytes_equal, dev, host, rel_err

pytestmark = pytest.mark.gpu


def _single_oracle_caches(L, msl, Hk, kv_bits):
    kv_dim = Hk * D
    if kv_bits == 0:
        return [[np.zeros((msl, kv_dim), np.float16), np.zeros((msl, kv_dim), np.float16), None, None] for _ in range(L)]
    kvp = kv_dim * kv_bits // 8
    return [[np.zeros((msl, kvp), np.uint8), np.zeros((msl, kvp), np.uint8), np.zeros((msl, Hk), np.float16),
             np.zeros((msl, Hk), np.float16)] for _ in range(L)]


def _oracle_single_layer(oracle, c, q, k, v, rot, pos, msl, H, Hk, kv_bits):
    """forward_layer steps 4-5 with the oracle's single-sequence functions: the token-list append with one token
    (engine.cpp:1082-1091) or the row copy (1071-1074), then the single-sequence attention (1094-1106)."""
    kv_dim = Hk * D
    want = np.zeros(H * D, np.float16)
    if kv_bits == 0:
        c[0][pos] = k; c[1][pos] = v
        oracle.gqa_attention(q, c[0], c[1], want, pos, msl, H, Hk, D)
    else:
        p = np.array([pos], np.int32)
        oracle.turbo_kv_quantize(c[0], c[2], k.reshape(1, kv_dim), rot, p, msl, 1, Hk, D, kv_dim, kv_bits)
        oracle.turbo_kv_quantize(c[1], c[3], v.reshape(1, kv_dim), rot, p, msl, 1, Hk, D, kv_dim, kv_bits)
        oracle.turbo_gqa_attention(q, c[0], c[1], c[2], c[3], rot, want, pos, msl, H, Hk, D, kv_bits)
    return want


@pytest.mark.parametrize("kv_bits,H,Hk", [(0, 16, 8), (4, 16, 8), (2, 32, 8), (4, 12, 3)])
def test_single_sequence_tokens_against_the_oracle(oracle, rotation_fixture, kv_bits, H, Hk):
    """Tokens through tw_engine_single_step / single_advance from position 0, then from a position set by hand after
    a reset: every cache byte and the output of every layer and token against the oracle."""
    import torch
    from triebwerk_amd import Engine
    L, msl = 3, 96
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(9300 + kv_bits + H)
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    assert not eng.single_is_allocated()
    eng.alloc_single()
    assert eng.single_is_allocated() and eng.single_pos() == 0
    rot = None
    if kv_bits:
        rot = host(eng.single_rotation())
        assert_bytes_equal(rot, rotation_fixture, "single-sequence rotation")
    caches = _single_oracle_caches(L, msl, Hk, kv_bits)
    worst = 0.0

    def run_tokens(n_tokens):
        nonlocal worst
        for _ in range(n_tokens):
            pos = eng.single_pos()
            print(f"single step kv_bits={kv_bits} H={H} Hk={Hk} pos={pos}", flush=True)
            for l in range(L):
                q = gen.normal_f16(r, (q_dim,)); k = gen.kv_rows_with_outliers(r, (1, kv_dim), kv_dim)[0][0]; v = gen.normal_f16(r, (kv_dim,))
                out = torch.zeros(q_dim, dtype=torch.float16, device="cuda")
                eng.single_step(l, dev(q), dev(k), dev(v), out)
                want = _oracle_single_layer(oracle, caches[l], q, k, v, rot, pos, msl, H, Hk, kv_bits)
                err = rel_err(host(out), want)
                worst = max(worst, err)
                assert err <= TOL, f"token at {pos}, layer {l}: {err}"
            eng.single_advance()
            assert eng.single_pos() == pos + 1

    run_tokens(37)
    for l in range(L):
        for i, t in enumerate(eng.single_cache(l)):
            if t is not None:
                assert_bytes_equal(host(t), caches[l][i], f"layer {l} array {i}")
    # reset(): caches zeroed, current_pos = 0 (engine.cpp:893-916); then a position set by hand
    eng.reset()
    assert eng.single_pos() == 0
    for t in eng.single_cache(L - 1):
        assert t is None or not host(t).view(np.uint8).any()
    caches = _single_oracle_caches(L, msl, Hk, kv_bits)
    eng.single_set_pos(msl - 3)
    run_tokens(3)
    assert eng.single_pos() == msl
    # the cache is full: the step is refused, nothing is launched
    q = torch.zeros(q_dim, dtype=torch.float16, device="cuda"); kv_row = torch.zeros(kv_dim, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="-8"):
        eng.single_step(0, q, kv_row, kv_row, q)
    with pytest.raises(RuntimeError, match="-8"):
        eng.single_advance()
    for l in range(L):
        for i, t in enumerate(eng.single_cache(l)):
            if t is not None:
                assert_bytes_equal(host(t), caches[l][i], f"after the hand-set position: layer {l} array {i}")


@pytest.mark.parametrize("kv_bits", [4, 2])
def test_single_sequence_long_context_is_shared_by_workgroups(oracle, kv_bits):
    """One sequence of a few thousand tokens: the layer step takes the one-launch kernel with the context shared by
    workgroups (the engine hands its tickets over); random cache bytes, three tokens in a row against the oracle."""
    import torch
    from triebwerk_amd import Engine, kvcache
    L, H, Hk, msl = 2, 16, 8, 4200
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(9340 + kv_bits)
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_single()
    rot = host(eng.single_rotation())
    kvp = kv_dim * kv_bits // 8
    caches = []
    for l in range(L):
        c = [r.integers(0, 256, (msl, kvp), dtype=np.uint8), r.integers(0, 256, (msl, kvp), dtype=np.uint8),
             (11.3 + 0.7 * r.standard_normal((msl, Hk))).astype(np.float16), (11.3 + 0.7 * r.standard_normal((msl, Hk))).astype(np.float16)]
        for t, a in zip(eng.single_cache(l), c):
            t.copy_(dev(a))
        caches.append(c)
    start = 4100
    eng.single_set_pos(start)
    for tok in range(3):
        pos = eng.single_pos()
        print(f"single long context kv_bits={kv_bits} pos={pos}", flush=True)
        for l in range(L):
            q = gen.normal_f16(r, (q_dim,)); k = gen.normal_f16(r, (kv_dim,)); v = gen.normal_f16(r, (kv_dim,))
            out = torch.zeros(q_dim, dtype=torch.float16, device="cuda")
            eng.single_step(l, dev(q), dev(k), dev(v), out)
            assert "context shared" in kvcache.last_scan_kernel(), kvcache.last_scan_kernel()
            want = _oracle_single_layer(oracle, caches[l], q, k, v, rot, pos, msl, H, Hk, kv_bits)
            assert rel_err(host(out), want) <= TOL, f"token at {pos}, layer {l}"
        eng.single_advance()
    for l in range(L):
        for i, t in enumerate(eng.single_cache(l)):
            assert_bytes_equal(host(t)[start - 2:start + 5], caches[l][i][start - 2:start + 5], f"layer {l} array {i}")


def test_single_state_sleep_wake_and_batch_side_by_side(oracle):
    """sleep frees the single-sequence caches, wake re-allocates them (zeroed, position 0) when the engine had them;
    an engine that never had them gets none from wake; the batch arena and the single-sequence state do not touch
    each other's memory."""
    import torch
    from triebwerk_amd import Engine
    L, H, Hk, msl, kv_bits = 2, 16, 8, 48, 4
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(9351)
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.wake()
    assert not eng.single_is_allocated(), "wake re-allocates only what a sleep freed"
    eng.alloc_single()
    eng.alloc_batch(2, msl)
    rot = host(eng.single_rotation())
    caches = _single_oracle_caches(L, msl, Hk, kv_bits)
    dq = dev(gen.normal_f16(r, (L, 2, q_dim))); dk = dev(gen.normal_f16(r, (L, 2, kv_dim))); dv = dev(gen.normal_f16(r, (L, 2, kv_dim)))
    dout = torch.zeros((L, 2, q_dim), dtype=torch.float16, device="cuda")
    for tok in range(5):
        for l in range(L):
            q = gen.normal_f16(r, (q_dim,)); k = gen.normal_f16(r, (kv_dim,)); v = gen.normal_f16(r, (kv_dim,))
            out = torch.zeros(q_dim, dtype=torch.float16, device="cuda")
            eng.single_step(l, dev(q), dev(k), dev(v), out)
            want = _oracle_single_layer(oracle, caches[l], q, k, v, rot, tok, msl, H, Hk, kv_bits)
            assert rel_err(host(out), want) <= TOL
        eng.single_advance()
        eng.decode_step(dq, dk, dv, dout)                      # the batch path in between
    torch.cuda.synchronize()
    for l in range(L):
        for i, t in enumerate(eng.single_cache(l)):
            assert_bytes_equal(host(t), caches[l][i], f"layer {l} array {i}")
    assert host(eng.positions()).tolist() == [5, 5]
    eng.sleep()
    assert not eng.single_is_allocated() and not eng.is_allocated()
    q = torch.zeros(q_dim, dtype=torch.float16, device="cuda"); kv_row = torch.zeros(kv_dim, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="-1"):
        eng.single_step(0, q, kv_row, kv_row, q)
    eng.wake()
    assert eng.single_is_allocated() and eng.single_pos() == 0 and not eng.is_allocated()
    for t in eng.single_cache(0):
        assert not host(t).view(np.uint8).any()
    caches = _single_oracle_caches(L, msl, Hk, kv_bits)
    qh = gen.normal_f16(r, (q_dim,)); kh = gen.normal_f16(r, (kv_dim,)); vh = gen.normal_f16(r, (kv_dim,))
    out = torch.zeros(q_dim, dtype=torch.float16, device="cuda")
    eng.single_step(1, dev(qh), dev(kh), dev(vh), out)
    want = _oracle_single_layer(oracle, caches[1], qh, kh, vh, rot, 0, msl, H, Hk, kv_bits)
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("kv_bits", [0, 4])
def test_decode_goes_on_without_a_graph_when_capture_fails(oracle, capfd, kv_bits):
    """The capture is made to fail from the host (recorded, then treated as failed): the step runs eagerly, says so on
    stderr once, reports state 2, later steps with the same buffers do not try again, and other buffers do -- with the
    oracle's results throughout."""
    import torch
    from triebwerk_amd import Engine, _lib
    lib = _lib.load()
    L, H, Hk, G, msl = 2, 16, 8, 3, 40
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(9360 + kv_bits)
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    rot = host(eng.rotation()) if kv_bits else None
    if kv_bits:
        kvp = kv_dim * kv_bits // 8
        oc = [[np.zeros((G, msl, kvp), np.uint8), np.zeros((G, msl, kvp), np.uint8), np.zeros((G, msl, Hk), np.float16),
               np.zeros((G, msl, Hk), np.float16)] for _ in range(L)]
    else:
        oc = [[np.zeros((G, msl, kv_dim), np.float16), np.zeros((G, msl, kv_dim), np.float16)] for _ in range(L)]
    pos = np.zeros(G, np.int32)
    bufs = [[torch.zeros((L, G, n), dtype=torch.float16, device="cuda") for n in (q_dim, kv_dim, kv_dim, q_dim)] for _ in range(2)]
    lib.tw_engine_debug_fail_captures(eng._h, 1)
    states = []
    capfd.readouterr()
    for step, which in enumerate((0, 0, 0, 1, 1)):
        d_q, d_k, d_v, d_out = bufs[which]
        q = gen.normal_f16(r, (L, G, q_dim)); k = gen.normal_f16(r, (L, G, kv_dim)); v = gen.normal_f16(r, (L, G, kv_dim))
        d_q.copy_(dev(q)); d_k.copy_(dev(k)); d_v.copy_(dev(v))
        torch.cuda.synchronize()
        eng.decode_step(d_q, d_k, d_v, d_out, use_graph=True)
        states.append(eng.graph_state())
        got = host(d_out)
        for l in range(L):
            want = np.zeros((G, q_dim), np.float16)
            if kv_bits:
                oracle.turbo_kv_quantize_batch(oc[l][0], oc[l][2], k[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_kv_quantize_batch(oc[l][1], oc[l][3], v[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_gqa_attention_batch(want, q[l], oc[l][0], oc[l][1], oc[l][2], oc[l][3], rot, pos, msl, G, H, Hk, D,
                                                 q_dim, kv_dim, kv_bits)
            else:
                oracle.kv_cache_write_batch(oc[l][0], oc[l][1], k[l], v[l], pos, msl, G, kv_dim)
                oracle.gqa_attention_batch(want, q[l], oc[l][0], oc[l][1], pos, msl, G, H, Hk, D, q_dim, kv_dim)
            assert rel_err(got[l], want) <= TOL, f"step {step} layer {l}"
        pos += 1
        assert np.array_equal(host(eng.positions()), pos), f"positions after step {step}"
    # failed capture -> eager (2), same buffers stay eager, new buffers capture (1) and replay (1)
    assert states == [2, 2, 2, 1, 1]
    err = capfd.readouterr().err
    assert err.count("hipGraph capture FAILED") == 1
    eng.decode_step(*bufs[1], use_graph=False)
    assert eng.graph_state() == 0
    for l in range(L):
        c = eng.cache(l)
        for i in range(len(oc[l])):
            assert_bytes_equal(host(c[i])[:, :5], oc[l][i][:, :5], f"layer {l} array {i}")


def test_graph_replay_equals_the_eager_step_across_a_plan_flip_at_full_size():
    """28 layers, 16 heads over 8 KV heads, 2 bit, 80 sequences around the context where tw_kv_decode_step_plan2 changes
    its answer for a caller with tickets: an engine that replays a captured step and one that runs every step eagerly
    take the same plan at every step (both go by the positions the host knows), so their outputs and caches are equal
    bit for bit before, at and after the change, and the change happens inside the run."""
    import torch
    from triebwerk_amd import Engine, _lib
    lib = _lib.load()
    L, H, Hk, G, bits = 28, 16, 8, 80, 2
    kv_dim, q_dim = Hk * D, H * D
    msl = 4352
    flip = next(c for c in range(2, msl) if lib.tw_kv_decode_step_plan2(G, H, Hk, bits, msl, c, c, 1) == 0)
    assert lib.tw_kv_decode_step_plan2(G, H, Hk, bits, msl, flip - 1, flip - 1, 1) == 1 and flip + 8 < msl
    start = flip - 5                     # contexts of the steps: start + 1 .. start + 8, the flip among them
    gt = torch.Generator(device="cuda"); gt.manual_seed(97)
    engines = []
    for _ in range(2):
        e = Engine(max_seq_len=msl, kv_bits=bits)
        e.set_shape(L, H, Hk, D)
        e.alloc_batch(G, msl)
        engines.append(e)
    # the same random cache contents in both
    for l in range(L):
        a, b = engines[0].cache(l), engines[1].cache(l)
        for i in range(2):
            a[i].view(torch.int32).copy_(torch.randint(-2 ** 31, 2 ** 31 - 1, (a[i].numel() // 4,), generator=gt, device="cuda",
                                                      dtype=torch.int32).view(a[i].view(torch.int32).shape))
            b[i].copy_(a[i])
        for i in (2, 3):
            a[i].copy_((11.3 + 0.7 * torch.randn(a[i].shape, generator=gt, device="cuda")).to(torch.float16))
            b[i].copy_(a[i])
    for e in engines:
        e.set_positions([start] * G)
    q = torch.randn((L, G, q_dim), generator=gt, device="cuda", dtype=torch.float16)
    k = torch.randn((L, G, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
    v = torch.randn((L, G, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
    outs = [torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda") for _ in range(2)]
    one_launch_steps = []
    for step in range(8):
        print(f"plan flip run: step {step}, context {start + step + 1}", flush=True)
        n0 = lib.tw_kv_decode_fused_launches()
        engines[1].decode_step(q, k, v, outs[1], use_graph=False)
        one_launch_steps.append(lib.tw_kv_decode_fused_launches() - n0 == L)
        engines[0].decode_step(q, k, v, outs[0], use_graph=True)
        assert engines[0].graph_state() == 1
        torch.cuda.synchronize()
        assert torch.isfinite(outs[0].float()).all()
        assert torch.equal(outs[0], outs[1]), f"step {step}: graph replay differs from the eager step"
    assert one_launch_steps[0] and not one_launch_steps[-1], f"no flip inside the run: {one_launch_steps}"
    assert host(engines[0].positions()).tolist() == [start + 8] * G
    for l in (0, L - 1):
        for x, y in zip(engines[0].cache(l), engines[1].cache(l)):
            assert torch.equal(x[:, start:start + 9], y[:, start:start + 9])


def test_trace_ranges_switch():
    """The roctx ranges: switching them on finds the library (or reports that there is none), steps run with them on
    and off, and the results do not depend on the switch."""
    import torch
    from triebwerk_amd import Engine, _lib
    lib = _lib.load()
    L, H, Hk, G, msl = 1, 16, 8, 2, 24
    eng = Engine(max_seq_len=msl, kv_bits=4)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    gt = torch.Generator(device="cuda"); gt.manual_seed(5)
    q = torch.randn((L, G, H * D), generator=gt, device="cuda", dtype=torch.float16)
    k = torch.randn((L, G, Hk * D), generator=gt, device="cuda", dtype=torch.float16)
    v = torch.randn((L, G, Hk * D), generator=gt, device="cuda", dtype=torch.float16)
    out = [torch.zeros_like(q) for _ in range(2)]
    rc = lib.tw_kv_set_trace_ranges(1)
    assert rc in (0, -1)
    eng.decode_step(q, k, v, out[0])
    assert lib.tw_kv_set_trace_ranges(0) == 0
    eng.set_positions([0] * G)
    eng.decode_step(q, k, v, out[1])
    torch.cuda.synchronize()
    assert torch.equal(out[0], out[1])
