"""The entry point that allocates nothing (tw_turbo_gqa_attention_batch_noalloc), through the C ABI,
against the entry point it is a variant of (launch_turbo_gqa_attention_batch) and against the CPU oracle.

Two calls in a row share the library's device array; the second is smaller, so it runs over what the first
left there.  Bars: attention outputs within 2e-3 of the oracle (per head vector, ||gpu - oracle||_inf /
||oracle||_inf) and -- the array gives every (sequence, head) the room the caller's scratch would, so both entry
points make the same plan -- equal to the existing entry point's output bit for bit.
"""
import numpy as np
import pytest

import gen
from test_gpu_parity import D, TOL, build_turbo_cache, dev, host, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kv():
    import torch
    from triebwerk_amd import kvcache
    assert torch.cuda.is_available()
    return kvcache


def _case(kv, oracle, rot, seed, bits, H, Hk, lens, msl):
    import torch
    r = gen.rng(seed)
    G = len(lens)
    kv_dim, q_dim = Hk * D, H * D
    ck, cv, kn, vn = build_turbo_cache(oracle, rot, r, G, Hk, msl, lens, bits, outliers=False)
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.array(lens, np.int32) - 1
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rot, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    d = [dev(x) for x in (q, ck, cv, kn, vn, rot, pos)]
    ref = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.launch_turbo_gqa_attention_batch(ref, d[0], d[1], d[2], d[3], d[4], d[5], scratch, d[6], msl, G, H, Hk, D,
                                        q_dim, kv_dim, bits)
    out = torch.full((G, q_dim), float("nan"), dtype=torch.float16, device="cuda")
    print(f"noalloc case seed={seed} bits={bits} G={G} H={H} Hk={Hk} msl={msl}", flush=True)
    kv.tw_turbo_gqa_attention_batch_noalloc(out, d[0], d[1], d[2], d[3], d[4], d[5], d[6], msl, G, H, Hk, D, q_dim,
                                            kv_dim, bits)
    got, ref = host(out), host(ref)
    assert rel_err(got, want) <= TOL
    assert rel_err(ref, want) <= TOL
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), "differs from launch_turbo_gqa_attention_batch"


@pytest.mark.parametrize("bits,H,Hk", [(4, 16, 8), (2, 32, 8)])
def test_noalloc_two_calls_second_smaller(kv, oracle, rotation_fixture, bits, H, Hk):
    big = [1536, 1000, 257, 129, 64, 33, 1200, 1535]
    small = [300, 17, 640]
    _case(kv, oracle, rotation_fixture, 9100 + bits, bits, H, Hk, big, 1536)
    _case(kv, oracle, rotation_fixture, 9200 + bits, bits, H, Hk, small, 640)


def test_noalloc_allocates_nothing_and_replays_from_a_graph(kv, oracle, rotation_fixture):
    """What the entry point is for: after the first call on the GPU has looked the array up, a call leaves the free
    device memory as it was, and a call recorded into a graph on a side stream replays -- several times, with eager
    work of the program in between -- to the eager call's bits."""
    import torch
    bits, H, Hk, msl = 4, 16, 8, 512
    lens = [512, 300, 77, 401]
    G = len(lens)
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(9301)
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits, outliers=False)
    d = [dev(x) for x in (ck, cv, kn, vn, rotation_fixture, np.array(lens, np.int32) - 1)]
    dq = dev(gen.normal_f16(r, (G, q_dim)))
    eager = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    replayed = torch.zeros_like(eager)

    def call(out, stream=None):
        kv.tw_turbo_gqa_attention_batch_noalloc(out, dq, d[0], d[1], d[2], d[3], d[4], d[5], msl, G, H, Hk, D, q_dim, kv_dim,
                                                bits, stream=stream)
    call(eager)                                   # first call on this GPU: looks the array up
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    call(eager)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "a call changed the free device memory"
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, host(dq), ck, cv, kn, vn, rotation_fixture, host(d[5]), msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert rel_err(host(eager), want) <= TOL
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        call(replayed, stream=side)
    for rep in range(3):
        replayed.zero_()
        dq.copy_(dev(gen.normal_f16(r, (G, q_dim))))          # the program's own eager work between the replays
        call(eager)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(replayed, eager), f"replay {rep} differs from the eager call"


def test_noalloc_return_value_is_the_calls_own(kv, oracle, rotation_fixture):
    """An error that an earlier call left uncleared on the thread does not turn a good call into a failure or hide a
    bad call's message (raw ctypes: the Python wrappers clear the error after every call)."""
    import torch
    from triebwerk_amd import _lib
    lib = _lib.load()
    bits, H, Hk, msl = 4, 16, 8, 128
    lens = [128, 40]
    G = len(lens)
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(9302)
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits, outliers=False)
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.array(lens, np.int32) - 1
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    d = [dev(x) for x in (q, ck, cv, kn, vn, rotation_fixture, pos)]
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    args = [x.data_ptr() for x in d]
    lib.tw_kv_clear_error()
    try:
        # a validation error (bits = 3), left uncleared
        lib.launch_turbo_gqa_attention_batch(out.data_ptr(), *args[:6], None, args[6], msl, G, H, Hk, D, q_dim, kv_dim, 3, s)
        assert lib.tw_kv_last_error() != 0 and b"bits=3" in lib.tw_kv_last_error_string()
        rc = lib.tw_turbo_gqa_attention_batch_noalloc(out.data_ptr(), *args, msl, G, H, Hk, D, q_dim, kv_dim, bits, s)
        assert rc == 0, "a good call reported the earlier call's error"
        assert rel_err(host(out), want) <= TOL
        assert b"bits=3" in lib.tw_kv_last_error_string(), "the earlier error is still the thread's"
        rc = lib.tw_turbo_gqa_attention_batch_noalloc(out.data_ptr(), *args, msl, 2048, H, Hk, D, q_dim, kv_dim, bits, s)
        assert rc != 0 and b"exceeds" in lib.tw_kv_last_error_string()
    finally:
        lib.tw_kv_clear_error()


def test_noalloc_less_room_than_max_seq_len(kv, oracle):
    """16384 (sequence, head) pairs share the array: 512 floats each where max_seq_len is 2048, so the plan has to fit
    two partials and the query.  Random cache bytes (any bytes are a valid cache), ragged lengths with a few long
    sequences; against the oracle on every sequence, equal to a second call bit for bit, and within the tolerance of
    launch_turbo_gqa_attention_batch -- which has max_seq_len floats per pair, plans more pieces for the long
    sequences, and therefore need not give the same bits."""
    import torch
    bits, H, Hk, msl, G = 4, 16, 8, 2048, 1024
    kv_dim, q_dim, kvp = Hk * D, H * D, Hk * D * bits // 8
    r = gen.rng(9303)
    lens = r.integers(1, 200, size=G)
    lens[::97] = r.integers(1500, msl + 1, size=len(lens[::97]))
    lens[5] = msl; lens[6] = 1
    pos = (lens - 1).astype(np.int32)
    ck = r.integers(0, 256, (G, msl, kvp), dtype=np.uint8); cv = r.integers(0, 256, (G, msl, kvp), dtype=np.uint8)
    kn = (11.3 + 0.7 * r.standard_normal((G, msl, Hk))).astype(np.float16)
    vn = (11.3 + 0.7 * r.standard_normal((G, msl, Hk))).astype(np.float16)
    rot, _ = oracle.make_rotation(128, 42)
    q = gen.normal_f16(r, (G, q_dim))
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rot, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    d = [dev(x) for x in (q, ck, cv, kn, vn, rot, pos)]
    outs = [torch.full((G, q_dim), float("nan"), dtype=torch.float16, device="cuda") for _ in range(2)]
    print(f"noalloc case room < msl: G={G} H={H} msl={msl}", flush=True)
    for o in outs:
        kv.tw_turbo_gqa_attention_batch_noalloc(o, d[0], d[1], d[2], d[3], d[4], d[5], d[6], msl, G, H, Hk, D, q_dim, kv_dim, bits)
    ref = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.launch_turbo_gqa_attention_batch(ref, d[0], d[1], d[2], d[3], d[4], d[5], scratch, d[6], msl, G, H, Hk, D, q_dim, kv_dim, bits)
    got = host(outs[0])
    assert rel_err(got, want) <= TOL
    assert torch.equal(outs[0], outs[1]), "two calls on the same inputs differ"
    assert rel_err(host(ref), want) <= TOL and rel_err(got, host(ref)) <= TOL


def test_noalloc_rejects_what_the_array_cannot_serve(kv):
    """More (sequence, head) pairs than the array serves: a clear error, nothing launched (the arguments are
    never dereferenced, so small stand-in tensors do)."""
    import torch
    t16 = torch.zeros(8, dtype=torch.float16, device="cuda")
    t8 = torch.zeros(8, dtype=torch.uint8, device="cuda")
    ti = torch.zeros(8, dtype=torch.int32, device="cuda")
    G, H, Hk = 2048, 16, 8          # 32768 pairs > 16384
    with pytest.raises(RuntimeError, match="exceeds"):
        kv.tw_turbo_gqa_attention_batch_noalloc(t16, t16, t8, t8, t16, t16, t16, ti, 64, G, H, Hk, D, H * D, Hk * D, 4)
    torch.cuda.synchronize()
    assert float(t16.abs().sum()) == 0.0
