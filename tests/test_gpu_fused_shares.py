"""The one-launch decode step with a sequence's context shared by two or four workgroups (small batches, whose
(sequence, head group) units alone leave compute units idle): through tw_layer_attention_step with tickets, every
combination of heads per workgroup and shares, against the CPU oracle -- appended rows bit for bit, outputs within 2e-3
per head vector -- and launch after launch on the same tickets (each launch must leave them zero).
"""
import numpy as np
import pytest

import gen
from test_gpu_parity import D, TOL, assert_bytes_equal, build_turbo_cache, dev, host, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kv():
    import torch
    from triebwerk_amd import kvcache
    assert torch.cuda.is_available()
    yield kvcache
    kvcache.set_fused_shape(0, 0)
    kvcache.set_decode_fused(0)


@pytest.mark.parametrize("bits,H,Hk,G", [(4, 16, 8, 5), (2, 32, 8, 3), (4, 8, 8, 8), (2, 16, 8, 4), (4, 12, 3, 4)])
@pytest.mark.parametrize("hkw,shares", [(1, 2), (1, 4), (1, 8), (2, 2), (2, 4), (2, 8), (4, 4), (8, 2)])
def test_shared_context_step_against_the_oracle(kv, oracle, rotation_fixture, bits, H, Hk, G, hkw, shares):
    """Contexts that leave shares empty (fewer tiles than shares), that end on tile and share edges, and long ones;
    three steps in a row on the same tickets and scratch."""
    import torch
    if Hk % hkw:
        pytest.skip("heads per workgroup must divide the KV heads")
    msl = 1400
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(9500 + 10 * bits + H + hkw + shares)
    lens = ([0, 1, 31, 32, 33, 64, 95, 127, 128, 129, 255, 256, 257, 1023, 1024, 1300, msl - 3] * 2)
    lens = [lens[(3 * i + G + hkw) % len(lens)] for i in range(G)]
    lens[-1] = msl - 3
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits)
    d_c = [dev(x) for x in (ck, cv, kn, vn)]
    d_rot = dev(rotation_fixture)
    scratch = torch.full((G * H * msl,), float("nan"), dtype=torch.float32, device="cuda")
    tickets = torch.zeros(G * Hk, dtype=torch.int32, device="cuda")
    pos = np.array(lens, np.int32)
    lib = kv._lib.load()
    kv.set_decode_fused(1)
    kv.set_fused_shape(hkw, shares)
    try:
        for step in range(3):
            q = gen.normal_f16(r, (G, q_dim)); k = gen.kv_rows_with_outliers(r, (G, kv_dim), kv_dim)[0]; v = gen.normal_f16(r, (G, kv_dim))
            out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
            n0 = lib.tw_kv_decode_fused_launches()
            print(f"shared-context step bits={bits} H={H} Hk={Hk} G={G} hkw={hkw} shares={shares} step={step}", flush=True)
            kv.tw_layer_attention_step(out, dev(q), dev(k), dev(v), dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, d_c[0], d_c[1],
                                       scratch, kv_bits=bits, k_norms=d_c[2], v_norms=d_c[3], rotation=d_rot, tickets=tickets)
            assert lib.tw_kv_decode_fused_launches() == n0 + 1
            assert "context shared" in kv.last_scan_kernel()
            oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
            oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
            want = np.zeros((G, q_dim), np.float16)
            oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
            got = host(out)
            worst = [(rel_err(got[g], want[g]), g, int(pos[g])) for g in range(G)]
            assert max(worst)[0] <= TOL, f"step {step}: worst (error, sequence, position): {sorted(worst)[-3:]}"
            assert not host(tickets).any(), f"step {step}: tickets were not left zero"
            pos = pos + 1
    finally:
        kv.set_fused_shape(0, 0)
        kv.set_decode_fused(0)
    for got, want_arr, what in zip(d_c, (ck, cv, kn, vn), ("K codes", "V codes", "K norms", "V norms")):
        assert_bytes_equal(host(got), want_arr, what)


def test_shared_context_is_chosen_for_small_batches_and_is_deterministic(kv, oracle, rotation_fixture):
    """BASELINE config 4's shape with the library's own choice: the engine hands over tickets, the plan takes the one
    launch with shares, two runs from the same state give the same bits, and the result is the oracle's."""
    import torch
    from triebwerk_amd import Engine
    lib = kv._lib.load()
    L, H, Hk, G, bits, msl, ctx = 2, 32, 8, 16, 2, 4352, 4096
    kv_dim, q_dim = Hk * D, H * D
    assert lib.tw_kv_decode_step_plan2(G, H, Hk, bits, msl, ctx + 1, ctx + 1, 1) == 1
    eng = Engine(max_seq_len=msl, kv_bits=bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    gt = torch.Generator(device="cuda"); gt.manual_seed(41)
    for l in range(L):
        c = eng.cache(l)
        for i in range(2):
            c[i].view(torch.int32).copy_(torch.randint(-2 ** 31, 2 ** 31 - 1, tuple(c[i].view(torch.int32).shape), generator=gt,
                                                      device="cuda", dtype=torch.int32))
        for i in (2, 3):
            c[i].copy_((11.3 + 0.7 * torch.randn(c[i].shape, generator=gt, device="cuda")).to(torch.float16))
    q = torch.randn((L, G, q_dim), generator=gt, device="cuda", dtype=torch.float16)
    k = torch.randn((L, G, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
    v = torch.randn((L, G, kv_dim), generator=gt, device="cuda", dtype=torch.float16)
    outs = []
    for rep in range(2):
        eng.set_positions([ctx] * G)
        out = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
        eng.decode_step(q, k, v, out, use_graph=(rep == 1))
        torch.cuda.synchronize()
        assert "context shared" in kv.last_scan_kernel(), kv.last_scan_kernel()
        outs.append(out)
    assert torch.equal(outs[0], outs[1]), "two runs from the same state differ"
    rot = host(eng.rotation())
    pos = np.full(G, ctx, np.int32)
    for l in range(L):
        c = [host(t) for t in eng.cache(l)]
        want = np.zeros((G, q_dim), np.float16)
        oracle.turbo_gqa_attention_batch(want, host(q[l]), c[0], c[1], c[2], c[3], rot, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
        assert rel_err(host(outs[0][l]), want) <= TOL
