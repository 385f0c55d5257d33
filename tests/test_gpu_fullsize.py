"""GPU parity at the benchmark's full sizes (one layer of each): batch 64, context 8192,
Qwen3-0.6B KV shape; the ragged paged case with contexts in [512, 8192]; the 2-bit case
with 32 query heads at context 4097.

The oracle is too slow to quantize 64 x 8192 tokens, so the cache is built on the GPU by
the T-token append and checked three ways: a few whole sequences against the oracle bit
for bit, every other sequence against the one it replicates (the same rows must give the
same bytes wherever they are written), and a checksum of the per-sequence checksums.
Attention is then checked for EVERY sequence against the oracle run over the cache the GPU
wrote, for both kernel families, and the two families against each other.
"""
import zlib

import numpy as np
import pytest

import gen
import parity_log

pytestmark = pytest.mark.gpu

TOL = 2e-3
D = 128


@pytest.fixture(scope="module")
def kv():
    import torch
    from triebwerk_amd import kvcache
    assert torch.cuda.is_available()
    yield kvcache
    kvcache.set_attention_variant(0)
    kvcache.set_num_splits(0)


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.cpu().numpy()


def rel_err_rows(got, want, against_oracle=True):
    """Per head vector; `against_oracle` False for comparisons of one GPU path with another (they have their own
    bars and stay out of the log of how much of the oracle tolerance was used)."""
    got = got.astype(np.float64).reshape(-1, D)
    want = want.astype(np.float64).reshape(-1, D)
    err = np.max(np.abs(got - want), axis=1) / np.max(np.abs(want), axis=1)
    if against_oracle:
        parity_log.record(err.max())
    return err


def build_target_cache(kv, rotation_fixture, bits, G, Hk, ctx, n_base):
    """The target shape's cache through the T-token append (kernels.cu:1482-1560), one sequence per call;
    sequence g replicates base sequence g % n_base.  Returns the base rows and the device arrays."""
    import torch
    kv_dim = Hk * D
    kvp = kv_dim * bits // 8
    msl = ctx
    r = gen.rng(900 + bits)
    rot = dev(rotation_fixture)
    base_k = [gen.kv_rows_with_outliers(r, (ctx, kv_dim), kv_dim)[0] for _ in range(n_base)]
    base_v = [gen.kv_rows_with_outliers(r, (ctx, kv_dim), kv_dim)[0] for _ in range(n_base)]   # BASELINE config 2's rows: K and V
    d_base_k = [dev(x) for x in base_k]
    d_base_v = [dev(x) for x in base_v]
    ck = torch.zeros((G, msl, kvp), dtype=torch.uint8, device="cuda")
    cv = torch.zeros_like(ck)
    kn = torch.zeros((G, msl, Hk), dtype=torch.float16, device="cuda")
    vn = torch.zeros_like(kn)
    tok = dev(np.arange(ctx, dtype=np.int32))
    for g in range(G):
        kv.launch_turbo_kv_quantize(ck[g], kn[g], d_base_k[g % n_base], rot, tok, msl, ctx, Hk, D, kv_dim, bits)
        kv.launch_turbo_kv_quantize(cv[g], vn[g], d_base_v[g % n_base], rot, tok, msl, ctx, Hk, D, kv_dim, bits)
    return r, rot, base_k, base_v, ck, cv, kn, vn


@pytest.mark.parametrize("bits", [4, 2])
def test_target_shape_decode_step_in_one_launch(kv, oracle, rotation_fixture, bits):
    """The benchmark's default path at its full size: one decode step of a layer as one kernel (batch 64, contexts
    8187..8191 + the appended token; cached and appended K and V rows with BASELINE config 2's outlier channels).
    Appended rows equal the oracle's bytes, every other byte of the cache is
    untouched, outputs within tolerance of the oracle and of the three-kernel path."""
    import torch
    G, H, Hk, ctx = 64, 16, 8, 8192
    kv_dim, q_dim = Hk * D, H * D
    msl = ctx
    r, rot, _, _, ck, cv, kn, vn = build_target_cache(kv, rotation_fixture, bits, G, Hk, ctx, n_base=4)
    before = [host(x).copy() for x in (ck, cv, kn, vn)]
    pos = (ctx - 1 - (np.arange(G) % 5)).astype(np.int32)       # the append overwrites row pos[g]
    q = gen.normal_f16(r, (G, q_dim))
    k = gen.kv_rows_with_outliers(r, (G, kv_dim), kv_dim)[0]; v = gen.kv_rows_with_outliers(r, (G, kv_dim), kv_dim)[0]
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    outs, caches = {}, {}
    for mode in (1, 2):
        c = [dev(x) for x in before]
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        kv.set_decode_fused(mode)
        try:
            kv.tw_turbo_append_attention_batch(out, dev(q), dev(k), dev(v), c[0], c[1], c[2], c[3], rot, scratch, dev(pos),
                                               msl, G, H, Hk, D, q_dim, kv_dim, bits)
        finally:
            kv.set_decode_fused(0)
        outs[mode] = host(out)
        caches[mode] = [host(x) for x in c]
        del c
    want_c = [x.copy() for x in before]
    oracle.turbo_kv_quantize_batch(want_c[0], want_c[2], k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(want_c[1], want_c[3], v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    for mode in (1, 2):
        for got, want_arr, what in zip(caches[mode], want_c, ("K codes", "V codes", "K norms", "V norms")):
            assert np.array_equal(got.view(np.uint8), want_arr.view(np.uint8)), f"mode {mode}: {what}"
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, want_c[0], want_c[1], want_c[2], want_c[3], rotation_fixture, pos, msl, G,
                                     H, Hk, D, q_dim, kv_dim, bits)
    for mode in (1, 2):
        err = rel_err_rows(outs[mode], want)
        assert err.max() <= TOL, f"mode {mode}: max rel err {err.max():.3e} at head vector {err.argmax()}"
    assert rel_err_rows(outs[1], outs[2], against_oracle=False).max() <= TOL


@pytest.mark.parametrize("bits", [4, 2])
def test_target_shape_append_and_attention(kv, oracle, rotation_fixture, bits):
    import torch
    G, H, Hk, ctx = 64, 16, 8, 8192
    kv_dim, q_dim = Hk * D, H * D
    kvp = kv_dim * bits // 8
    msl = ctx
    n_base = 4                                   # distinct sequences; sequence g replicates g % n_base
    r, rot, base_k, base_v, ck, cv, kn, vn = build_target_cache(kv, rotation_fixture, bits, G, Hk, ctx, n_base)
    h_ck, h_cv, h_kn, h_vn = host(ck), host(cv), host(kn), host(vn)

    # (1) base sequences against the oracle, every byte
    for b in range(n_base):
        for rows, codes, norms, what in ((base_k[b], h_ck[b], h_kn[b], "K"), (base_v[b], h_cv[b], h_vn[b], "V")):
            oq = np.zeros((msl, kvp), np.uint8); on = np.zeros((msl, Hk), np.float16)
            oracle.turbo_kv_quantize(oq, on, rows, rotation_fixture, np.arange(ctx, dtype=np.int32), msl, ctx, Hk, D,
                                     kv_dim, bits)
            assert np.array_equal(codes, oq), f"{what} codes of sequence {b}: {(codes != oq).sum()} bytes differ"
            assert np.array_equal(norms.view(np.uint16), on.view(np.uint16)), f"{what} norms of sequence {b}"
    # (2) replicas equal their base; (3) checksum of checksums over the whole cache
    sums = []
    for g in range(G):
        b = g % n_base
        assert np.array_equal(h_ck[g], h_ck[b]) and np.array_equal(h_cv[g], h_cv[b]), f"sequence {g} != its base {b}"
        assert np.array_equal(h_kn[g].view(np.uint16), h_kn[b].view(np.uint16))
        assert np.array_equal(h_vn[g].view(np.uint16), h_vn[b].view(np.uint16))
        sums.append(zlib.crc32(h_ck[g].tobytes()) ^ zlib.crc32(h_cv[g].tobytes()))
    base_sums = [sums[b] for b in range(n_base)]
    assert zlib.crc32(np.array(sums, np.uint32).tobytes()) == \
        zlib.crc32(np.array([base_sums[g % n_base] for g in range(G)], np.uint32).tobytes())

    # attention over the whole batch, every sequence with its own query and (ragged by a few) position
    q = gen.normal_f16(r, (G, q_dim))
    pos = (ctx - 1 - (np.arange(G) % 5)).astype(np.int32)
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, h_ck, h_cv, h_kn, h_vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim,
                                     kv_dim, bits)
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    outs = {}
    for variant in (0, 1, 3):
        kv.set_attention_variant(variant)
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        kv.launch_turbo_gqa_attention_batch(out, dev(q), ck, cv, kn, vn, rot, scratch, dev(pos), msl, G, H, Hk, D,
                                            q_dim, kv_dim, bits)
        outs[variant] = host(out)
        err = rel_err_rows(outs[variant], want)
        assert err.max() <= TOL, f"variant {variant}: max rel err {err.max():.3e} at head vector {err.argmax()}"
    kv.set_attention_variant(0)
    cross = rel_err_rows(outs[0], outs[1], against_oracle=False)
    assert cross.max() <= TOL, f"MFMA vs vector-ALU kernels: {cross.max():.3e}"
    # same cache and query in two batch slots give the same output bits (no dependence on placement)
    q2 = q.copy(); q2[n_base:2 * n_base] = q2[:n_base]
    pos2 = pos.copy(); pos2[n_base:2 * n_base] = pos2[:n_base]
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    kv.launch_turbo_gqa_attention_batch(out, dev(q2), ck, cv, kn, vn, rot, scratch, dev(pos2), msl, G, H, Hk, D,
                                        q_dim, kv_dim, bits)
    o = host(out)
    assert np.array_equal(o[:n_base].view(np.uint16), o[n_base:2 * n_base].view(np.uint16))


def test_target_shape_fp16_cache(kv, oracle):
    """The 16-bit figure of the metric is quoted at batch 64 x context 8192: the whole batch in one launch (and the
    append + attention call of the engine path), every sequence against the oracle -- in four passes of 16
    sequences, which bounds the host memory the oracle's copy of the cache needs."""
    import torch
    G, H, Hk, ctx = 64, 16, 8, 8192
    kv_dim, q_dim = Hk * D, H * D
    msl = ctx
    r = gen.rng(950)
    g_ = torch.Generator(device="cuda"); g_.manual_seed(951)
    ck = torch.randn((G, msl, kv_dim), generator=g_, device="cuda", dtype=torch.float16)
    cv = torch.randn((G, msl, kv_dim), generator=g_, device="cuda", dtype=torch.float16)
    pos = (ctx - 1 - (np.arange(G) % 3)).astype(np.int32)
    k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim)); q = gen.normal_f16(r, (G, q_dim))
    kv.launch_kv_cache_write_batch(ck, cv, dev(k), dev(v), dev(pos), msl, G, kv_dim)
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    kv.launch_gqa_attention_batch(out, dev(q), ck, cv, scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    got = host(out)
    # the engine path: append inside the attention launch, on a cache whose appended rows were wiped
    for g in range(G):
        ck[g, pos[g]] = 0; cv[g, pos[g]] = 0
    out2 = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    kv.tw_append_attention_batch(out2, dev(q), dev(k), dev(v), ck, cv, scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    got2 = host(out2)
    worst = 0.0
    for g0 in range(0, G, 16):
        sl = slice(g0, g0 + 16)
        h_ck, h_cv = host(ck[sl]), host(cv[sl])
        for i, g in enumerate(range(g0, g0 + 16)):   # appended rows land where they should
            assert np.array_equal(h_ck[i, pos[g]].view(np.uint16), k[g].view(np.uint16))
            assert np.array_equal(h_cv[i, pos[g]].view(np.uint16), v[g].view(np.uint16))
        want = np.zeros((16, q_dim), np.float16)
        oracle.gqa_attention_batch(want, q[sl], h_ck, h_cv, pos[sl], msl, 16, H, Hk, D, q_dim, kv_dim)
        for name, o in (("attention launcher", got[sl]), ("append + attention call", got2[sl])):
            err = rel_err_rows(o, want)
            worst = max(worst, float(err.max()))
            assert err.max() <= TOL, f"{name}, sequences {g0}..{g0 + 15}: max rel err {err.max():.3e}"
    print(f"fp16 cache, batch 64 x 8192: max rel err {worst:.2e}")


@pytest.mark.parametrize("H,Hk", [(16, 8), (32, 16)])
@pytest.mark.parametrize("lens", [[8191, 8190, 8189, 8191, 8188], [8191, 7000, 4099, 100, 1]])
def test_fp16_small_batch_long_context(kv, oracle, lens, H, Hk):
    """Five sequences of up to 8192 tokens over the fp16 cache: the whole-row scan with its 64 chunks per sequence
    (equal lengths) or its balanced walk (ragged), and the merge over up to 64 partials per head, with the append
    inside the launch.  With 16 KV heads a sequence's chunks are two workgroups' work each, more items than the grid
    holds at once, and there is no balanced walk."""
    import torch
    G, msl = len(lens), 8192
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(960 + lens[1] % 7)
    ck, cv = gen.normal_f16(r, (G, msl, kv_dim)), gen.normal_f16(r, (G, msl, kv_dim))
    pos = np.array(lens, np.int32)
    for g in range(G):
        ck[g, pos[g]:] = 0; cv[g, pos[g]:] = 0
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    d_ck, d_cv = dev(ck), dev(cv)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.tw_append_attention_batch(out, dev(q), dev(k), dev(v), d_ck, d_cv, scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    assert kv.last_scan_kernel() == "attention_rows_kernel"
    oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
    want = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    assert np.array_equal(host(d_ck).view(np.uint16), ck.view(np.uint16)) and np.array_equal(host(d_cv).view(np.uint16), cv.view(np.uint16))
    err = rel_err_rows(host(out), want)
    assert err.max() <= TOL, f"max rel err {err.max():.3e} (per sequence {err})"


@pytest.mark.parametrize("bits", [4, 2])
def test_ragged_paged_batch64(kv, oracle, rotation_fixture, bits):
    """Contexts uniform in [512, 8192], 16-token pages in random order."""
    import torch
    G, H, Hk = 64, 16, 8
    kv_dim, q_dim = Hk * D, H * D
    kvp = kv_dim * bits // 8
    r = gen.rng(960 + bits)
    lens = gen.ragged_contexts(r, G, 512, 8192)
    lens[0], lens[1] = 512, 8192
    pages_per_seq = 8192 // 16
    msl = pages_per_seq * 16
    bt = gen.shuffled_block_table(r, G, pages_per_seq)
    n_pages = G * pages_per_seq
    g_ = torch.Generator(device="cuda"); g_.manual_seed(961)
    p_ck = torch.randint(0, 256, (n_pages, 16, kvp), generator=g_, device="cuda", dtype=torch.uint8)
    p_cv = torch.randint(0, 256, (n_pages, 16, kvp), generator=g_, device="cuda", dtype=torch.uint8)
    p_kn = (11.3 + 0.7 * torch.randn((n_pages, 16, Hk), generator=g_, device="cuda")).to(torch.float16)
    p_vn = (11.3 + 0.7 * torch.randn((n_pages, 16, Hk), generator=g_, device="cuda")).to(torch.float16)
    rot = dev(rotation_fixture)
    # one appended token per sequence through the paged append, then attention
    pos = (lens - 1).astype(np.int32)
    k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim)); q = gen.normal_f16(r, (G, q_dim))
    d_bt = dev(bt)
    kv.tw_paged_turbo_kv_append_batch(p_ck, p_kn, p_cv, p_vn, dev(k), dev(v), rot, dev(pos), d_bt, pages_per_seq, G,
                                      Hk, D, kv_dim, bits)
    idx = torch.from_numpy(bt.astype(np.int64)).cuda()

    def gather(pool):                            # pages in block-table order = the contiguous layout
        return host(pool[idx].reshape(G, msl, pool.shape[-1]))
    ck, cv, kn, vn = gather(p_ck), gather(p_cv), gather(p_kn), gather(p_vn)
    # the appended rows equal the oracle's contiguous append, bit for bit
    ock, ocv, okn, ovn = ck.copy(), cv.copy(), kn.copy(), vn.copy()
    for g in range(G):
        ock[g, pos[g]] = 0; ocv[g, pos[g]] = 0; okn[g, pos[g]] = 0; ovn[g, pos[g]] = 0
    oracle.turbo_kv_quantize_batch(ock, okn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(ocv, ovn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    assert np.array_equal(ck, ock) and np.array_equal(cv, ocv)
    assert np.array_equal(kn.view(np.uint16), okn.view(np.uint16)) and np.array_equal(vn.view(np.uint16), ovn.view(np.uint16))
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    ws = torch.zeros(kv.attention_workspace_floats(G, H, msl), dtype=torch.float32, device="cuda")
    for variant in (0, 1, 3):
        kv.set_attention_variant(variant)
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        kv.tw_paged_turbo_gqa_attention_batch(out, dev(q), p_ck, p_cv, p_kn, p_vn, rot, ws, dev(pos), d_bt,
                                              pages_per_seq, msl, G, H, Hk, D, q_dim, kv_dim, bits)
        err = rel_err_rows(host(out), want)
        assert err.max() <= TOL, f"variant {variant}: max rel err {err.max():.3e} (sequence {err.argmax() // H})"
    kv.set_attention_variant(0)
    # the layer step in one call (append + attention, three launches): the appended rows are wiped first, so the
    # call has to write them again -- same bytes through the block-table gather, same outputs
    for g in range(G):
        page, slot = int(bt[g, pos[g] // 16]), int(pos[g] % 16)
        for pool in (p_ck, p_cv, p_kn, p_vn):
            pool[page, slot] = 0
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    kv.tw_paged_turbo_append_attention_batch(out, dev(q), dev(k), dev(v), p_ck, p_cv, p_kn, p_vn, rot, ws, dev(pos), d_bt,
                                             pages_per_seq, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert np.array_equal(gather(p_ck), ock) and np.array_equal(gather(p_cv), ocv)
    assert np.array_equal(gather(p_kn).view(np.uint16), okn.view(np.uint16))
    assert np.array_equal(gather(p_vn).view(np.uint16), ovn.view(np.uint16))
    err = rel_err_rows(host(out), want)
    assert err.max() <= TOL, f"one call: max rel err {err.max():.3e} (sequence {err.argmax() // H})"


def test_tq2_gqa4_context4097(kv, oracle, rotation_fixture):
    """2-bit codes, 32 query heads on 8 KV heads, batch 16, context 4096 + 1."""
    import torch
    bits, G, H, Hk, ctx = 2, 16, 32, 8, 4097
    kv_dim, q_dim = Hk * D, H * D
    kvp = kv_dim * bits // 8
    msl = ctx
    r = gen.rng(970)
    g_ = torch.Generator(device="cuda"); g_.manual_seed(971)
    ck = torch.randint(0, 256, (G, msl, kvp), generator=g_, device="cuda", dtype=torch.uint8)
    cv = torch.randint(0, 256, (G, msl, kvp), generator=g_, device="cuda", dtype=torch.uint8)
    kn = (11.3 + 0.7 * torch.randn((G, msl, Hk), generator=g_, device="cuda")).to(torch.float16)
    vn = (11.3 + 0.7 * torch.randn((G, msl, Hk), generator=g_, device="cuda")).to(torch.float16)
    rot = dev(rotation_fixture)
    pos = np.full(G, ctx - 1, np.int32)
    k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim)); q = gen.normal_f16(r, (G, q_dim))
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    kv.tw_turbo_append_attention_batch(out, dev(q), dev(k), dev(v), ck, cv, kn, vn, rot, scratch, dev(pos), msl, G, H,
                                       Hk, D, q_dim, kv_dim, bits)
    h_ck, h_cv, h_kn, h_vn = host(ck), host(cv), host(kn), host(vn)
    ock, ocv, okn, ovn = h_ck.copy(), h_cv.copy(), h_kn.copy(), h_vn.copy()
    ock[:, ctx - 1] = 0; ocv[:, ctx - 1] = 0; okn[:, ctx - 1] = 0; ovn[:, ctx - 1] = 0
    oracle.turbo_kv_quantize_batch(ock, okn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(ocv, ovn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    assert np.array_equal(h_ck, ock) and np.array_equal(h_cv, ocv)
    assert np.array_equal(h_kn.view(np.uint16), okn.view(np.uint16)) and np.array_equal(h_vn.view(np.uint16), ovn.view(np.uint16))
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ock, ocv, okn, ovn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    err = rel_err_rows(host(out), want)
    assert err.max() <= TOL, f"max rel err {err.max():.3e}"


@pytest.mark.parametrize("bits", [4, 2])
def test_extremely_ragged_batch(kv, oracle, rotation_fixture, bits):
    """Lengths from 1 token to 8192 in one batch of 100: the scan cuts such a batch by tiles, not
    by sequence, and a sequence's partials come from a varying number of wave groups."""
    import torch
    G, H, Hk = 100, 16, 8
    kv_dim, q_dim = Hk * D, H * D
    kvp = kv_dim * bits // 8
    msl = 8192
    r = gen.rng(980 + bits)
    lens = np.concatenate([np.array([1, 2, 31, 32, 33, 63, 64, 65, 8192, 8191, 4097, 1000]),
                           r.integers(1, 300, size=G - 12)]).astype(np.int32)
    r.shuffle(lens)
    g_ = torch.Generator(device="cuda"); g_.manual_seed(981 + bits)
    ck = torch.randint(0, 256, (G, msl, kvp), generator=g_, device="cuda", dtype=torch.uint8)
    cv = torch.randint(0, 256, (G, msl, kvp), generator=g_, device="cuda", dtype=torch.uint8)
    kn = (11.3 + 0.7 * torch.randn((G, msl, Hk), generator=g_, device="cuda")).to(torch.float16)
    vn = (11.3 + 0.7 * torch.randn((G, msl, Hk), generator=g_, device="cuda")).to(torch.float16)
    rot = dev(rotation_fixture)
    pos = (lens - 1).astype(np.int32)
    q = gen.normal_f16(r, (G, q_dim))
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, host(ck), host(cv), host(kn), host(vn), rotation_fixture, pos, msl, G, H, Hk,
                                     D, q_dim, kv_dim, bits)
    scratch = torch.full((G * H * msl,), float("nan"), dtype=torch.float32, device="cuda")   # nothing may rely on its content
    for variant in (0, 1, 3):
        kv.set_attention_variant(variant)
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        kv.launch_turbo_gqa_attention_batch(out, dev(q), ck, cv, kn, vn, rot, scratch, dev(pos), msl, G, H, Hk, D,
                                            q_dim, kv_dim, bits)
        err = rel_err_rows(host(out), want)
        assert err.max() <= TOL, f"variant {variant}: max rel err {err.max():.3e} (sequence {err.argmax() // H}, length {lens[err.argmax() // H]})"
    kv.set_attention_variant(0)


@pytest.mark.parametrize("H,T", [(16, 2500), (16, 5000), (32, 4100)])
def test_fp16_prefill_long_prompts_kernel_families_agree(kv, H, T):
    """Prompt lengths at which the matrix-core prefill kernel switches to mirrored block pairs and to two
    query blocks per wave, against the vector-ALU kernel (which the small cases pin to the oracle):
    both within the attention tolerance of each other, row by row."""
    import torch
    Hk = 8
    kv_dim, q_dim = Hk * D, H * D
    g_ = torch.Generator(device="cuda"); g_.manual_seed(990 + T)
    q = torch.randn((T, q_dim), generator=g_, device="cuda").to(torch.float16)
    ck = torch.randn((T, kv_dim), generator=g_, device="cuda").to(torch.float16)
    cv = torch.randn((T, kv_dim), generator=g_, device="cuda").to(torch.float16)
    ck[T - 2] *= 5
    scratch = torch.zeros(H * T * 1024, dtype=torch.float32, device="cuda")
    outs = []
    for variant in (0, 1):
        kv.set_attention_variant(variant)
        try:
            out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
            kv.launch_gqa_prefill_attention(out, q, ck, cv, scratch, T, T, H, Hk, D, q_dim, kv_dim)
            outs.append(host(out))
        finally:
            kv.set_attention_variant(0)
    err = rel_err_rows(outs[0], outs[1], against_oracle=False)
    assert err.max() <= TOL, f"max rel err {err.max():.3e} at row {err.argmax() // H}"


@pytest.mark.parametrize("bits", [4, 2])
def test_compressed_prefill_8192_tokens(kv, oracle, rotation_fixture, bits):
    """A prompt of 8192 tokens over the compressed cache (16 heads over 8 KV heads): the cache comes from the
    T-token append, the matrix-core prompt kernel (one launch: query rotation, attention, rotation back) is
    compared row by row with the vector-ALU kernel, and rows at the ends, at tile and block borders and in
    the middle with the oracle's decode attention at that position over the same cache (prefill row t is
    decode at position t, kernels.cu:1874-1960 against 1641-1870)."""
    import torch
    H, Hk, T = 16, 8, 8192
    kv_dim, q_dim = Hk * D, H * D
    r, rot, base_k, base_v, ck, cv, kn, vn = build_target_cache(kv, rotation_fixture, bits, 1, Hk, T, 1)
    q = gen.normal_f16(r, (T, q_dim))
    d_q = dev(q)
    scratch = torch.full((H * T * 1024,), float("nan"), dtype=torch.float32, device="cuda")
    outs = []
    for variant in (0, 1):
        kv.set_attention_variant(variant)
        try:
            out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
            kv.launch_turbo_gqa_prefill_attention(out, d_q, ck[0], cv[0], kn[0], vn[0], rot, scratch, T, T, H, Hk, D,
                                                  q_dim, kv_dim, bits)
            outs.append(host(out))
        finally:
            kv.set_attention_variant(0)
        if variant == 0:
            assert bool(torch.isnan(scratch).all()), "the prompt kernel keeps nothing in the scratch"
    err = rel_err_rows(outs[0], outs[1], against_oracle=False)
    assert err.max() <= 2 * TOL, f"kernel families: max rel err {err.max():.3e} at row {err.argmax() // H}"
    h_ck, h_cv, h_kn, h_vn = host(ck[0]), host(cv[0]), host(kn[0]), host(vn[0])
    for t in (0, 1, 31, 32, 63, 64, 1000, 4095, 4096, 6143, 8190, 8191):
        want = np.zeros(q_dim, np.float16)
        oracle.turbo_gqa_attention(q[t], h_ck, h_cv, h_kn, h_vn, rotation_fixture, want, t, T, H, Hk, D, bits)
        for name, got in (("matrix-core", outs[0][t]), ("vector-ALU", outs[1][t])):
            e = rel_err_rows(got, want).max()
            assert e <= TOL, f"{name} kernel, row {t}: rel err {e:.3e}"


@pytest.mark.parametrize("bits,T", [(4, 4100), (2, 8200)])
def test_compressed_prefill_per_wave_kernel_long_prompt(kv, rotation_fixture, bits, T):
    """The prompt kernel that expands tiles per wave (form 4) keeps the three-launch shape: query rotation,
    scan with partials, merge + rotate-back.  At these lengths its two small kernels walk several tiles per
    wave / workgroup (more than 2048 tiles of 16 vectors); its output must agree row by row with the
    one-launch kernel, which the test above pins to the oracle."""
    import torch
    H, Hk = 16, 8
    kv_dim, q_dim = Hk * D, H * D
    r, rot, base_k, base_v, ck, cv, kn, vn = build_target_cache(kv, rotation_fixture, bits, 1, Hk, T, 1)
    d_q = dev(gen.normal_f16(r, (T, q_dim)))
    scratch = torch.zeros(H * T * 1024, dtype=torch.float32, device="cuda")
    outs = []
    for form in (0, 4):
        kv.set_prefill_form(form)
        try:
            out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
            kv.launch_turbo_gqa_prefill_attention(out, d_q, ck[0], cv[0], kn[0], vn[0], rot, scratch, T, T, H, Hk, D,
                                                  q_dim, kv_dim, bits)
            outs.append(host(out))
        finally:
            kv.set_prefill_form(0)
    assert outs[1].any()
    err = rel_err_rows(outs[0], outs[1], against_oracle=False)
    assert err.max() <= 2 * TOL, f"max rel err {err.max():.3e} at row {err.argmax() // H}"


@pytest.mark.parametrize("bits", [4, 2])
def test_prompt_step_8192_tokens_same_cache_and_output(kv, rotation_fixture, bits):
    """tw_layer_prompt_step over 8192 tokens (K and V rows appended in one launch, 131072 vectors) leaves the
    bytes that two launch_turbo_kv_quantize calls leave (pinned to the oracle above and in the small cases),
    and the output of the prefill launcher on that cache."""
    import torch
    H, Hk, T = 16, 8, 8192
    kv_dim, q_dim = Hk * D, H * D
    r, rot, base_k, base_v, ck, cv, kn, vn = build_target_cache(kv, rotation_fixture, bits, 1, Hk, T, 1)
    q = dev(gen.normal_f16(r, (T, q_dim)))
    scratch = torch.zeros(H * T * 1024, dtype=torch.float32, device="cuda")
    want = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    kv.launch_turbo_gqa_prefill_attention(want, q, ck[0], cv[0], kn[0], vn[0], rot, scratch, T, T, H, Hk, D, q_dim, kv_dim, bits)
    ck2, cv2, kn2, vn2 = torch.zeros_like(ck[0]), torch.zeros_like(cv[0]), torch.zeros_like(kn[0]), torch.zeros_like(vn[0])
    out = torch.zeros_like(want)
    pos = dev(np.arange(T, dtype=np.int32))
    kv.tw_layer_prompt_step(out, q, dev(base_k[0]), dev(base_v[0]), pos, T, T, H, Hk, D, q_dim, kv_dim, ck2, cv2, scratch,
                            kv_bits=bits, k_norms=kn2, v_norms=vn2, rotation=rot)
    for name, a, b in (("K codes", ck2, ck[0]), ("V codes", cv2, cv[0]), ("K norms", kn2, kn[0]), ("V norms", vn2, vn[0]),
                       ("output", out, want)):
        assert torch.equal(a, b), name
