"""A seeded random sweep over the layer step's argument space (compressed caches): shapes, context mixes, kernel
forms, contexts shared by workgroups, producers, gate, host knowledge of the contexts.  Every case is checked like
the hand-picked ones: appended rows bit for bit, tickets back at zero, outputs within tolerance of the oracle."""
import numpy as np
import pytest

import gen
import test_gpu_parity as tp
from test_gpu_parity import kv  # noqa: F401  (fixture)

D = 128
pytestmark = pytest.mark.gpu


def draw_case(r):
    bits = int(r.choice([4, 2]))
    Hk = int(r.choice([1, 2, 4, 8, 8, 8]))
    R = int(r.choice([1, 2, 2, 4]))
    G = int(r.choice([1, 2, 3, 4, 7, 8, 16, 17, 33, 64]))
    msl = int(r.choice([40, 96, 300, 700, 1100]))
    G = min(G, max(1, (32 * 1100 * 8) // (msl * Hk * 4)))            # keeps the oracle's share of a case under a second
    kind = int(r.integers(0, 4))
    if kind == 0:
        lens = [int(x) for x in r.integers(0, msl - 1, size=G)]                                   # ragged
    elif kind == 1:
        lens = [int(r.integers(max(0, msl - 40), msl - 1))] * G                                    # uniform, long
    elif kind == 2:
        lens = [int(x) for x in r.integers(max(0, msl * 7 // 8 - 2), msl - 1, size=G)]            # nearly uniform
    else:
        lens = [int(r.integers(0, min(msl - 1, 70)))] * G                                          # uniform, short
    mode = int(r.choice([0, 0, 1, 2, 3]))
    with_tickets = bool(r.integers(0, 2))
    shape = None
    if mode in (0, 1) and with_tickets and r.integers(0, 2):
        shape = (int(r.choice([h for h in (1, 2, 4, 8) if h <= Hk])), int(r.choice([1, 2, 4, 8])))
    return dict(bits=bits, Hk=Hk, H=Hk * R, G=G, msl=msl, lens=lens, mode=mode, producers=bool(r.integers(0, 2)),
                gated=bool(r.integers(0, 2)), with_tickets=with_tickets, known=bool(r.integers(0, 2)), shape=shape,
                outliers=bool(r.integers(0, 2)))


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_layer_steps(kv, oracle, rotation_fixture, seed):
    import torch
    failures = []
    for case in range(25):
        r = gen.rng(700000 + 1000 * seed + case)
        c = draw_case(r)
        bits, Hk, H, G, msl, lens = c["bits"], c["Hk"], c["H"], c["G"], c["msl"], c["lens"]
        kv_dim, q_dim = Hk * D, H * D
        ck, cv, kn, vn = tp.build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits, outliers=c["outliers"])
        pos = np.array(lens, np.int32)
        q, k, qw, kw = tp.producer_inputs(r, G, H, Hk, q_dim, kv_dim)
        if not c["producers"]:
            q = gen.normal_f16(r, (G, q_dim))          # producer_inputs scales a row by 30 for the RMSNorm to undo
        v = gen.normal_f16(r, (G, kv_dim))
        gate = gen.normal_f16(r, (G, q_dim))
        ct, st = tp.rope_tables(msl, 128)
        d_ck, d_cv, d_kn, d_vn = tp.dev(ck), tp.dev(cv), tp.dev(kn), tp.dev(vn)
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        scratch = torch.zeros(G * H * msl + 8 * 132 * G * H, dtype=torch.float32, device="cuda")
        tickets = torch.zeros(G * Hk, dtype=torch.int32, device="cuda") if c["with_tickets"] else None
        kw_args = dict(kv_bits=bits, k_norms=d_kn, v_norms=d_vn, rotation=tp.dev(rotation_fixture), tickets=tickets)
        if c["producers"]:
            kw_args.update(q_weight=tp.dev(qw), k_weight=tp.dev(kw), eps=1e-6, cos_table=tp.dev(ct), sin_table=tp.dev(st), rope_dim=128)
        if c["gated"]:
            kw_args.update(gate=tp.dev(gate), gate_stride=q_dim)
        if c["known"]:
            kw_args.update(ctx_min=min(lens) + 1, ctx_max=max(lens) + 1)
        kv.set_decode_fused(c["mode"])
        if c["shape"]:
            kv.set_fused_shape(*c["shape"])
        try:
            kv.tw_layer_attention_step(out, tp.dev(q), tp.dev(k), tp.dev(v), tp.dev(pos), msl, G, H, Hk, D, q_dim, kv_dim,
                                       d_ck, d_cv, scratch, **kw_args)
        finally:
            kv.set_decode_fused(0)
            kv.set_fused_shape(0, 0)
        if c["producers"]:
            oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, 1e-6, q_dim, kv_dim, False)
            oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, 128)
        oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
        oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
        want = np.zeros((G, q_dim), np.float16)
        oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
        if c["gated"]:
            oracle.sigmoid_gate_batch(want, gate, q_dim, G)
        what = []
        for name, got, ref in (("K codes", d_ck, ck), ("V codes", d_cv, cv), ("K norms", d_kn, kn), ("V norms", d_vn, vn)):
            if not np.array_equal(tp.host(got).view(np.uint8), ref.view(np.uint8)):
                what.append(name)
        if tickets is not None and int(tickets.abs().sum()) != 0:
            what.append("tickets left non-zero")
        err = tp.rel_err(tp.host(out), want)
        if err > tp.TOL:
            what.append(f"rel err {err:.2e}")
        if what:
            failures.append((case, {k_: v_ for k_, v_ in c.items() if k_ != "lens"}, what))
    assert not failures, failures


@pytest.mark.parametrize("seed", [1, 2])
def test_random_fp16_layer_steps(kv, oracle, seed):
    """The same sweep over the fp16 cache: append inside the attention launch or before it, forced split counts,
    producers, gate, GQA groups 1 to 4."""
    import torch
    failures = []
    for case in range(25):
        r = gen.rng(800000 + 1000 * seed + case)
        Hk = int(r.choice([1, 2, 4, 8, 8]))
        H = Hk * int(r.choice([1, 2, 2, 3, 4]))
        G = int(r.choice([1, 2, 3, 5, 8, 16, 17, 40]))
        msl = int(r.choice([40, 96, 300, 700]))
        G = min(G, max(1, (16 * 700 * 8) // (msl * Hk)))
        lens = [int(x) for x in r.integers(0, msl - 1, size=G)] if r.integers(0, 2) else [int(r.integers(0, msl - 1))] * G
        nsplit = int(r.choice([0, 0, 1, 3, 7]))
        producers, gated, known = bool(r.integers(0, 2)), bool(r.integers(0, 2)), bool(r.integers(0, 2))
        variant = int(r.choice([0, 0, 1]))
        kv_dim, q_dim = Hk * D, H * D
        ck, cv = tp.build_fp16_cache(r, G, msl, kv_dim)
        for g in range(G):
            ck[g, lens[g]:] = 0; cv[g, lens[g]:] = 0
        pos = np.array(lens, np.int32)
        q, k, qw, kw = tp.producer_inputs(r, G, H, Hk, q_dim, kv_dim)
        if not producers:
            q = gen.normal_f16(r, (G, q_dim))
        v = gen.normal_f16(r, (G, kv_dim))
        gate = gen.normal_f16(r, (G, q_dim))
        ct, st = tp.rope_tables(msl, 128)
        d_ck, d_cv = tp.dev(ck), tp.dev(cv)
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
        kw_args = dict(kv_bits=0)
        if producers:
            kw_args.update(q_weight=tp.dev(qw), k_weight=tp.dev(kw), eps=1e-6, cos_table=tp.dev(ct), sin_table=tp.dev(st), rope_dim=128)
        if gated:
            kw_args.update(gate=tp.dev(gate), gate_stride=q_dim)
        if known:
            kw_args.update(ctx_min=min(lens) + 1, ctx_max=max(lens) + 1)
        kv.set_num_splits(nsplit)
        kv.set_attention_variant(variant)
        try:
            kv.tw_layer_attention_step(out, tp.dev(q), tp.dev(k), tp.dev(v), tp.dev(pos), msl, G, H, Hk, D, q_dim, kv_dim,
                                       d_ck, d_cv, scratch, **kw_args)
        finally:
            kv.set_num_splits(0)
            kv.set_attention_variant(0)
        if producers:
            oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, 1e-6, q_dim, kv_dim, False)
            oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, 128)
        oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
        want = np.zeros((G, q_dim), np.float16)
        oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
        if gated:
            oracle.sigmoid_gate_batch(want, gate, q_dim, G)
        what = []
        if not np.array_equal(tp.host(d_ck).view(np.uint16), ck.view(np.uint16)):
            what.append("K cache")
        if not np.array_equal(tp.host(d_cv).view(np.uint16), cv.view(np.uint16)):
            what.append("V cache")
        err = tp.rel_err(tp.host(out), want)
        if err > tp.TOL:
            what.append(f"rel err {err:.2e}")
        if what:
            failures.append((case, dict(G=G, H=H, Hk=Hk, msl=msl, nsplit=nsplit, producers=producers, gated=gated,
                                        known=known, variant=variant), what))
    assert not failures, failures


@pytest.mark.parametrize("seed", [1, 2])
def test_random_paged_attention(kv, oracle, rotation_fixture, seed):
    """Random paged batches, every cache width: pages in shuffled order, one appended row per sequence through the
    block table (bit for bit where it lands), then attention over the pages against the oracle on the contiguous cache."""
    import torch
    failures = []
    for case in range(20):
        r = gen.rng(900000 + 1000 * seed + case)
        bits = int(r.choice([4, 2, 0]))
        Hk = int(r.choice([2, 4, 8, 8]))
        H = Hk * int(r.choice([1, 2, 4]))
        G = int(r.choice([1, 2, 5, 9, 16, 33]))
        pages_per_seq = int(r.choice([3, 9, 20, 45]))
        msl = pages_per_seq * 16
        G = min(G, max(1, (16 * 720 * 8) // (msl * Hk)))
        lens = np.array([int(x) for x in r.integers(1, msl + 1, size=G)])            # tokens after the append
        kv_dim, q_dim = Hk * D, H * D
        bt = gen.shuffled_block_table(r, G, pages_per_seq)
        n_pages = G * pages_per_seq
        rot = tp.dev(rotation_fixture)
        if bits == 0:
            ck, cv = tp.build_fp16_cache(r, G, msl, kv_dim)
            for g in range(G):
                ck[g, lens[g] - 1:] = 0; cv[g, lens[g] - 1:] = 0
            width, dtype = kv_dim, np.float16
        else:
            ck, cv, kn, vn = tp.build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens - 1, bits)
            width, dtype = kv_dim * bits // 8, np.uint8

        def scatter(contig, w, dt):
            pool = np.zeros((n_pages, 16, w), dt)
            for g in range(G):
                for i in range(pages_per_seq):
                    pool[bt[g, i]] = contig[g, 16 * i:16 * (i + 1)]
            return pool

        def gather(pool):
            return np.stack([np.concatenate([pool[bt[g, i]] for i in range(pages_per_seq)]) for g in range(G)])

        p_ck, p_cv = tp.dev(scatter(ck, width, dtype)), tp.dev(scatter(cv, width, dtype))
        if bits:
            p_kn, p_vn = tp.dev(scatter(kn, Hk, np.float16)), tp.dev(scatter(vn, Hk, np.float16))
        d_bt = tp.dev(bt)
        pos = (lens - 1).astype(np.int32)
        k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
        q = gen.normal_f16(r, (G, q_dim))
        want = np.zeros((G, q_dim), np.float16)
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        ws = torch.zeros(kv.attention_workspace_floats(G, H, msl), dtype=torch.float32, device="cuda")
        what = []
        if bits == 0:
            oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
            kv.tw_paged_kv_cache_write_batch(p_ck, p_cv, tp.dev(k), tp.dev(v), tp.dev(pos), d_bt, pages_per_seq, G, kv_dim)
            oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
            kv.tw_paged_gqa_attention_batch(out, tp.dev(q), p_ck, p_cv, ws, tp.dev(pos), d_bt, pages_per_seq, msl, G, H, Hk, D,
                                            q_dim, kv_dim)
        else:
            oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
            oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
            kv.tw_paged_turbo_kv_append_batch(p_ck, p_kn, p_cv, p_vn, tp.dev(k), tp.dev(v), rot, tp.dev(pos), d_bt,
                                              pages_per_seq, G, Hk, D, kv_dim, bits)
            oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
            kv.tw_paged_turbo_gqa_attention_batch(out, tp.dev(q), p_ck, p_cv, p_kn, p_vn, rot, ws, tp.dev(pos), d_bt,
                                                  pages_per_seq, msl, G, H, Hk, D, q_dim, kv_dim, bits)
            if not np.array_equal(gather(tp.host(p_kn)).view(np.uint16), kn.view(np.uint16)):
                what.append("paged K norms")
            if not np.array_equal(gather(tp.host(p_vn)).view(np.uint16), vn.view(np.uint16)):
                what.append("paged V norms")
        if not np.array_equal(gather(tp.host(p_ck)).view(np.uint8), ck.view(np.uint8)):
            what.append("paged K")
        if not np.array_equal(gather(tp.host(p_cv)).view(np.uint8), cv.view(np.uint8)):
            what.append("paged V")
        err = tp.rel_err(tp.host(out), want)
        if err > tp.TOL:
            what.append(f"rel err {err:.2e}")
        if what:
            failures.append((case, dict(bits=bits, G=G, H=H, Hk=Hk, pages_per_seq=pages_per_seq), what))
    assert not failures, failures
