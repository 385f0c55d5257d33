"""GPU parity: the HIP library, called through its C ABI, against the CPU oracle
on the same seeded inputs.

Bars (from the task statement of this path):
  - packed codes, norms and every piece of cache bookkeeping: bit-exact;
  - attention outputs: max relative error <= 2e-3 in fp16, measured per head
    vector as ||gpu - oracle||_inf / ||oracle||_inf.
"""
from pathlib import Path

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
    return kvcache


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch
    torch.cuda.synchronize()
    return t.cpu().numpy()


def rel_err(got, want):
    got = got.astype(np.float64).reshape(-1, D)
    want = want.astype(np.float64).reshape(-1, D)
    err = float(np.max(np.max(np.abs(got - want), axis=1) / np.max(np.abs(want), axis=1)))
    parity_log.record(err)
    return err


def assert_bytes_equal(got, want, what, margin=None):
    got = np.ascontiguousarray(got).view(np.uint8)
    want = np.ascontiguousarray(want).view(np.uint8)
    if np.array_equal(got, want):
        return
    bad = np.argwhere(got != want)
    msg = f"{what}: {len(bad)} of {got.size} bytes differ; first at {bad[0].tolist()}"
    if margin is not None:
        msg += f"; smallest boundary margin in the call: {float(margin.min()):.3e}"
    raise AssertionError(msg)


# ------------------------------------------------------------------ fp16 append
def test_fp16_append_bit_exact(kv, oracle):
    r = gen.rng(101)
    G, msl, kv_dim = 4, 24, 1024
    ck = np.zeros((G, msl, kv_dim), np.float16); cv = np.zeros_like(ck)
    d_ck, d_cv = dev(ck), dev(cv)
    pos = np.array([0, 5, 23, 11], np.int32)
    for step in range(3):
        k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
        oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
        kv.launch_kv_cache_write_batch(d_ck, d_cv, dev(k), dev(v), dev(pos), msl, G, kv_dim)
        pos = (pos + 7) % msl
    assert_bytes_equal(host(d_ck), ck, "fp16 K cache")
    assert_bytes_equal(host(d_cv), cv, "fp16 V cache")


def test_fp16_append_unaligned_width(kv, oracle):
    r = gen.rng(102)
    G, msl, kv_dim = 3, 5, 132  # not a multiple of 8 halves: scalar path
    ck = np.zeros((G, msl, kv_dim), np.float16); cv = np.zeros_like(ck)
    d_ck, d_cv = dev(ck), dev(cv)
    pos = np.array([4, 0, 2], np.int32)
    k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
    kv.launch_kv_cache_write_batch(d_ck, d_cv, dev(k), dev(v), dev(pos), msl, G, kv_dim)
    assert_bytes_equal(host(d_ck), ck, "fp16 K cache")
    assert_bytes_equal(host(d_cv), cv, "fp16 V cache")


def test_increment_positions(kv):
    pos = np.array([0, 7, 100, 65535], np.int32)
    d = dev(pos)
    for _ in range(3):
        kv.launch_increment_positions(d, 4)
    assert np.array_equal(host(d), pos + 3)


# ------------------------------------------------------------------ compressed append
def special_rows(r, G, kv_dim):
    rows, _ = gen.kv_rows_with_outliers(r, (G, kv_dim), kv_dim)
    rows[1, :D] = 0
    rows[2] = (rows[2].astype(np.float32) * 1e-3).astype(np.float16)
    rows[3] = (rows[3].astype(np.float32) * 30).astype(np.float16)
    rows[4, D:2 * D] = np.float16(6e-8)  # fp16 subnormals
    return rows


@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_append_batch_bit_exact(kv, oracle, rotation_fixture, bits):
    r = gen.rng(110 + bits)
    G, Hk, msl = 64, 8, 12
    kv_dim = Hk * D
    kvp = kv_dim * bits // 8
    rows = special_rows(r, G, kv_dim)
    pos = r.integers(0, msl, G).astype(np.int32)
    cq = np.zeros((G, msl, kvp), np.uint8); cn = np.zeros((G, msl, Hk), np.float16)
    margin = np.zeros((G, kv_dim), np.float32)
    oracle.turbo_kv_quantize_batch(cq, cn, rows, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits, None, margin)
    d_cq, d_cn = dev(np.zeros_like(cq)), dev(np.zeros_like(cn))
    kv.launch_turbo_kv_quantize_batch(d_cq, d_cn, dev(rows), dev(rotation_fixture), dev(pos), msl, G, Hk, D, kv_dim, bits)
    assert_bytes_equal(host(d_cq), cq, f"{bits}-bit codes", margin)
    assert_bytes_equal(host(d_cn), cn, "norms")


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_append_many_rows_bit_exact(kv, oracle, rotation_fixture, bits, variant):
    """A few hundred thousand coordinates: the tie set, if any, shows up here.
    variant 0 = MFMA rotation kernel, 1 = vector-ALU kernel; both must give the oracle's bytes."""
    r = gen.rng(120 + bits)
    G, Hk, msl = 512, 8, 1
    kv_dim = Hk * D
    kvp = kv_dim * bits // 8
    rows = gen.normal_f16(r, (G, kv_dim))
    pos = np.zeros(G, np.int32)
    cq = np.zeros((G, msl, kvp), np.uint8); cn = np.zeros((G, msl, Hk), np.float16)
    margin = np.zeros((G, kv_dim), np.float32)
    oracle.turbo_kv_quantize_batch(cq, cn, rows, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits, None, margin)
    d_cq, d_cn = dev(np.zeros_like(cq)), dev(np.zeros_like(cn))
    kv.set_attention_variant(variant)
    try:
        kv.launch_turbo_kv_quantize_batch(d_cq, d_cn, dev(rows), dev(rotation_fixture), dev(pos), msl, G, Hk, D, kv_dim, bits)
    finally:
        kv.set_attention_variant(0)
    assert_bytes_equal(host(d_cq), cq, f"{bits}-bit codes", margin)
    assert_bytes_equal(host(d_cn), cn, "norms")


@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_append_token_list_and_fused(kv, oracle, rotation_fixture, bits):
    r = gen.rng(130 + bits)
    T, Hk, msl = 37, 8, 64
    kv_dim = Hk * D
    kvp = kv_dim * bits // 8
    rows = gen.normal_f16(r, (T, kv_dim))
    positions = r.permutation(msl)[:T].astype(np.int32)
    cq = np.zeros((msl, kvp), np.uint8); cn = np.zeros((msl, Hk), np.float16)
    oracle.turbo_kv_quantize(cq, cn, rows, rotation_fixture, positions, msl, T, Hk, D, kv_dim, bits)
    d_cq, d_cn = dev(np.zeros_like(cq)), dev(np.zeros_like(cn))
    kv.launch_turbo_kv_quantize(d_cq, d_cn, dev(rows), dev(rotation_fixture), dev(positions), msl, T, Hk, D, kv_dim, bits)
    assert_bytes_equal(host(d_cq), cq, "token-list codes")
    assert_bytes_equal(host(d_cn), cn, "token-list norms")

    # K and V through one launch == two reference-style launches
    G = 9
    k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    pos = r.integers(0, msl, G).astype(np.int32)
    want = []
    for src in (k, v):
        q_ = np.zeros((G, msl, kvp), np.uint8); n_ = np.zeros((G, msl, Hk), np.float16)
        oracle.turbo_kv_quantize_batch(q_, n_, src, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
        want += [q_, n_]
    bufs = [dev(np.zeros_like(w)) for w in want]
    kv.tw_turbo_kv_append_batch(bufs[0], bufs[1], bufs[2], bufs[3], dev(k), dev(v), dev(rotation_fixture),
                                dev(pos), msl, G, Hk, D, kv_dim, bits)
    for b, w, name in zip(bufs, want, ("K codes", "K norms", "V codes", "V norms")):
        assert_bytes_equal(host(b), w, "fused " + name)


# ------------------------------------------------------------------ attention helpers
def build_fp16_cache(r, G, msl, kv_dim):
    return gen.normal_f16(r, (G, msl, kv_dim)), gen.normal_f16(r, (G, msl, kv_dim))


def build_turbo_cache(oracle, rot, r, G, Hk, msl, lens, bits, outliers=True):
    """Quantize lens[g] rows per sequence with the oracle's token-list append."""
    kv_dim = Hk * D
    kvp = kv_dim * bits // 8
    ck = np.zeros((G, msl, kvp), np.uint8); cv = np.zeros_like(ck)
    kn = np.zeros((G, msl, Hk), np.float16); vn = np.zeros_like(kn)
    for g in range(G):
        n = int(lens[g])
        if outliers:
            k_rows, _ = gen.kv_rows_with_outliers(r, (n, kv_dim), kv_dim)
            v_rows, _ = gen.kv_rows_with_outliers(r, (n, kv_dim), kv_dim)
        else:
            k_rows = gen.normal_f16(r, (n, kv_dim)); v_rows = gen.normal_f16(r, (n, kv_dim))
        p = np.arange(n, dtype=np.int32)
        oracle.turbo_kv_quantize(ck[g], kn[g], k_rows, rot, p, msl, n, Hk, D, kv_dim, bits)
        oracle.turbo_kv_quantize(cv[g], vn[g], v_rows, rot, p, msl, n, Hk, D, kv_dim, bits)
    return ck, cv, kn, vn


# ------------------------------------------------------------------ fp16 attention
@pytest.mark.parametrize("nsplit", [0, 1, 3])
def test_fp16_attention_batch_config1(kv, oracle, nsplit):
    """Single layer, 16 query heads, 8 KV heads, batch 4, context 612 + the appended token."""
    r = gen.rng(201)
    G, H, Hk, msl = 4, 16, 8, 640
    kv_dim, q_dim = Hk * D, H * D
    ck, cv = build_fp16_cache(r, G, msl, kv_dim)
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.full(G, 612, np.int32)
    want = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    import torch
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.set_num_splits(nsplit)
    try:
        kv.launch_gqa_attention_batch(out, dev(q), dev(ck), dev(cv), scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    finally:
        kv.set_num_splits(0)
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("nsplit", [0, 1, 3])
@pytest.mark.parametrize("H,Hk", [(16, 8), (8, 2), (4, 4), (8, 1)])
def test_fp16_append_attention_step(kv, oracle, H, Hk, nsplit, mode):
    """fp16 cache, append + attention in one call: with the append inside the attention launch (mode 0) and
    as the reference's two launches (mode 2).  Cache bytes equal the oracle's row copy (nothing else
    touched), outputs within tolerance of the oracle's attention over the appended cache."""
    import torch
    r = gen.rng(210 + H + Hk)
    lens = [0, 1, 15, 16, 63, 64, 65, 255, 256, 700, 1023]
    G, msl = len(lens), 1024
    kv_dim, q_dim = Hk * D, H * D
    ck, cv = build_fp16_cache(r, G, msl, kv_dim)
    pos = np.array(lens, np.int32)
    for g in range(G):
        ck[g, pos[g]:] = 0; cv[g, pos[g]:] = 0
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    d_ck, d_cv = dev(ck), dev(cv)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.set_num_splits(nsplit)
    kv.set_decode_fused(mode)
    try:
        kv.tw_append_attention_batch(out, dev(q), dev(k), dev(v), d_ck, d_cv, scratch, dev(pos), msl, G, H, Hk, D,
                                     q_dim, kv_dim)
    finally:
        kv.set_num_splits(0)
        kv.set_decode_fused(0)
    oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
    want = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    assert_bytes_equal(host(d_ck), ck, "K rows"); assert_bytes_equal(host(d_cv), cv, "V rows")
    assert rel_err(host(out), want) <= TOL


def test_fp16_attention_ragged_and_strided(kv, oracle):
    r = gen.rng(202)
    G, H, Hk, msl = 6, 8, 2, 1500   # GQA group 4
    kv_dim, q_dim = Hk * D, H * D + 64   # q_dim is a row stride
    ck, cv = build_fp16_cache(r, G, msl, kv_dim)
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.array([0, 1, 63, 64, 777, 1499], np.int32)
    want = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    import torch
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.launch_gqa_attention_batch(out, dev(q), dev(ck), dev(cv), scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    got = host(out)
    assert rel_err(got[:, :H * D], want[:, :H * D]) <= TOL
    assert not got[:, H * D:].any()


def test_fp16_attention_single_sequence(kv, oracle):
    r = gen.rng(203)
    H, Hk, msl = 16, 8, 700
    kv_dim, q_dim = Hk * D, H * D
    ck, cv = build_fp16_cache(r, 1, msl, kv_dim)
    q = gen.normal_f16(r, (q_dim,))
    import torch
    for pos in (0, 129, 699):
        want = np.zeros(q_dim, np.float16)
        oracle.gqa_attention(q, ck[0], cv[0], want, pos, msl, H, Hk, D)
        out = torch.zeros(q_dim, dtype=torch.float16, device="cuda")
        scratch = torch.zeros(H * msl, dtype=torch.float32, device="cuda")
        kv.launch_gqa_attention(dev(q), dev(ck[0]), dev(cv[0]), out, scratch, pos, msl, H, Hk, D)
        assert rel_err(host(out), want) <= TOL


ROW_SCAN_LENS = {
    # ragged: the balanced walk (lengths differ by more than 1/8), pieces cut at sequence ends, every wave of a
    # workgroup meets the appended token somewhere
    "ragged": [0, 1, 7, 8, 9, 15, 16, 17, 63, 64, 65, 100, 255, 256, 257, 300, 511, 512, 513, 700, 900, 1021, 1022, 1023],
    # nearly equal: even chunks in units of 8 tokens
    "even": [700 + i for i in range(20)],
    # very short: most even chunks hold no token
    "short": [0, 1, 2, 3, 5, 8, 9, 11, 13, 16, 17, 19, 21, 24, 25, 27, 30],
}


@pytest.mark.parametrize("append", [False, True])
@pytest.mark.parametrize("nsplit", [0, 1, 5])
@pytest.mark.parametrize("lens_kind", ["ragged", "even", "short"])
@pytest.mark.parametrize("H,Hk", [(16, 8), (8, 8), (32, 8), (32, 16)])
def test_fp16_whole_row_scan(kv, oracle, H, Hk, lens_kind, nsplit, append):
    """fp16 cache with KV heads in blocks of eight and 16 or more sequences: the scan whose waves read whole cache
    rows (groups of 1, 2 and 4 query heads per KV head, one and two blocks of KV heads), attention alone and with
    the append inside the launch, == the oracle's attention; the appended rows are the oracle's row copy."""
    import torch
    r = gen.rng(230 + H + Hk + nsplit)
    lens = ROW_SCAN_LENS[lens_kind]
    G, msl = len(lens), 1024
    kv_dim, q_dim = Hk * D, H * D
    ck, cv = build_fp16_cache(r, G, msl, kv_dim)
    pos = np.array(lens, np.int32)
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    if append:
        for g in range(G):
            ck[g, pos[g]:] = 0; cv[g, pos[g]:] = 0
    d_ck, d_cv = dev(ck), dev(cv)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.set_num_splits(nsplit)
    try:
        if append:
            kv.tw_append_attention_batch(out, dev(q), dev(k), dev(v), d_ck, d_cv, scratch, dev(pos), msl, G, H, Hk, D,
                                         q_dim, kv_dim)
        else:
            kv.launch_gqa_attention_batch(out, dev(q), d_ck, d_cv, scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    finally:
        kv.set_num_splits(0)
    assert kv.last_scan_kernel() == "attention_rows_kernel"
    if append:
        oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
    want = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    assert_bytes_equal(host(d_ck), ck, "K rows"); assert_bytes_equal(host(d_cv), cv, "V rows")
    assert rel_err(host(out), want) <= TOL


def test_fp16_whole_row_scan_without_workspace_and_paged(kv, oracle):
    """The same kernel where the caller's scratch is too small for partials (every workgroup walks a whole
    sequence and writes the output itself), and over 16-token pages in shuffled order."""
    import torch
    r = gen.rng(236)
    G, H, Hk = 18, 16, 8
    kv_dim, q_dim = Hk * D, H * D
    pages_per_seq = 12
    msl = pages_per_seq * 16                       # 192 floats per (sequence, head): no room for a partial and q_rot
    ck, cv = build_fp16_cache(r, G, msl, kv_dim)
    pos = np.array([0, 1, 15, 16, 17, 31, 32, 33, 47, 64, 100, 127, 128, 150, 170, 189, 190, 191], np.int32)
    q = gen.normal_f16(r, (G, q_dim))
    want = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.launch_gqa_attention_batch(out, dev(q), dev(ck), dev(cv), scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    assert kv.last_scan_kernel() == "attention_rows_kernel"
    assert rel_err(host(out), want) <= TOL

    bt = gen.shuffled_block_table(r, G, pages_per_seq)
    pool_k = np.zeros((G * pages_per_seq, 16, kv_dim), np.float16); pool_v = np.zeros_like(pool_k)
    for g in range(G):
        for i in range(pages_per_seq):
            pool_k[bt[g, i]] = ck[g, 16 * i:16 * (i + 1)]; pool_v[bt[g, i]] = cv[g, 16 * i:16 * (i + 1)]
    for nsplit in (0, 1, 3):
        out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
        ws = torch.zeros(kv.attention_workspace_floats(G, H, msl), dtype=torch.float32, device="cuda")
        kv.set_num_splits(nsplit)
        try:
            kv.tw_paged_gqa_attention_batch(out, dev(q), dev(pool_k), dev(pool_v), ws, dev(pos), dev(bt), pages_per_seq, msl,
                                            G, H, Hk, D, q_dim, kv_dim)
        finally:
            kv.set_num_splits(0)
        assert kv.last_scan_kernel() == "attention_rows_kernel"
        assert rel_err(host(out), want) <= TOL, nsplit


def test_fp16_prefill_attention(kv, oracle):
    r = gen.rng(204)
    T, H, Hk, msl = 70, 4, 2, 96
    kv_dim, q_dim = Hk * D, H * D
    ck, cv = build_fp16_cache(r, 1, msl, kv_dim)
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    oracle.gqa_prefill_attention(want, q, ck[0], cv[0], T, msl, H, Hk, D, q_dim, kv_dim)
    import torch
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * T, dtype=torch.float32, device="cuda")
    kv.launch_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), scratch, T, msl, H, Hk, D, q_dim, kv_dim)
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("H,Hk,T,pad", [(16, 8, 700, 0), (8, 8, 333, 0), (16, 4, 530, 256), (12, 4, 100, 0), (4, 2, 1, 0),
                                        (4, 2, 17, 0), (16, 8, 64, 0)])
def test_fp16_prefill_attention_long(kv, oracle, H, Hk, T, pad, variant):
    """Causal prefill over the fp16 cache: GQA groups 1, 2 and 4 take the matrix-core kernel (variant 0),
    group 3 and variant 1 the vector-ALU one; block edges (T = 1, 17, 64), a q row stride wider than
    H*D, outlier keys that move the running maximum late in the row."""
    import torch
    r = gen.rng(250 + H + T)
    msl = T + 5
    kv_dim, q_dim = Hk * D, H * D + pad
    ck, cv = build_fp16_cache(r, 1, msl, kv_dim)
    if T > 40:
        ck[0, T - 3] = (ck[0, T - 3].astype(np.float32) * 6).astype(np.float16)   # a late, large key
        ck[0, 35] = (ck[0, 35].astype(np.float32) * 5).astype(np.float16)
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    oracle.gqa_prefill_attention(want, q, ck[0], cv[0], T, msl, H, Hk, D, q_dim, kv_dim)
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * T, dtype=torch.float32, device="cuda")
    kv.set_attention_variant(variant)
    try:
        kv.launch_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), scratch, T, msl, H, Hk, D, q_dim, kv_dim)
    finally:
        kv.set_attention_variant(0)
    got = host(out)
    assert rel_err(got[:, :H * D], want[:, :H * D]) <= TOL
    assert not got[:, H * D:].any()


@pytest.mark.parametrize("form", [1, 2, 3, 5, 6])
@pytest.mark.parametrize("H,Hk,T", [(16, 8, 300), (8, 8, 129), (16, 4, 97), (16, 8, 31), (16, 4, 777)])
def test_fp16_prefill_every_form_of_the_mfma_kernel(kv, oracle, H, Hk, T, form):
    """The matrix-core prefill kernel picks one of five forms from the prompt length (one or two query
    blocks per wave, with or without mirrored block pairs, four or eight waves per workgroup); each is forced
    here at lengths that put the diagonal, the middle block of an odd count and a ragged last block in
    different places."""
    import torch
    r = gen.rng(270 + H + T)
    msl = T
    kv_dim, q_dim = Hk * D, H * D
    ck, cv = build_fp16_cache(r, 1, msl, kv_dim)
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    oracle.gqa_prefill_attention(want, q, ck[0], cv[0], T, msl, H, Hk, D, q_dim, kv_dim)
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * T, dtype=torch.float32, device="cuda")
    kv.set_prefill_form(form)
    try:
        kv.launch_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), scratch, T, msl, H, Hk, D, q_dim, kv_dim)
    finally:
        kv.set_prefill_form(0)
    assert rel_err(host(out), want) <= TOL


# ------------------------------------------------------------------ compressed attention
@pytest.mark.parametrize("variant", [1, 0, 3])
@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_attention_batch_config2_layer(kv, oracle, rotation_fixture, bits, variant):
    """One layer of the 28-layer TurboQuant case: batch 4, context 612 + 1, 1 % outlier channels x8."""
    r = gen.rng(300 + bits)
    G, H, Hk, msl = 4, 16, 8, 640
    kv_dim, q_dim = Hk * D, H * D
    lens = [613] * G
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits)
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.array(lens, np.int32) - 1
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    import torch
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.set_attention_variant(variant)
    try:
        kv.launch_turbo_gqa_attention_batch(out, dev(q), dev(ck), dev(cv), dev(kn), dev(vn), dev(rotation_fixture),
                                            scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, bits)
    finally:
        kv.set_attention_variant(0)
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("variant", [1, 0, 3])
@pytest.mark.parametrize("bits,H,Hk", [(4, 16, 8), (2, 32, 8), (4, 4, 4)])
def test_turbo_attention_ragged_splits(kv, oracle, rotation_fixture, bits, H, Hk, variant):
    """Ragged contexts around every tile / chunk edge, with forced split counts."""
    r = gen.rng(310 + bits + H)
    lens = [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 257, 1000, 1535, 1536]
    G, msl = len(lens), 1536
    kv_dim, q_dim = Hk * D, H * D
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits, outliers=False)
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.array(lens, np.int32) - 1
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    import torch
    d = [dev(x) for x in (q, ck, cv, kn, vn, rotation_fixture, pos)]
    kv.set_attention_variant(variant)
    try:
        for nsplit in (0, 1, 2, 7):
            kv.set_num_splits(nsplit)
            out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
            scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
            kv.launch_turbo_gqa_attention_batch(out, d[0], d[1], d[2], d[3], d[4], d[5], scratch, d[6], msl, G, H, Hk,
                                                D, q_dim, kv_dim, bits)
            err = rel_err(host(out), want)
            assert err <= TOL, f"nsplit={nsplit}: {err}"
    finally:
        kv.set_num_splits(0)
        kv.set_attention_variant(0)


@pytest.mark.parametrize("bits", [4, 2])
def test_fused_append_attention_equals_two_calls(kv, oracle, rotation_fixture, bits):
    """append + attention in one call == oracle append, then oracle attention."""
    r = gen.rng(340 + bits)
    G, H, Hk, msl = 7, 16, 8, 320
    kv_dim, q_dim = Hk * D, H * D
    lens = [1, 33, 64, 100, 257, 300, 319]
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits)
    pos = np.array(lens, np.int32)            # the appended token goes right behind the cache
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    import torch
    d_ck, d_cv, d_kn, d_vn = dev(ck), dev(cv), dev(kn), dev(vn)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.tw_turbo_append_attention_batch(out, dev(q), dev(k), dev(v), d_ck, d_cv, d_kn, d_vn, dev(rotation_fixture),
                                       scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert_bytes_equal(host(d_ck), ck, "K codes"); assert_bytes_equal(host(d_cv), cv, "V codes")
    assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("mode", [1, 2])
@pytest.mark.parametrize("bits", [4, 2])
@pytest.mark.parametrize("H,Hk,lens", [
    (16, 8, [0, 1, 31, 32, 33, 511, 512, 513, 1023, 1500, 2047]),          # every tile edge, 11 sequences
    (32, 8, [5, 64, 700, 1299, 95, 96, 97, 1, 0, 255, 256, 257, 640, 641, 2, 1111]),   # GQA 4, 16 sequences
    (4, 4, [40, 0, 1000]),                                                   # no grouping, 4 KV heads
    (4, 2, [3, 77, 1999]), (2, 1, [130, 12]), (8, 2, [300, 301, 1024])])     # few KV heads
def test_decode_step_in_one_launch(kv, oracle, rotation_fixture, bits, H, Hk, lens, mode):
    """tw_turbo_append_attention_batch as one kernel (mode 1) and as three (mode 2): the appended rows equal the
    oracle's bytes, the rest of the cache is untouched, outputs within tolerance of oracle append + attention."""
    import torch
    r = gen.rng(900 + bits + H + Hk)
    G, msl = len(lens), 2048
    kv_dim, q_dim = Hk * D, H * D
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits)
    pos = np.array(lens, np.int32)
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    d_ck, d_cv, d_kn, d_vn = dev(ck), dev(cv), dev(kn), dev(vn)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.set_decode_fused(mode)
    try:
        kv.tw_turbo_append_attention_batch(out, dev(q), dev(k), dev(v), d_ck, d_cv, d_kn, d_vn, dev(rotation_fixture),
                                           scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, bits)
    finally:
        kv.set_decode_fused(0)
    oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert_bytes_equal(host(d_ck), ck, "K codes"); assert_bytes_equal(host(d_cv), cv, "V codes")
    assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("mode", [1, 3])
@pytest.mark.parametrize("bits", [4, 2])
@pytest.mark.parametrize("G,H,Hk,producers", [(64, 16, 8, False), (128, 16, 8, True), (256, 16, 8, False), (264, 32, 8, True),
                                              (520, 8, 8, False), (130, 8, 2, True)])
def test_decode_step_in_one_launch_every_head_grouping(kv, oracle, rotation_fixture, bits, G, H, Hk, producers, mode):
    """The one-launch step with 2, 4 and 8 KV heads per workgroup (batches of 64, 128 and 256 and more sequences on a
    256-CU GPU; 8 heads make units of more than 16 vectors, two rotation tiles), batch sizes that are and are not
    multiples of 8 (the workgroup numbering differs), with and without the producers: cache bytes and outputs
    against the oracle.  Mode 1 takes the 4-bit kernel whose waves scan two KV heads each where the shape admits
    it, mode 3 keeps one head per wave."""
    import torch
    r = gen.rng(950 + bits + G)
    msl = 96
    kv_dim, q_dim = Hk * D, H * D
    lens = [int(x) for x in r.integers(0, msl - 1, size=G)]
    lens[0], lens[1], lens[G - 1] = 0, msl - 1, 33
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits, outliers=False)
    pos = np.array(lens, np.int32)
    q, k, qw, kw = producer_inputs(r, G, H, Hk, q_dim, kv_dim)
    v = gen.normal_f16(r, (G, kv_dim))
    ct, st = rope_tables(msl, 128)
    d_ck, d_cv, d_kn, d_vn = dev(ck), dev(cv), dev(kn), dev(vn)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    launches = kv._lib.load().tw_kv_decode_fused_launches()
    kv.set_decode_fused(mode)
    try:
        if producers:
            kv.tw_qk_norm_rope_turbo_append_attention_batch(
                out, dev(q), dev(k), dev(v), dev(qw), dev(kw), 1e-6, False, dev(ct), dev(st), 128, d_ck, d_cv, d_kn, d_vn,
                dev(rotation_fixture), scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, bits)
        else:
            kv.tw_turbo_append_attention_batch(out, dev(q), dev(k), dev(v), d_ck, d_cv, d_kn, d_vn, dev(rotation_fixture),
                                               scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, bits)
    finally:
        kv.set_decode_fused(0)
    assert kv._lib.load().tw_kv_decode_fused_launches() == launches + 1      # it was the one-launch kernel
    if producers:
        oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, 1e-6, q_dim, kv_dim, False)
        oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, 128)
    oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert_bytes_equal(host(d_ck), ck, "K codes"); assert_bytes_equal(host(d_cv), cv, "V codes")
    assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("mode", [1, 3])
@pytest.mark.parametrize("G,H,Hk,msl", [(64, 16, 8, 2048), (64, 8, 8, 1100), (64, 32, 8, 1100), (128, 16, 8, 700), (256, 16, 8, 400),
                                        (128, 8, 4, 520)])
def test_decode_step_two_heads_per_wave_long_contexts(kv, oracle, rotation_fixture, G, H, Hk, msl, mode):
    """The 4-bit one-launch step at batch sizes where a workgroup owns 2, 4 or 8 KV heads (mode 1: its waves scan
    two heads each, every load a whole cache line; mode 3: one head per wave), over contexts that hit every tile and
    part edge up to max_seq_len - 1, query groups of 1, 2 and 4: appended rows bit for bit, outputs within tolerance."""
    import torch
    bits = 4
    r = gen.rng(990 + G + H + Hk)
    kv_dim, q_dim = Hk * D, H * D
    edges = [0, 1, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 512, 513, 767, 1023,
             1024, 1025, 1500, 2046, 2047]
    lens = [e for e in edges if e < msl] + [msl - 1, msl - 2]
    lens = (lens + [int(x) for x in r.integers(0, msl - 1, size=G)])[:G]
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits)
    pos = np.array(lens, np.int32)
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    d_ck, d_cv, d_kn, d_vn = dev(ck), dev(cv), dev(kn), dev(vn)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    launches = kv._lib.load().tw_kv_decode_fused_launches()
    kv.set_decode_fused(mode)
    try:
        kv.tw_turbo_append_attention_batch(out, dev(q), dev(k), dev(v), d_ck, d_cv, d_kn, d_vn, dev(rotation_fixture),
                                           scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, bits)
    finally:
        kv.set_decode_fused(0)
    assert kv._lib.load().tw_kv_decode_fused_launches() == launches + 1
    oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert_bytes_equal(host(d_ck), ck, "K codes"); assert_bytes_equal(host(d_cv), cv, "V codes")
    assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")
    got = host(out)
    worst = [(rel_err(got[g], want[g]), g, lens[g]) for g in range(G)]
    assert max(worst)[0] <= TOL, f"worst (error, sequence, context): {sorted(worst)[-3:]}"


@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_attention_single_and_tiny_scratch(kv, oracle, rotation_fixture, bits):
    """Single-sequence entry point; max_seq_len 40 leaves no room for split partials."""
    r = gen.rng(320 + bits)
    H, Hk, msl = 4, 2, 40
    kv_dim, q_dim = Hk * D, H * D
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, 1, Hk, msl, [37], bits)
    q = gen.normal_f16(r, (q_dim,))
    import torch
    for pos in (0, 36):
        want = np.zeros(q_dim, np.float16)
        oracle.turbo_gqa_attention(q, ck[0], cv[0], kn[0], vn[0], rotation_fixture, want, pos, msl, H, Hk, D, bits)
        out = torch.zeros(q_dim, dtype=torch.float16, device="cuda")
        scratch = torch.zeros(H * msl, dtype=torch.float32, device="cuda")
        kv.launch_turbo_gqa_attention(dev(q), dev(ck[0]), dev(cv[0]), dev(kn[0]), dev(vn[0]), dev(rotation_fixture),
                                      out, scratch, pos, msl, H, Hk, D, bits)
        assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_prefill_attention(kv, oracle, rotation_fixture, bits):
    r = gen.rng(330 + bits)
    T, H, Hk, msl = 70, 4, 2, 96
    kv_dim, q_dim = Hk * D, H * D
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, 1, Hk, msl, [T], bits)
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    oracle.turbo_gqa_prefill_attention(want, q, ck[0], cv[0], kn[0], vn[0], rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    import torch
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * T, dtype=torch.float32, device="cuda")
    kv.launch_turbo_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), dev(kn[0]), dev(vn[0]),
                                          dev(rotation_fixture), scratch, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("bits,H,Hk,T", [(4, 16, 8, 700), (2, 16, 8, 645), (4, 8, 2, 601), (2, 4, 4, 530), (4, 4, 1, 1111)])
def test_turbo_prefill_attention_long(kv, oracle, rotation_fixture, bits, H, Hk, T):
    """Prompts long enough for the scratch (T floats per query token and head) to hold split
    partials: the prefill runs on the matrix cores, several query tokens per wave, for
    GQA groups of 2, 4 and 1 and prompt lengths that are not multiples of the token block."""
    import torch
    r = gen.rng(340 + bits + H + T)
    msl = T + 3
    kv_dim, q_dim = Hk * D, H * D
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, 1, Hk, msl, [T], bits)
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    oracle.turbo_gqa_prefill_attention(want, q, ck[0], cv[0], kn[0], vn[0], rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    scratch = torch.full((T * H * T,), float("nan"), dtype=torch.float32, device="cuda")
    for variant in (0, 1):
        kv.set_attention_variant(variant)
        out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
        kv.launch_turbo_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), dev(kn[0]), dev(vn[0]),
                                              dev(rotation_fixture), scratch, T, msl, H, Hk, D, q_dim, kv_dim, bits)
        assert rel_err(host(out), want) <= TOL, f"variant {variant}"
    kv.set_attention_variant(0)


@pytest.mark.parametrize("form", [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("bits,H,Hk,T", [(4, 16, 8, 300), (2, 8, 8, 129), (4, 16, 4, 97), (2, 16, 8, 31), (4, 8, 4, 1),
                                         (2, 4, 4, 7), (4, 4, 1, 16), (2, 8, 4, 33), (2, 16, 4, 777), (4, 8, 4, 515)])
def test_turbo_prefill_every_form(kv, oracle, rotation_fixture, bits, H, Hk, T, form):
    """Compressed prefill: the five forms of the kernel that expands a tile once per workgroup (four or eight
    waves per workgroup, one or two query blocks per wave, with or without mirrored block pairs) and (form 4)
    the kernel that expands per wave, each against the oracle."""
    import torch
    r = gen.rng(380 + bits + H + T)
    msl = T + 3
    kv_dim, q_dim = Hk * D, H * D
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, 1, Hk, msl, [T], bits)
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    oracle.turbo_gqa_prefill_attention(want, q, ck[0], cv[0], kn[0], vn[0], rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * max(T, 1024), dtype=torch.float32, device="cuda")
    kv.set_prefill_form(form)
    try:
        kv.launch_turbo_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), dev(kn[0]), dev(vn[0]),
                                              dev(rotation_fixture), scratch, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    finally:
        kv.set_prefill_form(0)
    err = rel_err(host(out), want)
    assert err <= TOL, err


@pytest.mark.parametrize("form", [3, 5, 6])
@pytest.mark.parametrize("R,T", [(1, 255), (1, 256), (1, 257), (2, 127), (2, 128), (2, 129), (2, 383), (4, 63), (4, 64), (4, 65), (4, 193)])
@pytest.mark.parametrize("bits", [0, 2])
def test_prefill_lengths_around_the_token_blocks(kv, oracle, rotation_fixture, bits, R, T, form):
    """Prompt lengths one below, at and one above a multiple of the workgroup's token block (64 to 256 tokens,
    by GQA group and form): the last block is ragged or exactly full, the mirrored pair of a block may be the
    block itself, and the steady part of the tile loop may be empty."""
    import torch
    Hk = 2
    H = Hk * R
    r = gen.rng(1300 + 17 * R + T + bits)
    msl = T + 1
    kv_dim, q_dim = Hk * D, H * D
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * max(T, 1024), dtype=torch.float32, device="cuda")
    kv.set_prefill_form(form)
    try:
        if bits:
            ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, 1, Hk, msl, [T], bits)
            oracle.turbo_gqa_prefill_attention(want, q, ck[0], cv[0], kn[0], vn[0], rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, bits)
            kv.launch_turbo_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), dev(kn[0]), dev(vn[0]),
                                                  dev(rotation_fixture), scratch, T, msl, H, Hk, D, q_dim, kv_dim, bits)
        else:
            ck, cv = build_fp16_cache(r, 1, msl, kv_dim)
            oracle.gqa_prefill_attention(want, q, ck[0], cv[0], T, msl, H, Hk, D, q_dim, kv_dim)
            kv.launch_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), scratch, T, msl, H, Hk, D, q_dim, kv_dim)
    finally:
        kv.set_prefill_form(0)
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("form", [1, 3, 6])
@pytest.mark.parametrize("Hk,R,T", [(1, 2, 290), (2, 1, 97), (2, 2, 418), (3, 1, 150), (4, 2, 163), (6, 2, 130), (16, 1, 200), (24, 1, 70)])
@pytest.mark.parametrize("bits", [0, 4])
def test_prefill_workgroup_placement_covers_every_block(kv, oracle, rotation_fixture, bits, Hk, R, T, form):
    """The prompt kernels place the workgroups of a KV head on one XCD (8, 16, 24 heads), on 8 / heads of them
    (1, 2, 4 heads, when the block count divides) or leave the grid as it is (3, 6 heads, odd block counts):
    whatever the branch, every (token block, head) is computed exactly once -- the output equals the oracle's
    for head counts and block counts that take each branch, with and without mirrored block pairs."""
    import torch
    H = Hk * R
    r = gen.rng(900 + 31 * Hk + T + bits)
    msl = T + 2
    kv_dim, q_dim = Hk * D, H * D
    q = gen.normal_f16(r, (T, q_dim))
    want = np.zeros((T, q_dim), np.float16)
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * max(T, 1024), dtype=torch.float32, device="cuda")
    kv.set_prefill_form(form)
    try:
        if bits:
            ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, 1, Hk, msl, [T], bits)
            oracle.turbo_gqa_prefill_attention(want, q, ck[0], cv[0], kn[0], vn[0], rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, bits)
            kv.launch_turbo_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), dev(kn[0]), dev(vn[0]),
                                                  dev(rotation_fixture), scratch, T, msl, H, Hk, D, q_dim, kv_dim, bits)
        else:
            ck, cv = build_fp16_cache(r, 1, msl, kv_dim)
            oracle.gqa_prefill_attention(want, q, ck[0], cv[0], T, msl, H, Hk, D, q_dim, kv_dim)
            kv.launch_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), scratch, T, msl, H, Hk, D, q_dim, kv_dim)
    finally:
        kv.set_prefill_form(0)
    got = host(out)
    assert np.abs(got.astype(np.float32)).sum(axis=1).min() > 0, "a token block was left out"
    assert rel_err(got, want) <= TOL


@pytest.mark.parametrize("bits,H,Hk,T,pad", [(4, 16, 8, 333, 64), (2, 8, 4, 200, 8), (4, 8, 4, 150, 4), (2, 4, 4, 95, 1024)])
def test_turbo_prefill_strided_rows_scratch_untouched(kv, oracle, rotation_fixture, bits, H, Hk, T, pad):
    """Compressed prefill with rows of q and out wider than the heads (q_dim = H * 128 + pad; a pad of 4 halves
    leaves the rows 8-byte aligned only, which the matrix-core prompt kernel does not take).  That kernel keeps
    nothing in the scratch: it comes back as it went in.  The padding of out stays untouched."""
    import torch
    r = gen.rng(390 + bits + H + T)
    msl = T + 5
    kv_dim, q_dim = Hk * D, H * D + pad
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, 1, Hk, msl, [T], bits)
    q = gen.normal_f16(r, (T, q_dim))
    want = np.full((T, q_dim), 7.0, np.float16)
    oracle.turbo_gqa_prefill_attention(want, q, ck[0], cv[0], kn[0], vn[0], rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    assert (want[:, H * D:] == 7.0).all()
    out = torch.full((T, q_dim), 7.0, dtype=torch.float16, device="cuda")
    scratch = torch.full((T * H * T,), float("nan"), dtype=torch.float32, device="cuda")
    kv.launch_turbo_gqa_prefill_attention(out, dev(q), dev(ck[0]), dev(cv[0]), dev(kn[0]), dev(vn[0]),
                                          dev(rotation_fixture), scratch, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    got = host(out)
    if pad % 8 == 0:
        assert bool(torch.isnan(scratch).all())
    assert (got[:, H * D:] == 7.0).all()
    err = rel_err(got[:, :H * D], want[:, :H * D])
    assert err <= TOL, err


@pytest.mark.parametrize("bits", [4, 2])
def test_golden_case_on_gpu(kv, rotation_fixture, bits):
    """Committed vectors: append 37 tokens on the GPU, compare every byte, then attention."""
    z = np.load(Path(__file__).parent / "golden" / f"case_tq{bits}_g2_h4_ctx37.npz")
    G, H, Hk, ctx, msl = (int(z[k]) for k in ("G", "H", "Hk", "ctx", "msl"))
    kv_dim, q_dim = Hk * D, H * D
    import torch
    bufs = [dev(np.zeros_like(z[k])) for k in ("ck", "kn", "cv", "vn")]
    pos = torch.zeros(G, dtype=torch.int32, device="cuda")
    rot = dev(rotation_fixture)
    for t in range(ctx + 1):
        kv.tw_turbo_kv_append_batch(bufs[0], bufs[1], bufs[2], bufs[3], dev(z["k_rows"][t]), dev(z["v_rows"][t]), rot,
                                    pos, msl, G, Hk, D, kv_dim, bits)
        if t < ctx:
            kv.launch_increment_positions(pos, G)
    for b, k in zip(bufs, ("ck", "kn", "cv", "vn")):
        assert_bytes_equal(host(b), z[k], k, z["last_margin"])
    assert np.array_equal(host(pos), z["pos"])
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.launch_turbo_gqa_attention_batch(out, dev(z["q"]), bufs[0], bufs[2], bufs[1], bufs[3], rot, scratch, pos, msl, G,
                                        H, Hk, D, q_dim, kv_dim, bits)
    assert rel_err(host(out), z["out"]) <= TOL


# ------------------------------------------------------------------ paged cache
@pytest.mark.parametrize("bits", [4, 2, 0])
def test_paged_cache_equals_contiguous(kv, oracle, rotation_fixture, bits):
    """16-token pages in shuffled order: pages gathered in block-table order are the
    contiguous oracle cache byte for byte, and attention over them is the same."""
    import torch
    r = gen.rng(400 + bits)
    G, H, Hk = 5, 8, 4
    kv_dim, q_dim = Hk * D, H * D
    pages_per_seq = 9
    msl = pages_per_seq * 16
    lens = np.array([1, 16, 17, 100, 144])
    steps = 3                                   # append 3 more tokens on the GPU per sequence
    bt = gen.shuffled_block_table(r, G, pages_per_seq)
    n_pages = G * pages_per_seq
    rot = dev(rotation_fixture)
    if bits == 0:
        ck, cv = build_fp16_cache(r, G, msl, kv_dim)
        for g in range(G):
            ck[g, lens[g] - steps:] = 0; cv[g, lens[g] - steps:] = 0
        row_bytes = kv_dim * 2
    else:
        ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, np.maximum(lens - steps, 0), bits)
        row_bytes = kv_dim * bits // 8

    def scatter(contig, width, dtype):
        pool = np.zeros((n_pages, 16, width), dtype)
        for g in range(G):
            for i in range(pages_per_seq):
                pool[bt[g, i]] = contig[g, 16 * i:16 * (i + 1)]
        return pool

    def gather(pool):
        return np.stack([np.concatenate([pool[bt[g, i]] for i in range(pages_per_seq)]) for g in range(G)])

    start = np.maximum(lens - steps, 0).astype(np.int32)
    if bits == 0:
        p_ck, p_cv = dev(scatter(ck, kv_dim, np.float16)), dev(scatter(cv, kv_dim, np.float16))
    else:
        p_ck, p_cv = dev(scatter(ck, row_bytes, np.uint8)), dev(scatter(cv, row_bytes, np.uint8))
        p_kn, p_vn = dev(scatter(kn, Hk, np.float16)), dev(scatter(vn, Hk, np.float16))
    d_bt = dev(bt)
    pos = start.copy()
    for s in range(steps):
        live = pos < lens
        k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
        # sequences shorter than `steps` tokens stay where they are and rewrite the same row
        wpos = np.where(live, pos, lens - 1).astype(np.int32)
        if bits == 0:
            oracle.kv_cache_write_batch(ck, cv, k, v, wpos, msl, G, kv_dim)
            kv.tw_paged_kv_cache_write_batch(p_ck, p_cv, dev(k), dev(v), dev(wpos), d_bt, pages_per_seq, G, kv_dim)
        else:
            oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, wpos, msl, G, Hk, D, kv_dim, bits)
            oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, wpos, msl, G, Hk, D, kv_dim, bits)
            kv.tw_paged_turbo_kv_append_batch(p_ck, p_kn, p_cv, p_vn, dev(k), dev(v), rot, dev(wpos), d_bt,
                                              pages_per_seq, G, Hk, D, kv_dim, bits)
        pos = np.where(live, pos + 1, pos)
    assert_bytes_equal(gather(host(p_ck)), ck, "paged K")
    assert_bytes_equal(gather(host(p_cv)), cv, "paged V")
    if bits:
        assert_bytes_equal(gather(host(p_kn)), kn, "paged K norms")
        assert_bytes_equal(gather(host(p_vn)), vn, "paged V norms")

    apos = (lens - 1).astype(np.int32)
    q = gen.normal_f16(r, (G, q_dim))
    want = np.zeros((G, q_dim), np.float16)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    ws = torch.zeros(kv.attention_workspace_floats(G, H, msl), dtype=torch.float32, device="cuda")
    if bits == 0:
        oracle.gqa_attention_batch(want, q, ck, cv, apos, msl, G, H, Hk, D, q_dim, kv_dim)
        kv.tw_paged_gqa_attention_batch(out, dev(q), p_ck, p_cv, ws, dev(apos), d_bt, pages_per_seq, msl, G, H, Hk, D,
                                        q_dim, kv_dim)
    else:
        oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, apos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
        kv.tw_paged_turbo_gqa_attention_batch(out, dev(q), p_ck, p_cv, p_kn, p_vn, rot, ws, dev(apos), d_bt,
                                              pages_per_seq, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("ragged", [False, True])
@pytest.mark.parametrize("H", [8, 16, 32])
def test_tq2_eight_kv_heads_paged_and_contiguous(kv, oracle, rotation_fixture, H, ragged):
    """2-bit cache with 8 KV heads (256-byte rows: the scan whose waves load whole rows together), GQA
    groups of 1, 2 and 4, over shuffled 16-token pages and over the contiguous layout, with nearly equal
    lengths (even chunks) and with very unequal ones (balanced walk), for several split counts."""
    import torch
    bits, Hk = 2, 8
    r = gen.rng(430 + H + int(ragged))
    lens = np.array([1, 15, 16, 17, 31, 32, 33, 64, 65, 700, 1023, 1024] if ragged else [1000, 1001, 1023, 1024, 990, 1024])
    G = len(lens)
    kv_dim, q_dim = Hk * D, H * D
    pages_per_seq = 64
    msl = pages_per_seq * 16
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits, outliers=False)
    bt = gen.shuffled_block_table(r, G, pages_per_seq)
    n_pages = G * pages_per_seq

    def scatter(contig, width, dtype):
        pool = np.full((n_pages, 16, width), 0, dtype)
        for g in range(G):
            for i in range(pages_per_seq):
                pool[bt[g, i]] = contig[g, 16 * i:16 * (i + 1)]
        return pool

    p_ck, p_cv = dev(scatter(ck, kv_dim // 4, np.uint8)), dev(scatter(cv, kv_dim // 4, np.uint8))
    p_kn, p_vn = dev(scatter(kn, Hk, np.float16)), dev(scatter(vn, Hk, np.float16))
    q = gen.normal_f16(r, (G, q_dim))
    pos = (lens - 1).astype(np.int32)
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    rot, d_q, d_pos, d_bt = dev(rotation_fixture), dev(q), dev(pos), dev(bt)
    d_c = [dev(x) for x in (ck, cv, kn, vn)]
    ws = torch.full((kv.attention_workspace_floats(G, H, msl),), float("nan"), dtype=torch.float32, device="cuda")
    try:
        for nsplit in (0, 1, 3, 8):
            kv.set_num_splits(nsplit)
            out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
            kv.tw_paged_turbo_gqa_attention_batch(out, d_q, p_ck, p_cv, p_kn, p_vn, rot, ws, d_pos, d_bt,
                                                  pages_per_seq, msl, G, H, Hk, D, q_dim, kv_dim, bits)
            err = rel_err(host(out), want)
            assert err <= TOL, f"paged, nsplit={nsplit}: {err}"
            out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
            scratch = torch.full((G * H * msl,), float("nan"), dtype=torch.float32, device="cuda")
            kv.launch_turbo_gqa_attention_batch(out, d_q, d_c[0], d_c[1], d_c[2], d_c[3], rot, scratch, d_pos, msl, G, H, Hk,
                                                D, q_dim, kv_dim, bits)
            err = rel_err(host(out), want)
            assert err <= TOL, f"contiguous, nsplit={nsplit}: {err}"
    finally:
        kv.set_num_splits(0)


# ------------------------------------------------------------------ producers of q and k: RMSNorm and RoPE
def rope_tables(msl, rope_dim, theta=1e6):
    d = np.arange(rope_dim // 2, dtype=np.float64)
    ang = np.arange(msl, dtype=np.float64)[:, None] * theta ** (-2.0 * d / rope_dim)[None, :]
    return np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)


def producer_inputs(r, G, H, Hk, q_dim, kv_dim):
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim))
    q[0] = (q[0].astype(np.float32) * 30).astype(np.float16)
    k[G - 1] = (k[G - 1].astype(np.float32) * 1e-3).astype(np.float16)
    k[0, :D] = 0                                         # a zero head: rms = 1/sqrt(eps)
    qw = (1.0 + 0.3 * r.standard_normal(D)).astype(np.float16)
    kw = (1.0 + 0.3 * r.standard_normal(D)).astype(np.float16)
    return q, k, qw, kw


@pytest.mark.parametrize("biased", [False, True])
def test_qk_norm_batch_bit_exact(kv, oracle, biased):
    r = gen.rng(700 + biased)
    G, H, Hk = 37, 16, 8
    q_dim, kv_dim = 2 * H * D, Hk * D            # gated projection: the second half of a q row is the gate
    q, k, qw, kw = producer_inputs(r, G, H, Hk, q_dim, kv_dim)
    d_q, d_k = dev(q), dev(k)
    kv.launch_qk_norm_batch(d_q, d_k, dev(qw), dev(kw), H, Hk, D, G, 1e-6, q_dim, kv_dim, biased=biased)
    oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, 1e-6, q_dim, kv_dim, biased)
    assert_bytes_equal(host(d_q), q, "normalised q")
    assert_bytes_equal(host(d_k), k, "normalised k")


@pytest.mark.parametrize("rope_dim", [128, 64, 32, 48])
def test_rope_batch_bit_exact(kv, oracle, rope_dim):
    r = gen.rng(710 + rope_dim)
    G, H, Hk, msl = 29, 8, 2, 4096
    q_dim, kv_dim = H * D + 64, Hk * D
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim))
    ct, st = rope_tables(msl, rope_dim)
    pos = r.integers(0, msl, G).astype(np.int32); pos[0] = 0; pos[1] = msl - 1
    d_q, d_k = dev(q), dev(k)
    kv.launch_rope_batch(d_q, d_k, dev(ct), dev(st), dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, rope_dim)
    oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, rope_dim)
    assert_bytes_equal(host(d_q), q, "rotated q")
    assert_bytes_equal(host(d_k), k, "rotated k")


def test_qk_norm_and_rope_single_sequence_bit_exact(kv, oracle):
    r = gen.rng(720)
    H, Hk, msl = 16, 8, 777
    q = gen.normal_f16(r, (H * D,)); k = gen.normal_f16(r, (Hk * D,))
    qw = (1.0 + 0.3 * r.standard_normal(D)).astype(np.float16); kw = (0.7 * r.standard_normal(D)).astype(np.float16)
    ct, st = rope_tables(msl, D, theta=10000.0)
    d_q, d_k = dev(q), dev(k)
    kv.launch_qk_norm(d_q, d_k, dev(qw), dev(kw), H, Hk, D, 1e-6)
    oracle.qk_norm(q, k, qw, kw, H, Hk, D, 1e-6)
    assert_bytes_equal(host(d_q), q, "normalised q"); assert_bytes_equal(host(d_k), k, "normalised k")
    kv.launch_rope(d_q, d_k, dev(ct), dev(st), 613, msl, H, Hk, D)
    oracle.rope(q, k, ct, st, 613, msl, H, Hk, D)
    assert_bytes_equal(host(d_q), q, "rotated q"); assert_bytes_equal(host(d_k), k, "rotated k")


def test_producer_rejects_unsupported_shapes(kv):
    import torch
    q = torch.zeros(2, 256, dtype=torch.float16, device="cuda"); k = torch.zeros(2, 256, dtype=torch.float16, device="cuda")
    w = torch.ones(128, dtype=torch.float16, device="cuda")
    pos = torch.zeros(2, dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="head_dim"):
        kv.launch_qk_norm_batch(q, k, w, w, 4, 4, 64, 2, 1e-6, 256, 256)
    with pytest.raises(RuntimeError, match="rope_dim"):
        kv.launch_rope_batch(q, k, w, w, pos, 16, 2, 2, 2, 128, 256, 256, 96)


@pytest.mark.parametrize("variant,one_launch", [(0, 1), (0, 2), (1, 0)])
@pytest.mark.parametrize("bits,H,Hk,norm,rope_dim,biased", [
    (4, 16, 8, True, 128, False), (2, 16, 8, True, 128, False), (4, 32, 8, True, 64, False), (2, 8, 8, False, 128, False),
    (4, 16, 8, True, 0, False), (4, 16, 8, True, 48, True), (2, 32, 8, True, 32, True), (4, 8, 2, True, 16, False)])
def test_fused_norm_rope_turbo_step(kv, oracle, rotation_fixture, bits, H, Hk, norm, rope_dim, biased, variant, one_launch):
    """RMSNorm + RoPE + append + attention in one call == the oracle's four steps: cache bytes bit for
    bit, output within the attention tolerance.  One kernel for the whole step (one_launch 1), the three-kernel
    path with the producers inside its rotation launch (2), and variant 1: the kernels of their own."""
    import torch
    r = gen.rng(730 + bits + H + rope_dim)
    G, msl = 9, 384
    kv_dim, q_dim = Hk * D, H * D
    lens = [1, 33, 64, 100, 257, 300, 319, 200, 383]
    ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, bits, outliers=False)
    pos = np.array(lens, np.int32)
    pos[8] = 383
    q, k, qw, kw = producer_inputs(r, G, H, Hk, q_dim, kv_dim)
    v = gen.normal_f16(r, (G, kv_dim))
    ct, st = rope_tables(msl, rope_dim) if rope_dim else (None, None)
    d_ck, d_cv, d_kn, d_vn = dev(ck), dev(cv), dev(kn), dev(vn)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.set_attention_variant(variant)
    kv.set_decode_fused(one_launch)
    try:
        kv.tw_qk_norm_rope_turbo_append_attention_batch(
            out, dev(q), dev(k), dev(v), dev(qw) if norm else None, dev(kw) if norm else None, 1e-6, biased,
            dev(ct) if rope_dim else None, dev(st) if rope_dim else None, rope_dim, d_ck, d_cv, d_kn, d_vn,
            dev(rotation_fixture), scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, bits)
    finally:
        kv.set_attention_variant(0)
        kv.set_decode_fused(0)
    if norm:
        oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, 1e-6, q_dim, kv_dim, biased)
    if rope_dim:
        oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, rope_dim)
    oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
    want = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert_bytes_equal(host(d_ck), ck, "K codes"); assert_bytes_equal(host(d_cv), cv, "V codes")
    assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")
    assert rel_err(host(out), want) <= TOL


@pytest.mark.parametrize("rope_dim", [128, 64])
def test_fused_norm_rope_fp16_step(kv, oracle, rope_dim):
    """fp16 cache: one launch normalises and rotates q in place and writes the transformed K rows and the
    V rows to the cache; q and the cache are the oracle's bit for bit."""
    import torch
    r = gen.rng(740 + rope_dim)
    G, H, Hk, msl = 6, 16, 8, 160
    kv_dim, q_dim = Hk * D, H * D
    ck, cv = build_fp16_cache(r, G, msl, kv_dim)
    pos = np.array([0, 1, 17, 64, 100, 159], np.int32)
    for g in range(G):
        ck[g, pos[g]:] = 0; cv[g, pos[g]:] = 0
    q, k, qw, kw = producer_inputs(r, G, H, Hk, q_dim, kv_dim)
    v = gen.normal_f16(r, (G, kv_dim))
    ct, st = rope_tables(msl, rope_dim)
    d_q, d_ck, d_cv = dev(q), dev(ck), dev(cv)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.tw_qk_norm_rope_append_attention_batch(out, d_q, dev(k), dev(v), dev(qw), dev(kw), 1e-6, True, dev(ct), dev(st),
                                              rope_dim, d_ck, d_cv, scratch, dev(pos), msl, G, H, Hk, D, q_dim, kv_dim)
    oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, 1e-6, q_dim, kv_dim, True)
    oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, rope_dim)
    oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
    want = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    assert_bytes_equal(host(d_q), q, "q after the call")
    assert_bytes_equal(host(d_ck), ck, "K cache"); assert_bytes_equal(host(d_cv), cv, "V cache")
    assert rel_err(host(out), want) <= TOL


# ------------------------------------------------------------------ gated attention and the whole layer step
def test_sigmoid_gate_batch(kv, oracle):
    """Elementwise floating point (expf, division): within one fp16 step of the oracle."""
    r = gen.rng(750)
    dim, G = 2048, 37
    data = gen.normal_f16(r, (G, dim)); gate = (3 * r.standard_normal((G, dim))).astype(np.float16)
    d_data = dev(data)
    kv.launch_sigmoid_gate_batch(d_data, dev(gate), dim, G)
    oracle.sigmoid_gate_batch(data, gate, dim, G)
    got = host(d_data).astype(np.float64); want = data.astype(np.float64)
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-4)) <= 2 ** -10
    assert np.mean(host(d_data).view(np.uint16) == data.view(np.uint16)) > 0.999


@pytest.mark.parametrize("kv_bits,nsplit,G", [(4, 0, 6), (2, 0, 6), (0, 0, 6), (0, 1, 6), (4, 1, 6), (0, 0, 18)])
def test_layer_attention_step_with_gate(kv, oracle, rotation_fixture, kv_bits, nsplit, G):
    """Producers + append + attention + sigmoid gate through one call, with the gate in the second half of
    the q rows (gated q projection: row stride 2*H*D) == the oracle's six steps."""
    import torch
    r = gen.rng(760 + kv_bits + nsplit)
    H, Hk, msl = 16, 8, 160
    kv_dim, q_dim = Hk * D, 2 * H * D
    lens = np.resize(np.array([1, 2, 17, 64, 100, 159]), G)     # 18 sequences: the fp16 scan that reads whole rows
    pos = lens.astype(np.int32)
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
    qw = (1.0 + 0.2 * r.standard_normal(D)).astype(np.float16); kw = (1.0 + 0.2 * r.standard_normal(D)).astype(np.float16)
    ct, st = rope_tables(msl, D)
    if kv_bits:
        ck, cv, kn, vn = build_turbo_cache(oracle, rotation_fixture, r, G, Hk, msl, lens, kv_bits, outliers=False)
        d_kn, d_vn, d_rot = dev(kn), dev(vn), dev(rotation_fixture)
    else:
        ck, cv = build_fp16_cache(r, G, msl, kv_dim)
        for g in range(G):
            ck[g, pos[g]:] = 0; cv[g, pos[g]:] = 0
        d_kn = d_vn = d_rot = None
    d_q, d_ck, d_cv = dev(q), dev(ck), dev(cv)
    out = torch.zeros((G, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(G * H * msl, dtype=torch.float32, device="cuda")
    kv.set_num_splits(nsplit)
    try:
        kv.tw_layer_attention_step(out, d_q, dev(k), dev(v), dev(pos), msl, G, H, Hk, D, q_dim, kv_dim, d_ck, d_cv, scratch,
                                   kv_bits=kv_bits, k_norms=d_kn, v_norms=d_vn, rotation=d_rot, q_weight=dev(qw),
                                   k_weight=dev(kw), eps=1e-6, cos_table=dev(ct), sin_table=dev(st), rope_dim=D,
                                   gate=d_q, gate_stride=q_dim, gate_offset=H * D)
    finally:
        kv.set_num_splits(0)
    gate_rows = q[:, H * D:].copy()
    oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, 1e-6, q_dim, kv_dim, False)
    oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, D)
    want = np.zeros((G, q_dim), np.float16)
    if kv_bits:
        oracle.turbo_kv_quantize_batch(ck, kn, k, rotation_fixture, pos, msl, G, Hk, D, kv_dim, kv_bits)
        oracle.turbo_kv_quantize_batch(cv, vn, v, rotation_fixture, pos, msl, G, Hk, D, kv_dim, kv_bits)
        oracle.turbo_gqa_attention_batch(want, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, kv_bits)
        assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")
    else:
        oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
        oracle.gqa_attention_batch(want, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    assert_bytes_equal(host(d_ck), ck, "K cache"); assert_bytes_equal(host(d_cv), cv, "V cache")
    attn = np.ascontiguousarray(want[:, :H * D])
    oracle.sigmoid_gate_batch(attn, np.ascontiguousarray(gate_rows), H * D, G)
    got = host(out)
    assert rel_err(got[:, :H * D], attn) <= TOL
    assert not got[:, H * D:].any(), "the gate half of the output rows is not written"
    # the gate half of q is an input only
    assert_bytes_equal(host(d_q)[:, H * D:], gate_rows, "gate rows")


@pytest.mark.parametrize("bits,T", [(4, 77), (2, 300)])
def test_turbo_kv_append_tokens(kv, oracle, rotation_fixture, bits, T):
    """K and V rows of a prompt in one launch == the oracle's two T-token appends, bit for bit; positions in
    any order, rows that are not written stay as they are."""
    r = gen.rng(810 + bits)
    Hk, msl = 8, T + 20
    kv_dim = Hk * D
    kvp = kv_dim * bits // 8
    pos = r.permutation(msl)[:T].astype(np.int32)
    k = gen.kv_rows_with_outliers(r, (T, kv_dim), kv_dim)[0]; v = gen.normal_f16(r, (T, kv_dim))
    ck = r.integers(0, 256, (msl, kvp), dtype=np.uint8); cv = r.integers(0, 256, (msl, kvp), dtype=np.uint8)
    kn = gen.normal_f16(r, (msl, Hk)); vn = gen.normal_f16(r, (msl, Hk))
    d_ck, d_cv, d_kn, d_vn = dev(ck), dev(cv), dev(kn), dev(vn)
    kv.tw_turbo_kv_append_tokens(d_ck, d_kn, d_cv, d_vn, dev(k), dev(v), dev(rotation_fixture), dev(pos), msl, T, Hk, D,
                                 kv_dim, bits)
    oracle.turbo_kv_quantize(ck, kn, k, rotation_fixture, pos, msl, T, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize(cv, vn, v, rotation_fixture, pos, msl, T, Hk, D, kv_dim, bits)
    assert_bytes_equal(host(d_ck), ck, "K codes"); assert_bytes_equal(host(d_cv), cv, "V codes")
    assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")


@pytest.mark.parametrize("kv_bits,T,producers,gated", [(4, 333, True, True), (2, 200, True, False), (0, 150, True, True),
                                                       (4, 97, False, False), (0, 70, False, True), (2, 40, False, True)])
def test_layer_prompt_step(kv, oracle, rotation_fixture, kv_bits, T, producers, gated):
    """A layer over a prompt in one call (producers of q and k, T-token append into sequence 0, causal
    attention, sigmoid gate; prefill_chunked, engine.cpp:2097-2150) == the oracle's steps one by one: the
    cache bit for bit, the output within the attention tolerance.  Gated rows: q_dim = 2*H*D, the gate in the
    second half of the q rows."""
    import torch
    r = gen.rng(820 + kv_bits + T)
    H, Hk, msl = 8, 4, T + 11
    kv_dim = Hk * D
    q_dim = 2 * H * D if gated else H * D
    pos = np.arange(T, dtype=np.int32)
    q = gen.normal_f16(r, (T, q_dim)); k = gen.kv_rows_with_outliers(r, (T, kv_dim), kv_dim)[0]; v = gen.normal_f16(r, (T, kv_dim))
    qw = (1.0 + 0.2 * r.standard_normal(D)).astype(np.float16); kw = (1.0 + 0.2 * r.standard_normal(D)).astype(np.float16)
    ct, st = rope_tables(msl, D)
    kvp = kv_dim * kv_bits // 8 if kv_bits else kv_dim
    ck = np.zeros((msl, kvp), np.uint8 if kv_bits else np.float16); cv = np.zeros_like(ck)
    kn = np.zeros((msl, Hk), np.float16); vn = np.zeros_like(kn)
    d_q, d_k, d_ck, d_cv, d_kn, d_vn = dev(q), dev(k), dev(ck), dev(cv), dev(kn), dev(vn)
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    scratch = torch.zeros(T * H * max(T, 1024), dtype=torch.float32, device="cuda")
    extra = {}
    if producers:
        extra = dict(q_weight=dev(qw), k_weight=dev(kw), eps=1e-6, cos_table=dev(ct), sin_table=dev(st), rope_dim=D)
    if gated:
        extra.update(gate=d_q, gate_stride=q_dim, gate_offset=H * D)
    kv.tw_layer_prompt_step(out, d_q, d_k, dev(v), dev(pos), msl, T, H, Hk, D, q_dim, kv_dim, d_ck, d_cv, scratch,
                            kv_bits=kv_bits, k_norms=d_kn if kv_bits else None, v_norms=d_vn if kv_bits else None,
                            rotation=dev(rotation_fixture) if kv_bits else None, **extra)
    gate_rows = q[:, H * D:].copy()
    if producers:
        oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, T, 1e-6, q_dim, kv_dim, False)
        oracle.rope_batch(q, k, ct, st, pos, msl, T, H, Hk, D, q_dim, kv_dim, D)
    want = np.zeros((T, q_dim), np.float16)
    if kv_bits:
        oracle.turbo_kv_quantize(ck, kn, k, rotation_fixture, pos, msl, T, Hk, D, kv_dim, kv_bits)
        oracle.turbo_kv_quantize(cv, vn, v, rotation_fixture, pos, msl, T, Hk, D, kv_dim, kv_bits)
        oracle.turbo_gqa_prefill_attention(want, q, ck, cv, kn, vn, rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, kv_bits)
        assert_bytes_equal(host(d_kn), kn, "K norms"); assert_bytes_equal(host(d_vn), vn, "V norms")
    else:
        ck[:T] = k; cv[:T] = v                                    # engine.cpp:2115-2118
        oracle.gqa_prefill_attention(want, q, ck, cv, T, msl, H, Hk, D, q_dim, kv_dim)
    assert_bytes_equal(host(d_ck), ck, "K cache"); assert_bytes_equal(host(d_cv), cv, "V cache")
    assert_bytes_equal(host(d_q)[:, :H * D], q[:, :H * D], "q after its producers")
    attn = np.ascontiguousarray(want[:, :H * D])
    if gated:
        oracle.sigmoid_gate_batch(attn, np.ascontiguousarray(gate_rows), H * D, T)
        assert_bytes_equal(host(d_q)[:, H * D:], gate_rows, "gate rows")
    got = host(out)
    assert rel_err(got[:, :H * D], attn) <= TOL
    assert not got[:, H * D:].any()


# ------------------------------------------------------------------ engine: append -> attention -> positions, eager and graph
@pytest.mark.parametrize("kv_bits", [0, 4, 2])
@pytest.mark.parametrize("use_graph", [False, True])
def test_engine_decode_steps(oracle, kv_bits, use_graph):
    import torch
    from triebwerk_amd import Engine
    r = gen.rng(500 + kv_bits)
    L, H, Hk, G, msl, steps = 3, 16, 8, 5, 48, 6
    kv_dim, q_dim = Hk * D, H * D
    eng = Engine(max_seq_len=1024, kv_bits=kv_bits)
    assert eng.kv_bits() == kv_bits
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    start = np.array([0, 3, 10, 31, 41], np.int32)
    eng.set_positions(start)
    rot = None
    if kv_bits:
        rot = host(eng.rotation())
        assert np.array_equal(rot.view(np.uint16), oracle.make_rotation(128, 42)[0].view(np.uint16))
    # oracle-side caches
    if kv_bits == 0:
        o_k = [np.zeros((G, msl, kv_dim), np.float16) for _ in range(L)]
        o_v = [np.zeros((G, msl, kv_dim), np.float16) for _ in range(L)]
    else:
        kvp = kv_dim * kv_bits // 8
        o_k = [np.zeros((G, msl, kvp), np.uint8) for _ in range(L)]; o_v = [np.zeros((G, msl, kvp), np.uint8) for _ in range(L)]
        o_kn = [np.zeros((G, msl, Hk), np.float16) for _ in range(L)]; o_vn = [np.zeros((G, msl, Hk), np.float16) for _ in range(L)]
    pos = start.copy()
    # the graph replays fixed buffers: inputs are copied into them before every step
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
            eng.decode_step(d_q, d_k, d_v, d_out, use_graph=use_graph, stream=stream)
        stream.synchronize()
        got = host(d_out)
        for l in range(L):
            want = np.zeros((G, q_dim), np.float16)
            if kv_bits == 0:
                oracle.kv_cache_write_batch(o_k[l], o_v[l], k[l], v[l], pos, msl, G, kv_dim)
                oracle.gqa_attention_batch(want, q[l], o_k[l], o_v[l], pos, msl, G, H, Hk, D, q_dim, kv_dim)
            else:
                oracle.turbo_kv_quantize_batch(o_k[l], o_kn[l], k[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_kv_quantize_batch(o_v[l], o_vn[l], v[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_gqa_attention_batch(want, q[l], o_k[l], o_v[l], o_kn[l], o_vn[l], rot, pos, msl, G, H, Hk, D,
                                                 q_dim, kv_dim, kv_bits)
            err = rel_err(got[l], want)
            assert err <= TOL, f"step {step} layer {l}: {err}"
        oracle.increment_positions(pos, G)
        assert np.array_equal(host(eng.positions()), pos)
    for l in range(L):
        c = eng.cache(l)
        assert_bytes_equal(host(c[0]), o_k[l], f"layer {l} K cache")
        assert_bytes_equal(host(c[1]), o_v[l], f"layer {l} V cache")
        if kv_bits:
            assert_bytes_equal(host(c[2]), o_kn[l], f"layer {l} K norms")
            assert_bytes_equal(host(c[3]), o_vn[l], f"layer {l} V norms")
    eng.reset()
    assert not host(eng.cache(0)[0]).any() and not host(eng.positions()).any()


@pytest.mark.parametrize("kv_bits", [0, 4, 2])
@pytest.mark.parametrize("mode", [1, 2])
def test_engine_decode_steps_with_producers(oracle, kv_bits, mode):
    """The engine's step with per-layer QK RMSNorm and RoPE, fused (mode 1) or as launches of their own
    (mode 2), captured in a graph: caches bit for bit and outputs within tolerance of the oracle's
    norm -> rope -> append -> attention, over several steps (positions advance, so the table row does)."""
    import torch
    from triebwerk_amd import Engine
    r = gen.rng(560 + kv_bits + mode)
    L, H, Hk, G, msl, steps = 3, 16, 8, 5, 48, 4
    kv_dim, q_dim = Hk * D, H * D
    eng = Engine(max_seq_len=1024, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    start = np.array([0, 3, 10, 31, 41], np.int32)
    eng.set_positions(start)
    rot = host(eng.rotation()) if kv_bits else None
    qn = (1.0 + 0.2 * r.standard_normal((L, D))).astype(np.float16); kn_w = (1.0 + 0.2 * r.standard_normal((L, D))).astype(np.float16)
    ct, st = rope_tables(msl, D)
    eng.set_producers(mode, dev(qn), dev(kn_w), 1e-6, False, dev(ct), dev(st), D)
    if kv_bits == 0:
        o_k = [np.zeros((G, msl, kv_dim), np.float16) for _ in range(L)]
        o_v = [np.zeros((G, msl, kv_dim), np.float16) for _ in range(L)]
    else:
        kvp = kv_dim * kv_bits // 8
        o_k = [np.zeros((G, msl, kvp), np.uint8) for _ in range(L)]; o_v = [np.zeros((G, msl, kvp), np.uint8) for _ in range(L)]
        o_kn = [np.zeros((G, msl, Hk), np.float16) for _ in range(L)]; o_vn = [np.zeros((G, msl, Hk), np.float16) for _ in range(L)]
    pos = start.copy()
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
            ql, kl = q[l].copy(), k[l].copy()
            oracle.qk_norm_batch(ql, kl, qn[l], kn_w[l], H, Hk, D, G, 1e-6, q_dim, kv_dim, False)
            oracle.rope_batch(ql, kl, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, D)
            if kv_bits == 0:
                oracle.kv_cache_write_batch(o_k[l], o_v[l], kl, v[l], pos, msl, G, kv_dim)
                oracle.gqa_attention_batch(want, ql, o_k[l], o_v[l], pos, msl, G, H, Hk, D, q_dim, kv_dim)
            else:
                oracle.turbo_kv_quantize_batch(o_k[l], o_kn[l], kl, rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_kv_quantize_batch(o_v[l], o_vn[l], v[l], rot, pos, msl, G, Hk, D, kv_dim, kv_bits)
                oracle.turbo_gqa_attention_batch(want, ql, o_k[l], o_v[l], o_kn[l], o_vn[l], rot, pos, msl, G, H, Hk, D,
                                                 q_dim, kv_dim, kv_bits)
            err = rel_err(got[l], want)
            assert err <= TOL, f"step {step} layer {l}: {err}"
        oracle.increment_positions(pos, G)
    for l in range(L):
        c = eng.cache(l)
        assert_bytes_equal(host(c[0]), o_k[l], f"layer {l} K cache")
        assert_bytes_equal(host(c[1]), o_v[l], f"layer {l} V cache")
        if kv_bits:
            assert_bytes_equal(host(c[2]), o_kn[l], f"layer {l} K norms")
            assert_bytes_equal(host(c[3]), o_vn[l], f"layer {l} V norms")
    eng.set_producers(0)


def test_engine_sleep_and_wake(oracle):
    """sleep() hands the cache memory back and drops the captured step; after wake() + alloc_batch the
    caches are zero again and a captured step works on the new memory."""
    import torch
    from triebwerk_amd import Engine
    r = gen.rng(570)
    L, H, Hk, G, msl = 2, 16, 8, 3, 32
    kv_dim, q_dim = Hk * D, H * D
    eng = Engine(kv_bits=4)
    eng.set_shape(L, H, Hk, D)
    d_q = dev(gen.normal_f16(r, (L, G, q_dim))); d_k = dev(gen.normal_f16(r, (L, G, kv_dim))); d_v = dev(gen.normal_f16(r, (L, G, kv_dim)))
    d_out = torch.zeros((L, G, q_dim), dtype=torch.float16, device="cuda")
    stream = torch.cuda.Stream()
    outs = []
    for cycle in range(2):
        eng.alloc_batch(G, msl)
        assert eng.is_allocated()
        assert not host(eng.cache(0)[0]).any() and not host(eng.positions()).any()
        with torch.cuda.stream(stream):
            for _ in range(3):
                eng.decode_step(d_q, d_k, d_v, d_out, use_graph=True, stream=stream)
        stream.synchronize()
        assert host(eng.positions()).tolist() == [3] * G
        assert host(eng.cache(1)[0])[:, :3].any()
        outs.append(host(d_out).copy())
        eng.sleep()
        assert not eng.is_allocated()
        with pytest.raises(RuntimeError):
            eng.decode_step(d_q, d_k, d_v, d_out, use_graph=True, stream=stream)
        eng.wake()
    assert_bytes_equal(outs[0], outs[1], "same steps after a sleep / wake cycle")


def test_engine_stop_check_cadence():
    """record_tokens + check_stops against a plain restatement of the reference's loop (engine.cpp:2496-2534):
    checks on steps 7, 15, ... and the last; eos and a two-token stop sequence; sequences that finished keep
    their output; the loop ends on the first check at which all have finished."""
    import torch
    from triebwerk_amd import Engine
    r = gen.rng(580)
    L, H, Hk, G, msl, max_new = 1, 4, 2, 6, 64, 21
    eos, stop = 9, [3, 4]
    eng = Engine(kv_bits=0)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    toks = r.integers(0, 12, (max_new, G)).astype(np.int32)
    toks[:, 5] = 1                      # never stops
    toks[2, 0] = eos                    # stops early
    toks[9, 1], toks[10, 1] = 3, 4      # stop sequence across a check boundary? (steps 9, 10 are in one block)
    toks[7, 2], toks[8, 2] = 3, 4       # stop sequence across the check at step 7
    eng.begin_generation(max_new, eos, stop)
    # model
    outputs = [[] for _ in range(G)]; finished = [False] * G
    last_checked, want_checks, want_done_step = -1, [], None
    for step in range(max_new):
        if not ((step + 1) % 8 == 0 or step + 1 == max_new):
            continue
        want_checks.append(step)
        all_done = True
        for st in range(last_checked + 1, step + 1):
            for g in range(G):
                if finished[g]:
                    continue
                t = int(toks[st, g]); outputs[g].append(t)
                if t == eos or (len(outputs[g]) >= 2 and outputs[g][-2:] == stop):
                    finished[g] = True
                if not finished[g]:
                    all_done = False
        last_checked = step
        if all_done:
            want_done_step = step
            break
    stream = torch.cuda.Stream()
    got_checks, done_step = [], None
    d_tok = torch.zeros(G, dtype=torch.int32, device="cuda")
    for step in range(max_new):
        d_tok.copy_(dev(toks[step]))
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            eng.record_tokens(d_tok, step, stream=stream)
        done, checked = eng.check_stops(step, stream=stream)
        if checked:
            got_checks.append(step)
        if done:
            done_step = step
            break
    assert got_checks == want_checks and done_step == want_done_step
    for g in range(G):
        out, fin = eng.output(g)
        assert out == outputs[g] and fin == finished[g], g
    assert not finished[5] and finished[0] and outputs[0] == [int(x) for x in toks[:3, 0]]


@pytest.mark.parametrize("kv_bits,Hk", [(4, 2), (2, 1), (0, 2), (4, 8)])
@pytest.mark.parametrize("src,dst", [(0, (1, 4)), (2, (0, 5)), (4, (1, 3))])
def test_engine_prefix_broadcast(oracle, kv_bits, Hk, src, dst):
    """Rows [0, T) of the source sequence reach every destination in all arrays of all layers (one launch per
    layer); the source, sequences outside the range and rows from T on keep their bytes."""
    import torch
    from triebwerk_amd import Engine
    L, H, G, msl, T = 2, 8, 5, 32, 7
    eng = Engine(kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    gt = torch.Generator(device="cuda"); gt.manual_seed(600 + kv_bits)
    before = []
    for l in range(L):
        arrs = []
        for arr in eng.cache(l):
            if arr is None:
                continue
            raw = arr.view(torch.uint8) if arr.dtype != torch.uint8 else arr
            raw.copy_(torch.randint(0, 256, raw.shape, generator=gt, device="cuda", dtype=torch.uint8))
            arrs.append(host(raw).copy())
        before.append(arrs)
    eng.broadcast_prefix(src, dst[0], dst[1], T)
    torch.cuda.synchronize()
    for l in range(L):
        live = [a for a in eng.cache(l) if a is not None]
        assert len(live) == (2 if kv_bits == 0 else 4)
        for arr, was in zip(live, before[l]):
            now = host(arr.view(torch.uint8) if arr.dtype != torch.uint8 else arr)
            for g in range(G):
                if dst[0] <= g < dst[1] and g != src:
                    assert np.array_equal(now[g, :T], was[src, :T]), (l, g)
                    assert np.array_equal(now[g, T:], was[g, T:]), (l, g)
                else:
                    assert np.array_equal(now[g], was[g]), (l, g)


@pytest.mark.parametrize("kv_bits,mode", [(4, 1), (2, 2), (0, 1), (4, 0)])
def test_engine_prompt_layer_then_broadcast(oracle, rotation_fixture, kv_bits, mode):
    """The engine's prompt call for one sequence of the batch (producers fused, as the reference's two launches,
    or none), then the prefix broadcast: that sequence's cache rows and the output equal the oracle's steps, the
    destinations hold the same rows, everything else keeps its bytes."""
    import torch
    from triebwerk_amd import Engine
    L, H, Hk, G, msl, T, seq = 2, 8, 4, 4, 96, 50, 2
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(880 + kv_bits + mode)
    eng = Engine(max_seq_len=msl, kv_bits=kv_bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    qw = (1.0 + 0.2 * r.standard_normal((L, D))).astype(np.float16); kw = (1.0 + 0.2 * r.standard_normal((L, D))).astype(np.float16)
    ct, st = rope_tables(msl, D)
    if mode:
        eng.set_producers(mode, dev(qw), dev(kw), 1e-6, False, dev(ct), dev(st), D)
    pos = np.arange(T, dtype=np.int32)
    layer = 1
    marks = []
    for arr in eng.cache(layer):
        if arr is not None:
            raw = arr.view(torch.uint8)
            raw.fill_(0x5A)
            marks.append(raw)
    q = gen.normal_f16(r, (T, q_dim)); k = gen.kv_rows_with_outliers(r, (T, kv_dim), kv_dim)[0]; v = gen.normal_f16(r, (T, kv_dim))
    out = torch.zeros((T, q_dim), dtype=torch.float16, device="cuda")
    eng.prompt_layer(layer, seq, dev(q), dev(k), dev(v), out, dev(pos))
    if mode:
        oracle.qk_norm_batch(q, k, qw[layer], kw[layer], H, Hk, D, T, 1e-6, q_dim, kv_dim, False)
        oracle.rope_batch(q, k, ct, st, pos, msl, T, H, Hk, D, q_dim, kv_dim, D)
    want = np.zeros((T, q_dim), np.float16)
    if kv_bits:
        kvp = kv_dim * kv_bits // 8
        ck = np.full((msl, kvp), 0x5A, np.uint8); cv = ck.copy()
        kn = np.full((msl, Hk), 0x5A5A, np.uint16).view(np.float16); vn = kn.copy()
        oracle.turbo_kv_quantize(ck, kn, k, rotation_fixture, pos, msl, T, Hk, D, kv_dim, kv_bits)
        oracle.turbo_kv_quantize(cv, vn, v, rotation_fixture, pos, msl, T, Hk, D, kv_dim, kv_bits)
        oracle.turbo_gqa_prefill_attention(want, q, ck, cv, kn, vn, rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, kv_bits)
        expect = [ck, cv, kn.view(np.uint8).reshape(msl, -1), vn.view(np.uint8).reshape(msl, -1)]
    else:
        ck = np.full((msl, kv_dim), 0x5A5A, np.uint16).view(np.float16); cv = ck.copy()
        ck[:T] = k; cv[:T] = v
        oracle.gqa_prefill_attention(want, q, ck, cv, T, msl, H, Hk, D, q_dim, kv_dim)
        expect = [ck.view(np.uint8).reshape(msl, -1), cv.view(np.uint8).reshape(msl, -1)]
    assert rel_err(host(out), want) <= TOL
    for raw, exp in zip(marks, expect):
        now = host(raw).reshape(G, msl, -1)
        assert np.array_equal(now[seq], exp)
        for g in range(G):
            if g != seq:
                assert (now[g] == 0x5A).all()
    eng.broadcast_prefix(seq, 0, G, T)
    for raw, exp in zip(marks, expect):
        now = host(raw).reshape(G, msl, -1)
        for g in range(G):
            assert np.array_equal(now[g, :T], exp[:T]), g
            assert g == seq or (now[g, T:] == 0x5A).all()


def test_plain_read_bandwidth_probe(kv):
    """The calibration kernel the benchmark quotes: plausible on a large buffer, an error on a bad one."""
    import ctypes as C
    import torch
    from triebwerk_amd import _lib
    lib = _lib.load()
    buf = torch.ones(1 << 30, dtype=torch.uint8, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    gbps = lib.tw_kv_measure_read_bandwidth(C.c_void_p(buf.data_ptr()), C.c_size_t(buf.numel()), 2, C.c_void_p(s))
    assert 1000.0 < gbps < 8000.0, gbps          # above any PCIe or cache-less rate, below the HBM peak
    assert torch.all(buf == 1)                   # it only reads
    lib.tw_kv_clear_error()
    assert lib.tw_kv_measure_read_bandwidth(C.c_void_p(buf.data_ptr() + 1), C.c_size_t(1 << 20), 1, C.c_void_p(s)) == 0.0
    assert lib.tw_kv_last_error() != 0
    lib.tw_kv_clear_error()
