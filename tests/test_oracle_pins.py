"""Pins for the CPU oracle (oracle/kv_oracle.cpp).

The reference ships no golden vector for the KV path, so each oracle function is
pinned against something that does not share its code: closed forms, library
routines, exhaustive enumeration, or a second restatement written differently
(numpy, vectorised over other axes, FMA emulated in float64).
"""
import ctypes
import math

import numpy as np
import pytest
from scipy.stats import norm

import gen

SIGMA = 1.0 / math.sqrt(128.0)  # kernels.cu:1422-1423


# ------------------------------------------------------------------ fp16 conversions
def test_f16_to_f32_all_patterns(oracle):
    allh = np.arange(65536, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib.tw_oracle_f16_to_f32(int(h)) for h in allh], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_round_to_nearest_even(oracle):
    r = gen.rng(7)
    vals = np.concatenate([
        r.standard_normal(20000, dtype=np.float32) * np.float32(10.0) ** r.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-6, 5.96e-8, 2.98e-8, 2.9802322e-8, 3e-8,
                  6.1e-5, 6.097e-5, np.inf, -np.inf], dtype=np.float32),
        # exact ties between neighbouring halves
        (np.arange(1024, 1100, dtype=np.float32) + 0.5) * np.float32(2.0 ** -10),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.lib.tw_oracle_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ tables
@pytest.mark.parametrize("bits", [4, 2])
def test_tables_antisymmetric_and_midpoints(oracle, bits):
    c, b = oracle.centroids(bits), oracle.bounds(bits)
    assert np.array_equal(c, -c[::-1])
    assert np.array_equal(b, -b[::-1])
    assert np.all(np.diff(c) > 0) and np.all(np.diff(b) > 0)
    mid = (c[:-1].astype(np.float64) + c[1:]) / 2
    assert np.max(np.abs(mid - b)) <= 1.5e-5  # printed to 5 decimals


@pytest.mark.parametrize("bits", [4, 2])
def test_tables_are_the_lloyd_max_quantizer_of_the_rotated_coordinate(oracle, bits):
    """Run Lloyd's iteration for N(0, 1/128) from scratch and compare."""
    n = 1 << bits
    levels = np.linspace(-2.5, 2.5, n)
    for _ in range(3000):
        edges = np.concatenate([[-np.inf], (levels[:-1] + levels[1:]) / 2, [np.inf]])
        mass = norm.cdf(edges[1:]) - norm.cdf(edges[:-1])
        new = (norm.pdf(edges[:-1]) - norm.pdf(edges[1:])) / mass  # E[x | bin]
        if np.max(np.abs(new - levels)) < 1e-12:
            break
        levels = new
    # the reference's literals are the published N(0,1) levels to 4 digits, times sigma
    assert np.max(np.abs(levels * SIGMA - oracle.centroids(bits))) < 6e-5
    assert np.max(np.abs((levels[:-1] + levels[1:]) / 2 * SIGMA - oracle.bounds(bits))) < 6e-5
    # textbook values quoted in the reference's comments (kernels.cu:1425)
    if bits == 2:
        assert abs(levels[2] - 0.4528) < 1e-4 and abs(levels[3] - 1.5104) < 1e-4


# ------------------------------------------------------------------ turbo_quantize
@pytest.mark.parametrize("bits", [4, 2])
def test_quantize_bin_edges_nan_inf(oracle, bits):
    b = oracle.bounds(bits)
    n = 1 << bits
    for i, edge in enumerate(b):
        below = np.nextafter(np.float32(edge), np.float32(-np.inf))
        above = np.nextafter(np.float32(edge), np.float32(np.inf))
        assert oracle.quantize(below, bits) == i
        assert oracle.quantize(edge, bits) == i + 1  # on the boundary: upper bin
        assert oracle.quantize(above, bits) == i + 1
    assert oracle.quantize(-np.inf, bits) == 0
    assert oracle.quantize(np.inf, bits) == n - 1
    # NaN: every `<` fails in the 4-bit tree (-> 15); every `>=` fails in the 2-bit count (-> 0)
    assert oracle.quantize(float("nan"), bits) == (15 if bits == 4 else 0)
    assert oracle.quantize(-0.0, bits) == n // 2  # -0.0 is not < 0


@pytest.mark.parametrize("bits", [4, 2])
def test_quantize_equals_searchsorted_and_nearest_centroid(oracle, bits):
    b, c = oracle.bounds(bits), oracle.centroids(bits)
    vals = np.concatenate([np.linspace(-0.4, 0.4, 20001, dtype=np.float32),
                           gen.rng(3).standard_normal(20000, dtype=np.float32) * np.float32(SIGMA)])
    got = np.array([oracle.quantize(v, bits) for v in vals])
    assert np.array_equal(got, np.searchsorted(b, vals, side="right"))
    assert np.all(np.diff(got[:20001]) >= 0)
    # away from the boundaries the bin is the nearest centroid
    margin = np.min(np.abs(vals[:, None] - b[None, :]), axis=1)
    far = margin > 2e-5
    nearest = np.argmin(np.abs(vals[:, None].astype(np.float64) - c[None, :]), axis=1)
    assert np.array_equal(got[far], nearest[far])


# ------------------------------------------------------------------ rotation
def _libstdcpp_normal_f32(seed: int, count: int) -> np.ndarray:
    """std::normal_distribution<float>(0,1) over std::mt19937(seed), libstdc++:
    Marsaglia polar method on generate_canonical<float,24>, one saved value."""
    libm = ctypes.CDLL("libm.so.6")
    libm.logf.restype = ctypes.c_float
    libm.logf.argtypes = [ctypes.c_float]
    mt = np.random.RandomState()
    mt.set_state(("MT19937", np.random.RandomState(0).get_state()[1], 624))
    # std::mt19937(seed) is init_genrand(seed), which is numpy's legacy seeding
    mt = np.random.RandomState(seed)
    f = np.float32

    def canonical():
        u = f(int(mt.randint(0, 2 ** 32, dtype=np.uint64))) / f(4294967296.0)
        return np.nextafter(f(1), f(0)) if u >= f(1) else u

    out, saved = [], None
    while len(out) < count:
        if saved is not None:
            out.append(saved)
            saved = None
            continue
        while True:
            x = f(f(2.0) * canonical() - 1.0)
            y = f(f(2.0) * canonical() - 1.0)
            r2 = f(f(x * x) + f(y * y))
            if not (r2 > f(1.0) or r2 == f(0.0)):
                break
        mult = f(np.sqrt(f(f(f(-2.0) * f(libm.logf(float(r2)))) / r2)))
        saved = f(x * mult)
        out.append(f(y * mult))
    return np.array(out[:count], dtype=np.float32)


def _mgs_rows_f32(mat: np.ndarray) -> np.ndarray:
    """engine.cpp:375-385 with sequential fp32 accumulation (cumsum is sequential)."""
    mat = mat.copy()
    d = mat.shape[0]
    for i in range(d):
        for j in range(i):
            dot = np.cumsum(mat[i] * mat[j], dtype=np.float32)[-1]
            mat[i] = mat[i] - dot * mat[j]
        nrm = np.cumsum(mat[i] * mat[i], dtype=np.float32)[-1]
        mat[i] = mat[i] * (np.float32(1.0) / np.sqrt(nrm))
    return mat


def test_mt19937_known_answer():
    # first output of std::mt19937 seeded with 42
    assert int(np.random.RandomState(42).randint(0, 2 ** 32, dtype=np.uint64)) == 1608637542


def test_rotation_matches_independent_restatement(oracle, rotation_fixture):
    f16, f32 = oracle.make_rotation(128, 42)
    assert np.array_equal(f16.view(np.uint16), rotation_fixture.view(np.uint16))
    raw = _libstdcpp_normal_f32(42, 128 * 128).reshape(128, 128)
    mine = _mgs_rows_f32(raw)
    assert np.array_equal(mine.view(np.uint32), f32.view(np.uint32))
    assert np.array_equal(mine.astype(np.float16).view(np.uint16), rotation_fixture.view(np.uint16))


def test_rotation_is_orthogonal(oracle, rotation_fixture):
    _, f32 = oracle.make_rotation(128, 42)
    q = f32.astype(np.float64)
    assert np.max(np.abs(q @ q.T - np.eye(128))) < 2e-5
    r = rotation_fixture.astype(np.float64)
    assert np.max(np.abs(r @ r.T - np.eye(128))) < 2e-3  # fp16 entry rounding
    assert np.max(np.abs(np.linalg.norm(r, axis=1) - 1)) < 1e-3
    other, _ = oracle.make_rotation(128, 43)
    assert not np.array_equal(other, rotation_fixture)


# ------------------------------------------------------------------ compressed append
def _fma32(a, b, c):
    """fp32 fused multiply-add emulated in float64: the product of two fp32 values is
    exact in float64; the sum is rounded once to float64 and once to fp32, which equals
    the single fp32 rounding unless the float64 sum was inexact AND sits on an fp32 tie."""
    p = a.astype(np.float64) * b.astype(np.float64)
    c = c.astype(np.float64)
    t = p + c
    bb = t - p
    err = (p - (t - bb)) + (c - bb)          # two-sum: exact rounding error of p + c
    low = t.view(np.uint64) & np.uint64((1 << 29) - 1)
    assert not np.any((low == np.uint64(1 << 28)) & (err != 0)), "double-rounding hazard"
    return t.astype(np.float32)


def _tree_sum_128(sq: np.ndarray) -> np.ndarray:
    """kernels.cu:1509-1520 for (..., 128) fp32: shuffle-down tree per 32, then (s0+s2)+(s1+s3)."""
    v = sq.reshape(sq.shape[:-1] + (4, 32)).copy()
    for off in (16, 8, 4, 2, 1):
        v[..., :off] = v[..., :off] + v[..., off:2 * off]
    s = v[..., 0]
    return (s[..., 0] + s[..., 2]) + (s[..., 1] + s[..., 3])


def numpy_quantize_rows(x_f16: np.ndarray, rot_f16: np.ndarray, bits: int):
    """Second restatement of kernels.cu:1586-1635 for (N,128) rows: returns codes (N,128), norms (N,), rotated."""
    x = x_f16.astype(np.float32)
    n2 = _tree_sum_128(x * x)
    inv = np.float32(1.0) / np.sqrt(n2 + np.float32(1e-12))
    u = x * inv[:, None]
    rot = rot_f16.astype(np.float32)
    acc = np.zeros((x.shape[0], 128), np.float32)
    for k in range(128):
        acc = _fma32(np.broadcast_to(rot[:, k], acc.shape), np.broadcast_to(u[:, k:k + 1], acc.shape), acc)
    bounds = np.array([-0.21224, -0.16299, -0.12701, -0.09715, -0.07068, -0.04619, -0.02284, 0.0,
                       0.02284, 0.04619, 0.07068, 0.09715, 0.12701, 0.16299, 0.21224], np.float32) \
        if bits == 4 else np.array([-0.08677, 0.0, 0.08677], np.float32)
    codes = np.searchsorted(bounds, acc, side="right").astype(np.uint8)
    norms = np.sqrt(n2 + np.float32(1e-12)).astype(np.float16)
    return codes, norms, acc


def pack_codes(codes: np.ndarray, bits: int) -> np.ndarray:
    vpb = 8 // bits
    c = codes.reshape(codes.shape[:-1] + (codes.shape[-1] // vpb, vpb)).astype(np.uint32)
    out = np.zeros(c.shape[:-1], np.uint32)
    for j in range(vpb):
        out |= c[..., j] << (j * bits)
    return out.astype(np.uint8)


def unpack_codes(packed: np.ndarray, bits: int) -> np.ndarray:
    vpb = 8 // bits
    p = packed.astype(np.uint32)
    parts = [(p >> (j * bits)) & ((1 << bits) - 1) for j in range(vpb)]
    return np.stack(parts, axis=-1).reshape(packed.shape[:-1] + (packed.shape[-1] * vpb,)).astype(np.uint8)


@pytest.mark.parametrize("bits", [4, 2])
def test_pack_order_exhaustive(oracle, rotation_fixture, bits):
    """Every byte pattern: field j of byte b is coordinate b*vpb + j, low field first."""
    for byte in range(256):
        codes = unpack_codes(np.array([[byte]], np.uint8), bits)[0]
        vpb = 8 // bits
        expect = [(byte >> (j * bits)) & ((1 << bits) - 1) for j in range(vpb)]
        assert list(codes) == expect
        assert pack_codes(codes[None, :], bits)[0, 0] == byte


@pytest.mark.parametrize("bits", [4, 2])
def test_append_matches_numpy_restatement(oracle, rotation_fixture, bits):
    r = gen.rng(11 + bits)
    G, Hk, D, msl = 6, 4, 128, 9
    kv_dim = Hk * D
    rows, _ = gen.kv_rows_with_outliers(r, (G, kv_dim), kv_dim)
    rows[1, :D] = 0                      # an all-zero head vector
    rows[2] = (rows[2].astype(np.float32) * 1e-3).astype(np.float16)   # tiny
    rows[3] = (rows[3].astype(np.float32) * 30).astype(np.float16)     # large
    pos = np.array([0, 3, 8, 1, 5, 2], np.int32)
    kvp = kv_dim * bits // 8
    cq = np.zeros((G, msl, kvp), np.uint8)
    cn = np.zeros((G, msl, Hk), np.float16)
    rotated = np.zeros((G, kv_dim), np.float32)
    margin = np.zeros((G, kv_dim), np.float32)
    oracle.turbo_kv_quantize_batch(cq, cn, rows, rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits, rotated, margin)

    codes, norms, acc = numpy_quantize_rows(rows.reshape(G * Hk, D), rotation_fixture, bits)
    assert np.array_equal(acc.reshape(G, kv_dim).view(np.uint32), rotated.view(np.uint32))
    packed = pack_codes(codes, bits).reshape(G, kvp)
    for g in range(G):
        assert np.array_equal(cq[g, pos[g]], packed[g])
        assert np.array_equal(cn[g, pos[g]].view(np.uint16), norms.reshape(G, Hk)[g].view(np.uint16))
    # bookkeeping: nothing else was written
    mask = np.ones((G, msl), bool)
    mask[np.arange(G), pos] = False
    assert not cq[mask].any() and not cn[mask].view(np.uint16).any()
    # zero vector: norm = fp16(1e-6), every code is the first non-negative bin
    assert cn[1, pos[1], 0] == np.float16(1e-6)
    zero_codes = unpack_codes(cq[1, pos[1], :D * bits // 8][None, :], bits)
    assert np.all(zero_codes == (8 if bits == 4 else 2))
    # margins are the distance to the nearest boundary
    b = oracle.bounds(bits)
    assert np.allclose(margin, np.min(np.abs(rotated[..., None] - b), axis=-1))


@pytest.mark.parametrize("bits", [4, 2])
def test_token_list_variant_equals_batch_variant(oracle, rotation_fixture, bits):
    r = gen.rng(21)
    T, Hk, D, msl = 5, 2, 128, 16
    kv_dim = Hk * D
    rows = gen.normal_f16(r, (T, kv_dim))
    positions = np.array([4, 0, 9, 2, 15], np.int32)
    kvp = kv_dim * bits // 8
    q1 = np.zeros((msl, kvp), np.uint8); n1 = np.zeros((msl, Hk), np.float16)
    oracle.turbo_kv_quantize(q1, n1, rows, rotation_fixture, positions, msl, T, Hk, D, kv_dim, bits)
    for t in range(T):  # one batch-variant call per token with G=1
        q2 = np.zeros((1, msl, kvp), np.uint8); n2 = np.zeros((1, msl, Hk), np.float16)
        oracle.turbo_kv_quantize_batch(q2, n2, rows[t:t + 1], rotation_fixture, positions[t:t + 1], msl, 1, Hk, D, kv_dim, bits)
        assert np.array_equal(q1[positions[t]], q2[0, positions[t]])
        assert np.array_equal(n1[positions[t]], n2[0, positions[t]])


@pytest.mark.parametrize("bits,rel", [(4, math.sqrt(0.009497)), (2, math.sqrt(0.1175))])
def test_append_reconstruction_error_is_the_lloyd_max_distortion(oracle, rotation_fixture, bits, rel):
    r = gen.rng(31)
    G, Hk, D = 64, 8, 128
    kv_dim = Hk * D
    rows = gen.normal_f16(r, (G, kv_dim))
    pos = np.zeros(G, np.int32)
    kvp = kv_dim * bits // 8
    cq = np.zeros((G, 1, kvp), np.uint8); cn = np.zeros((G, 1, Hk), np.float16)
    oracle.turbo_kv_quantize_batch(cq, cn, rows, rotation_fixture, pos, 1, G, Hk, D, kv_dim, bits)
    codes = unpack_codes(cq.reshape(G * Hk, D * bits // 8), bits)
    c = oracle.centroids(bits).astype(np.float64)
    R = rotation_fixture.astype(np.float64)
    recon = (c[codes] @ R) * cn.reshape(G * Hk, 1).astype(np.float64)  # n * R^T c
    x = rows.reshape(G * Hk, D).astype(np.float64)
    err = np.linalg.norm(x - recon, axis=1) / np.linalg.norm(x, axis=1)
    assert abs(err.mean() - rel) < 0.06 * rel
    # code histogram = Gaussian bin masses
    edges = np.concatenate([[-np.inf], oracle.bounds(bits) / SIGMA, [np.inf]])
    mass = norm.cdf(edges[1:]) - norm.cdf(edges[:-1])
    hist = np.bincount(codes.ravel(), minlength=1 << bits) / codes.size
    assert np.max(np.abs(hist - mass)) < 0.004


# ------------------------------------------------------------------ fp16 append + attention
def test_fp16_write_bookkeeping_bruteforce(oracle):
    r = gen.rng(41)
    G, msl, kv_dim = 3, 5, 16
    ck = np.zeros((G, msl, kv_dim), np.float16); cv = np.zeros_like(ck)
    model_k, model_v = {}, {}
    pos = np.array([0, 2, 4], np.int32)
    for step in range(2):
        k = gen.normal_f16(r, (G, kv_dim)); v = gen.normal_f16(r, (G, kv_dim))
        oracle.kv_cache_write_batch(ck, cv, k, v, pos, msl, G, kv_dim)
        for g in range(G):
            model_k[(g, int(pos[g]))] = k[g].copy(); model_v[(g, int(pos[g]))] = v[g].copy()
        if step == 0:
            pos = np.array([1, 3, 0], np.int32)
    for g in range(G):
        for p in range(msl):
            wk = model_k.get((g, p), np.zeros(kv_dim, np.float16))
            wv = model_v.get((g, p), np.zeros(kv_dim, np.float16))
            assert np.array_equal(ck[g, p], wk) and np.array_equal(cv[g, p], wv)
    before = pos.copy()
    oracle.increment_positions(pos, G)
    assert np.array_equal(pos, before + 1)


def f64_attention(q, K, V, n, group):
    """softmax(q K^T / sqrt(D)) V in float64. q (H,D); K,V (n_max,Hk,D)."""
    H, D = q.shape
    out = np.zeros((H, D))
    for h in range(H):
        kh = h // group
        s = K[:n, kh] @ q[h] / math.sqrt(D)
        w = np.exp(s - s.max()); w /= w.sum()
        out[h] = w @ V[:n, kh]
    return out


def rel_err(got, want):
    """max over head vectors of ||got - want||_inf / ||want||_inf."""
    got = got.astype(np.float64).reshape(-1, 128); want = np.asarray(want, np.float64).reshape(-1, 128)
    return float(np.max(np.max(np.abs(got - want), axis=1) / np.max(np.abs(want), axis=1)))


def test_fp16_attention_is_textbook_attention(oracle):
    r = gen.rng(51)
    G, H, Hk, D, msl = 3, 4, 2, 128, 300
    kv_dim, q_dim = Hk * D, H * D
    ck = gen.normal_f16(r, (G, msl, kv_dim)); cv = gen.normal_f16(r, (G, msl, kv_dim))
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.array([0, 130, 299], np.int32)   # 1 token, just past one block, full
    out = np.zeros((G, q_dim), np.float16)
    oracle.gqa_attention_batch(out, q, ck, cv, pos, msl, G, H, Hk, D, q_dim, kv_dim)
    for g in range(G):
        want = f64_attention(q[g].reshape(H, D).astype(np.float64), ck[g].reshape(msl, Hk, D).astype(np.float64),
                             cv[g].reshape(msl, Hk, D).astype(np.float64), int(pos[g]) + 1, H // Hk)
        assert rel_err(out[g], want) < 1e-3
        # single-sequence kernel (pos by value) gives the same bits as the batch kernel
        single = np.zeros(q_dim, np.float16)
        oracle.gqa_attention(q[g], ck[g], cv[g], single, int(pos[g]), msl, H, Hk, D)
        assert np.array_equal(single, out[g])
    # q_dim is a row stride: padded rows give the same heads
    q_pad = np.zeros((G, q_dim + 64), np.float16); q_pad[:, :q_dim] = q
    out_pad = np.zeros_like(q_pad)
    oracle.gqa_attention_batch(out_pad, q_pad, ck, cv, pos, msl, G, H, Hk, D, q_dim + 64, kv_dim)
    assert np.array_equal(out_pad[:, :q_dim], out)


def test_fp16_prefill_row_equals_decode_at_that_position(oracle):
    r = gen.rng(52)
    T, H, Hk, D, msl = 9, 4, 2, 128, 12
    kv_dim, q_dim = Hk * D, H * D
    ck = gen.normal_f16(r, (msl, kv_dim)); cv = gen.normal_f16(r, (msl, kv_dim))
    q = gen.normal_f16(r, (T, q_dim))
    out = np.zeros((T, q_dim), np.float16)
    oracle.gqa_prefill_attention(out, q, ck, cv, T, msl, H, Hk, D, q_dim, kv_dim)
    for t in range(T):
        single = np.zeros(q_dim, np.float16)
        oracle.gqa_attention(q[t], ck, cv, single, t, msl, H, Hk, D)
        assert rel_err(out[t], single.astype(np.float64)) < 1e-6  # same arithmetic, block size 128 both


# ------------------------------------------------------------------ compressed attention
def dequantize(cq, cn, rot_f16, bits, centroids):
    """K_hat[p,h,:] = n[p,h] * R^T c(codes[p,h]) in float64. cq (n,Hk*bph), cn (n,Hk)."""
    n, Hk = cn.shape
    codes = unpack_codes(cq.reshape(n * Hk, -1), bits)
    R = rot_f16.astype(np.float64)
    return ((centroids.astype(np.float64)[codes] @ R) * cn.reshape(n * Hk, 1).astype(np.float64)).reshape(n, Hk, 128)


@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_attention_is_attention_on_the_dequantized_cache(oracle, rotation_fixture, bits):
    r = gen.rng(61 + bits)
    G, H, Hk, D, msl = 3, 8, 2, 128, 200
    kv_dim, q_dim = Hk * D, H * D
    kvp = kv_dim * bits // 8
    ck = np.zeros((G, msl, kvp), np.uint8); cv = np.zeros_like(ck)
    kn = np.zeros((G, msl, Hk), np.float16); vn = np.zeros_like(kn)
    pos = np.zeros(G, np.int32)
    lens = [1, 129, 200]
    for t in range(msl):
        live = np.array([t < L for L in lens])
        if not live.any():
            break
        k_rows, _ = gen.kv_rows_with_outliers(r, (G, kv_dim), kv_dim)
        v_rows = gen.normal_f16(r, (G, kv_dim))
        p = np.where(live, t, [L - 1 for L in lens]).astype(np.int32)
        # sequences that are already full rewrite their last row with the same data: skip them
        for g in range(G):
            if live[g]:
                oracle.turbo_kv_quantize_batch(ck[g:g + 1], kn[g:g + 1], k_rows[g:g + 1], rotation_fixture,
                                               p[g:g + 1], msl, 1, Hk, D, kv_dim, bits)
                oracle.turbo_kv_quantize_batch(cv[g:g + 1], vn[g:g + 1], v_rows[g:g + 1], rotation_fixture,
                                               p[g:g + 1], msl, 1, Hk, D, kv_dim, bits)
    pos = np.array([L - 1 for L in lens], np.int32)
    q = gen.normal_f16(r, (G, q_dim))
    out = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(out, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    c = oracle.centroids(bits)
    for g in range(G):
        Kh = dequantize(ck[g], kn[g], rotation_fixture, bits, c)
        Vh = dequantize(cv[g], vn[g], rotation_fixture, bits, c)
        want = f64_attention(q[g].reshape(H, D).astype(np.float64), Kh, Vh, lens[g], H // Hk)
        # R is orthogonal only to fp16 precision (|R R^T - I| ~ 1e-3), which is what separates
        # "rotate q, dot with codes" from "dot q with R^T codes"; both use the same R, so they agree.
        assert rel_err(out[g], want) < 1.5e-3
        single = np.zeros(q_dim, np.float16)
        oracle.turbo_gqa_attention(q[g], ck[g], cv[g], kn[g], vn[g], rotation_fixture, single,
                                   int(pos[g]), msl, H, Hk, D, bits)
        assert np.array_equal(single, out[g])


@pytest.mark.parametrize("bits", [4, 2])
def test_turbo_prefill_row_equals_decode_at_that_position(oracle, rotation_fixture, bits):
    r = gen.rng(71)
    T, H, Hk, D, msl = 7, 4, 2, 128, 8
    kv_dim, q_dim = Hk * D, H * D
    kvp = kv_dim * bits // 8
    ck = np.zeros((msl, kvp), np.uint8); cv = np.zeros_like(ck)
    kn = np.zeros((msl, Hk), np.float16); vn = np.zeros_like(kn)
    positions = np.arange(T, dtype=np.int32)
    oracle.turbo_kv_quantize(ck, kn, gen.normal_f16(r, (T, kv_dim)), rotation_fixture, positions, msl, T, Hk, D, kv_dim, bits)
    oracle.turbo_kv_quantize(cv, vn, gen.normal_f16(r, (T, kv_dim)), rotation_fixture, positions, msl, T, Hk, D, kv_dim, bits)
    q = gen.normal_f16(r, (T, q_dim))
    out = np.zeros((T, q_dim), np.float16)
    oracle.turbo_gqa_prefill_attention(out, q, ck, cv, kn, vn, rotation_fixture, T, msl, H, Hk, D, q_dim, kv_dim, bits)
    for t in range(T):
        single = np.zeros(q_dim, np.float16)
        oracle.turbo_gqa_attention(q[t], ck, cv, kn, vn, rotation_fixture, single, t, msl, H, Hk, D, bits)
        assert np.array_equal(single, out[t])


# ------------------------------------------------------------------ committed fixtures
@pytest.mark.parametrize("bits", [4, 2])
def test_golden_case_reproduces(oracle, rotation_fixture, bits):
    from pathlib import Path
    z = np.load(Path(__file__).parent / "golden" / f"case_tq{bits}_g2_h4_ctx37.npz")
    G, H, Hk, ctx, msl = (int(z[k]) for k in ("G", "H", "Hk", "ctx", "msl"))
    D, kv_dim, q_dim = 128, Hk * 128, H * 128
    ck = np.zeros_like(z["ck"]); cv = np.zeros_like(z["cv"]); kn = np.zeros_like(z["kn"]); vn = np.zeros_like(z["vn"])
    pos = np.zeros(G, np.int32)
    for t in range(ctx + 1):
        oracle.turbo_kv_quantize_batch(ck, kn, np.ascontiguousarray(z["k_rows"][t]), rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
        oracle.turbo_kv_quantize_batch(cv, vn, np.ascontiguousarray(z["v_rows"][t]), rotation_fixture, pos, msl, G, Hk, D, kv_dim, bits)
        if t < ctx:
            oracle.increment_positions(pos, G)
    assert np.array_equal(ck, z["ck"]) and np.array_equal(cv, z["cv"])
    assert np.array_equal(kn, z["kn"]) and np.array_equal(vn, z["vn"])
    assert np.array_equal(pos, z["pos"]) and np.all(pos == ctx)
    out = np.zeros((G, q_dim), np.float16)
    oracle.turbo_gqa_attention_batch(out, np.ascontiguousarray(z["q"]), ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    assert np.array_equal(out, z["out"])


# ------------------------------------------------------------------ producers: QK RMSNorm and RoPE
def _f64(a):
    return a.astype(np.float64)


@pytest.mark.parametrize("biased", [False, True])
def test_qk_norm_is_rmsnorm(oracle, biased):
    """x / sqrt(mean(x^2) + eps) * w in float64, per head; the gap between the heads and the row
    stride (gate half of a gated q projection) is not touched."""
    r = gen.rng(610 + biased)
    G, H, Hk, D = 3, 4, 2, 128
    q_dim, kv_dim = 2 * H * D, Hk * D + 64
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim))
    q[1] = (q[1].astype(np.float32) * 40).astype(np.float16)        # large row
    k[2] = (k[2].astype(np.float32) * 1e-3).astype(np.float16)      # tiny row: eps matters
    qw = (1.0 + 0.3 * r.standard_normal(D)).astype(np.float16)
    kw = (0.5 * r.standard_normal(D)).astype(np.float16)
    eps = 1e-6
    q0, k0 = q.copy(), k.copy()
    oracle.qk_norm_batch(q, k, qw, kw, H, Hk, D, G, eps, q_dim, kv_dim, biased)
    for x, x0, w, heads in ((q, q0, qw, H), (k, k0, kw, Hk)):
        ww = _f64(w) + (1.0 if biased else 0.0)
        for g in range(G):
            for h in range(heads):
                v = _f64(x0[g, h * D:(h + 1) * D])
                want = v / np.sqrt(np.mean(v * v) + eps) * ww
                got = _f64(x[g, h * D:(h + 1) * D])
                assert np.max(np.abs(got - want)) <= 1e-3 * np.max(np.abs(want)) + 1e-7
            assert np.array_equal(x[g, heads * D:].view(np.uint16), x0[g, heads * D:].view(np.uint16))


def test_qk_norm_single_equals_batch_of_one_and_scaling(oracle):
    """The single-sequence kernel (128 threads striding the head) and the batch kernel (one thread
    per element) agree on 128-wide heads; scaling the input by a power of two does not change the
    result when eps is negligible (RMSNorm is scale-free), which a dropped 1/head_dim would break
    together with the float64 check above."""
    r = gen.rng(612)
    H, Hk, D = 6, 2, 128
    q = gen.normal_f16(r, (H * D,)); k = gen.normal_f16(r, (Hk * D,))
    qw = (1.0 + 0.1 * r.standard_normal(D)).astype(np.float16); kw = (1.0 + 0.1 * r.standard_normal(D)).astype(np.float16)
    q1, k1, q2, k2 = q.copy(), k.copy(), q.copy().reshape(1, -1), k.copy().reshape(1, -1)
    oracle.qk_norm(q1, k1, qw, kw, H, Hk, D, 1e-6)
    oracle.qk_norm_batch(q2, k2, qw, kw, H, Hk, D, 1, 1e-6, H * D, Hk * D, False)
    assert np.array_equal(q1.view(np.uint16), q2[0].view(np.uint16))
    assert np.array_equal(k1.view(np.uint16), k2[0].view(np.uint16))
    q3 = (q.astype(np.float32) * 4).astype(np.float16); k3 = (k.astype(np.float32) * 4).astype(np.float16)
    oracle.qk_norm(q3, k3, qw, kw, H, Hk, D, 0.0)
    q4, k4 = q.copy(), k.copy()
    oracle.qk_norm(q4, k4, qw, kw, H, Hk, D, 0.0)
    assert np.array_equal(q3.view(np.uint16), q4.view(np.uint16))
    assert np.array_equal(k3.view(np.uint16), k4.view(np.uint16))


def test_qk_norm_unit_weight_gives_unit_rms(oracle):
    r = gen.rng(613)
    H, Hk, D, G = 2, 2, 128, 4
    q = gen.normal_f16(r, (G, H * D)); k = gen.normal_f16(r, (G, Hk * D))
    one = np.ones(D, np.float16)
    oracle.qk_norm_batch(q, k, one, one, H, Hk, D, G, 1e-6, H * D, Hk * D, False)
    rms = np.sqrt(np.mean(_f64(q.reshape(G, H, D)) ** 2, axis=-1))
    assert np.all(np.abs(rms - 1.0) < 2e-3)
    zero = np.zeros(D, np.float16)                       # biased: weight 0 means scale 1
    q2 = gen.normal_f16(r, (G, H * D)); k2 = gen.normal_f16(r, (G, Hk * D))
    q3, k3 = q2.copy(), k2.copy()
    oracle.qk_norm_batch(q2, k2, one, one, H, Hk, D, G, 1e-6, H * D, Hk * D, False)
    oracle.qk_norm_batch(q3, k3, zero, zero, H, Hk, D, G, 1e-6, H * D, Hk * D, True)
    assert np.array_equal(q2.view(np.uint16), q3.view(np.uint16)) and np.array_equal(k2.view(np.uint16), k3.view(np.uint16))


def _tables(r, msl, rope_dim, theta=1e6):
    """cos/sin of pos * theta^(-2d/rope_dim) in float64, rounded to fp16 (engine.cpp:554-574)."""
    d = np.arange(rope_dim // 2, dtype=np.float64)
    ang = np.arange(msl, dtype=np.float64)[:, None] * theta ** (-2.0 * d / rope_dim)[None, :]
    return np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)


@pytest.mark.parametrize("rope_dim", [128, 64])
def test_rope_batch_is_a_complex_rotation(oracle, rope_dim):
    """(x_d + i x_{d+half}) * (c + i s) in float64 with the fp16 table values; coordinates past
    rope_dim, the gap behind the heads and other sequences' rows are left alone."""
    r = gen.rng(620 + rope_dim)
    G, H, Hk, D, msl = 4, 4, 2, 128, 300
    q_dim, kv_dim = H * D + 32, Hk * D
    ct, st = _tables(r, msl, rope_dim)
    q = gen.normal_f16(r, (G, q_dim)); k = gen.normal_f16(r, (G, kv_dim))
    pos = np.array([0, 1, 137, 299], np.int32)
    q0, k0 = q.copy(), k.copy()
    oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, q_dim, kv_dim, rope_dim)
    half = rope_dim // 2
    for x, x0, heads in ((q, q0, H), (k, k0, Hk)):
        for g in range(G):
            c, s = _f64(ct[pos[g]]), _f64(st[pos[g]])
            for h in range(heads):
                v = _f64(x0[g, h * D:(h + 1) * D]); got = _f64(x[g, h * D:(h + 1) * D])
                z = (v[:half] + 1j * v[half:rope_dim]) * (c + 1j * s)
                assert np.max(np.abs(got[:half] - z.real)) <= 2e-3 * np.max(np.abs(v)) + 1e-6
                assert np.max(np.abs(got[half:rope_dim] - z.imag)) <= 2e-3 * np.max(np.abs(v)) + 1e-6
                assert np.array_equal(x[g, h * D + rope_dim:(h + 1) * D].view(np.uint16),
                                      x0[g, h * D + rope_dim:(h + 1) * D].view(np.uint16))
            assert np.array_equal(x[g, heads * D:].view(np.uint16), x0[g, heads * D:].view(np.uint16))
    # position 0: cos = 1 and sin = 0 exactly, so the row comes back bit for bit
    assert np.array_equal(q[0].view(np.uint16), q0[0].view(np.uint16))
    assert np.array_equal(k[0].view(np.uint16), k0[0].view(np.uint16))


def test_rope_single_rotates_like_batch_and_differs_only_in_operand_order(oracle):
    """Same rotation from both kernels; exactly representable inputs (small integers, table entries
    that are powers of two) make every product exact, so the two operand orders give equal bits."""
    r = gen.rng(630)
    H, Hk, D, msl = 3, 2, 128, 8
    ct = np.full((msl, D // 2), 0.5, np.float16); st = np.full((msl, D // 2), -0.25, np.float16)
    q = r.integers(-8, 9, H * D).astype(np.float16); k = r.integers(-8, 9, Hk * D).astype(np.float16)
    q1, k1 = q.copy(), k.copy()
    q2, k2 = q.copy().reshape(1, -1), k.copy().reshape(1, -1)
    oracle.rope(q1, k1, ct, st, 5, msl, H, Hk, D)
    oracle.rope_batch(q2, k2, ct, st, np.array([5], np.int32), msl, 1, H, Hk, D, H * D, Hk * D, D)
    assert np.array_equal(q1.view(np.uint16), q2[0].view(np.uint16)) and np.array_equal(k1.view(np.uint16), k2[0].view(np.uint16))
    v = _f64(q.reshape(H, D))
    want0 = v[:, :64] * 0.5 - v[:, 64:] * -0.25
    want1 = v[:, 64:] * 0.5 + v[:, :64] * -0.25
    got = _f64(q1.reshape(H, D))
    assert np.array_equal(got[:, :64], want0) and np.array_equal(got[:, 64:], want1)
    # general inputs: within one fp16 step of each other and of the float64 rotation
    ct, st = _tables(r, msl, D)
    q = gen.normal_f16(r, (H * D,)); k = gen.normal_f16(r, (Hk * D,))
    q1, k1, q2, k2 = q.copy(), k.copy(), q.copy().reshape(1, -1), k.copy().reshape(1, -1)
    oracle.rope(q1, k1, ct, st, 7, msl, H, Hk, D)
    oracle.rope_batch(q2, k2, ct, st, np.array([7], np.int32), msl, 1, H, Hk, D, H * D, Hk * D, D)
    assert np.max(np.abs(_f64(q1) - _f64(q2[0]))) <= 2 ** -8 * np.max(np.abs(_f64(q)))


def test_rope_keeps_pair_norms_and_inverts(oracle):
    """A rotation keeps |x_d|^2 + |x_{d+half}|^2 (to the tables' fp16 rounding), and the table with
    the sine negated undoes it."""
    r = gen.rng(640)
    G, H, Hk, D, msl = 2, 2, 2, 128, 64
    ct, st = _tables(r, msl, D, theta=10000.0)
    q = gen.normal_f16(r, (G, H * D)); k = gen.normal_f16(r, (G, Hk * D))
    q0 = q.copy()
    pos = np.array([17, 63], np.int32)
    oracle.rope_batch(q, k, ct, st, pos, msl, G, H, Hk, D, H * D, Hk * D, D)
    a = _f64(q0.reshape(G, H, 2, 64)); b = _f64(q.reshape(G, H, 2, 64))
    n0 = (a ** 2).sum(axis=2); n1 = (b ** 2).sum(axis=2)
    assert np.max(np.abs(n1 - n0) / (n0 + 1e-3)) < 5e-3
    oracle.rope_batch(q, k, ct, (-st.astype(np.float32)).astype(np.float16), pos, msl, G, H, Hk, D, H * D, Hk * D, D)
    assert np.max(np.abs(_f64(q) - _f64(q0))) <= 4e-3 * np.max(np.abs(_f64(q0)))


def test_rope_tables_follow_the_recipe(oracle):
    ct, st = oracle.rope_tables(200, 64, 1e6)
    want_c, want_s = _tables(None, 200, 64, 1e6)
    # float32 powf/cosf against float64: a few fp16 steps at large angles
    assert np.max(np.abs(_f64(ct) - _f64(want_c))) < 4e-3 and np.max(np.abs(_f64(st) - _f64(want_s))) < 4e-3
    assert np.all(ct[0] == 1.0) and np.all(st[0] == 0.0)


# ------------------------------------------------------------------ gated attention output
def test_sigmoid_gate_is_x_times_sigmoid(oracle):
    """data * 1/(1 + exp(-gate)) in float64; gate 0 halves exactly, a large gate leaves the bits alone,
    a very negative one gives zero; only dim*G elements are touched."""
    r = gen.rng(650)
    dim, G = 256, 5
    data = gen.normal_f16(r, (G * dim + 16,)); gate = (4 * r.standard_normal(G * dim + 16)).astype(np.float16)
    gate[:4] = [0.0, 30.0, -30.0, -0.0]
    data[:4] = [3.0, -1.2345, 7.0, 5.0]
    d0 = data.copy()
    oracle.sigmoid_gate_batch(data, gate, dim, G)
    n = dim * G
    want = _f64(d0[:n]) / (1.0 + np.exp(-_f64(gate[:n])))
    assert np.max(np.abs(_f64(data[:n]) - want)) <= 2 ** -10 * np.max(np.abs(want))
    assert data[0] == np.float16(1.5) and data[3] == np.float16(2.5)
    assert data[1].view(np.uint16) == d0[1].view(np.uint16)
    assert data[2] == 0
    assert np.array_equal(data[n:].view(np.uint16), d0[n:].view(np.uint16))


def test_o3_build_of_the_oracle_gives_the_same_bits(oracle, rotation_fixture):
    """The benchmark times the oracle's source built -O3 -march=x86-64-v3 (oracle/Makefile); it must be the same
    arithmetic: compressed append and attention of a small case, bit for bit against the -O2 build the tests use."""
    import oracle_lib
    o3 = oracle_lib.load_o3()
    r = gen.rng(4242)
    G, H, Hk, msl, D = 3, 8, 4, 70, 128
    kv_dim, q_dim = Hk * D, H * D
    for bits in (4, 2):
        outs = []
        for o in (oracle, o3):
            rr = gen.rng(4242 + bits)
            kvp = kv_dim * bits // 8
            ck = np.zeros((G, msl, kvp), np.uint8); cv = np.zeros_like(ck)
            kn = np.zeros((G, msl, Hk), np.float16); vn = np.zeros_like(kn)
            for g in range(G):
                n = 40 + 10 * g
                k_rows = gen.normal_f16(rr, (n, kv_dim)); v_rows = gen.normal_f16(rr, (n, kv_dim))
                p = np.arange(n, dtype=np.int32)
                o.turbo_kv_quantize(ck[g], kn[g], k_rows, rotation_fixture, p, msl, n, Hk, D, kv_dim, bits)
                o.turbo_kv_quantize(cv[g], vn[g], v_rows, rotation_fixture, p, msl, n, Hk, D, kv_dim, bits)
            q = gen.normal_f16(rr, (G, q_dim))
            pos = np.array([39, 49, 59], np.int32)
            out = np.zeros((G, q_dim), np.float16)
            o.turbo_gqa_attention_batch(out, q, ck, cv, kn, vn, rotation_fixture, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
            outs.append((ck.copy(), cv.copy(), kn.copy(), vn.copy(), out.copy()))
        for a, b in zip(*outs):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
