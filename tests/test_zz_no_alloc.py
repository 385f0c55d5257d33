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
