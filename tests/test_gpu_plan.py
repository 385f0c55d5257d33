"""The automatic choice between the forms of a compressed decode step (one launch, one launch with a sequence's context
shared by workgroups, three launches) against the forms themselves, timed on the GPU at hand: the choice rests on
rates and fixed costs measured on one device (plan_constants in kv_decode_fused.hip), and this is the check that they
still describe the device the library runs on.  Each form runs graph-replayed steps of a few layers; the automatic
choice must be within 5 % of the faster forced form (medians of several timings)."""
import statistics

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

D = 128


def _time_steps(eng, q, k, v, out, start, steps, stream):
    import torch
    eng.set_positions([start] * q.shape[1])
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        eng.decode_step(q, k, v, out, use_graph=True, stream=stream)        # capture (or replay) outside the timing
        e0.record(stream)
        for _ in range(steps):
            eng.decode_step(q, k, v, out, use_graph=True, stream=stream)
        e1.record(stream)
    stream.synchronize()
    return e0.elapsed_time(e1) / steps


@pytest.mark.parametrize("G,ctx,bits,H", [(64, 8192, 4, 16), (16, 8192, 4, 16), (96, 8192, 2, 16), (128, 512, 4, 16), (16, 4096, 2, 32)])
def test_automatic_choice_is_the_faster_form(G, ctx, bits, H):
    import torch
    from triebwerk_amd import Engine, kvcache
    L, Hk, steps, reps = 4, 8, 12, 5
    msl = ctx + (reps * 3 + 2) * (steps + 1) + 64
    msl = (msl + 255) // 256 * 256
    eng = Engine(max_seq_len=msl, kv_bits=bits)
    eng.set_shape(L, H, Hk, D)
    eng.alloc_batch(G, msl)
    gt = torch.Generator(device="cuda"); gt.manual_seed(3)
    for l in range(L):
        c = eng.cache(l)
        for i in range(2):
            c[i].view(torch.int32).copy_(torch.randint(-2 ** 31, 2 ** 31 - 1, tuple(c[i].view(torch.int32).shape), generator=gt,
                                                      device="cuda", dtype=torch.int32))
        for i in (2, 3):
            c[i].copy_((11.3 + 0.7 * torch.randn(c[i].shape, generator=gt, device="cuda")).to(torch.float16))
    q = torch.randn((L, G, H * D), generator=gt, device="cuda", dtype=torch.float16)
    k = torch.randn((L, G, Hk * D), generator=gt, device="cuda", dtype=torch.float16)
    v = torch.randn((L, G, Hk * D), generator=gt, device="cuda", dtype=torch.float16)
    out = torch.zeros_like(q)
    stream = torch.cuda.Stream()
    times = {0: [], 1: [], 2: []}
    try:
        for rep in range(reps):
            for mode in (0, 1, 2):          # automatic, one launch (shared where the library would share), three launches
                kvcache.set_decode_fused(mode)
                # a change of mode does not invalidate the captured step: other buffers make the engine capture again
                times[mode].append(_time_steps(eng, q, k, v, out, ctx - 1, steps, stream))
                q = q.clone()
    finally:
        kvcache.set_decode_fused(0)
    auto, one, three = (statistics.median(times[m]) for m in (0, 1, 2))
    print(f"plan check G={G} ctx={ctx} bits={bits}: automatic {auto:.4f} ms, one launch {one:.4f}, three launches {three:.4f}", flush=True)
    assert auto <= 1.05 * min(one, three), (auto, one, three)
