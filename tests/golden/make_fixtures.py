"""Writes the committed fixtures under tests/golden/.

  rotation_seed42.f16  the engine's rotation matrix (engine.cpp:366-392):
                       mt19937(42) + libstdc++ normal_distribution<float> +
                       modified Gram-Schmidt, fp16.  libstdc++'s normal
                       distribution is library-defined, hence a fixture.
  case_*.npz           small append + attention cases computed by the CPU oracle
                       (oracle/kv_oracle.cpp), inputs and expected outputs.

The reference ships no vectors for this path; these pin the oracle against
itself over time (a change in its arithmetic shows up as a diff) and give the
GPU tests inputs that do not depend on a random generator.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))

import gen  # noqa: E402
import oracle_lib  # noqa: E402


def make_case(o, rot, seed, bits, G, H, Hk, ctx, msl):
    D = 128
    kv_dim, q_dim = Hk * D, H * D
    r = gen.rng(seed)
    kvp = kv_dim * bits // 8
    ck = np.zeros((G, msl, kvp), np.uint8)
    cv = np.zeros((G, msl, kvp), np.uint8)
    kn = np.zeros((G, msl, Hk), np.float16)
    vn = np.zeros((G, msl, Hk), np.float16)
    k_rows = gen.normal_f16(r, (ctx + 1, G, kv_dim))
    v_rows = gen.normal_f16(r, (ctx + 1, G, kv_dim))
    q = gen.normal_f16(r, (G, q_dim))
    pos = np.zeros(G, np.int32)
    for t in range(ctx + 1):
        o.turbo_kv_quantize_batch(ck, kn, k_rows[t], rot, pos, msl, G, Hk, D, kv_dim, bits)
        o.turbo_kv_quantize_batch(cv, vn, v_rows[t], rot, pos, msl, G, Hk, D, kv_dim, bits)
        if t < ctx:
            o.increment_positions(pos, G)
    rotated = np.zeros((G, kv_dim), np.float32)
    margin = np.zeros((G, kv_dim), np.float32)
    scratch_q = np.zeros_like(ck)
    scratch_n = np.zeros_like(kn)
    o.turbo_kv_quantize_batch(scratch_q, scratch_n, k_rows[ctx], rot, pos, msl, G, Hk, D, kv_dim, bits,
                              rotated, margin)
    out = np.zeros((G, q_dim), np.float16)
    o.turbo_gqa_attention_batch(out, q, ck, cv, kn, vn, rot, pos, msl, G, H, Hk, D, q_dim, kv_dim, bits)
    return dict(bits=bits, G=G, H=H, Hk=Hk, ctx=ctx, msl=msl, k_rows=k_rows, v_rows=v_rows, q=q,
                ck=ck, cv=cv, kn=kn, vn=vn, pos=pos, out=out, last_margin=margin)


def main():
    o = oracle_lib.load()
    f16, _ = o.make_rotation(128, 42)
    f16.tofile(HERE / "rotation_seed42.f16")
    for bits in (4, 2):
        case = make_case(o, f16, seed=1000 + bits, bits=bits, G=2, H=4, Hk=2, ctx=36, msl=40)
        np.savez_compressed(HERE / f"case_tq{bits}_g2_h4_ctx37.npz", **case)
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
