"""Writes the small golden fixtures of this folder: for every function of the CPU oracle, one .npz
holding seeded inputs and the outputs the oracle gave for them when the fixture was made.

The reference ships no golden vectors for this path (its test scripts draw unseeded random inputs and
compare with eager execution on the device), so these are made from the oracle itself, after the
mathematics pinned it (tests/test_oracle.py).  What they add: an edit of the oracle that changes any
output fails tests/test_golden.py, and the HIP kernels are checked against numbers that do not move.

Run from the repository root:  python tests/golden/make_fixtures.py
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import oracle as O  # noqa: E402


def _bf16(rng, shape, scale=1.0):
    return O.f32_to_bf16_bits((rng.standard_normal(shape) * scale).astype(np.float32))


def cases():
    rng = np.random.default_rng(20240611)

    x = rng.standard_normal((8, 96)).astype(np.float32) * 3
    x[0, :4] = [0.0, -0.0, 88.0, -104.0]  # zeros and the ends of exp's range
    x[1] = -np.abs(x[1])                   # a row that relu empties
    yield "relu_sigmoid_rowsum", dict(x=x), dict(y=O.relu_sigmoid_rowsum(x))

    h, r = _bf16(rng, (6, 128)), _bf16(rng, (6, 128))
    w = O.f32_to_bf16_bits((1 + 0.02 * rng.standard_normal(128)).astype(np.float32))
    h[5], r[5] = 0, 0                      # an all-zero row: eps alone under the root
    out, s = O.add_rmsnorm_bf16(h, r, w, 1e-6)
    yield "add_rmsnorm_bf16", dict(h=h, r=r, w=w, eps=np.float64(1e-6)), dict(out=out, h_plus_r=s)

    x = rng.standard_normal((33, 20)).astype(np.float32)
    x[:, 3] = 1.5                          # constant column: variance 0, argmax 0
    x[[4, 17], 7] = 9.0                    # tie: first index wins
    x[:, 11] += 1000.0                     # large offset: cancellation in the variance
    m0, v0, a0 = O.col_mean_var_argmax(x, 0.0)
    m1, v1, a1 = O.col_mean_var_argmax(x, 1.0)
    yield "col_mean_var_argmax", dict(x=x), dict(mean=m0, var_c0=v0, var_c1=v1, argmax=a0)
    assert np.array_equal(m0, m1) and np.array_equal(a0, a1)

    table = _bf16(rng, (16, 8))
    idx = np.array([[3, 3, 0, 15], [7, 1, 15, 0], [9, 9, 9, 2]], dtype=np.int64)
    yield "gather_rows", dict(table=table, idx=idx), dict(out=O.gather_rows(table, idx))

    t = _bf16(rng, (2, 3, 4, 8))
    yield "permute4_0213", dict(t=t), dict(out=O.permute4(t, (0, 2, 1, 3)))

    q, k, v = (_bf16(rng, (1, 1, 128, 128)) for _ in range(3))
    scale = 128 ** -0.5
    oc, mc, lc = O.attention_bf16(q, k, v, scale, True)
    of, mf, lf = O.attention_bf16(q, k, v, scale, False)
    yield "attention_bf16", dict(q=q, k=k, v=v, scale=np.float64(scale)), dict(
        out_causal=oc, max_causal=mc[..., 0].copy(), sum_causal=lc[..., 0].copy(),
        out_full=of, max_full=mf[..., 0].copy(), sum_full=lf[..., 0].copy())

    q, k, v, do = (_bf16(rng, (1, 1, 128, 128)) for _ in range(4))
    dq, dk, dv = O.attention_bwd(q, k, v, do, scale, True)
    yield "attention_bwd_causal", dict(q=q, k=k, v=v, dout=do, scale=np.float64(scale)), dict(
        dq=dq.astype(np.float32), dk=dk.astype(np.float32), dv=dv.astype(np.float32))

    S, B, N, D = 16, 2, 3, 8
    po, co = (rng.standard_normal((S, B, N * D)).astype(np.float32) for _ in range(2))
    stat = lambda a: np.ascontiguousarray(np.broadcast_to(a[..., None], a.shape + (8,))).astype(np.float32)  # noqa: E731
    pm, cm = (stat(rng.standard_normal((B, N, S)) * 4) for _ in range(2))
    ps, cs = (stat(rng.uniform(1, 50, (B, N, S))) for _ in range(2))
    cm[0, 0, :4] = pm[0, 0, :4]            # equal maxima: both factors 1
    out, mx, sm = O.forward_update(po, pm, ps, co, cm, cs)
    yield "ring_forward_update", dict(prev_out=po, prev_max=pm, prev_sum=ps, cur_out=co, cur_max=cm, cur_sum=cs), dict(
        out=out.astype(np.float32), max=mx.astype(np.float32), sum=sm.astype(np.float32))

    po, co = (rng.standard_normal((1, 3, 16, 8)).astype(np.float32) for _ in range(2))
    pl, cl = (rng.standard_normal((1, 3, 16, 1)).astype(np.float32) * 5 for _ in range(2))
    out, lse = O.forward_update_lse(po, pl, co, cl)
    yield "ring_forward_update_lse", dict(prev_out=po, prev_lse=pl, cur_out=co, cur_lse=cl), dict(
        out=out.astype(np.float32), lse=lse.astype(np.float32))

    a, b = _bf16(rng, (5, 64)), _bf16(rng, (5, 64))
    yield "add_bf16", dict(dst=a, src=b), dict(out=O.add_bf16(a, b))


def main():
    total = 0
    for name, inputs, outputs in cases():
        path = os.path.join(HERE, name + ".npz")
        arrays = {"in_" + k: np.asarray(v) for k, v in inputs.items()}
        arrays.update({"out_" + k: np.asarray(v) for k, v in outputs.items()})
        np.savez_compressed(path, **arrays)
        total += os.path.getsize(path)
        print(f"{name}.npz  {os.path.getsize(path)} bytes")
    print(f"total {total} bytes")


if __name__ == "__main__":
    main()
