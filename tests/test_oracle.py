"""Pins the CPU oracle (oracle/oracle.c) before it is trusted as the checker.

The reference ships no golden vectors for this path (its tests draw unseeded
inputs and compare compiled with eager on the device), so each oracle function
is pinned by what the mathematics fixes: an independent fp64 evaluation with a
library routine, hand-computed tiny cases, and invariants chosen so that a
dropped term, a wrong sign or index or a transposed operand fails.
"""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.helpers import bits


def bf16(x: torch.Tensor) -> np.ndarray:
    return bits(x.bfloat16())


# ------------------------------------------------------------------ rowsum
def test_rowsum_tiny_by_hand():
    x = np.array([[0.0, 1.0, -1.0, -0.5]], dtype=np.float32)
    # relu(2x+1)*sigmoid(x): [1*0.5, 3*sig(1), 0, 0*...] ; -0.5 -> relu(0) = 0
    expect = 0.5 + 3.0 / (1.0 + math.exp(-1.0))
    assert abs(O.relu_sigmoid_rowsum(x)[0] - expect) < 1e-6


@pytest.mark.parametrize("shape", [(3, 5), (37, 64), (7, 9, 11), (2053, 13)])
def test_rowsum_vs_fp64(shape):
    torch.manual_seed(0)
    x = torch.randn(*shape)
    ref = (torch.relu(2 * x.double() + 1) * torch.sigmoid(x.double())).sum(-1)
    np.testing.assert_allclose(O.relu_sigmoid_rowsum(x.numpy()), ref.numpy(), rtol=2e-6, atol=1e-6)


def test_rowsum_invariants():
    torch.manual_seed(1)
    x = torch.randn(16, 128)
    y = O.relu_sigmoid_rowsum(x.numpy())
    perm = torch.randperm(16)
    assert np.array_equal(O.relu_sigmoid_rowsum(x[perm].numpy()), y[perm.numpy()])  # rows independent
    cperm = torch.randperm(128)
    np.testing.assert_allclose(O.relu_sigmoid_rowsum(x[:, cperm].numpy()), y, rtol=1e-6)  # order-free sum
    both = O.relu_sigmoid_rowsum(torch.cat([x, x], 1).numpy())
    np.testing.assert_allclose(both, 2 * y, rtol=1e-6)  # additive over the row
    assert O.relu_sigmoid_rowsum(np.full((1, 8), -0.5, np.float32))[0] == 0.0  # relu cuts exactly at 2x+1=0


# ------------------------------------------------------------------ add + rmsnorm
def test_add_rmsnorm_vs_fp64_and_rounding():
    torch.manual_seed(0)
    h = torch.randn(33, 256).bfloat16()
    r = torch.randn(33, 256).bfloat16()
    w = (1 + 0.02 * torch.randn(256)).bfloat16()
    out, s = O.add_rmsnorm_bf16(bits(h), bits(r), bits(w), 1e-6)
    s32 = h.float() + r.float()
    assert np.array_equal(s, bits(s32.bfloat16()))  # rounded once, round-to-nearest-even
    sd = s32.double()  # the norm uses the unrounded sum
    ref = sd * torch.rsqrt((sd * sd).mean(-1, keepdim=True) + 1e-6) * w.double()
    got = torch.from_numpy(O.bf16_bits_to_f32(out))
    assert (got.double() - ref).abs().max() <= 2 ** -7 * ref.abs().max()  # within bf16 rounding of fp64
    assert np.array_equal(out, bits(ref.float().bfloat16())) or (out != bits(ref.float().bfloat16())).mean() < 0.01


def test_add_rmsnorm_special_cases():
    torch.manual_seed(2)
    h = torch.randn(9, 64).bfloat16()
    zero = torch.zeros_like(h)
    ones = torch.ones(64).bfloat16()
    out, s = O.add_rmsnorm_bf16(bits(h), bits(zero), bits(ones), 0.0)
    assert np.array_equal(s, bits(h))  # h + 0 = h
    o = O.bf16_bits_to_f32(out)
    assert np.abs((o * o).mean(-1) - 1).max() < 1e-2  # textbook RMSNorm: unit mean square
    out2, _ = O.add_rmsnorm_bf16(bits(zero), bits(h), bits(ones), 0.0)
    assert np.array_equal(out, out2)  # symmetric in h and r
    two = (2 * torch.ones(64)).bfloat16()
    out3, _ = O.add_rmsnorm_bf16(bits(h), bits(zero), bits(two), 0.0)
    assert np.array_equal(O.bf16_bits_to_f32(out3), 2 * o)  # weight multiplies the result
    # a constant row: every element becomes sign * w
    c = torch.full((1, 64), -3.0).bfloat16()
    outc, _ = O.add_rmsnorm_bf16(bits(c), bits(torch.zeros_like(c)), bits(ones), 0.0)
    assert np.allclose(O.bf16_bits_to_f32(outc), -1.0)


def test_bf16_round_to_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -1.00390625, np.inf], dtype=np.float32)  # ties at bit 16
    got = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x))
    assert np.array_equal(got, torch.from_numpy(x).bfloat16().float().numpy())
    assert np.isnan(O.bf16_bits_to_f32(O.f32_to_bf16_bits(np.array([np.nan], np.float32))))[0]


# ------------------------------------------------------------------ column stats
@pytest.mark.parametrize("rows,cols", [(1, 3), (2, 4), (513, 64), (4096, 8)])
def test_col_stats_vs_fp64(rows, cols):
    torch.manual_seed(0)
    x = torch.randn(rows, cols)
    mean, var, arg = O.col_mean_var_argmax(x.numpy(), 0.0)
    np.testing.assert_allclose(mean, x.double().mean(0).numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(var, x.double().var(0, unbiased=False).numpy(), rtol=1e-6, atol=1e-12)
    assert np.array_equal(arg, torch.argmax(x, 0).numpy())


def test_col_stats_by_hand_and_correction():
    x = np.array([[1.0, 5.0], [3.0, 5.0], [5.0, 5.0], [7.0, -1.0]], dtype=np.float32)
    mean, var, arg = O.col_mean_var_argmax(x, 0.0)
    assert list(mean) == [4.0, 3.5] and list(var) == [5.0, 6.75] and list(arg) == [3, 0]
    _, var1, _ = O.col_mean_var_argmax(x, 1.0)
    np.testing.assert_allclose(var1, [20.0 / 3, 9.0])  # divisor N - correction


def test_col_stats_invariants_and_ties():
    torch.manual_seed(3)
    x = torch.randn(1000, 16)
    m, v, a = O.col_mean_var_argmax(x.numpy())
    m2, v2, a2 = O.col_mean_var_argmax((x * 2 + 3).numpy())
    np.testing.assert_allclose(v2, 4 * v, rtol=1e-5)  # var(kx + c) = k^2 var(x)
    np.testing.assert_allclose(m2, 2 * m + 3, rtol=1e-5, atol=1e-5)
    assert np.array_equal(a, a2)
    y = x.clone()
    y[700, 0] = 100.0
    y[20, 0] = 100.0
    y[500, 1] = float("nan")
    y[600, 1] = float("nan")
    y[:, 2] = float("-inf")
    _, vy, ay = O.col_mean_var_argmax(y.numpy())
    assert ay[0] == 20 and ay[1] == 500 and ay[2] == 0  # first index on ties, NaN is the maximum
    assert np.array_equal(ay, torch.argmax(y, 0).numpy())
    assert np.isnan(vy[1])


# ------------------------------------------------------------------ gather / permute
def test_gather_and_permute_definitions():
    torch.manual_seed(0)
    table = torch.randn(11, 6).bfloat16()
    idx = torch.tensor([0, 10, 10, 3, -1, -11], dtype=torch.int64)
    out = O.gather_rows(bits(table), idx.numpy())
    assert np.array_equal(out, bits(table[idx]))
    with pytest.raises(IndexError):
        O.gather_rows(bits(table), np.array([11], dtype=np.int64))
    t = torch.randn(2, 3, 4, 5).bfloat16()
    for perm in [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 3, 2), (0, 1, 2, 3)]:
        assert np.array_equal(O.permute4(bits(t), perm), bits(t.permute(*perm).contiguous()))
    once = O.permute4(bits(t), (0, 2, 1, 3))
    assert np.array_equal(O.permute4(once, (0, 2, 1, 3)), bits(t))  # involution
    f = torch.randn(2, 3, 4, 5)
    assert np.array_equal(O.permute4(f.numpy(), (0, 2, 1, 3)), f.permute(0, 2, 1, 3).contiguous().numpy())


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("causal", [True, False])
def test_attention_vs_fp64(causal):
    torch.manual_seed(0)
    q, k, v = (torch.randn(2, 3, 24, 16).bfloat16() for _ in range(3))
    scale = 16 ** -0.5
    out, smax, ssum = O.attention_bf16(bits(q), bits(k), bits(v), scale, causal)
    s = (q.double() @ k.double().transpose(-1, -2)) * scale
    if causal:
        s = s.masked_fill(torch.ones(24, 24, dtype=torch.bool).triu(1), float("-inf"))
    ref = torch.softmax(s, -1) @ v.double()
    assert np.array_equal(out, bits(ref.float().bfloat16())) or \
        np.abs(O.bf16_bits_to_f32(out) - ref.float().numpy()).max() < 2 ** -8 * ref.abs().max().item()
    np.testing.assert_allclose(smax[..., 0], s.max(-1).values.numpy(), rtol=1e-6)
    np.testing.assert_allclose(ssum[..., 0], torch.exp(s - s.max(-1, keepdim=True).values).sum(-1).numpy(), rtol=1e-6)
    assert (smax == smax[..., :1]).all() and (ssum == ssum[..., :1]).all()  # repeated over the axis of 8
    sdpa = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=causal)
    assert np.abs(O.bf16_bits_to_f32(out) - sdpa.float().numpy()).max() < 1e-2


def test_attention_closed_forms():
    torch.manual_seed(1)
    q, k, v = (torch.randn(1, 2, 12, 8).bfloat16() for _ in range(3))
    ones = torch.ones_like(v)
    out, _, _ = O.attention_bf16(bits(q), bits(k), bits(ones), 0.3, True)
    assert np.array_equal(out, bits(ones))  # probabilities sum to one
    out, _, ssum = O.attention_bf16(bits(q), bits(k), bits(v), 0.3, True)
    assert np.array_equal(out[:, :, 0], bits(v)[:, :, 0])  # first causal row sees one key
    assert np.allclose(ssum[:, :, 0], 1.0)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 6:] = 7.0
    v2[:, :, 6:] = -7.0
    out2, _, _ = O.attention_bf16(bits(q), bits(k2), bits(v2), 0.3, True)
    assert np.array_equal(out[:, :, :6], out2[:, :, :6])  # causal: no dependence on later keys
    kc = k[:, :, :1].expand(-1, -1, 12, -1).contiguous()
    out3, _, ssum3 = O.attention_bf16(bits(q), bits(kc), bits(v), 0.3, False)
    mean = v.double().mean(2, keepdim=True).expand(-1, -1, 12, -1)
    assert np.abs(O.bf16_bits_to_f32(out3) - mean.float().numpy()).max() < 1e-2  # equal keys: plain mean
    assert np.allclose(ssum3, 12.0)


@pytest.mark.parametrize("causal", [True, False])
def test_attention_backward_vs_central_differences(causal):
    """The backward oracle against central differences of an independent fp64 forward (numpy),
    entry by entry: a wrong sign, a dropped rowsum term or a missing scale factor all fail."""
    rng = np.random.default_rng(3)
    B, N, S, D = 1, 2, 6, 4
    mk = lambda: torch.from_numpy(rng.standard_normal((B, N, S, D)).astype(np.float32)).bfloat16()  # noqa: E731
    q, k, v, g = mk(), mk(), mk(), mk()
    scale = 0.37
    dq, dk, dv = O.attention_bwd(bits(q), bits(k), bits(v), bits(g), scale, causal)

    def loss(qa, ka, va):
        s = np.einsum("bnid,bnjd->bnij", qa, ka) * scale
        if causal:
            s = np.where(np.triu(np.ones((S, S), bool), 1), -np.inf, s)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        return float((np.einsum("bnij,bnjd->bnid", p, va) * g.double().numpy()).sum())

    base = [t.double().numpy() for t in (q, k, v)]
    eps = 1e-5
    for which, grad in enumerate((dq, dk, dv)):
        fd = np.zeros_like(grad)
        it = np.nditer(base[which], flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            plus = [a.copy() for a in base]
            minus = [a.copy() for a in base]
            plus[which][idx] += eps
            minus[which][idx] -= eps
            fd[idx] = (loss(*plus) - loss(*minus)) / (2 * eps)
        np.testing.assert_allclose(grad, fd, rtol=1e-6, atol=1e-8)


def test_attention_backward_invariants():
    """dV with dO = 1 holds the column sums of P (which total S per head); a V that is constant
    along the sequence makes dQ = dK = 0; the gradients are linear in dO."""
    torch.manual_seed(4)
    q, k, v, g = (torch.randn(1, 2, 10, 8).bfloat16() for _ in range(4))
    dq, dk, dv = O.attention_bwd(bits(q), bits(k), bits(v), bits(torch.ones_like(g)), 0.3, True)
    assert np.allclose(dv, dv[..., :1]) and np.allclose(dv[..., 0].sum(-1), 10.0)
    vc = v[:, :, :1].expand(-1, -1, 10, -1).contiguous()
    dq, dk, _ = O.attention_bwd(bits(q), bits(k), bits(vc), bits(g), 0.3, True)
    assert np.abs(dq).max() < 1e-12 and np.abs(dk).max() < 1e-12
    a = O.attention_bwd(bits(q), bits(k), bits(v), bits(g), 0.3, False)
    b = O.attention_bwd(bits(q), bits(k), bits(v), bits((g.float() * 2).bfloat16()), 0.3, False)
    for x, y in zip(a, b):
        assert np.allclose(2 * x, y)


# ---------------------------------------------------------------- ring-attention merges
def _softmax_partials(scores, v):
    """Attention over one key range in float64 with numpy: (out, row max, row sum of exp(s - max))."""
    m = scores.max(-1, keepdims=True)
    p = np.exp(scores - m)
    l = p.sum(-1, keepdims=True)
    return (p / l) @ v, m[..., 0], l[..., 0]


def test_forward_update_equals_softmax_over_the_union():
    """Merging the partial results of two key ranges must give the softmax attention over their
    union: out, row maximum and row sum (reference test/npu_indexing/attn_cp_test.py:36-59).
    A swapped weight, a missing rescale or statistics read from the wrong row fails this."""
    rng = np.random.default_rng(0)
    B, N, S, D, K1, K2 = 2, 3, 5, 4, 7, 6
    q = rng.standard_normal((B, N, S, D))
    k = rng.standard_normal((B, N, K1 + K2, D)) * 2.0
    v = rng.standard_normal((B, N, K1 + K2, D))
    s = q @ k.transpose(0, 1, 3, 2)
    o1, m1, l1 = _softmax_partials(s[..., :K1], v[:, :, :K1])
    o2, m2, l2 = _softmax_partials(s[..., K1:], v[:, :, K1:])
    o, m, l = _softmax_partials(s, v)
    sbh = lambda t: np.ascontiguousarray(t.transpose(2, 0, 1, 3).reshape(S, B, N * D)).astype(np.float32)  # noqa: E731
    st8 = lambda t: np.ascontiguousarray(np.repeat(t[..., None], 8, -1)).astype(np.float32)  # noqa: E731
    out, mx, sm = O.forward_update(sbh(o1), st8(m1), st8(l1), sbh(o2), st8(m2), st8(l2))
    np.testing.assert_allclose(out, sbh(o).astype(np.float64), rtol=2e-6, atol=2e-6)
    np.testing.assert_allclose(mx[..., 0], m, rtol=1e-6)
    np.testing.assert_allclose(sm[..., 0], l, rtol=2e-6)
    assert (mx == mx[..., :1]).all() and (sm == sm[..., :1]).all()
    # the order of the two partials does not matter
    out_b, mx_b, sm_b = O.forward_update(sbh(o2), st8(m2), st8(l2), sbh(o1), st8(m1), st8(l1))
    np.testing.assert_allclose(out_b, out, rtol=1e-12, atol=1e-12)
    assert np.array_equal(mx_b, mx)
    # a partner whose sum is zero leaves the other side unchanged
    zero = np.zeros_like(st8(l2))
    out_z, mx_z, sm_z = O.forward_update(sbh(o1), st8(m1), st8(l1), sbh(o2), st8(m1) - 1.0, zero)
    np.testing.assert_allclose(out_z, sbh(o1).astype(np.float64), rtol=0, atol=0)
    np.testing.assert_allclose(sm_z, st8(l1).astype(np.float64))


def test_forward_update_scales_come_from_the_first_statistic_lane():
    """The output weights read element 0 of the trailing axis of 8 (reference
    attn_cp_test.py:24-32, `x[..., 0]`), while max and sum merge element by element."""
    rng = np.random.default_rng(1)
    S, B, N, D = 3, 1, 2, 2
    po, co = rng.standard_normal((S, B, N * D)).astype(np.float32), rng.standard_normal((S, B, N * D)).astype(np.float32)
    pm, cm = rng.random((B, N, S, 8)).astype(np.float32), rng.random((B, N, S, 8)).astype(np.float32)
    ps, cs = rng.random((B, N, S, 8)).astype(np.float32) + 0.5, rng.random((B, N, S, 8)).astype(np.float32) + 0.5
    out, mx, sm = O.forward_update(po, pm, ps, co, cm, cs)
    m = np.maximum(pm.astype(np.float64), cm)
    a, b = ps * np.exp(pm - m), cs * np.exp(cm - m)
    np.testing.assert_allclose(mx, m)
    np.testing.assert_allclose(sm, a + b, rtol=1e-12)
    wa = (a / (a + b))[..., 0].transpose(2, 0, 1)[..., None].repeat(D, -1).reshape(S, B, N * D)
    np.testing.assert_allclose(out, po * wa + co * (1 - wa), rtol=1e-12, atol=1e-12)


def test_forward_update_lse_equals_softmax_over_the_union():
    """Same identity in log-sum-exp form, lse = max + log(sum)
    (reference test/npu_indexing/written/test_attn_cp.py:361-367)."""
    rng = np.random.default_rng(2)
    R, D, K1, K2 = 11, 8, 5, 9
    q = rng.standard_normal((R, D))
    k = rng.standard_normal((K1 + K2, D)) * 1.5
    v = rng.standard_normal((K1 + K2, D))
    s = q @ k.T
    o1, m1, l1 = _softmax_partials(s[:, :K1], v[:K1])
    o2, m2, l2 = _softmax_partials(s[:, K1:], v[K1:])
    o, m, l = _softmax_partials(s, v)
    f = lambda t: np.ascontiguousarray(t).astype(np.float32)  # noqa: E731
    out, lse = O.forward_update_lse(f(o1), f((m1 + np.log(l1))[:, None]), f(o2), f((m2 + np.log(l2))[:, None]))
    np.testing.assert_allclose(out, f(o).astype(np.float64), rtol=3e-6, atol=3e-6)
    np.testing.assert_allclose(lse[:, 0], m + np.log(l), rtol=2e-6, atol=2e-6)
    # merging a result with itself doubles the weight sum and keeps the output
    out2, lse2 = O.forward_update_lse(f(o1), f((m1 + np.log(l1))[:, None]), f(o1), f((m1 + np.log(l1))[:, None]))
    np.testing.assert_allclose(out2, f(o1).astype(np.float64), rtol=1e-12)
    np.testing.assert_allclose(lse2[:, 0], f(m1 + np.log(l1)).astype(np.float64) + np.log(2.0), rtol=1e-12)


def test_add_bf16_rounds_once_to_nearest_even():
    """1 + 2^-8 is a tie between two bf16 values and goes to the even one; 1 + 3 * 2^-9 rounds up;
    the sum is formed in fp32 before the single rounding."""
    one = O.f32_to_bf16_bits(np.array([1.0, 1.0, 256.0, -3.0], np.float32))
    add = O.f32_to_bf16_bits(np.array([2.0 ** -8, 3 * 2.0 ** -9, 1.0, 3.0], np.float32))
    got = O.bf16_bits_to_f32(O.add_bf16(one, add))
    assert list(got) == [1.0, 1.0078125, 256.0, 0.0]  # 257 is a tie between 256 and 258 -> even mantissa (256)
    rng = np.random.default_rng(3)
    a = O.f32_to_bf16_bits(rng.standard_normal(1000).astype(np.float32))
    b = O.f32_to_bf16_bits(rng.standard_normal(1000).astype(np.float32))
    ref = torch.from_numpy(O.bf16_bits_to_f32(a)).bfloat16() + torch.from_numpy(O.bf16_bits_to_f32(b)).bfloat16()
    assert np.array_equal(O.bf16_bits_to_f32(O.add_bf16(a, b)), ref.float().numpy())
