"""Fused attention (bf16 / fp16 MFMA kernel) against the CPU oracle and against the
closed-form properties of softmax attention.  Tolerance: 2e-2 absolute on the
16-bit output; the fp32 statistics to 1e-3 relative (they depend only on q, k).
"""
import numpy as np
import pytest
import torch

from tests.helpers import announce, bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def K():
    from inductor_x_amd import kernels

    return kernels


@pytest.fixture(scope="module")
def O():
    from oracle import oracle

    return oracle


def _check_against_oracle(K, O, q, k, v, scale, causal):
    """q, k, v: CPU tensors whose values bf16 represents exactly (the oracle reads bf16 bits)."""
    out, smax, ssum = K.fused_attention(q.to(DEV), k.to(DEV), v.to(DEV), scale, causal)
    o_ref, m_ref, l_ref = O.attention_bf16(bits(q.bfloat16()), bits(k.bfloat16()), bits(v.bfloat16()), scale, causal)
    assert out.dtype == q.dtype and out.shape == q.shape
    err = np.abs(out.float().cpu().numpy() - O.bf16_bits_to_f32(o_ref)).max()
    assert err <= 2e-2, err
    np.testing.assert_allclose(smax.cpu().numpy(), m_ref, rtol=1e-3, atol=1e-3)
    np.testing.assert_allclose(ssum.cpu().numpy(), l_ref, rtol=2e-3)


@pytest.mark.parametrize(
    "B,N,S,causal,qmul",
    [
        (1, 2, 256, True, 1.0),
        (1, 2, 256, False, 1.0),
        (2, 3, 512, True, 1.0),
        (1, 9, 512, False, 1.0),  # heads not a multiple of the 8 dies
        (1, 2, 768, True, 1.0),  # odd number of query blocks: the middle one has no partner
        (1, 2, 1024, True, 8.0),  # large scores: the reference maximum moves more than once
        (1, 2, 512, False, 8.0),
        (1, 20, 1280, True, 1.0),  # more work items than one pass of a small grid: the persistent walk
    ],
)
def test_attention_vs_oracle(K, O, B, N, S, causal, qmul):
    """Lengths that are multiples of 256: the instantiations without bounds handling."""
    announce(f"attention B={B} N={N} S={S} causal={causal} qmul={qmul}")
    torch.manual_seed(3)
    q, k, v = (torch.randn(B, N, S, 128).bfloat16() for _ in range(3))
    q = (q.float() * qmul).bfloat16()
    _check_against_oracle(K, O, q, k, v, 128 ** -0.5, causal)


@pytest.mark.parametrize(
    "B,N,Sq,Sk,causal",
    [
        (1, 1, 128, 128, True),
        (1, 9, 128, 128, False),
        (2, 3, 384, 384, True),
        (1, 2, 1, 1, True),
        (1, 2, 1, 1, False),
        (1, 2, 63, 63, True),
        (1, 2, 64, 64, False),
        (1, 3, 65, 65, True),
        (1, 2, 100, 100, False),
        (1, 2, 257, 257, True),  # a second query block with one row
        (1, 2, 300, 300, True),
        (1, 2, 300, 300, False),
        (1, 2, 1000, 1000, True),
        (1, 2, 1000, 1000, False),
        (1, 2, 100, 333, False),  # queries and keys of different lengths
        (1, 2, 512, 128, False),  # ... both aligned
        (1, 2, 256, 64, False),
        (1, 3, 700, 50, False),
        (1, 2, 30, 1100, False),
    ],
)
def test_attention_ragged_lengths_vs_oracle(K, O, B, N, Sq, Sk, causal):
    """Any sequence lengths (the reference's fused op takes them as they come, reference
    inductor_x/npu_fusion_attention_graph.py:20-35): partly filled last key tile, partly filled last
    query block, query and key lengths that differ."""
    announce(f"attention B={B} N={N} Sq={Sq} Sk={Sk} causal={causal}")
    torch.manual_seed(7)
    q = torch.randn(B, N, Sq, 128).bfloat16()
    k, v = (torch.randn(B, N, Sk, 128).bfloat16() for _ in range(2))
    _check_against_oracle(K, O, q, k, v, 128 ** -0.5, causal)


@pytest.mark.parametrize("B,N,Sq,Sk,causal", [(1, 2, 256, 256, True), (1, 3, 512, 512, False), (1, 2, 333, 333, True),
                                              (1, 2, 100, 200, False), (2, 2, 1024, 1024, True)])
def test_attention_fp16_vs_oracle(K, O, B, N, Sq, Sk, causal):
    """fp16 operands.  Inputs are multiples of 1/64 below 4 in magnitude, which both 16-bit formats
    represent exactly, so the bf16 oracle sees the same numbers."""
    announce(f"attention fp16 B={B} N={N} Sq={Sq} Sk={Sk} causal={causal}")
    torch.manual_seed(11)
    grid = lambda *shape: (torch.randint(-255, 256, shape).float() / 64).half()  # noqa: E731
    q, k, v = grid(B, N, Sq, 128), grid(B, N, Sk, 128), grid(B, N, Sk, 128)
    assert torch.equal(q.float(), q.float().bfloat16().float())
    _check_against_oracle(K, O, q, k, v, 128 ** -0.5, causal)


@pytest.mark.parametrize("dtype,B,N,Sq,Sk,D,causal", [
    (torch.bfloat16, 2, 3, 512, 512, 64, True), (torch.bfloat16, 1, 5, 300, 300, 64, True), (torch.float16, 2, 2, 256, 384, 64, False),
    (torch.float16, 1, 3, 77, 130, 40, False), (torch.bfloat16, 1, 9, 1024, 1024, 32, True), (torch.bfloat16, 1, 2, 1, 1, 8, True),
])
def test_attention_small_heads_skip_the_zero_half(K, dtype, B, N, Sq, Sk, D, causal):
    """Heads of at most 64 columns, zero-padded to 128: the instantiation that skips the all-zero d
    slices and d blocks returns bit for bit what the full-width kernel returns on the same padded
    operands (the skipped products only add zeros), and that is right against fp32 attention."""
    announce(f"attention, 64 data columns {dtype} B={B} N={N} Sq={Sq} Sk={Sk} D={D} causal={causal}")
    torch.manual_seed(31)
    pad = lambda t: torch.nn.functional.pad(t, (0, 128 - D))  # noqa: E731
    q = torch.randn(B, N, Sq, D, device=DEV).to(dtype)
    k, v = (torch.randn(B, N, Sk, D, device=DEV).to(dtype) for _ in range(2))
    scale = D ** -0.5
    narrow = K.fused_attention(pad(q), pad(k), pad(v), scale, causal, data_columns=64)
    wide = K.fused_attention(pad(q), pad(k), pad(v), scale, causal)
    assert torch.equal(narrow[0][..., :64], wide[0][..., :64])
    assert torch.equal(narrow[1], wide[1]) and torch.equal(narrow[2], wide[2])
    s = (q.float() @ k.float().transpose(-1, -2)) * scale
    if causal:
        s = s.masked_fill(torch.ones(Sq, Sk, device=DEV, dtype=torch.bool).triu(1), float("-inf"))
    ref = torch.softmax(s, -1) @ v.float()
    assert (narrow[0][..., :D].float() - ref).abs().max().item() <= 2e-2
    with pytest.raises(ValueError):
        K.fused_attention(pad(q), pad(k), pad(v), scale, causal, data_columns=0)


@pytest.mark.parametrize("dtype,B,N,Sq,Sk,causal,mshape", [
    (torch.bfloat16, 2, 3, 256, 256, False, (2, 1, 256, 256)), (torch.bfloat16, 1, 4, 300, 300, True, (300, 300)),
    (torch.float16, 2, 2, 130, 200, False, (1, 2, 130, 200)), (torch.bfloat16, 1, 2, 512, 1024, False, (1, 1, 512, 1024)),
    (torch.float16, 1, 3, 65, 68, False, (1, 3, 65, 68)), (torch.bfloat16, 2, 2, 1, 4, False, (2, 2, 1, 4)),
    (torch.bfloat16, 1, 2, 77, 131, False, (77, 131)), (torch.float16, 1, 1, 333, 333, True, (1, 1, 333, 333)),
])
def test_attention_with_a_mask(K, dtype, B, N, Sq, Sk, causal, mshape):
    """A general mask (non-zero = hidden) in the fused kernel, alone and together with the causal mask,
    broadcast over batch and / or heads: output and statistics against fp32 attention with the same mask;
    rows with every key hidden (planted) give zeros, maximum 0 and sum 1; a mask of zeros changes nothing."""
    announce(f"attention with a mask {dtype} B={B} N={N} Sq={Sq} Sk={Sk} causal={causal} mask={mshape}")
    torch.manual_seed(41)
    q = torch.randn(B, N, Sq, 128, device=DEV).to(dtype)
    k, v = (torch.randn(B, N, Sk, 128, device=DEV).to(dtype) for _ in range(2))
    mask = torch.rand(*mshape, device=DEV) < 0.4
    mask[..., 0] = False          # every row keeps its first key ...
    if Sq > 2:
        mask[..., Sq // 2, :] = True  # ... but one, which loses them all
    if Sk > 70:
        mask[..., 1, : 64] = True     # and one whose first tile is hidden entirely
        mask[..., 1, 64] = False
    scale = 0.11
    out, smax, ssum = K.fused_attention(q, k, v, scale, causal, mask=mask)
    s = (q.float() @ k.float().transpose(-1, -2)) * scale
    hide = mask if mask.dim() == 4 else mask.view(1, 1, Sq, Sk)
    hide = hide.expand(B, N, Sq, Sk).clone()
    if causal:
        hide |= torch.ones(Sq, Sk, device=DEV, dtype=torch.bool).triu(1)
    s = s.masked_fill(hide, float("-inf"))
    dead = hide.all(-1)
    m = torch.where(dead, torch.zeros_like(s[..., 0]), s.amax(-1))
    p = torch.exp(s - m.unsqueeze(-1))
    l = torch.where(dead, torch.ones_like(m), p.sum(-1))
    ref = torch.where(dead.unsqueeze(-1), torch.zeros_like(v.float()[..., :1, :]).expand(B, N, Sq, 128), (p / l.unsqueeze(-1)) @ v.float())
    assert torch.isfinite(out).all() and (out.float() - ref).abs().max().item() <= 2e-2
    torch.testing.assert_close(smax[..., 0], m, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(ssum[..., 0], l, rtol=3e-3, atol=1e-6)
    if Sq > 2:
        assert dead.any() and out[dead].abs().max().item() == 0
    # other mask types, and a mask that hides nothing
    out8 = K.fused_attention(q, k, v, scale, causal, mask=mask.to(torch.int32) * 7)[0]
    assert torch.equal(out8, out)
    packed = K.attention_mask_bits(mask, B, N, Sq, Sk)
    assert packed.dtype == torch.uint8 and packed.shape[-1] == 8 * ((Sk + 63) // 64)
    assert torch.equal(K.fused_attention(q, k, v, scale, causal, mask=packed, mask_is_packed=True)[0], out)
    plain = K.fused_attention(q, k, v, scale, causal)
    none = K.fused_attention(q, k, v, scale, causal, mask=torch.zeros(Sq, Sk, device=DEV, dtype=torch.bool))
    assert (none[0].float() - plain[0].float()).abs().max().item() <= 1e-2
    torch.testing.assert_close(none[1], plain[1], rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError):
        K.fused_attention(q, k, v, scale, causal, mask=torch.zeros(Sq + 1, Sk, device=DEV, dtype=torch.bool))


def test_attention_closed_forms(K):
    """V = 1 gives O = 1 (probabilities sum to one); with a causal mask the first
    query row returns V[0]; identical keys give the running mean of V."""
    announce("attention closed forms")
    torch.manual_seed(1)
    B, N, S = 1, 2, 256
    q = torch.randn(B, N, S, 128, device=DEV).bfloat16()
    k = torch.randn(B, N, S, 128, device=DEV).bfloat16()
    v = torch.randn(B, N, S, 128, device=DEV).bfloat16()
    ones = torch.ones_like(v)
    for causal in (True, False):
        out, _, _ = K.fused_attention(q, k, ones, 0.1, causal)
        assert (out.float() - 1).abs().max().item() <= 8e-3
    out, smax, ssum = K.fused_attention(q, k, v, 0.1, True)
    assert torch.equal(out[:, :, 0], v[:, :, 0])
    assert (ssum[:, :, 0] - 1).abs().max().item() < 1e-6  # one key: sum of exp(0)
    kc = k[:, :, :1].expand(-1, -1, S, -1).contiguous()  # all keys equal -> uniform weights
    out, _, ssum = K.fused_attention(q, kc, v, 0.1, True)
    mean = torch.cumsum(v.float(), 2) / torch.arange(1, S + 1, device=DEV).view(1, 1, S, 1)
    assert (out.float() - mean).abs().max().item() <= 2e-2
    n = torch.arange(1, S + 1, device=DEV, dtype=torch.float32).view(1, 1, S, 1).expand(B, N, S, 8)
    assert torch.allclose(ssum, n, rtol=1e-5)
    # a ragged length leaves what lies behind the last row untouched
    S = 200
    big = torch.full((B, N, S + 56, 128), 7.0, device=DEV).bfloat16()
    out, _, _ = K.fused_attention(q[:, :, :S].contiguous(), k[:, :, :S].contiguous(), ones[:, :, :S].contiguous(), 0.1, False)
    assert out.shape == (B, N, S, 128) and (out.float() - 1).abs().max().item() <= 8e-3
    assert (big == 7.0).all()


def test_attention_causality_and_sdpa_full_size_slice(K):
    """Causal output must not depend on later keys/values; and two heads at the
    BASELINE sequence length match the fp32 definition evaluated on the GPU."""
    announce("attention causality / S=4096")
    torch.manual_seed(2)
    B, N, S = 1, 2, 4096
    q, k, v = (torch.randn(B, N, S, 128, device=DEV).bfloat16() for _ in range(3))
    scale = 128 ** -0.5
    out, smax, ssum = K.fused_attention(q, k, v, scale, True)
    again = K.fused_attention(q, k, v, scale, True)
    assert torch.equal(out, again[0]) and torch.equal(smax, again[1]) and torch.equal(ssum, again[2])
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 2048:] = torch.randn_like(k2[:, :, 2048:])
    v2[:, :, 2048:] = torch.randn_like(v2[:, :, 2048:])
    out2, _, _ = K.fused_attention(q, k2, v2, scale, True)
    assert torch.equal(out[:, :, :2048], out2[:, :, :2048])
    s = (q.float() @ k.float().transpose(-1, -2)) * scale
    full = torch.softmax(s, -1) @ v.float()
    outf, smaxf, ssumf = K.fused_attention(q, k, v, scale, False)
    assert (outf.float() - full).abs().max().item() <= 2e-2
    assert torch.allclose(smaxf[..., 0], s.max(-1).values, rtol=1e-3, atol=1e-3)
    s = s.masked_fill(torch.ones(S, S, device=DEV, dtype=torch.bool).triu(1), float("-inf"))
    ref = torch.softmax(s, -1) @ v.float()
    assert (out.float() - ref).abs().max().item() <= 2e-2
    assert torch.allclose(smax[..., 0], s.max(-1).values, rtol=1e-3, atol=1e-3)
    assert torch.allclose(ssum[..., 0], torch.exp(s - s.max(-1, keepdim=True).values).sum(-1), rtol=2e-3)
    # the ragged instantiation on aligned lengths is the same arithmetic: one row fewer changes nothing above it
    out3, smax3, _ = K.fused_attention(q[:, :, :4095].contiguous(), k[:, :, :4095].contiguous(), v[:, :, :4095].contiguous(), scale, True)
    assert (out3.float() - out[:, :, :4095].float()).abs().max().item() <= 1.6e-2
    assert torch.allclose(smax3, smax[:, :, :4095], rtol=1e-6)


def test_attention_rejects_bad_operands(K):
    q = torch.randn(1, 1, 128, 64, device=DEV).bfloat16()
    with pytest.raises(ValueError):
        K.fused_attention(q, q, q, 0.1, True)  # head dim
    q = torch.randn(1, 1, 128, 128, device=DEV)
    with pytest.raises(ValueError):
        K.fused_attention(q, q, q, 0.1, True)  # dtype
    q = torch.randn(1, 1, 128, 128, device=DEV).bfloat16()
    with pytest.raises(ValueError):
        K.fused_attention(q, q[:, :, :64].contiguous(), q[:, :, :64].contiguous(), 0.1, True)  # causal with Sq != Sk
    with pytest.raises(ValueError):
        K.fused_attention(q, q.half(), q.half(), 0.1, False)  # mixed element types
    with pytest.raises(ValueError):
        K.fused_attention(q, q[:, :, :0].contiguous(), q[:, :, :0].contiguous(), 0.1, False)  # no keys


@pytest.mark.parametrize("B,N,S,causal", [(1, 2, 256, True), (2, 3, 512, False), (1, 4, 1024, True), (1, 1, 128, True)])
def test_attention_backward_vs_autograd(B, N, S, causal):
    """npu_fa_backward through the autograd wrapper against autograd of the fp32 definition.
    Tolerance: 1 % of the largest gradient entry (P and dS enter the GEMMs rounded to bf16)."""
    announce(f"attention backward B={B} N={N} S={S} causal={causal}")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(5)
    q, k, v = (torch.randn(B, N, S, 128, device=DEV).bfloat16().requires_grad_() for _ in range(3))
    do = torch.randn(B, N, S, 128, device=DEV).bfloat16()
    inv = 128 ** 0.5
    out = npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv, sparse_mode=3 if causal else 0)[0]
    out.backward(do)
    qf, kf, vf = (t.detach().float().requires_grad_() for t in (q, k, v))
    s = (qf @ kf.transpose(-1, -2)) / inv
    if causal:
        s = s.masked_fill(torch.ones(S, S, device=DEV, dtype=torch.bool).triu(1), float("-inf"))
    (torch.softmax(s, -1) @ vf).backward(do.float())
    for got, ref in ((q.grad, qf.grad), (k.grad, kf.grad), (v.grad, vf.grad)):
        assert got.dtype == torch.bfloat16 and got.shape == ref.shape
        assert (got.float() - ref).abs().max().item() <= 1e-2 * ref.abs().max().item() + 1e-3


def test_attention_backward_closed_forms():
    """V gets gradient P^T dO: with dO = 1 every row of dV is the column sum of the probabilities,
    and those sum to the number of queries over all keys; dQ and dK vanish when V is constant
    along the sequence (the output does not depend on the probabilities)."""
    announce("attention backward closed forms")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(6)
    B, N, S = 1, 2, 256
    q, k, v = (torch.randn(B, N, S, 128, device=DEV).bfloat16().requires_grad_() for _ in range(3))
    out = npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=128 ** 0.5, sparse_mode=3)[0]
    out.backward(torch.ones_like(out))
    col_sums = v.grad.float()[..., 0]  # identical along d
    assert (v.grad.float() - col_sums.unsqueeze(-1)).abs().max().item() <= 2e-2
    assert (col_sums.sum(-1) - S).abs().max().item() <= 0.02 * S
    vc = torch.randn(B, N, 1, 128, device=DEV).bfloat16().expand(B, N, S, 128).contiguous().requires_grad_()
    q2, k2 = (t.detach().clone().requires_grad_() for t in (q, k))
    out = npu_fusion_attention_graph(q2, k2, vc, N, "BNSD", scale=128 ** 0.5, sparse_mode=3)[0]
    out.backward(torch.randn_like(out))
    assert q2.grad.float().abs().max().item() <= 2e-2 and k2.grad.float().abs().max().item() <= 2e-2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,N,S,causal", [(1, 2, 256, True), (1, 3, 384, False), (1, 3, 384, True), (2, 4, 1024, True),
                                          (1, 9, 128, False), (1, 2, 128, True), (1, 2, 640, True), (1, 5, 1280, False)])
def test_attention_backward_kernels_vs_gemm_path(K, B, N, S, causal, dtype):
    """The fused backward kernels (bf16 and fp16) against the same gradients computed with library
    GEMMs from the same saved statistics.  Both round P and dS to the operand type once, so they
    agree to two bf16 ulps of the largest entry.  Sequence lengths include last blocks of 128 rows."""
    announce(f"attention backward vs GEMM path {dtype} B={B} N={N} S={S} causal={causal}")
    from inductor_x_amd import attention_backward as AB

    torch.manual_seed(7)
    q, k, v, do = (torch.randn(B, N, S, 128, device=DEV).to(dtype) for _ in range(4))
    scale = 128 ** -0.5
    o, m, l = K.fused_attention(q, k, v, scale, causal)
    a = K.fused_attention_backward(q, k, v, o, do, m, l, scale, causal)
    b = AB.fused_attention_backward(q, k, v, o, do, m, l, scale, causal, use_kernels=False)
    for x, y in zip(a, b):
        assert (x.float() - y.float()).abs().max().item() <= 8e-3 * max(y.float().abs().max().item(), 1.0)
    with pytest.raises(ValueError):
        K.fused_attention_backward(q[:, :, :32].contiguous(), k[:, :, :32].contiguous(), v[:, :, :32].contiguous(),
                                   o[:, :, :32].contiguous(), do[:, :, :32].contiguous(), m[:, :, :32].contiguous(),
                                   l[:, :, :32].contiguous(), scale, causal)


@pytest.mark.parametrize("dtype,B,N,S,D", [(torch.bfloat16, 1, 3, 100, 128), (torch.float16, 2, 2, 333, 128), (torch.bfloat16, 1, 2, 77, 64),
                                            (torch.bfloat16, 1, 2, 1, 128), (torch.float16, 1, 1, 65, 128)])
def test_attention_backward_causal_any_length(K, dtype, B, N, S, D):
    """The gradient kernels serve any sequence length on zero-padded rows: under a causal mask as they are
    (the mask hides the padded keys), without it through the instantiations with a bit mask that hides
    them.  The same gradients as the GEMM formulation from the same saved statistics."""
    announce(f"attention backward causal, padded length {dtype} B={B} N={N} S={S} D={D}")
    from inductor_x_amd import attention_backward as AB
    from inductor_x_amd import launcher

    torch.manual_seed(17)
    q, k, v, do = (torch.randn(B, N, S, D, device=DEV).to(dtype) for _ in range(4))
    scale = D ** -0.5
    o, m, l = AB.attention_forward_over_gemms(q, k, v, scale, True)
    launcher.launch_log = []
    try:
        a = AB.fused_attention_backward(q, k, v, o, do, m, l, scale, True)
        torch.cuda.synchronize()
    finally:
        log, launcher.launch_log = launcher.launch_log, None
    assert any(sym.startswith("attention_bwd8_dq_") for sym in log), log
    b = AB.fused_attention_backward(q, k, v, o, do, m, l, scale, True, use_kernels=False)
    for x, y in zip(a, b):
        assert x.shape == q.shape and x.dtype == dtype and torch.isfinite(x).all()
        assert (x.float() - y.float()).abs().max().item() <= 8e-3 * max(y.float().abs().max().item(), 1.0)
    if S % 64:
        # without the causal mask the padded keys are hidden by a bit mask: the masked kernels run
        o2, m2, l2 = AB.attention_forward_over_gemms(q, k, v, scale, False)
        launcher.launch_log = []
        try:
            a2 = AB.fused_attention_backward(q, k, v, o2, do, m2, l2, scale, False)
            torch.cuda.synchronize()
        finally:
            log, launcher.launch_log = launcher.launch_log, None
        assert sum(sym.startswith("attention_bwd8_") and sym.endswith("_masked") for sym in log) == 3, log
        b2 = AB.fused_attention_backward(q, k, v, o2, do, m2, l2, scale, False, use_kernels=False)
        for x, y in zip(a2, b2):
            assert x.shape == q.shape and torch.isfinite(x).all()
            assert (x.float() - y.float()).abs().max().item() <= 8e-3 * max(y.float().abs().max().item(), 1.0)


@pytest.mark.parametrize("dtype,B,N,S,D,causal", [(torch.bfloat16, 2, 3, 512, 64, True), (torch.float16, 1, 5, 320, 64, False),
                                                   (torch.bfloat16, 1, 2, 256, 32, True), (torch.bfloat16, 1, 3, 1024, 48, False)])
def test_attention_backward_small_heads_skip_the_zero_half(K, dtype, B, N, S, D, causal):
    """Gradient kernels for heads of at most 64 columns, zero-padded to 128: the instantiations that
    skip the all-zero d slices and d blocks return bit for bit what the full-width kernels return on
    the same padded operands, and the op-level path (which picks them) agrees with the GEMM formulation."""
    announce(f"attention backward, 64 data columns {dtype} B={B} N={N} S={S} D={D} causal={causal}")
    from inductor_x_amd import attention_backward as AB

    torch.manual_seed(33)
    pad = lambda t: torch.nn.functional.pad(t, (0, 128 - D))  # noqa: E731
    q, k, v, do = (torch.randn(B, N, S, D, device=DEV).to(dtype) for _ in range(4))
    scale = D ** -0.5
    o, m, l = K.fused_attention(pad(q), pad(k), pad(v), scale, causal, data_columns=64)
    o[..., D:] = 0
    narrow = K.fused_attention_backward(pad(q), pad(k), pad(v), o, pad(do), m, l, scale, causal, data_columns=64)
    wide = K.fused_attention_backward(pad(q), pad(k), pad(v), o, pad(do), m, l, scale, causal)
    for a, b in zip(narrow, wide):
        assert torch.equal(a[..., :64], b[..., :64])
    got = AB.fused_attention_backward(q, k, v, o[..., :D].contiguous(), do, m, l, scale, causal)
    ref = AB.fused_attention_backward(q, k, v, o[..., :D].contiguous(), do, m, l, scale, causal, use_kernels=False)
    for a, b, n in zip(got, ref, narrow):
        assert a.shape == q.shape and torch.equal(a, n[..., :D])
        assert (a.float() - b.float()).abs().max().item() <= 8e-3 * max(b.float().abs().max().item(), 1.0)


@pytest.mark.parametrize("dtype,B,N,S,D,causal,mshape", [
    (torch.bfloat16, 2, 3, 256, 128, False, (2, 1, 256, 256)), (torch.float16, 1, 2, 320, 128, True, (320, 320)),
    (torch.bfloat16, 1, 4, 512, 64, False, (1, 4, 512, 512)), (torch.bfloat16, 1, 2, 64, 128, False, (1, 1, 64, 64)),
])
def test_attention_backward_with_a_mask(K, dtype, B, N, S, D, causal, mshape):
    """Gradients under a general mask on the fused kernels (bit-packed mask for dQ, its transpose for
    dK and dV), alone and together with the causal mask, with planted rows that lose every key: against
    fp32 autograd of the unfused graph and against the GEMM formulation from the same saved statistics;
    the masked kernels are what ran (through npu_fa as well, where the mask is not paired with a causal
    mode: under those the op does not read the mask tensor, as in the reference)."""
    announce(f"attention backward with a mask {dtype} B={B} N={N} S={S} D={D} causal={causal} mask={mshape}")
    from inductor_x_amd import attention_backward as AB
    from inductor_x_amd import launcher
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(43)
    q, k, v = (torch.randn(B, N, S, D, device=DEV).to(dtype) for _ in range(3))
    do = torch.randn(B, N, S, D, device=DEV).to(dtype)
    mask = torch.rand(*mshape, device=DEV) < 0.35
    mask[..., 0] = False
    mask[..., S // 3, :] = True   # a query that sees nothing
    mask[..., :, 5] = True        # a key nobody sees
    mask[..., 0, 5] = False
    scale = D ** -0.5
    pad = (lambda t: torch.nn.functional.pad(t, (0, 128 - D))) if D < 128 else (lambda t: t)  # noqa: E731
    launcher.launch_log = []
    try:
        o, m, l = K.fused_attention(pad(q), pad(k), pad(v), scale, causal, mask=mask)
        o = o[..., :D].contiguous()
        got = AB.fused_attention_backward(q, k, v, o, do, m, l, scale, causal, atten_mask=mask)
        torch.cuda.synchronize()
    finally:
        log, launcher.launch_log = launcher.launch_log, None
    assert sum(sym.endswith("_masked") and sym.startswith("attention_bwd8_") for sym in log) == 3, log
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    hide = (mask if mask.dim() == 4 else mask.view(1, 1, S, S)).expand(B, N, S, S).clone()
    if causal:
        hide |= torch.ones(S, S, device=DEV, dtype=torch.bool).triu(1)
    s = ((qf @ kf.transpose(-1, -2)) * scale).masked_fill(hide, float("-inf"))
    dead = hide.all(-1, keepdim=True)
    p = torch.where(dead, torch.zeros_like(s), torch.softmax(torch.where(dead, torch.zeros_like(s), s), -1))
    ref = p @ vf
    ref.backward(do.float())
    assert (o.float() - ref).abs().max().item() <= 2e-2
    for g, r in zip(got[:3], (qf.grad, kf.grad, vf.grad)):
        assert g.shape == q.shape and torch.isfinite(g).all()
        assert (g.float() - r).abs().max().item() <= 3e-2 * max(r.abs().max().item(), 1.0)
    gemm = AB.fused_attention_backward(q, k, v, o, do, m, l, scale, causal, atten_mask=mask, use_kernels=False)
    for x, y in zip(got[:3], gemm[:3]):
        assert (x.float() - y.float()).abs().max().item() <= 8e-3 * max(y.float().abs().max().item(), 1.0)
    if not causal:
        qo, ko, vo = (t.clone().requires_grad_() for t in (q, k, v))
        launcher.launch_log = []
        try:
            npu_fusion_attention_graph(qo, ko, vo, N, "BNSD", atten_mask=mask, scale=1 / scale)[0].backward(do)
            torch.cuda.synchronize()
        finally:
            log, launcher.launch_log = launcher.launch_log, None
        assert any(sym.endswith("_masked") and sym.startswith("fused_attention_fwd_") for sym in log), log
        assert sum(sym.endswith("_masked") and sym.startswith("attention_bwd8_") for sym in log) == 3, log
        for g, x in zip((qo.grad, ko.grad, vo.grad), got[:3]):
            assert torch.equal(g, x)


@pytest.mark.parametrize("S,causal", [(64, True), (192, False), (320, True), (576, True)])
def test_attention_backward_sequence_multiple_of_64(K, S, causal):
    """The backward kernels take any multiple of 64: last blocks of 64 and 192 rows (the output and
    the row statistics come from fp32 torch here, independent of the forward kernel)."""
    announce(f"attention backward S={S} causal={causal}")
    from inductor_x_amd import attention_backward as AB

    torch.manual_seed(11)
    B, N = 1, 3
    q, k, v, do = (torch.randn(B, N, S, 128, device=DEV).bfloat16() for _ in range(4))
    scale = 128 ** -0.5
    sc = (q.float() @ k.float().transpose(-1, -2)) * scale
    if causal:
        sc = sc.masked_fill(torch.ones(S, S, device=DEV, dtype=torch.bool).triu(1), float("-inf"))
    mx = sc.max(-1, keepdim=True).values
    e = torch.exp(sc - mx)
    sm = e.sum(-1, keepdim=True)
    o = ((e / sm) @ v.float()).bfloat16()
    m, l = mx.expand(B, N, S, 8).contiguous(), sm.expand(B, N, S, 8).contiguous()
    a = K.fused_attention_backward(q, k, v, o, do, m, l, scale, causal)
    b = AB.fused_attention_backward(q, k, v, o, do, m, l, scale, causal, use_kernels=False)
    for x, y in zip(a, b):
        assert (x.float() - y.float()).abs().max().item() <= 8e-3 * max(y.float().abs().max().item(), 1.0)


def test_attention_backward_full_length_causal_independence(K):
    """S = 4096, causal: when only the first half of the queries carries upstream gradient, the
    later queries get dQ = 0 and the later keys (which those queries cannot see) get dK = dV = 0;
    and the gradients are linear in dO."""
    announce("attention backward S=4096 structure")
    torch.manual_seed(8)
    B, N, S = 1, 2, 4096
    q, k, v = (torch.randn(B, N, S, 128, device=DEV).bfloat16() for _ in range(3))
    scale = 128 ** -0.5
    o, m, l = K.fused_attention(q, k, v, scale, True)
    do = torch.randn_like(o)
    do[:, :, 2048:] = 0  # only the first 2048 queries carry gradient
    dq, dk, dv = K.fused_attention_backward(q, k, v, o, do, m, l, scale, True)
    assert dq[:, :, 2048:].float().abs().max().item() == 0.0
    assert dk[:, :, 2048:].float().abs().max().item() == 0.0 and dv[:, :, 2048:].float().abs().max().item() == 0.0
    assert dq[:, :, :2048].float().abs().max().item() > 0
    # linear in dO
    dq2, dk2, dv2 = K.fused_attention_backward(q, k, v, o, (do.float() * 2).bfloat16(), m, l, scale, True)
    for a, b in ((dq, dq2), (dk, dk2), (dv, dv2)):
        assert (b.float() - 2 * a.float()).abs().max().item() <= 2e-2 * max(b.float().abs().max().item(), 1.0)


@pytest.mark.parametrize("B,N,S,causal", [(1, 2, 128, True), (1, 1, 256, False), (2, 2, 256, True), (1, 1, 384, True)])
def test_attention_backward_vs_oracle(K, O, B, N, S, causal):
    """Fused backward kernels against the fp64 oracle on the same bf16 inputs (the kernels take the
    forward kernel's output and statistics).  Bar: 1 % of the largest entry of each gradient."""
    announce(f"attention backward vs oracle B={B} N={N} S={S} causal={causal}")
    torch.manual_seed(9)
    q, k, v, do = (torch.randn(B, N, S, 128).bfloat16() for _ in range(4))
    scale = 128 ** -0.5
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    o, m, l = K.fused_attention(qd, kd, vd, scale, causal)
    got = K.fused_attention_backward(qd, kd, vd, o, dod, m, l, scale, causal)
    ref = O.attention_bwd(bits(q), bits(k), bits(v), bits(do), scale, causal)
    for g, r in zip(got, ref):
        assert np.abs(g.float().cpu().numpy() - r).max() <= 1e-2 * np.abs(r).max() + 1e-3


@pytest.mark.parametrize("dtype,B,N,S,D,causal", [
    (torch.float16, 2, 3, 200, 64, True),    # fused forward on a padded head dimension, GEMM backward (fp16)
    (torch.bfloat16, 1, 4, 96, 80, False),   # fused forward (padded), GEMM backward (96 is no multiple of 64)
    (torch.float32, 1, 2, 130, 32, True),    # fp32: GEMMs both ways
    (torch.bfloat16, 1, 2, 192, 128, True),  # fused forward (ragged instantiation) and fused backward (a multiple of 64)
    (torch.bfloat16, 1, 2, 100, 160, False), (torch.float16, 1, 2, 64, 36, True),  # head dimensions the kernel does not take
])
def test_attention_op_outside_the_fused_kernels(dtype, B, N, S, D, causal):
    """npu_fa / npu_fa_backward for shapes and element types the MFMA kernels do not cover run the same
    mathematics over library GEMMs: outputs and gradients against fp32 autograd of the unfused graph."""
    announce(f"attention op over GEMMs {dtype} B={B} N={N} S={S} D={D} causal={causal}")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(12)
    q, k, v = (torch.randn(B, N, S, D, device=DEV).to(dtype).requires_grad_() for _ in range(3))
    do = torch.randn(B, N, S, D, device=DEV).to(dtype)
    inv = D ** 0.5
    res = npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv, sparse_mode=3 if causal else 0)
    out, smax, ssum = res[0], res[1], res[2]
    out.backward(do)
    got = (q.grad, k.grad, v.grad)
    qf, kf, vf = (t.detach().float().requires_grad_() for t in (q, k, v))
    s = (qf @ kf.transpose(-1, -2)) / inv
    if causal:
        s = s.masked_fill(torch.ones(S, S, device=DEV, dtype=torch.bool).triu(1), float("-inf"))
    ref = torch.softmax(s, -1) @ vf
    ref.backward(do.float())
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert out.dtype == dtype and (out.float() - ref).abs().max().item() <= tol * max(ref.abs().max().item(), 1.0)
    assert smax.shape == (B, N, S, 8) and ssum.dtype == torch.float32
    torch.testing.assert_close(smax[..., 0], s.amax(-1), rtol=1e-2, atol=1e-2)
    for g, r in zip(got, (qf.grad, kf.grad, vf.grad)):
        assert g.dtype == dtype
        assert (g.float() - r).abs().max().item() <= (1e-4 if dtype == torch.float32 else 3e-2) * max(r.abs().max().item(), 1.0)


@pytest.mark.parametrize("dtype,B,N,Sq,Sk,D", [
    (torch.bfloat16, 2, 3, 256, 384, 128),   # fused forward, gradients over GEMMs (the gradient kernels take one length)
    (torch.float16, 1, 2, 100, 333, 64),     # padded head, ragged lengths
    (torch.float32, 1, 2, 70, 45, 40),       # GEMMs both ways
])
def test_attention_op_cross_attention_gradients(dtype, B, N, Sq, Sk, D):
    """Query and key of different lengths through npu_fa and its backward: output and the three
    gradients (dk, dv in the key's shape) against fp32 autograd of the unfused graph."""
    announce(f"attention op cross attention {dtype} B={B} N={N} Sq={Sq} Sk={Sk} D={D}")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(21)
    q = torch.randn(B, N, Sq, D, device=DEV).to(dtype).requires_grad_()
    k, v = (torch.randn(B, N, Sk, D, device=DEV).to(dtype).requires_grad_() for _ in range(2))
    do = torch.randn(B, N, Sq, D, device=DEV).to(dtype)
    inv = D ** 0.5
    out = npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv)[0]
    out.backward(do)
    qf, kf, vf = (t.detach().float().requires_grad_() for t in (q, k, v))
    ref = torch.softmax((qf @ kf.transpose(-1, -2)) / inv, -1) @ vf
    ref.backward(do.float())
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert out.shape == q.shape and (out.float() - ref).abs().max().item() <= tol * max(ref.abs().max().item(), 1.0)
    for g, r, like in zip((q.grad, k.grad, v.grad), (qf.grad, kf.grad, vf.grad), (q, k, v)):
        assert g.shape == like.shape and g.dtype == dtype
        assert (g.float() - r).abs().max().item() <= (1e-4 if dtype == torch.float32 else 3e-2) * max(r.abs().max().item(), 1.0)
    with pytest.raises(ValueError):  # a causal mask is defined for equal lengths only
        npu_fusion_attention_graph(q.detach().float(), k.detach().float(), v.detach().float(), N, "BNSD", scale=inv, sparse_mode=3)


@pytest.mark.parametrize("dtype,B,N,Sq,Sk,causal,D", [
    (torch.float16, 1, 3, 200, 200, True, 128), (torch.float16, 2, 2, 512, 512, False, 128),
    (torch.bfloat16, 1, 2, 100, 300, False, 128), (torch.bfloat16, 1, 2, 77, 77, True, 128),
    (torch.bfloat16, 2, 3, 256, 256, True, 64), (torch.float16, 1, 2, 130, 130, False, 64), (torch.bfloat16, 1, 2, 192, 192, True, 80),
    (torch.float16, 2, 2, 320, 320, True, 128), (torch.float16, 1, 3, 128, 128, False, 96),
])
def test_attention_op_reaches_the_fused_kernel_for_fp16_and_any_length(dtype, B, N, Sq, Sk, causal, D):
    """npu_fa with fp16 operands, with sequence lengths that are no multiple of a tile, with
    different query and key lengths and with head dimensions below 128 (zero-padded) launches the
    MFMA kernel (not the GEMM formulation), and the training path still returns gradients where the
    backward applies (equal lengths)."""
    announce(f"attention op on the fused kernel {dtype} B={B} N={N} Sq={Sq} Sk={Sk} D={D} causal={causal}")
    from inductor_x_amd import launcher
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(13)
    q = torch.randn(B, N, Sq, D, device=DEV).to(dtype)
    k, v = (torch.randn(B, N, Sk, D, device=DEV).to(dtype) for _ in range(2))
    train = Sq == Sk
    if train:
        q, k, v = (t.requires_grad_() for t in (q, k, v))
    inv = D ** 0.5
    launcher.launch_log = []
    try:
        res = npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv, sparse_mode=3 if causal else 0)
        torch.cuda.synchronize()
    finally:
        log, launcher.launch_log = launcher.launch_log, None
    name = "f16" if dtype == torch.float16 else "bf16"
    assert any(sym.startswith(f"fused_attention_fwd_{name}_d{64 if D <= 64 else 128}_") for sym in log), log
    qf, kf, vf = (t.detach().float().requires_grad_() for t in (q, k, v))
    s = (qf @ kf.transpose(-1, -2)) / inv
    if causal:
        s = s.masked_fill(torch.ones(Sq, Sk, device=DEV, dtype=torch.bool).triu(1), float("-inf"))
    ref = torch.softmax(s, -1) @ vf
    assert res[0].dtype == dtype and res[0].shape == q.shape and (res[0].float() - ref).abs().max().item() <= 2e-2
    torch.testing.assert_close(res[1][..., 0], s.amax(-1), rtol=1e-3, atol=1e-3)
    if train:
        do = torch.randn_like(res[0])
        launcher.launch_log = []
        try:
            res[0].backward(do)
            torch.cuda.synchronize()
        finally:
            log, launcher.launch_log = launcher.launch_log, None
        if Sq % 64 == 0 or causal:
            assert any(sym.startswith(f"attention_bwd8_dq_{name}_") for sym in log), log
        ref.backward(do.float())
        for g, r in zip((q.grad, k.grad, v.grad), (qf.grad, kf.grad, vf.grad)):
            assert (g.float() - r).abs().max().item() <= 3e-2 * max(r.abs().max().item(), 1.0)


@pytest.mark.parametrize("dtype,B,N,S,D,pse_shape,mask_shape", [
    (torch.bfloat16, 2, 3, 128, 128, (1, 3, 128, 128), (2, 1, 128, 128)),
    (torch.float32, 1, 2, 100, 64, (100, 100), None),
    (torch.float16, 2, 2, 96, 128, None, (96, 96)),
    (torch.float32, 2, 2, 64, 32, (2, 2, 64, 64), (1, 1, 64, 64)),
])
def test_attention_op_positional_bias_and_mask(dtype, B, N, S, D, pse_shape, mask_shape):
    """pse (added to q k^T before the scaling) and a general atten_mask (non-zero = hidden) through
    npu_fa / npu_fa_backward: softmax(mask(scale * (pse + q k^T))) v, as the fused op of the
    reference's device library documents it (call site reference
    inductor_x/npu_fusion_attention_graph.py:31; PARITY UNPINNED against that library, pinned here by
    fp32 autograd of the written-out formula), outputs and gradients including the gradient of pse
    in pse's own (broadcast) shape.  One query row has every key hidden: it returns zeros."""
    announce(f"attention op pse {pse_shape} mask {mask_shape} {dtype} B={B} N={N} S={S} D={D}")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(31)
    q, k, v = (torch.randn(B, N, S, D, device=DEV).to(dtype).requires_grad_() for _ in range(3))
    pse = torch.randn(*pse_shape, device=DEV).to(dtype).requires_grad_() if pse_shape else None
    mask = None
    if mask_shape:
        mask = torch.rand(*mask_shape, device=DEV) < 0.3
        mask[..., 5, :] = True   # query 5 sees nothing
        mask[..., 6, :] = False  # query 6 sees everything
    inv = D ** 0.5
    res = npu_fusion_attention_graph(q, k, v, N, "BNSD", pse, None, mask, scale=inv)
    do = torch.randn_like(res[0])
    res[0].backward(do)
    qf, kf, vf = (t.detach().float().requires_grad_() for t in (q, k, v))
    pf = pse.detach().float().requires_grad_() if pse is not None else None
    s = qf @ kf.transpose(-1, -2)
    if pf is not None:
        s = s + pf
    s = s / inv
    if mask is not None:
        s = s.masked_fill(mask, float("-inf"))
    p = torch.softmax(s, -1)
    p = torch.nan_to_num(p, nan=0.0)  # the row with every key hidden
    ref = p @ vf
    ref.backward(do.float())
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert (res[0].float() - ref).abs().max().item() <= tol * max(ref.abs().max().item(), 1.0)
    if mask is not None:
        assert res[0][..., 5, :].abs().max().item() == 0.0
    gtol = 1e-4 if dtype == torch.float32 else 3e-2
    pairs = [(q.grad, qf.grad), (k.grad, kf.grad), (v.grad, vf.grad)]
    if pse is not None:
        assert pse.grad is not None and pse.grad.shape == pse.shape
        pairs.append((pse.grad, pf.grad))
    for g, r in pairs:
        assert (g.float() - r).abs().max().item() <= gtol * max(r.abs().max().item(), 1.0)


def _unfused_fp32(q, k, v, inv, causal, keep=None, keep_prob=1.0):
    """fp32 autograd-able definition on [B, N, S, D] tensors; `keep` is a [B, N, S, S] dropout mask."""
    S = q.size(2)
    s = (q @ k.transpose(-1, -2)) / inv
    if causal:
        s = s.masked_fill(torch.ones(S, S, device=q.device, dtype=torch.bool).triu(1), float("-inf"))
    p = torch.softmax(s, -1)
    if keep is not None:
        p = p * keep / keep_prob
    return p @ v


@pytest.mark.parametrize("layout", ["BSH", "SBH"])
@pytest.mark.parametrize("dtype,B,N,S,D,causal", [
    (torch.bfloat16, 2, 3, 256, 128, True),   # the fused kernels
    (torch.float16, 1, 4, 72, 64, False),     # the GEMM path
])
def test_attention_op_layouts(layout, dtype, B, N, S, D, causal):
    """Layouts BSH and SBH (reference inductor_x/npu_fusion_attention_graph.py:53-61): outputs and
    gradients come back in the caller's layout and equal the BNSD call on the same numbers bit for bit;
    the BNSD call itself is checked against fp32 autograd."""
    announce(f"attention op layout {layout} {dtype} B={B} N={N} S={S} D={D} causal={causal}")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(21)
    base = [torch.randn(B, N, S, D, device=DEV).to(dtype) for _ in range(4)]

    def to_layout(t):
        if layout == "BSH":
            return t.permute(0, 2, 1, 3).reshape(B, S, N * D).contiguous()
        return t.permute(2, 0, 1, 3).reshape(S, B, N * D).contiguous()

    def from_layout(t):
        if layout == "BSH":
            return t.view(B, S, N, D).permute(0, 2, 1, 3)
        return t.view(S, B, N, D).permute(1, 2, 0, 3)

    inv = D ** 0.5
    mode = 3 if causal else 0
    q, k, v = (t.clone().requires_grad_() for t in base[:3])
    ref = npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv, sparse_mode=mode)
    ref[0].backward(base[3])
    ql, kl, vl = (to_layout(t).requires_grad_() for t in base[:3])
    got = npu_fusion_attention_graph(ql, kl, vl, N, layout, scale=inv, sparse_mode=mode)
    assert got[0].shape == ql.shape and got[0].is_contiguous()
    assert got[1].shape == (B, N, S, 8) and torch.equal(got[1], ref[1]) and torch.equal(got[2], ref[2])
    got[0].backward(to_layout(base[3]))
    assert torch.equal(from_layout(got[0]), ref[0])
    for g, r in zip((ql.grad, kl.grad, vl.grad), (q.grad, k.grad, v.grad)):
        assert g.shape == ql.shape and torch.equal(from_layout(g), r)
    qf, kf, vf = (t.float().requires_grad_() for t in base[:3])
    want = _unfused_fp32(qf, kf, vf, inv, causal)
    want.backward(base[3].float())
    assert (ref[0].float() - want).abs().max().item() <= 2e-2 * max(want.abs().max().item(), 1.0)
    for g, r in zip((q.grad, k.grad, v.grad), (qf.grad, kf.grad, vf.grad)):
        assert (g.float() - r).abs().max().item() <= 3e-2 * max(r.abs().max().item(), 1.0)
    with pytest.raises(NotImplementedError):
        npu_fusion_attention_graph(ql, kl, vl, N, "TND", scale=inv)
    with pytest.raises(ValueError):
        npu_fusion_attention_graph(ql, kl, vl, 7, layout, scale=inv)  # 7 divides neither hidden size


@pytest.mark.parametrize("dtype,B,N,S,D,causal,keep_prob", [
    (torch.bfloat16, 2, 2, 256, 128, True, 0.8), (torch.float32, 1, 3, 100, 32, False, 0.5),
])
def test_attention_op_dropout(dtype, B, N, S, D, causal, keep_prob):
    """keep_prob < 1 (reference inductor_x/npu_fusion_attention_graph.py:150-164 passes
    keep_prob = 1 - dropout_p): output and gradients against fp32 autograd of the unfused graph under
    the mask that the op's seed output regenerates; the kept fraction; repeatability under
    torch.manual_seed; keep_prob 0 gives zeros, as torch's dropout with p = 1 does."""
    announce(f"attention op dropout {dtype} B={B} N={N} S={S} D={D} causal={causal} keep={keep_prob}")
    from inductor_x_amd.attention_backward import _heads_per_round, dropout_keep_mask
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(33)
    q, k, v = (torch.randn(B, N, S, D, device=DEV).to(dtype).requires_grad_() for _ in range(3))
    do = torch.randn(B, N, S, D, device=DEV).to(dtype)
    inv = D ** 0.5
    mode = 3 if causal else 0
    torch.manual_seed(5)
    res = npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv, keep_prob=keep_prob, sparse_mode=mode)
    out, seed, numels = res[0], res[4], res[6]
    assert seed.dtype == torch.int64 and seed.device.type == "cpu" and int(numels) == B * N * S * S
    out.backward(do)
    heads, step = B * N, _heads_per_round(B * N, S)
    keep = torch.cat([dropout_keep_mask(int(seed), h0, min(step, heads - h0), S, keep_prob, DEV)
                      for h0 in range(0, heads, step)]).view(B, N, S, S)
    assert abs(keep.float().mean().item() - keep_prob) < 0.01
    qf, kf, vf = (t.detach().float().requires_grad_() for t in (q, k, v))
    want = _unfused_fp32(qf, kf, vf, inv, causal, keep, keep_prob)
    want.backward(do.float())
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert (out.float() - want).abs().max().item() <= tol * max(want.abs().max().item(), 1.0)
    for g, r in zip((q.grad, k.grad, v.grad), (qf.grad, kf.grad, vf.grad)):
        assert (g.float() - r).abs().max().item() <= (1e-4 if dtype == torch.float32 else 3e-2) * max(r.abs().max().item(), 1.0)
    # the row statistics are those of the undropped softmax
    plain = npu_fusion_attention_graph(q.detach(), k.detach(), v.detach(), N, "BNSD", scale=inv, sparse_mode=mode)
    torch.testing.assert_close(res[1], plain[1], rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(res[2], plain[2], rtol=2e-2, atol=1e-2)
    torch.manual_seed(5)
    again = npu_fusion_attention_graph(q.detach(), k.detach(), v.detach(), N, "BNSD", scale=inv,
                                       keep_prob=keep_prob, sparse_mode=mode)
    assert int(again[4]) == int(seed) and torch.equal(again[0], out.detach())
    other = npu_fusion_attention_graph(q.detach(), k.detach(), v.detach(), N, "BNSD", scale=inv,
                                       keep_prob=keep_prob, sparse_mode=mode)
    assert int(other[4]) != int(seed) and not torch.equal(other[0], out.detach())
    zero = npu_fusion_attention_graph(q.detach(), k.detach(), v.detach(), N, "BNSD", scale=inv, keep_prob=0.0,
                                      sparse_mode=mode)
    assert zero[0].abs().max().item() == 0.0
    with pytest.raises(ValueError):
        npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv, keep_prob=1.5)


@pytest.mark.parametrize("dtype,B,N,Sq,Sk,D,pre,nxt,extra", [
    (torch.bfloat16, 2, 3, 320, 320, 128, 63, 0, False),     # causal sliding window of 64 keys
    (torch.float16, 1, 4, 256, 256, 64, 100, 17, False),      # a band around the diagonal, small heads
    (torch.bfloat16, 2, 2, 200, 200, 128, 40, 40, True),      # band joined with a key-padding mask, ragged length
    (torch.bfloat16, 1, 2, 130, 300, 128, 20, 150, False),    # query and key lengths differ (forward only)
    (torch.bfloat16, 1, 2, 256, 256, 128, 2147483647, 2147483647, False),  # the defaults: no band at all
])
def test_attention_op_sliding_window(dtype, B, N, Sq, Sk, D, pre, nxt, extra):
    """pre_tockens / next_tockens short of the sequence (op schema, reference
    inductor_x/npu_fusion_attention_graph.py:17): key j is visible to query i when -pre <= j - i <= next.
    The band runs on the fused kernels as a bit mask, forward and gradients, alone or joined with atten_mask."""
    announce(f"attention op sliding window {dtype} [{B},{N},{Sq}/{Sk},{D}] pre={pre} next={nxt} mask={extra}")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(17)
    same = Sq == Sk
    q = torch.randn(B, N, Sq, D, device=DEV).to(dtype).requires_grad_(same)
    k = torch.randn(B, N, Sk, D, device=DEV).to(dtype).requires_grad_(same)
    v = torch.randn(B, N, Sk, D, device=DEV).to(dtype).requires_grad_(same)
    user = None
    if extra:
        user = torch.zeros(B, 1, Sq, Sk, device=DEV, dtype=torch.bool)
        user[0, :, :, Sk - 30:] = True
    inv = D ** 0.5
    out = npu_fusion_attention_graph(q, k, v, N, "BNSD", atten_mask=user, scale=inv, pre_tockens=pre, next_tockens=nxt)[0]
    dist = torch.arange(Sk, device=DEV).view(1, Sk) - torch.arange(Sq, device=DEV).view(Sq, 1)
    hide = ((dist > nxt) | (dist < -pre)).view(1, 1, Sq, Sk)
    if user is not None:
        hide = hide | user
    qf, kf, vf = (t.detach().float().requires_grad_(same) for t in (q, k, v))
    s = (qf @ kf.transpose(-1, -2)) / inv
    s = s.masked_fill(hide, float("-inf"))
    gone = hide.expand(B, N, Sq, Sk).all(-1, keepdim=True)
    p = torch.softmax(s.masked_fill(gone, 0.0), -1).masked_fill(gone, 0.0)
    want = p @ vf
    assert (out.float() - want).abs().max().item() <= 2e-2
    if same:
        go = torch.randn_like(want)
        want.backward(go)
        out.backward(go.to(dtype))
        for g, r in zip((q.grad, k.grad, v.grad), (qf.grad, kf.grad, vf.grad)):
            assert torch.isfinite(g).all()
            assert (g.float() - r).abs().max().item() <= 3e-2 * max(r.abs().max().item(), 1.0)


def test_attention_op_sliding_window_launches_the_masked_kernels():
    announce("attention op sliding window launches the masked kernels")
    from inductor_x_amd import launcher as L
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(3)
    q, k, v = (torch.randn(1, 2, 256, 128, device=DEV).bfloat16().requires_grad_() for _ in range(3))
    L.launch_log = []
    try:
        out = npu_fusion_attention_graph(q, k, v, 2, "BNSD", scale=128 ** 0.5, pre_tockens=31, next_tockens=0)[0]
        out.sum().backward()
        torch.cuda.synchronize()
    finally:
        names, L.launch_log = L.launch_log, None
    assert "fused_attention_fwd_bf16_d128_full_v5_masked" in names, names
    assert {f"attention_bwd8_{w}_bf16_d128_full_masked" for w in ("dq", "dk", "dv")} <= set(names), names


@pytest.mark.parametrize("dtype,B,N,S,causal,kind", [
    (torch.bfloat16, 2, 3, 1024, False, "window"),     # keys i-200 .. i+100
    (torch.bfloat16, 1, 4, 1280, True, "window"),      # causal and the last 300 keys only
    (torch.float16, 2, 2, 777, False, "blocks"),       # block-diagonal (documents packed into one sequence), ragged length
    (torch.bfloat16, 1, 2, 512, False, "nothing"),     # one block of queries sees no key at all
])
def test_attention_mask_tile_ranges(K, dtype, B, N, S, causal, kind):
    """The masked kernel visits, per block of 256 queries, only the key tiles between the first and the last one in
    which a query of the block sees a key (kernels.attention_mask_tile_ranges): the result is bit-identical to the
    same launch over all tiles and matches the fp32 definition."""
    announce(f"attention mask tile ranges {dtype} [{B},{N},{S},128] causal={causal} {kind}")
    torch.manual_seed(23)
    q, k, v = (torch.randn(B, N, S, 128, device=DEV).to(dtype) for _ in range(3))
    i = torch.arange(S, device=DEV).view(S, 1)
    j = torch.arange(S, device=DEV).view(1, S)
    if kind == "window":
        hide = (j > i + (0 if causal else 100)) | (j < i - (299 if causal else 200))
    elif kind == "blocks":
        doc = torch.tensor([0, 130, 400, 401, 700, S], device=DEV)
        seg = torch.bucketize(torch.arange(S, device=DEV), doc[1:], right=True)
        hide = seg.view(S, 1) != seg.view(1, S)
    else:
        hide = torch.zeros(S, S, device=DEV, dtype=torch.bool)
        hide[256:512, :] = True
        hide[:256, 300:] = True
    hide = hide.view(1, 1, S, S).expand(B if kind == "blocks" else 1, 1, S, S).contiguous()
    packed = K.attention_mask_bits(hide, B, N, S, S)
    ranges = K.attention_mask_tile_ranges(packed, S, S, causal)
    assert ranges.shape == (packed.shape[0], 1, -(-S // 256), 2) and ranges.dtype == torch.int32
    lo, hi = ranges[..., 0], ranges[..., 1]
    assert (lo >= 0).all() and (hi >= lo).all() and (hi < -(-S // 64)).all()
    if kind == "window":
        assert (hi - lo).max().item() <= (256 + 300) // 64 + 2  # a band: a few tiles per block, not all of them
    scale = 128 ** -0.5
    got = K.fused_attention(q, k, v, scale, causal, mask=packed, mask_is_packed=True, tile_ranges=ranges)
    every = K.fused_attention(q, k, v, scale, causal, mask=packed, mask_is_packed=True)
    for a, b in zip(got, every):
        assert torch.equal(a, b)
    auto = K.fused_attention(q, k, v, scale, causal, mask=hide)
    assert torch.equal(auto[0], got[0])
    full_hide = hide | (torch.ones(S, S, device=DEV, dtype=torch.bool).triu(1) if causal else False)
    s = (q.float() @ k.float().transpose(-1, -2)) * scale
    s = s.masked_fill(full_hide, float("-inf"))
    gone = full_hide.expand(B, N, S, S).all(-1, keepdim=True)
    p = torch.softmax(s.masked_fill(gone, 0.0), -1).masked_fill(gone, 0.0)
    want = p @ v.float()
    assert (got[0].float() - want).abs().max().item() <= 2e-2
    assert torch.isfinite(got[1]).all() and torch.isfinite(got[2]).all()


@pytest.mark.parametrize("dtype,B,N,S,causal,kind", [
    (torch.bfloat16, 2, 2, 1024, False, "window"),
    (torch.bfloat16, 1, 3, 1280, True, "window"),
    (torch.float16, 1, 2, 768, False, "blocks"),
    (torch.bfloat16, 1, 2, 512, False, "nothing"),
])
def test_attention_backward_mask_tile_ranges(K, dtype, B, N, S, causal, kind):
    """The masked gradient kernels with tile ranges (dQ: key tiles per block of queries from the mask, dK / dV:
    query tiles per block of keys from its transpose) give bit-identical gradients to the same kernels over all
    tiles, and match autograd on the fp32 definition."""
    announce(f"attention backward mask tile ranges {dtype} [{B},{N},{S},128] causal={causal} {kind}")
    torch.manual_seed(29)
    q, k, v, go = (torch.randn(B, N, S, 128, device=DEV).to(dtype) for _ in range(4))
    i = torch.arange(S, device=DEV).view(S, 1)
    j = torch.arange(S, device=DEV).view(1, S)
    if kind == "window":
        hide = (j > i + (0 if causal else 100)) | (j < i - (299 if causal else 200))
    elif kind == "blocks":
        doc = torch.tensor([0, 130, 400, 401, 700, S], device=DEV)
        seg = torch.bucketize(torch.arange(S, device=DEV), doc[1:], right=True)
        hide = seg.view(S, 1) != seg.view(1, S)
    else:
        hide = torch.zeros(S, S, device=DEV, dtype=torch.bool)
        hide[256:512, :] = True
        hide[:256, 300:] = True
    hide = hide.view(1, 1, S, S).contiguous()
    scale = 128 ** -0.5
    out, smax, ssum = K.fused_attention(q, k, v, scale, causal, mask=hide)
    rows = K.attention_mask_bits(hide, B, N, S, S)
    cols = K.attention_mask_bits(hide.transpose(-1, -2), B, N, S, S)
    ranges = (K.attention_mask_tile_ranges(rows, S, S, causal), K.attention_mask_tile_ranges(cols, S, S, causal, transposed=True))
    got = K.fused_attention_backward(q, k, v, out, go, smax, ssum, scale, causal, packed_masks=(rows, cols), tile_ranges=ranges)
    every = K.fused_attention_backward(q, k, v, out, go, smax, ssum, scale, causal, packed_masks=(rows, cols))
    for a, b in zip(got, every):
        assert torch.equal(a, b)
    auto = K.fused_attention_backward(q, k, v, out, go, smax, ssum, scale, causal, mask=hide)
    for a, b in zip(got, auto):
        assert torch.equal(a, b)
    full_hide = hide | (torch.ones(S, S, device=DEV, dtype=torch.bool).triu(1) if causal else False)
    qf, kf, vf = (t.float().requires_grad_() for t in (q, k, v))
    s = (qf @ kf.transpose(-1, -2)) * scale
    s = s.masked_fill(full_hide, float("-inf"))
    gone = full_hide.expand(B, N, S, S).all(-1, keepdim=True)
    p = torch.softmax(s.masked_fill(gone, 0.0), -1).masked_fill(gone, 0.0)
    (p @ vf).backward(go.float())
    for g, r in zip(got, (qf.grad, kf.grad, vf.grad)):
        assert torch.isfinite(g).all()
        assert (g.float() - r).abs().max().item() <= 3e-2 * max(r.abs().max().item(), 1.0)
