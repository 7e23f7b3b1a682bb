"""Ring-attention merge steps compiled through the backend, at the shapes the reference runs them
on, against the fp64 oracle (oracle_forward_update, oracle_forward_update_lse, oracle_add_bf16).

Scenarios and shapes: reference test/npu_indexing/attn_cp_test.py:36-59,86-98 ((S,B,H,N) =
(4096,1,1536,12) fp32, sequence 2S), test/npu_indexing/written/test_attn_cp.py:186-198
((4096,1,6144,48) bf16), :267-287,329-336 (gradient accumulation, three cases) and :361-421
(log-sum-exp form, (S,B,N,D) = (4096,1,48,128) fp32).  Bars: 1e-5 relative for fp32 outputs,
2e-2 absolute for bf16 outputs, bit-exact for the bf16 accumulation.
"""
import numpy as np
import pytest
import torch

from tests.helpers import announce, bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32_BLK = 8


@pytest.fixture(scope="module", autouse=True)
def backend():
    import inductor_x_amd  # noqa: F401

    return inductor_x_amd


@pytest.fixture(scope="module")
def O():
    from oracle import oracle

    return oracle


def _compile(fn, *args, **kw):
    from torch._inductor.utils import run_and_get_code

    torch._dynamo.reset()
    out, codes = run_and_get_code(torch.compile(fn, **kw), *args)
    code = "\n".join(codes)
    assert "generated_kernel(" in code and "triton.jit" not in code and "@triton" not in code
    return out, code


def trans_bnsd2sbh(x):
    b, n, s, d = x.shape
    return x.permute(2, 0, 1, 3).reshape(s, b, n * d)


def broadcast_and_trans(x, h):
    n = x.shape[1]
    d = h // n
    return trans_bnsd2sbh(x[..., 0].unsqueeze(3).repeat(1, 1, 1, d))


def forward_update(prev_out, prev_max, prev_sum, cur_out, cur_max, cur_sum):
    org = prev_out.dtype
    smax = torch.maximum(prev_max, cur_max)
    prev_scale = torch.exp(prev_max - smax)
    cur_scale = torch.exp(cur_max - smax)
    ps = prev_sum * prev_scale
    cs = cur_sum * cur_scale
    ssum = ps + cs
    pso = broadcast_and_trans(ps / ssum, prev_out.shape[-1])
    cso = broadcast_and_trans(cs / ssum, prev_out.shape[-1])
    return (prev_out * pso + cur_out * cso).to(org), smax, ssum


@pytest.mark.parametrize("S,B,H,N,dtype", [(4096, 1, 6144, 48, torch.bfloat16), (4096, 1, 1536, 12, torch.float32)])
def test_forward_update_reference_shapes(O, S, B, H, N, dtype):
    announce(f"ring forward_update (2S,B,H,N)=({2 * S},{B},{H},{N}) {dtype}")
    torch.manual_seed(0)
    DS = 2 * S
    mk_out = lambda: torch.randn(DS, B, H).to(dtype)  # noqa: E731
    mk_st = lambda off: (torch.rand(B, N, DS) + off).unsqueeze(3).repeat(1, 1, 1, F32_BLK).contiguous()  # noqa: E731
    prev_out, cur_out = mk_out(), mk_out()
    prev_max, cur_max, prev_sum, cur_sum = mk_st(0.0), mk_st(0.0), mk_st(0.5), mk_st(0.5)
    args = (prev_out, prev_max, prev_sum, cur_out, cur_max, cur_sum)
    (out, smax, ssum), _ = _compile(forward_update, *(a.to(DEV) for a in args), options={"aggressive_fusion": True})
    ref_out, ref_max, ref_sum = O.forward_update(prev_out.float().numpy(), prev_max.numpy(), prev_sum.numpy(),
                                                 cur_out.float().numpy(), cur_max.numpy(), cur_sum.numpy())
    assert out.dtype == dtype and out.shape == (DS, B, H)
    np.testing.assert_allclose(smax.cpu().numpy(), ref_max, rtol=1e-6)
    np.testing.assert_allclose(ssum.cpu().numpy(), ref_sum, rtol=1e-5)
    got = out.float().cpu().numpy()
    if dtype == torch.bfloat16:
        assert np.abs(got - ref_out).max() <= 2e-2
    else:
        np.testing.assert_allclose(got, ref_out, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize(
    "S,B,H,N,dtype",
    [(4096, 1, 6144, 48, torch.bfloat16), (4096, 1, 1536, 12, torch.float32), (37, 2, 5 * 128, 5, torch.bfloat16),
     (100, 1, 3 * 64, 3, torch.float32), (33, 2, 17 * 128, 17, torch.float16), (65, 1, 9 * 64, 9, torch.float16)],
)
def test_forward_update_single_kernel(O, S, B, H, N, dtype):
    """The hand-written one-launch form (kernels.ring_forward_update; reference
    written/attn_cp_triton_kernel_3d.py:15-139) at the reference's two shapes and at extents that
    leave partly filled tiles along the sequence and the head axis, against the fp64 oracle; the
    previous step's statistics are a slice of a longer buffer (their head stride differs)."""
    from inductor_x_amd import kernels, launcher

    DS = 2 * S
    announce(f"ring forward_update, one kernel (2S,B,H,N)=({DS},{B},{H},{N}) {dtype}")
    torch.manual_seed(0)
    mk_out = lambda: torch.randn(DS, B, H).to(dtype)  # noqa: E731
    mk_st = lambda off, s=DS: (torch.rand(B, N, s) + off).unsqueeze(3).repeat(1, 1, 1, F32_BLK).contiguous()  # noqa: E731
    prev_out, cur_out = mk_out(), mk_out()
    cur_max, cur_sum = mk_st(0.0), mk_st(0.5)
    prev_max_buf, prev_sum_buf = mk_st(0.0, DS + 24), mk_st(0.5, DS + 24)
    prev_max, prev_sum = prev_max_buf[:, :, :DS], prev_sum_buf[:, :, :DS]
    dev = lambda t: t.to(DEV)  # noqa: E731
    pm_d, ps_d = dev(prev_max_buf)[:, :, :DS], dev(prev_sum_buf)[:, :, :DS]
    launcher.launch_log = []
    try:
        out, smax, ssum = kernels.ring_forward_update(dev(prev_out), pm_d, ps_d, dev(cur_out), dev(cur_max), dev(cur_sum))
        torch.cuda.synchronize()
    finally:
        log, launcher.launch_log = launcher.launch_log, None
    assert len(log) == 1 and log[0].startswith("ring_forward_update_"), log
    ref_out, ref_max, ref_sum = O.forward_update(prev_out.float().numpy(), prev_max.contiguous().numpy(), prev_sum.contiguous().numpy(),
                                                 cur_out.float().numpy(), cur_max.numpy(), cur_sum.numpy())
    assert out.dtype == dtype and out.shape == (DS, B, H) and smax.shape == cur_max.shape
    np.testing.assert_allclose(smax.cpu().numpy(), ref_max, rtol=1e-6)
    np.testing.assert_allclose(ssum.cpu().numpy(), ref_sum, rtol=1e-5)
    got = out.float().cpu().numpy()
    if dtype == torch.float32:
        np.testing.assert_allclose(got, ref_out, rtol=1e-5, atol=1e-5)
    else:
        assert np.abs(got - ref_out).max() <= 2e-2
    # both load forms give the same bits
    for variant in ((8, False), (8, True)):
        o2, m2, l2 = kernels.ring_forward_update(dev(prev_out), pm_d, ps_d, dev(cur_out), dev(cur_max), dev(cur_sum), variant=variant)
        assert torch.equal(o2, out) and torch.equal(m2, smax) and torch.equal(l2, ssum)


def test_forward_update_single_kernel_rejects_what_it_was_not_written_for():
    from inductor_x_amd import kernels

    announce("ring forward_update, one kernel: argument checks")
    o = torch.zeros(8, 1, 256, device=DEV, dtype=torch.bfloat16)
    st = torch.zeros(1, 2, 8, 8, device=DEV)
    with pytest.raises(ValueError):
        kernels.ring_forward_update(o, st, st, o.float(), st, st)  # mixed element types
    with pytest.raises(ValueError):
        kernels.ring_forward_update(o, st, st, o, st[..., :4].repeat(1, 1, 1, 2)[:, :, ::2], st)  # wrong sequence extent
    with pytest.raises(ValueError):
        kernels.ring_forward_update(o[:, :, :96].contiguous(), st, st, o[:, :, :96].contiguous(), st, st)  # head dimension 48
    assert kernels.ring_forward_update(o[:0], st[:, :, :0], st[:, :, :0], o[:0], st[:, :, :0], st[:, :, :0])[0].shape == (0, 1, 256)


def forward_update_la(prev_out, prev_lse, cur_out, cur_lse):
    lse = torch.log(torch.exp(cur_lse) + torch.exp(prev_lse))
    out = torch.exp(prev_lse - lse) * prev_out + torch.exp(cur_lse - lse) * cur_out
    return out, lse


def test_forward_update_lse_reference_shape(O):
    announce("ring forward_update_la (B,N,2S,D)=(1,48,8192,128) fp32")
    torch.manual_seed(1)
    B, N, DS, D = 1, 48, 8192, 128
    prev_out, cur_out = torch.randn(B, N, DS, D), torch.randn(B, N, DS, D)
    prev_lse, cur_lse = torch.rand(B, N, DS, 1), torch.rand(B, N, DS, 1)
    (out, lse), _ = _compile(forward_update_la, prev_out.to(DEV), prev_lse.to(DEV), cur_out.to(DEV), cur_lse.to(DEV))
    ref_out, ref_lse = O.forward_update_lse(prev_out.numpy(), prev_lse.numpy(), cur_out.numpy(), cur_lse.numpy())
    np.testing.assert_allclose(lse.cpu().numpy(), ref_lse, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(out.cpu().numpy(), ref_out, rtol=1e-5, atol=1e-5)
    # in place on the second half of the running buffers (strided views), as the reference's copy-back form
    S = DS // 2

    def forward_update_copy(prev_out, prev_lse, cur_out, cur_lse):
        o, l = forward_update_la(prev_out, prev_lse, cur_out, cur_lse)
        prev_out.copy_(o)
        prev_lse.copy_(l)

    run_out, run_lse = prev_out.to(DEV), prev_lse.to(DEV)
    cur_s, cur_lse_s = cur_out[:, :, :S].contiguous(), cur_lse[:, :, :S].contiguous()
    torch._dynamo.reset()
    torch.compile(forward_update_copy)(run_out.view(B, N, 2, S, D)[:, :, 1], run_lse.view(B, N, 2, S, 1)[:, :, 1],
                                       cur_s.to(DEV), cur_lse_s.to(DEV))
    ref_o2, ref_l2 = O.forward_update_lse(prev_out[:, :, S:].contiguous().numpy(), prev_lse[:, :, S:].contiguous().numpy(),
                                          cur_s.numpy(), cur_lse_s.numpy())
    np.testing.assert_allclose(run_out[:, :, S:].cpu().numpy(), ref_o2, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(run_lse[:, :, S:].cpu().numpy(), ref_l2, rtol=1e-5, atol=1e-6)
    assert torch.equal(run_out[:, :, :S].cpu(), prev_out[:, :, :S]) and torch.equal(run_lse[:, :, :S].cpu(), prev_lse[:, :, :S])


def backward_update(dq, dk, dv, cur_dq, cur_dk, cur_dv, i, rank=1):
    cp_size = 8
    if i >= cp_size - rank - 1:
        if i == cp_size - 1:
            dq.add_(cur_dq.view(dq.shape))
            dk.add_(cur_dk.view(dk.shape))
            dv.add_(cur_dv.view(dv.shape))
        else:
            dq.add_(cur_dq.view(dq.shape))
            dk[0].add_(cur_dk)
            dv[0].add_(cur_dv)
    else:
        dq[1].add_(cur_dq)
        dk.add_(cur_dk.view(dk.shape))
        dv.add_(cur_dv.view(dv.shape))


@pytest.mark.parametrize("case", [7, 6, 5])
def test_backward_update_reference_shape(O, case):
    """(S,B,H) = (16384,1,1536) bf16 (reference written/test_attn_cp.py:289-336): whole buffers
    (case 7), first halves of dk/dv (6), second half of dq (5); bit-exact single-rounding adds."""
    announce(f"ring backward_update case {case} (S,B,H)=(16384,1,1536) bf16")
    torch.manual_seed(case)
    S, B, H = 16384, 1, 1536
    mk2 = lambda: torch.randn(2, S, B, H).bfloat16()  # noqa: E731
    full = lambda: torch.randn(2 * S, B, H).bfloat16()  # noqa: E731
    half = lambda: torch.randn(S, B, H).bfloat16()  # noqa: E731
    acc = [mk2(), mk2(), mk2()]
    cur = {7: (full, full, full), 6: (full, half, half), 5: (half, full, full)}[case]
    cur = [f() for f in cur]
    dev_acc = [t.to(DEV) for t in acc]
    torch._dynamo.reset()
    torch.compile(lambda *a: backward_update(*a, case))(*dev_acc, *(c.to(DEV) for c in cur))
    for name, a0, got, c in zip(("dq", "dk", "dv"), acc, dev_acc, cur):
        exp = bits(a0).copy()
        if c.numel() == a0.numel():
            exp = O.add_bf16(exp.reshape(-1), bits(c).reshape(-1)).reshape(exp.shape)
        else:
            part = 1 if name == "dq" else 0
            exp[part] = O.add_bf16(exp[part], bits(c))
        assert np.array_equal(bits(got), exp), f"{name} differs from the oracle in case {case}"
