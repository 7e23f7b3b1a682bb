"""torch.compile through the backend's import hook vs eager and vs the oracle.

These read like the reference's own tests (compile with backend="inductor",
compare with eager, rtol = atol = 1e-3: reference
test/npu_indexing/reduction_test.py:28-30, permute_test.py:23-27,
argmax_test.py:19-23), plus the oracle comparison at the tolerances of the
benchmark definition.  Each test also checks that the generated wrapper calls
generated HIP kernels and no Triton kernel.
"""
import numpy as np
import pytest
import torch

from tests.helpers import announce, bits

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def backend():
    import inductor_x_amd  # noqa: F401  registration side effects

    return inductor_x_amd


@pytest.fixture(scope="module")
def O():
    from oracle import oracle

    return oracle


def compile_and_code(fn, *args):
    from torch._inductor.utils import run_and_get_code

    torch._dynamo.reset()
    out, codes = run_and_get_code(torch.compile(fn, backend="inductor"), *args)
    code = "\n".join(codes)
    assert "generated_kernel(" in code, "no generated HIP kernel in the wrapper"
    assert "triton.jit" not in code and "@triton" not in code, "Triton code was generated"
    return out, code


def test_pointwise_add_shapes():
    # reference test/npu_indexing/pointwise_test.py:12-31
    for shape in [(8, 8, 256, 128), (3, 5, 7), (1024,), (2, 3, 5, 9)]:
        announce(f"compile a+b {shape}")
        a, b = torch.randn(*shape, device=DEV), torch.randn(*shape, device=DEV)
        out, _ = compile_and_code(lambda a, b: a + b, a, b)
        torch.testing.assert_close(out, a + b, rtol=1e-3, atol=1e-3)


def test_graph1_pointwise_rowsum(O):
    announce("compile graph 1")
    torch.manual_seed(0)
    x = torch.randn(1024, 4096)
    f = lambda x: (torch.relu(2 * x + 1) * torch.sigmoid(x)).sum(-1)  # noqa: E731
    out, code = compile_and_code(f, x.to(DEV))
    assert code.count("generated_kernel(") == 1 and "'mode': 'row'" in code
    np.testing.assert_allclose(out.cpu().numpy(), O.relu_sigmoid_rowsum(x.numpy()), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(out, f(x.to(DEV)), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("shape", [(9, 1024), (32, 8, 2048), (2053, 7, 9), (8, 16, 512, 64), (1, 1, 7168), (77, 33000)])
def test_last_dim_sum_and_mean(shape):
    # reference test/npu_indexing/reduction_test.py:12-33, issue70_test.py:11-23
    announce(f"compile sum/mean {shape}")
    a, b = torch.randn(*shape, device=DEV), torch.randn(*shape, device=DEV)
    out, _ = compile_and_code(lambda a, b: ((a + b).sum(-1), (a + b).mean(-1)), a, b)
    torch.testing.assert_close(out[0], (a + b).sum(-1), rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(out[1], (a + b).mean(-1), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("dim", [0, 1, 2, 3])
def test_sum_every_dim(dim):
    # reference test/npu_indexing/reduction_test.py:36-42
    announce(f"compile sum dim={dim}")
    a = torch.randn(8, 16, 512, 64, device=DEV)
    out, _ = compile_and_code(lambda a: a.sum(dim), a)
    torch.testing.assert_close(out, a.sum(dim), rtol=1e-3, atol=1e-3)


def test_graph2_add_rmsnorm(O):
    announce("compile graph 2")
    torch.manual_seed(0)
    rows, cols = 2048, 4096
    h = torch.randn(rows, cols).bfloat16()
    r = torch.randn(rows, cols).bfloat16()
    w = (1 + 0.02 * torch.randn(cols)).bfloat16()

    def f(h, r, w):
        s = h + r
        sf = s.float()
        out = (sf * torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + 1e-6) * w.float()).to(torch.bfloat16)
        return out, s

    (out, s), code = compile_and_code(f, h.to(DEV), r.to(DEV), w.to(DEV))
    assert code.count("generated_kernel(") == 1 and "'mode': 'row'" in code
    o_ref, s_ref = O.add_rmsnorm_bf16(bits(h), bits(r), bits(w), 1e-6)
    assert np.array_equal(bits(s), s_ref)
    assert np.abs(O.bf16_bits_to_f32(bits(out)) - O.bf16_bits_to_f32(o_ref)).max() <= 2e-2


def test_graph3_col_mean_var_argmax(O):
    announce("compile graph 3")
    torch.manual_seed(0)
    x = torch.randn(65536, 512)
    f = lambda x: (x.mean(0), x.var(0, unbiased=False), x.argmax(0))  # noqa: E731
    (mean, var, arg), code = compile_and_code(f, x.to(DEV))
    assert "'mode': 'col'" in code
    m_ref, v_ref, a_ref = O.col_mean_var_argmax(x.numpy(), 0.0)
    assert np.array_equal(arg.cpu().numpy(), a_ref)
    scale = np.sqrt(v_ref)
    assert (np.abs(mean.cpu().numpy() - m_ref) <= 1e-5 * np.maximum(np.abs(m_ref), scale)).all()
    np.testing.assert_allclose(var.cpu().numpy(), v_ref, rtol=1e-5)


@pytest.mark.parametrize("shape,dim", [((512, 64), -1), ((513, 64), -1), ((513, 1024), -1), ((4096, 64), 0), ((300, 7, 12), 1)])
def test_argmax(shape, dim):
    # reference test/npu_indexing/argmax_test.py:10-25, argmax_unalign_test.py:36-58
    announce(f"compile argmax {shape} dim={dim}")
    torch.manual_seed(1)
    x = torch.randn(*shape, device=DEV) * 2000
    x[3] = x[1]  # ties between rows
    out, _ = compile_and_code(lambda x: torch.argmax(x, dim), x)
    assert torch.equal(out, torch.argmax(x, dim))


@pytest.mark.parametrize("dims", [[0, 2], [0, 1], [1, 2], [0], [1], [2]])
def test_var_mean_dims(dims):
    # reference test/npu_indexing/var_mean_test.py:8-36 (default correction)
    announce(f"compile var_mean {dims}")
    x = torch.randn(128, 8, 64, device=DEV)
    out, _ = compile_and_code(lambda x: torch.var_mean(x, dims), x)
    ref = torch.var_mean(x, dims)
    torch.testing.assert_close(out[0], ref[0], rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(out[1], ref[1], rtol=1e-3, atol=1e-3)


def test_graph4_gather_and_permute(O):
    announce("compile graph 4")
    torch.manual_seed(0)
    table = (0.02 * torch.randn(50304, 1024)).bfloat16()
    idx = torch.randint(0, 50304, (4096,), dtype=torch.int64)
    out, code = compile_and_code(lambda t, i: t[i], table.to(DEV), idx.to(DEV))
    assert np.array_equal(bits(out), O.gather_rows(bits(table), idx.numpy()))
    emb, _ = compile_and_code(lambda t, i: torch.nn.functional.embedding(i, t), table.to(DEV), idx.to(DEV))
    assert torch.equal(emb, out)
    t = torch.randn(4, 2048, 32, 128).bfloat16()
    out, code = compile_and_code(lambda t: t.permute(0, 2, 1, 3).contiguous(), t.to(DEV))
    assert "mi::vload_x<VEC, STREAM_READS>" in code and "mi::vstore<VEC" in code  # 16-byte accesses on both sides
    assert np.array_equal(bits(out), O.permute4(bits(t), (0, 2, 1, 3)))


@pytest.mark.parametrize("perm", [(0, 2, 1, 3), (0, 1, 3, 2), (3, 2, 1, 0), (1, 0, 2, 3), (0, 3, 1, 2)])
def test_permute_variants(perm):
    # reference test/npu_indexing/permute_test.py:7-30
    announce(f"compile permute {perm}")
    x = torch.randn(8, 8, 64, 128, device=DEV)
    out, _ = compile_and_code(lambda x: x.permute(*perm).contiguous() + 1.0, x)
    assert torch.equal(out, x.permute(*perm).contiguous() + 1.0)


def test_reduction_broadcast_permute():
    # reference test/npu_indexing/reduction_broadcast_permute_test.py:9-33
    announce("compile sum -> broadcast -> permute")
    a = torch.randn(8, 16, 64, 32, device=DEV)

    def f(a):
        s = a.sum(2, keepdim=True)
        return (a - s).permute(0, 2, 1, 3).contiguous()

    out, _ = compile_and_code(f, a)
    torch.testing.assert_close(out, f(a), rtol=1e-3, atol=1e-3)


def test_layernorm_fp16_and_softmax():
    # reference test/npu_indexing/issue62_test.py:8-47 (LayerNorm through var_mean + rsqrt)
    announce("compile layernorm / softmax")
    x = torch.randn(64, 1024, device=DEV, dtype=torch.float16)
    w = torch.randn(1024, device=DEV, dtype=torch.float16)
    b = torch.randn(1024, device=DEV, dtype=torch.float16)
    f = lambda x, w, b: torch.nn.functional.layer_norm(x, (1024,), w, b, 1e-5)  # noqa: E731
    out, _ = compile_and_code(f, x, w, b)
    torch.testing.assert_close(out, f(x, w, b), rtol=1e-2, atol=1e-2)
    y = torch.randn(33, 5000, device=DEV)
    out, _ = compile_and_code(lambda y: torch.softmax(y, -1), y)
    torch.testing.assert_close(out, torch.softmax(y, -1), rtol=1e-3, atol=1e-5)


def test_clamp_where_dtypes():
    # reference test/npu_indexing/clamp_test.py:28-114
    announce("compile clamp / where / dtypes")
    for dtype in (torch.float32, torch.bfloat16, torch.int32, torch.int64):
        x = (torch.randn(37, 129, device=DEV) * 10).to(dtype)
        f = lambda x: torch.where(x > 1, x.clamp(-3, 3), x * 2)  # noqa: E731
        out, _ = compile_and_code(f, x)
        torch.testing.assert_close(out, f(x), rtol=1e-3, atol=1e-3)


def test_attention_op_and_pattern():
    """The custom op under torch.compile, and the graph pattern rewriting the
    unfused matmul-softmax-matmul into it."""
    announce("compile attention op / pattern")
    from inductor_x_amd.fusion_attention_graph import npu_fusion_attention_graph

    torch.manual_seed(0)
    B, S, N, D = 2, 256, 4, 128
    q, k, v = (torch.randn(B, N, S, D, device=DEV).bfloat16() for _ in range(3))
    inv_scale = D ** 0.5

    def f(q, k, v):
        return npu_fusion_attention_graph(q, k, v, N, "BNSD", scale=inv_scale, sparse_mode=3)[0]

    torch._dynamo.reset()
    out = torch.compile(f)(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert (out.float() - ref).abs().max().item() <= 2e-2

    qs, ks, vs = (t.transpose(1, 2).contiguous() for t in (q, k, v))  # [B, S, N, D]

    def g(q, k, v):
        q, k, v = (t.permute(0, 2, 1, 3) for t in (q, k, v))
        return torch.matmul(q, k.transpose(-2, -1)).div(inv_scale).softmax(dim=-1).matmul(v)

    from torch._inductor.utils import run_and_get_code

    torch._dynamo.reset()
    with torch.no_grad():
        out, codes = run_and_get_code(torch.compile(g), qs, ks, vs)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert (out.float() - ref).abs().max().item() <= 2e-2
    # the compiled graph calls the fused op, not the library's scaled_dot_product_attention that
    # Inductor's own patterns would put there (the replacement counter also ticks while patterns
    # are traced at registration, so the generated code is what is checked)
    code = "\n".join(codes)
    assert "npu_graph.npu_fa" in code and "_scaled_dot_product" not in code

    # what the kernel cannot run (fp32) keeps Inductor's own rewrite
    torch._dynamo.reset()
    with torch.no_grad():
        out32, codes = run_and_get_code(torch.compile(g), qs.float(), ks.float(), vs.float())
    assert "npu_graph.npu_fa" not in "\n".join(codes)
    assert (out32 - ref).abs().max().item() <= 2e-2


def test_attention_pattern_cross_attention_fp16_and_negative_divisors():
    """Inference graphs: the pattern also fires for query and key of different sequence lengths
    (cross attention), for fp16 and for lengths that are no multiple of the kernel's tiles, which
    the fused kernel all runs; a negative divisor of the scores is not what the op runs and the
    pattern must not fire (Inductor's own pattern then hands the graph to the library's flash
    attention, whose result for a negative scale is the library's business, so only the rewrite is
    checked there)."""
    announce("compile attention pattern: cross attention / fp16 / ragged / negative divisor")
    from torch._inductor.utils import run_and_get_code

    from inductor_x_amd import launcher

    torch.manual_seed(1)
    N, D = 4, 128

    def make(div):
        def g(q, k, v):
            q, k, v = (t.permute(0, 2, 1, 3) for t in (q, k, v))
            return torch.matmul(q, k.transpose(-2, -1)).div(div).softmax(dim=-1).matmul(v)

        return g

    for dtype, B, Sq, Sk, div, fires in (
        (torch.bfloat16, 2, 256, 384, D ** 0.5, True),
        (torch.float16, 2, 333, 333, D ** 0.5, True),
        (torch.bfloat16, 1, 640, 640, D ** 0.5, True),
        (torch.float16, 2, 200, 77, 9.0, True),
        (torch.bfloat16, 2, 256, 256, -(D ** 0.5), False),
    ):
        q = torch.randn(B, Sq, N, D, device=DEV).to(dtype)
        k = torch.randn(B, Sk, N, D, device=DEV).to(dtype)
        v = torch.randn(B, Sk, N, D, device=DEV).to(dtype)
        g = make(div)
        torch._dynamo.reset()
        launched = []
        launcher.launch_log = launched
        try:
            with torch.no_grad():
                out, codes = run_and_get_code(torch.compile(g), q, k, v)
        finally:
            launcher.launch_log = None
        ref = g(q.float(), k.float(), v.float())
        assert ("npu_graph.npu_fa" in "\n".join(codes)) == fires, (dtype, Sq, Sk, div)
        if fires:
            assert any(name.startswith("fused_attention_fwd_") for name in launched), launched
            assert (out.float() - ref).abs().max().item() <= 3e-2
    torch._dynamo.reset()


def test_ring_attention_forward_update():
    """Merge step of ring attention: online-softmax rescale of two partial
    attention outputs (reference test/npu_indexing/attn_cp_test.py:19-59, shapes
    from :86-98 scaled down), compiled through the backend."""
    announce("compile ring-attention forward_update")
    F32_BLK = 8

    def trans_bnsd2sbh(x):
        b, n, s, d = x.shape
        return x.permute(2, 0, 1, 3).reshape(s, b, n * d)

    def broadcast_and_trans(x, h):
        n = x.shape[1]
        d = h // n
        new_x = x[..., 0].unsqueeze(3).repeat(1, 1, 1, d)
        return trans_bnsd2sbh(new_x)

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

    torch.manual_seed(0)
    S, B, H, N = 1024, 1, 1536, 12
    mk = lambda: torch.rand((B, N, S), device=DEV).unsqueeze(3).repeat(1, 1, 1, F32_BLK)  # noqa: E731
    args = (torch.randn(S, B, H, device=DEV), mk(), mk() + 0.5, torch.randn(S, B, H, device=DEV), mk(), mk() + 0.5)
    out, code = compile_and_code(forward_update, *args)
    ref = forward_update(*args)
    for a, b in zip(out, ref):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)
    bf = tuple(a.bfloat16() if i in (0, 3) else a for i, a in enumerate(args))  # bf16 outputs, fp32 statistics
    out, _ = compile_and_code(forward_update, *bf)
    ref = forward_update(*bf)
    assert out[0].dtype == torch.bfloat16 and (out[0].float() - ref[0].float()).abs().max().item() <= 2e-2
    # second half of a [2S, ...] run: non-contiguous views of every operand (the strided "1S" case the
    # reference keeps beside the contiguous one, attn_cp_test.py:113-123)
    big = (torch.randn(2 * S, B, H, device=DEV), torch.rand(B, N, 2 * S, device=DEV).unsqueeze(3).repeat(1, 1, 1, F32_BLK),
           torch.rand(B, N, 2 * S, device=DEV).unsqueeze(3).repeat(1, 1, 1, F32_BLK) + 0.5)
    prev_out_s = big[0].view(2, S, B, H)[1]
    prev_max_s = big[1].view(B, N, 2, S, F32_BLK)[:, :, 1]
    prev_sum_s = big[2].view(B, N, 2, S, F32_BLK)[:, :, 1]
    assert not prev_max_s.is_contiguous()
    sargs = (prev_out_s, prev_max_s, prev_sum_s, args[3], args[4], args[5])
    out, _ = compile_and_code(forward_update, *sargs)
    ref = forward_update(*sargs)
    for a, b in zip(out, ref):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)


def test_ring_attention_lse_merge_and_copy_back():
    """Log-sum-exp form of the ring-attention merge, functional and with the results copied
    back into the running buffers, on whole tensors and on the second-half views
    (reference test/npu_indexing/written/test_attn_cp.py:361-375, shapes from :403-421 scaled down)."""
    announce("compile ring-attention LSE merge")

    def forward_update_la(prev_out, prev_lse, cur_out, cur_lse):
        lse = torch.log(torch.exp(cur_lse) + torch.exp(prev_lse))
        out = torch.exp(prev_lse - lse) * prev_out + torch.exp(cur_lse - lse) * cur_out
        return out, lse

    def forward_update_copy(prev_out, prev_lse, cur_out, cur_lse):
        out, lse = forward_update_la(prev_out, prev_lse, cur_out, cur_lse)
        prev_out.copy_(out)
        prev_lse.copy_(lse)

    torch.manual_seed(0)
    S, B, N, D = 512, 1, 12, 128
    DS = 2 * S
    out = torch.randn(B, N, DS, D, device=DEV)
    lse = torch.rand(B, N, DS, 1, device=DEV)
    cur = torch.randn(B, N, DS, D, device=DEV)
    cur_lse = torch.rand(B, N, DS, 1, device=DEV)
    got, _ = compile_and_code(forward_update_la, out, lse, cur, cur_lse)
    ref = forward_update_la(out, lse, cur, cur_lse)
    for a, b in zip(got, ref):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)
    # in place, on the second half of the sequence (strided views of the running buffers)
    out_s = out.view(B, N, 2, S, D)
    lse_s = lse.view(B, N, 2, S, 1)
    cur_s = torch.randn(B, N, S, D, device=DEV)
    cur_lse_s = torch.rand(B, N, S, 1, device=DEV)
    out_ref, lse_ref = out.clone(), lse.clone()
    forward_update_copy(out_ref.view(B, N, 2, S, D)[:, :, 1], lse_ref.view(B, N, 2, S, 1)[:, :, 1], cur_s, cur_lse_s)
    torch._dynamo.reset()
    torch.compile(forward_update_copy)(out_s[:, :, 1], lse_s[:, :, 1], cur_s, cur_lse_s)
    torch.testing.assert_close(out, out_ref, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(lse, lse_ref, rtol=1e-5, atol=1e-6)
    assert torch.equal(out.view(B, N, 2, S, D)[:, :, 0], out_ref.view(B, N, 2, S, D)[:, :, 0])  # first half untouched


@pytest.mark.parametrize("case", [7, 6, 5])
def test_ring_attention_backward_update(case):
    """Gradient accumulation step of ring attention: in-place adds into whole buffers or into
    one half of them (reference test/npu_indexing/written/test_attn_cp.py:267-287, the three
    cases of :329-336), bf16, shapes scaled down."""
    announce(f"compile ring-attention backward_update case {case}")

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

    torch.manual_seed(case)
    S, B, H = 1024, 1, 1536
    mk2 = lambda: torch.randn(2, S, B, H, device=DEV).bfloat16()  # noqa: E731
    full = lambda: torch.randn(2 * S, B, H, device=DEV).bfloat16()  # noqa: E731
    half = lambda: torch.randn(S, B, H, device=DEV).bfloat16()  # noqa: E731
    dq, dk, dv = mk2(), mk2(), mk2()
    if case == 7:
        cur = (full(), full(), full())
    elif case == 6:
        cur = (full(), half(), half())
    else:
        cur = (half(), full(), full())
    ref = [t.clone() for t in (dq, dk, dv)]
    backward_update(*ref, *cur, case)
    torch._dynamo.reset()
    torch.compile(backward_update)(dq, dk, dv, *cur, case)
    for a, b in zip((dq, dk, dv), ref):
        assert torch.equal(a, b)  # one bf16 addition per element: bit-exact


def test_mamba_split_of_permuted_input():
    """Three-way split of a permuted tensor feeding a softplus-like tail (reference
    test/npu_indexing/mamba_test.py:7-17; the split sizes of :10 and the shapes of :20-22 scaled down)."""
    announce("compile mamba split")

    def foo(a, b):
        permute = a.permute(1, 0, 2).contiguous()
        _, _, bt = torch.split(permute, [2048, 4096, 32], 2)
        add = bt.contiguous().contiguous() + b
        y = torch.exp(add)
        where = torch.where(add < 20, add, torch.log1p(y))
        return add, where, bt

    torch.manual_seed(0)
    a = torch.randn(256, 3, 6176, device=DEV)
    b = torch.randn(32, device=DEV)
    got, _ = compile_and_code(foo, a, b)
    ref = foo(a, b)
    for x, y in zip(got, ref):
        torch.testing.assert_close(x, y, rtol=1e-5, atol=1e-6)


def test_dynamic_shapes_reuse_one_kernel():
    """dynamic=True: one compiled artefact serves several row counts (numel arguments are
    passed at launch, reference inductor_x/codegen/wrapper.py:21-38)."""
    announce("compile dynamic shapes")

    def f(x, w):
        return (torch.relu(x) * w).sum(-1), x * 2 + 1

    torch._dynamo.reset()
    cf = torch.compile(f, dynamic=True)
    w = torch.randn(1024, device=DEV)
    for rows in (64, 257, 1000, 3):
        x = torch.randn(rows, 1024, device=DEV)
        got = cf(x, w)
        ref = f(x, w)
        torch.testing.assert_close(got[0], ref[0], rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(got[1], ref[1])


def test_attention_pattern_training():
    """The unfused attention pattern in a graph that is differentiated: the joint-graph pass rewrites
    it to npu_fa / npu_fa_backward (reference inductor_x/npu_fusion_attention_graph.py:196-204), and
    the gradients agree with eager autograd to bf16 rounding."""
    announce("compile attention pattern, training")
    torch.manual_seed(0)
    B, S, N, D = 2, 256, 4, 128
    qs, ks, vs = (torch.randn(B, S, N, D, device=DEV).bfloat16().requires_grad_() for _ in range(3))
    inv = D ** 0.5

    def g(q, k, v):
        q, k, v = (t.permute(0, 2, 1, 3) for t in (q, k, v))
        return torch.matmul(q, k.transpose(-2, -1)).div(inv).softmax(dim=-1).matmul(v)

    from torch._inductor.utils import run_and_get_code

    torch._dynamo.reset()
    w = torch.randn(B, N, S, D, device=DEV).bfloat16()

    def step():
        out = torch.compile(g)(qs, ks, vs)
        (out * w).sum().backward()
        return out

    out, codes = run_and_get_code(step)
    code = "\n".join(codes)
    assert "npu_graph.npu_fa.default" in code and "npu_graph.npu_fa_backward" in code
    got = [t.grad.clone() for t in (qs, ks, vs)]
    for t in (qs, ks, vs):
        t.grad = None
    ref = g(qs, ks, vs)
    (ref * w).sum().backward()
    assert (out.float() - ref.float()).abs().max().item() <= 2e-2
    for a, t in zip(got, (qs, ks, vs)):
        assert (a.float() - t.grad.float()).abs().max().item() <= 3e-2 * max(t.grad.float().abs().max().item(), 1.0)


@pytest.mark.parametrize("case", ["all", "rows", "outer_inner", "bf16"])
def test_few_outputs_over_a_long_range(case):
    """Fewer outputs than compute units, each over a long range: the reduction is split into
    slices (two kernels: partials per slice, then a short second reduction) instead of running on
    a handful of workgroups.  The reference never splits (inductor_x/codegen/ir.py:13-24); results
    are the same sums, so the comparison with eager is the usual one."""
    announce(f"compile split reduction {case}")
    torch.manual_seed(0)
    if case == "all":
        x = torch.randn(8 * 1024 * 1024, device=DEV)
        f = lambda t: (t.sum(), t.mean(), t.var(), t.amax())  # noqa: E731
    elif case == "rows":
        x = torch.randn(16, 1024 * 1024, device=DEV)
        f = lambda t: (t.sum(-1), torch.var_mean(t, -1), t / t.abs().sum(-1, keepdim=True))  # noqa: E731
    elif case == "outer_inner":
        x = torch.randn(512, 64, 512, device=DEV)
        f = lambda t: (t.sum([0, 2]), torch.var_mean(t, [0, 2]))  # noqa: E731
    else:
        x = torch.randn(8, 1024 * 1024, device=DEV).bfloat16()
        f = lambda t: (t.float().mean(-1), t.float().amin(-1))  # noqa: E731
    got, code = compile_and_code(f, x)
    assert code.count("generated_kernel(") >= 2

    def flat(o):
        for v in o:
            if isinstance(v, (tuple, list)):
                yield from flat(v)
            else:
                yield v

    ref = f(x.double()) if case != "bf16" else f(x)
    for g, r in zip(flat(got), flat(ref)):
        torch.testing.assert_close(g.double(), r.double(), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("r", [4, 8, 32, 48, 100])
def test_short_strided_axis_reductions(r):
    """Reductions over a short axis that is not the contiguous one (the kept axis is): one kernel
    with the lanes along the kept axis and a loop over the reduced axis, no workspace."""
    announce(f"compile strided-axis reductions r={r}")
    torch.manual_seed(r)
    t = torch.randn(96, r, 320, device=DEV)
    t[3, r // 2, 7] = float("nan")
    t[5, :, 9] = 2.5  # ties: argmax must give the first index
    f = lambda t: (t.sum(1), torch.var_mean(t, 1), t.amax(1), t.argmax(1), t.amin(1))  # noqa: E731
    got, code = compile_and_code(f, t)
    if r > 8:  # shorter reductions are unrolled into a pointwise kernel by Inductor itself
        assert "'mode': 'colloop'" in code or "'mode': 'col'" in code
    ref = f(t)
    torch.testing.assert_close(got[0], ref[0], rtol=1e-5, atol=1e-5, equal_nan=True)
    torch.testing.assert_close(got[1][0], ref[1][0], rtol=1e-4, atol=1e-5, equal_nan=True)
    torch.testing.assert_close(got[1][1], ref[1][1], rtol=1e-5, atol=1e-5, equal_nan=True)
    torch.testing.assert_close(got[2], ref[2], rtol=0, atol=0, equal_nan=True)
    assert torch.equal(got[3], ref[3])
    torch.testing.assert_close(got[4], ref[4], rtol=0, atol=0, equal_nan=True)
    tb = torch.randn(64, r, 256, device=DEV).bfloat16()
    gb, _ = compile_and_code(lambda t: t.float().mean(1).bfloat16(), tb)
    torch.testing.assert_close(gb, tb.float().mean(1).bfloat16(), rtol=0, atol=1e-2)


def test_benchmark_helper(capsys):
    """The compiled-versus-eager timing helper (the reference's test scripts share one,
    test/npu_indexing/utils.py:26-65): both clocks give positive times and a line is printed."""
    announce("benchmark helper")
    from inductor_x_amd.testing import benchmark_test

    x = torch.randn(2048, 2048, device=DEV)
    f = lambda x: torch.relu(x) * 2 + 1  # noqa: E731
    torch._dynamo.reset()
    cf = torch.compile(f)
    for graph in (False, True):
        eager_us, compiled_us = benchmark_test(f, cf, (x,), name="relu_affine", times=5, repeat=4, graph=graph)
        assert eager_us > 0 and compiled_us > 0
    assert capsys.readouterr().out.count("benchmark_relu_affine") == 2


@pytest.mark.parametrize("mode", ["reduce-overhead", "max-autotune-no-cudagraphs", "max-autotune"])
def test_compile_modes(mode):
    """torch.compile's other modes over the same backend: HIP-graph capture of the generated
    launches (reduce-overhead) and autotuned library GEMMs around generated kernels, forward and
    one training step."""
    announce(f"compile mode {mode}")
    torch.manual_seed(0)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.l1 = torch.nn.Linear(512, 1024)
            self.ln = torch.nn.LayerNorm(1024)
            self.l2 = torch.nn.Linear(1024, 512)

        def forward(self, x):
            return x + self.l2(torch.nn.functional.gelu(self.ln(self.l1(x)))).softmax(-1)

    net = Net().to(DEV)
    x = torch.randn(256, 512, device=DEV)
    ref = net(x)
    torch._dynamo.reset()
    compiled = torch.compile(net, mode=mode, dynamic=False)
    with torch.no_grad():
        for _ in range(4):  # graph capture happens after the warm-up calls
            out = compiled(x).clone()
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-6)
    for _ in range(3):
        net.zero_grad()
        compiled(x).pow(2).mean().backward()
    got = net.l1.weight.grad.clone()
    net.zero_grad()
    net(x).pow(2).mean().backward()
    torch.testing.assert_close(got, net.l1.weight.grad, rtol=1e-4, atol=1e-7)


def test_generated_kernel_autotune_record_and_bandwidth_print(tmp_path, monkeypatch, capsys):
    """Generated kernels: with autotuning on, the run-time candidates of a column pair (split
    counts) are timed on the first call and the winner is written next to the code object and read
    back by a later kernel object; with the bandwidth switch on, `name: ms  GB  GB/s` is printed
    (reference inductor_x/npu_triton_heuristics.py:268-299,302-435)."""
    import glob
    import json

    from inductor_x_amd import config, hip_heuristics

    announce("generated kernel autotune record / bandwidth print")
    monkeypatch.setenv("INDUCTOR_X_AMD_CACHE", str(tmp_path))
    monkeypatch.setattr(config, "autotune", True)
    monkeypatch.setattr(config, "profile_bandwidth", True)
    made = []
    original = hip_heuristics.generated_kernel
    monkeypatch.setattr(hip_heuristics, "generated_kernel", lambda *a, **k: made.append(original(*a, **k)) or made[-1])
    torch.manual_seed(0)
    x = torch.randn(40000, 256, device=DEV) + 3.0  # unusual extents: no code object of another test matches
    f = lambda x: (x * 1.5).sum(0)  # noqa: E731
    out, code = compile_and_code(f, x)
    torch.testing.assert_close(out, f(x), rtol=1e-4, atol=1e-3)
    col = [k for k in made if k.mode == "col"]
    assert len(col) == 1
    k = col[0]
    recs = glob.glob(k.hsaco_path[: -len(".hsaco")] + ".*.best_config")
    assert len(recs) == 1, recs
    rec = json.loads(open(recs[0]).read())
    assert rec["best"] in rec["candidates"] and len(rec["candidates"]) > 1
    assert rec["timings_ms"][rec["candidates"].index(rec["best"])] == min(rec["timings_ms"])
    line = [l for l in capsys.readouterr().out.splitlines() if l.startswith(k.name + ":")]
    assert len(line) == 1 and line[0].endswith("GB/s") and " ms " in line[0]
    # a fresh kernel object over the same source reads the record and times nothing
    again = hip_heuristics.GeneratedKernel(k.name, k.meta, k.source)
    monkeypatch.setattr(again, "_autotune", lambda *a, **kw: pytest.fail("timed again despite a valid record"))
    monkeypatch.setattr(config, "profile_bandwidth", False)
    out2 = torch.empty_like(out)
    again.run(x, out2, xnumel=256, r0_numel=40000, stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert again._plans[(256, 40000)].candidate == rec["best"]
    torch.testing.assert_close(out2, out)


def test_timing_switches_leave_mutated_buffers_alone(tmp_path, monkeypatch, capsys):
    """With the bandwidth print (and autotuning) on, a generated kernel is launched several extra
    times for its timing.  A kernel that updates an operand in place (x.add_(y)) or accumulates
    through atomic stores (index_put with accumulate=True) must do that on copies: the caller's
    buffers see exactly one update (reference inductor_x/npu_triton_heuristics.py:395-429 passes the
    mutated argument names to its tuner for the same reason)."""
    from inductor_x_amd import config, hip_heuristics

    announce("timing switches on in-place and accumulating kernels")
    monkeypatch.setenv("INDUCTOR_X_AMD_CACHE", str(tmp_path))
    monkeypatch.setattr(config, "autotune", True)
    monkeypatch.setattr(config, "profile_bandwidth", True)
    made = []
    original = hip_heuristics.generated_kernel
    monkeypatch.setattr(hip_heuristics, "generated_kernel", lambda *a, **k: made.append(original(*a, **k)) or made[-1])
    torch.manual_seed(0)

    def inplace(x, y):
        x.add_(y * 3.0)
        return x

    x = torch.randn(3001, 517, device=DEV)
    y = torch.randn(3001, 517, device=DEV)
    want = x + y * 3.0
    torch._dynamo.reset()
    got = torch.compile(inplace)(x, y)
    torch.cuda.synchronize()
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(x, want, rtol=1e-6, atol=1e-6)

    def accumulate(base, idx, vals):
        return torch.index_put(base * 1.0, (idx,), vals, accumulate=True)

    base = torch.zeros(257, 64, device=DEV)
    idx = torch.randint(0, 257, (5000,), device=DEV)
    vals = torch.ones(5000, 64, device=DEV)  # integers-valued sums: exact whatever the order
    want = torch.index_put(base * 1.0, (idx,), vals, accumulate=True)
    torch._dynamo.reset()
    got = torch.compile(accumulate)(base, idx, vals)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert any(k.meta.get("mutated_args") for k in made), [k.meta.get("mutated_args") for k in made]
    assert "GB/s" in capsys.readouterr().out


def test_sum_fp32_switch_applies_to_inference_graphs_only(monkeypatch):
    """config.sum_returns_fp32 (the reference's `sum` returns the fp32 accumulator for 16-bit inputs,
    reference inductor_x/lowering.py:204-215): in an inference graph the fp32 sum is what a consumer
    reads and what the graph returns; a graph with a backward keeps the traced 16-bit type."""
    from inductor_x_amd import config

    announce("sum of bf16 returning fp32: inference graph, consumer, training graph")
    monkeypatch.setattr(config, "sum_returns_fp32", True)
    torch.manual_seed(0)
    x = torch.randn(64, 4096, device=DEV).bfloat16()
    f = lambda x: (x.sum(-1) * 2.0, x.sum(-1))  # noqa: E731
    exact = x.double().sum(-1)
    torch._dynamo.reset()
    with torch.no_grad():
        doubled, plain = torch.compile(f)(x)
    assert plain.dtype == torch.float32 and doubled.dtype == torch.float32
    # fp32 accumulation of 4096 terms of size ~1: far inside bf16's rounding step of 0.25 - 0.5 at |sum| ~ 64
    assert (plain.double() - exact).abs().max().item() < 1e-2
    assert (doubled.double() - 2 * exact).abs().max().item() < 2e-2
    xg = x.clone().requires_grad_(True)
    torch._dynamo.reset()
    out = torch.compile(lambda x: x.sum(-1))(xg)
    assert out.dtype == torch.bfloat16
    out.float().sum().backward()
    assert xg.grad is not None and xg.grad.dtype == torch.bfloat16 and torch.equal(xg.grad, torch.ones_like(xg))
    torch._dynamo.reset()


def test_fusion_benchmarking_times_generated_kernels(monkeypatch):
    """With Inductor's `benchmark_fusion` on, the scheduler asks the backend for the run time of
    candidate kernels (fused against separate) before it fuses: the backend compiles each
    candidate, runs it on random operands and returns milliseconds.  The compiled graph is the
    same function either way (the reference inherits this from Triton's scheduling, reference
    inductor_x/codegen/triton.py:525-526,550-553,613-614)."""
    import torch._inductor.config as inductor_config

    from inductor_x_amd.codegen.scheduling import HipScheduling

    announce("fusion benchmarking")
    timed = []
    original = HipScheduling.benchmark_codegened_module

    def counting(self, mod, *a, **k):
        ms, path = original(self, mod, *a, **k)
        timed.append((path, ms))
        return ms, path

    monkeypatch.setattr(HipScheduling, "benchmark_codegened_module", counting)
    torch.manual_seed(0)
    x = torch.randn(4096, 2048, device=DEV)
    w = torch.randn(2048, device=DEV)

    def f(x, w):
        y = torch.relu(x * w + 1.0)
        return y.sum(-1), (y * 2.0).amax(-1), y.mean(0)

    want = f(x, w)
    torch._dynamo.reset()
    with inductor_config.patch(benchmark_fusion=True):
        got = torch.compile(f)(x, w)
    torch.cuda.synchronize()
    for g, r in zip(got, want):
        torch.testing.assert_close(g, r, rtol=1e-4, atol=1e-3)
    assert timed and all(ms > 0 for _, ms in timed), timed
    torch._dynamo.reset()
