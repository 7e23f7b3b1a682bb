"""torch.compile through the backend vs eager for the view / slice / broadcast graphs of the
reference's regression tests: every access here reaches the kernel as a flattened index with
divisions and remainders that the code generator has to classify per lane.  Same convention as the
reference (compile, compare with eager at rtol = atol = 1e-3); copies and slices must be bit-exact.
"""
import pytest
import torch

from tests.helpers import announce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def backend():
    import inductor_x_amd  # noqa: F401  registration side effects

    return inductor_x_amd


def check(fn, *args, exact=False, **compile_kw):
    from torch._inductor.utils import run_and_get_code

    torch._dynamo.reset()
    got, codes = run_and_get_code(torch.compile(fn, backend="inductor", **compile_kw), *args)
    code = "\n".join(codes)
    assert "triton.jit" not in code and "@triton" not in code, "Triton code was generated"
    ref = fn(*args)
    got = got if isinstance(got, (tuple, list)) else (got,)
    ref = ref if isinstance(ref, (tuple, list)) else (ref,)
    assert len(got) == len(ref)
    for g, r in zip(got, ref):
        assert g.shape == r.shape and g.dtype == r.dtype
        if exact:
            assert torch.equal(g, r)
        else:
            torch.testing.assert_close(g, r, rtol=1e-3, atol=1e-3)
    return code


@pytest.mark.parametrize("reps", [(1, 2, 1), (2, 1, 1), (1, 2, 2), (2, 2, 2)])
def test_repeat(reps):
    # reference test/npu_indexing/repeat_test.py:27-30
    announce(f"compile repeat {reps}")
    a = torch.randn(8, 1024, 64, device=DEV)
    code = check(lambda a: a.repeat(*reps), a, exact=True)
    assert "generated_kernel(" in code


def test_permute_unsqueeze_broadcast_add():
    # reference test/npu_indexing/issue57_test.py:11-25: a [512, 512, 64] table permuted to
    # [64, 512, 512] under a [1, 64, 512, 512] activation, plus a row broadcast along the last axis
    announce("compile permute + unsqueeze + broadcast add")

    def f(act, table, row):
        return act + (table.permute(2, 0, 1).unsqueeze(0) + row)

    act = torch.randn(1, 64, 512, 512, device=DEV)
    table = torch.randn(512, 512, 64, device=DEV)
    row = torch.randn(1, 1, 1, 512, device=DEV)
    assert "generated_kernel(" in check(f, act, table, row)


def test_negative_slice_then_views():
    # reference test/npu_indexing/issue61_test.py:33-45: the last 128 rows of a permuted table
    # added to an activation that is then viewed twice
    announce("compile negative slice + views")

    def f(act, table):
        t = table.permute(2, 0, 1).unsqueeze(0)
        y = act + t[:, :, -128:, :]
        return y.view(384, 128, 128).view(64, 6, 128, 128)

    act = torch.randn(64, 6, 128, 128, device=DEV)
    table = torch.randn(128, 128, 6, device=DEV)
    assert "generated_kernel(" in check(f, act, table)


def test_rearrange_heads_to_sequence_major():
    # reference test/npu_indexing/permute_reshape_test.py:9-17: 'b n s d -> s b (n d)'
    announce("compile b n s d -> s b (n d)")
    B, N, S, D = 1, 12, 4096, 8

    def f(a, b, c):
        y = (a + b).permute(2, 0, 1, 3).reshape(S, B, N * D)
        return c + y.contiguous()

    a, b = torch.randn(B, N, S, D, device=DEV), torch.randn(B, N, S, D, device=DEV)
    c = torch.randn(S, B, N * D, device=DEV)
    assert "generated_kernel(" in check(f, a, b, c)


@pytest.mark.parametrize("shape", [(8, 2048, 4), (8, 2048, 3), (8, 526, 3), (50, 526, 3), (50, 526, 129)])
def test_reshape_then_transpose_odd_sizes(shape):
    # reference test/npu_indexing/inductor_test.py:8-27: inner extents that no vector width divides
    announce(f"compile reshape + transpose {shape}")
    a = torch.randn(shape[0], shape[1] * shape[2], device=DEV)
    d = torch.randn(shape[0], shape[2], shape[1], device=DEV)
    assert "generated_kernel(" in check(lambda a, d: a.reshape(shape).permute(0, 2, 1) + d, a, d)


def test_head_split_clones_around_gemms():
    # reference test/npu_indexing/issue54_test.py:14-50 (batch scaled down 64 -> 8): three
    # projections, heads split with permute(0, 2, 1, 3) / (0, 1, 3, 2), contiguous clones feeding bmm
    announce("compile QKV head split around addmm / bmm")
    Bt, S, H, NH, HD = 8, 512, 256, 4, 64

    def f(x, wq, bq, wk_t, bk, wv, bv):
        qp = torch.addmm(bq, x, wq.t()).view(Bt, S, NH, HD).permute(0, 2, 1, 3)
        kp = torch.addmm(bk, x, wk_t).view(Bt, S, NH, HD).permute(0, 2, 1, 3).permute(0, 1, 3, 2)
        vp = torch.addmm(bv, x, wv.t()).view(Bt, S, NH, HD).permute(0, 2, 1, 3)
        qc = qp.expand(Bt, NH, S, HD).clone(memory_format=torch.contiguous_format).view(Bt * NH, S, HD)
        kc = kp.expand(Bt, NH, HD, S).clone(memory_format=torch.contiguous_format).view(Bt * NH, HD, S)
        vc = vp.expand(Bt, NH, S, HD).clone(memory_format=torch.contiguous_format).view(Bt * NH, S, HD)
        return torch.bmm(qc, kc), vc

    torch.manual_seed(0)
    x = torch.randn(Bt * S, H, device=DEV)
    ws = [torch.randn(H, H, device=DEV) * H ** -0.5 for _ in range(3)]
    bs = [torch.randn(H, device=DEV) for _ in range(3)]
    code = check(f, x, ws[0], bs[0], ws[1], bs[1], ws[2], bs[2],
                 options={"unroll_reductions_threshold": 1, "aggressive_fusion": True})
    assert "generated_kernel(" in code


def test_full_tensor_sum_chain():
    # reference test/npu_indexing/issue59_test.py:7-27: two sums over the whole [1, 1024] tensor
    # with pointwise work between and after them
    announce("compile full-tensor sum chain")

    def f(x, y, z):
        s = torch.sum(x)
        mean = s / torch.numel(s)
        sub = x - mean
        s1 = torch.sum(sub * sub)
        r = torch.rsqrt(s1 / torch.numel(s1) + 1e-05)
        mul = sub * r
        return mul, mul * y + z, r / torch.numel(r)

    x, y, z = (torch.randn(1, 1024, device=DEV) for _ in range(3))
    assert "generated_kernel(" in check(f, x, y, z)


@pytest.mark.parametrize("sl", [(slice(None), slice(3, 67)), (slice(5, 100), slice(None)), (slice(1, None, 2), slice(None, None, 3)),
                                (slice(-40, -8), slice(-64, None))])
def test_slices_are_exact(sl):
    # reference test/npu_indexing/written/test_slice.py:73-101 compares slices with torch.equal
    announce(f"compile slice {sl}")
    a = torch.randn(128, 192, device=DEV)
    b = torch.randn(128, 192, device=DEV)
    check(lambda a, b: (a[sl] + 0, a[sl] * 2 + b[sl]), a, b, exact=True)


@pytest.mark.parametrize("dim", [0, 1, 2, 3])
@pytest.mark.parametrize("perm", [(0, 2, 1, 3), (3, 2, 1, 0), (1, 0, 2, 3), (0, 3, 1, 2), (2, 0, 3, 1)])
def test_sum_broadcast_permute_matrix(dim, perm):
    # reference test/npu_indexing/reduction_broadcast_permute_test.py:9-33: every reduced axis
    # against five permutations
    announce(f"compile sum(dim={dim}) broadcast permute{perm}")

    def f(a, b):
        s = (a + b).sum(dim, keepdim=True)
        return (a - s).permute(*perm).contiguous()

    a, b = torch.randn(8, 16, 128, 64, device=DEV), torch.randn(8, 16, 128, 64, device=DEV)
    check(f, a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16, torch.int32])
@pytest.mark.parametrize("shape", [(512, 1024), (128, 64), (3, 256, 384), (2, 5, 64, 128), (5, 72, 200), (2, 784, 256)])
def test_inner_transpose_uses_register_tiles(shape, dtype):
    """Swapping the two innermost axes: the operand is read along its own contiguous axis into
    VEC x VEC register tiles (no element-wise gather) and the copy is bit-exact.  The last two
    shapes have extents that the workgroup tile does not divide (tiles hang over the end)."""
    announce(f"compile inner transpose {shape} {dtype}")
    t = (torch.randn(*shape, device=DEV) * 100).to(dtype)
    code = check(lambda t: t.transpose(-1, -2).contiguous(), t, exact=True)
    vec = 16 // t.element_size()
    if shape != (5, 72, 200) or vec == 4:  # 9 x 25 vectors of eight leave every workgroup shape half empty
        assert "mi::Tile<" in code and "mi::gather(" not in code


def test_transposed_operand_beside_contiguous_ones():
    """One operand transposed, one in output order, one broadcast row, two outputs."""
    announce("compile transposed operand + contiguous operands")

    def f(a, b, row):
        y = a.transpose(1, 2) * 2 + b
        return y + row, torch.relu(y)

    a = torch.randn(6, 256, 192, device=DEV)
    b = torch.randn(6, 192, 256, device=DEV)
    row = torch.randn(256, device=DEV)
    code = check(f, a, b, row)
    assert "mi::Tile<" in code


@pytest.mark.parametrize("shape", [(50, 526, 129), (7, 33, 20), (8, 2048, 3)])
def test_transpose_with_extents_no_vector_divides(shape):
    """Extents that no vector width divides fall back to element-wise accesses and stay correct."""
    announce(f"compile transpose odd {shape}")
    t = torch.randn(*shape, device=DEV)
    check(lambda t: t.transpose(-1, -2).contiguous() + 1, t)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("perm", [(1, 3, 2, 0), (2, 3, 1, 0), (3, 1, 2, 0), (3, 2, 1, 0), (1, 2, 3, 0), (3, 0, 1, 2), (2, 0, 3, 1)])
def test_permutations_with_a_short_innermost_output_axis(perm, dtype):
    """Permuted copies whose output innermost axis is short (16 elements) or whose input
    contiguous axis lands anywhere in the output: bit-exact, and no element-wise gather for the
    permutations that move the input's contiguous axis outward."""
    announce(f"compile permute{perm} {dtype}")
    t = torch.randn(16, 32, 64, 128, device=DEV).to(dtype)
    code = check(lambda t: t.permute(*perm).contiguous(), t, exact=True)
    if perm[-1] != 3:
        assert "mi::Tile<" in code


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(8, 64, 56, 56), (4, 256, 28, 28), (2, 3, 64, 64), (3, 96, 55, 55)])
def test_channels_last_round_trip(shape, dtype):
    """NCHW -> NHWC -> NCHW through compiled copies (both are transposing kernels), bit-exact,
    including extents that no vector width divides."""
    announce(f"compile channels_last round trip {shape} {dtype}")
    x = torch.randn(*shape, device=DEV).to(dtype)
    check(lambda x: x.contiguous(memory_format=torch.channels_last) * 1, x, exact=True)
    xc = x.contiguous(memory_format=torch.channels_last)
    check(lambda x: x.contiguous() * 1, xc, exact=True)
