"""A sweep of operator kinds through torch.compile against eager: whatever a user graph contains
must either become generated HIP kernels or fall back to the library kernel, never fail to
compile.  The reference draws this line in its lowering tables (reference
inductor_x/lowering.py:89-144, 173-339: a whitelist of generated ops, everything else eager)."""
import pytest
import torch
import torch.nn.functional as F

from tests.helpers import announce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def backend():
    import inductor_x_amd  # noqa: F401  registration side effects

    return inductor_x_amd


def _t(*shape, dtype=torch.float32, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return torch.randn(*shape, generator=g).to(dtype).to(DEV)


CASES = {
    "cat_last": (lambda a, b: torch.cat([a, b * 2], -1) + 1, lambda: (_t(33, 64), _t(33, 24))),
    "cat_first_stack": (lambda a, b: torch.stack([a, b], 0).sum(0) + torch.cat([a, b], 0)[:17], lambda: (_t(17, 40), _t(17, 40))),
    "where_mask_bool": (lambda a, b: torch.where((a > 0) & (b < 0.5), a, b * 3), lambda: (_t(128, 96), _t(128, 96))),
    "clamp_abs_sign": (lambda a: torch.clamp(a, -0.5, 0.7).abs() * torch.sign(a), lambda: (_t(77, 130),)),
    "int_arith": (lambda a: (a * 3 + 7) // 2 % 5 - (a >> 1), lambda: (torch.randint(-50, 50, (64, 100), device=DEV),)),
    "int8_uint8": (lambda a, b: (a.to(torch.int32) + b.to(torch.int32)).clamp(0, 255).to(torch.uint8),
                   lambda: (torch.randint(-128, 127, (40, 64), dtype=torch.int8, device=DEV), torch.randint(0, 255, (40, 64), dtype=torch.uint8, device=DEV))),
    "fp16_mix": (lambda a, b: (a.half() * b.half()).float() + a, lambda: (_t(64, 256), _t(64, 256))),
    "fp64": (lambda a: (a.double() * 1.000000001).sum(-1), lambda: (_t(32, 128),)),
    "gelu_silu_tanh": (lambda a: F.gelu(a) + F.silu(a) * torch.tanh(a), lambda: (_t(128, 512),)),
    "exp_log_pow": (lambda a: torch.exp(a * 0.1) + torch.log(a.abs() + 1) + a.abs().pow(1.5) + a.pow(3), lambda: (_t(64, 300),)),
    "erf_sqrt_rsqrt": (lambda a: torch.erf(a) + torch.sqrt(a.abs()) + torch.rsqrt(a.abs() + 1), lambda: (_t(64, 300),)),
    "trig": (lambda a: torch.sin(a) * torch.cos(a) + torch.atan2(a, a + 2), lambda: (_t(50, 200),)),
    "floor_ceil_round_trunc": (lambda a: torch.floor(a * 3) + torch.ceil(a) + torch.round(a * 2) + torch.trunc(a * 5), lambda: (_t(64, 128),)),
    "fmod_remainder": (lambda a, b: torch.fmod(a, b.abs() + 0.5) + torch.remainder(a, b.abs() + 0.5), lambda: (_t(64, 128), _t(64, 128))),
    "isnan_isinf": (lambda a: torch.isnan(a / (a - a)).sum() + torch.isinf(1 / (a * 0)).sum(), lambda: (_t(32, 64),)),
    "softmax_logsoftmax": (lambda a: torch.softmax(a, -1) + torch.log_softmax(a, -1), lambda: (_t(100, 333),)),
    "layernorm_groupnorm": (lambda a: F.layer_norm(a, (64,)) + F.group_norm(a.view(8, 16, 64), 4).view(128, 64), lambda: (_t(128, 64),)),
    "batchnorm_eval": (lambda a: F.batch_norm(a, torch.zeros(16, device=DEV), torch.ones(16, device=DEV), training=False), lambda: (_t(8, 16, 14, 14),)),
    "amax_amin_prod_any_all": (lambda a: (a.amax(-1), a.amin(0), (a * 0.1 + 1).prod(-1), (a > 2).any(-1), (a > -5).all(0)), lambda: (_t(64, 48),)),
    "argmin_argmax_keepdim": (lambda a: (a.argmin(-1, keepdim=True), a.argmax(0)), lambda: (_t(37, 129),)),
    "cumsum_cumprod": (lambda a: torch.cumsum(a, -1) + torch.cumprod(a * 0.1 + 1, 0), lambda: (_t(33, 65),)),
    "sort_topk": (lambda a: (torch.sort(a, -1).values, torch.topk(a, 5, -1).indices), lambda: (_t(40, 100),)),
    "index_select_gather": (lambda a, i: (a.index_select(0, i), torch.gather(a, 1, i[:16].view(1, 16).expand(64, 16) % 48)),
                            lambda: (_t(64, 48), torch.randint(0, 64, (32,), device=DEV))),
    "embedding": (lambda w, i: F.embedding(i, w) * 2, lambda: (_t(1000, 64), torch.randint(0, 1000, (8, 33), device=DEV))),
    "index_put_scatter": (lambda a, i, v: (a.index_put((i,), v, accumulate=True), torch.zeros(64, 48, device=DEV).scatter_add(0, i.view(-1, 1).expand(32, 48), v)),
                          lambda: (_t(64, 48), torch.randint(0, 64, (32,), device=DEV), _t(32, 48))),
    "masked_fill_tril": (lambda a: a.masked_fill(torch.ones(96, 96, device=DEV, dtype=torch.bool).triu(1), float("-inf")).softmax(-1), lambda: (_t(4, 96, 96),)),
    "arange_iota": (lambda a: a + torch.arange(a.shape[-1], device=DEV) * 0.5 + torch.linspace(0, 1, a.shape[0], device=DEV)[:, None], lambda: (_t(64, 100),)),
    "expand_repeat_flip_roll": (lambda a: a[:, None, :].expand(16, 3, 40).reshape(48, 40) + a.repeat(3, 1) + a.flip(-1).repeat(3, 1) + a.roll(3, -1).repeat(3, 1), lambda: (_t(16, 40),)),
    "pad_unfold": (lambda a: F.pad(a, (1, 2, 3, 0), value=0.5).sum() + a.unfold(-1, 4, 2).sum(-1).sum(), lambda: (_t(8, 30),)),
    "avgpool_maxpool_upsample": (lambda a: F.avg_pool2d(a, 2) + F.max_pool2d(a, 2) + F.interpolate(a, scale_factor=0.5, mode="nearest"), lambda: (_t(2, 8, 16, 16),)),
    "conv_relu_bias": (lambda a, w, b: F.relu(F.conv2d(a, w, b, padding=1)) * 2, lambda: (_t(2, 8, 16, 16), _t(8, 8, 3, 3), _t(8))),
    "linear_gelu_residual": (lambda a, w, b: a + F.gelu(F.linear(a, w, b)), lambda: (_t(64, 128), _t(128, 128), _t(128))),
    "bmm_scale_mask": (lambda a, b: (torch.bmm(a, b.transpose(1, 2)) * 0.125).masked_fill(torch.eye(32, device=DEV, dtype=torch.bool), 0), lambda: (_t(4, 32, 64), _t(4, 32, 64))),
    "dropout_eval_rand_like_shape": (lambda a: F.dropout(a, 0.5, training=False) + torch.zeros_like(a) + torch.full_like(a, 2.0), lambda: (_t(64, 64),)),
    "mse_crossentropy": (lambda a, t: F.cross_entropy(a, t) + F.mse_loss(a, a * 0.5), lambda: (_t(64, 100), torch.randint(0, 100, (64,), device=DEV))),
    "scalar_outputs_and_views": (lambda a: (a.sum(), a.mean(), a.t(), a[::2, 1::3], a.view(-1)[5:50]), lambda: (_t(20, 30),)),
    "complex_broadcast_5d": (lambda a, b, c: a[:, :, None] * b[None, :, :, None, :] + c, lambda: (_t(3, 4, 5, 6), _t(4, 1, 6), _t(1, 1, 7, 5, 6))),
    "var_std_norm": (lambda a: (a.var(-1), a.std(0), a.norm(dim=-1), torch.linalg.vector_norm(a, ord=1, dim=0)), lambda: (_t(65, 130),)),
    "bf16_chain": (lambda a, b: (F.silu(a) * b + a).to(torch.bfloat16).float().sum(-1), lambda: (_t(64, 512, dtype=torch.bfloat16), _t(64, 512, dtype=torch.bfloat16))),
    # reference test/npu_indexing/test_AddLayerNorm.py:95-100 at (64, 512, 256), scaled down
    "add_layernorm_by_hand": (lambda a, b: (lambda x, m: (x - m) / torch.sqrt(((x - m) ** 2).mean(2, keepdim=True) + 1e-5))(a + b, (a + b).mean(2, keepdim=True)),
                              lambda: (_t(16, 128, 256), _t(16, 128, 256, seed=1))),
    # reference test/npu_indexing/test_sum.py:94-105: a one-row sum with a broadcast scalar operand
    "one_row_sum_broadcast": (lambda a, b, c: (a + b + c).sum(1), lambda: (_t(1, 1024), _t(1, 1024, seed=1), _t(1, 1))),
    "logsumexp_sigmoid_bce": (lambda a, t: torch.logsumexp(a, -1).sum() + F.binary_cross_entropy_with_logits(a, torch.sigmoid(t)), lambda: (_t(32, 77), _t(32, 77))),
}


ROUNDED_IN_CHAIN = {"bf16_chain", "fp16_mix"}


@pytest.mark.parametrize("name", sorted(CASES))
def test_operator_kinds(name):
    announce(f"compile op sweep: {name}")
    fn, make = CASES[name]
    args = make()
    torch._dynamo.reset()
    # 16-bit intermediates stay in fp32 inside a generated kernel unless the
    # rounding of every eager op is asked for; the two cases that round in the
    # middle of a chain ask for it so that the comparison stays tight.
    from torch._inductor import config as inductor_config

    with inductor_config.patch(emulate_precision_casts=name in ROUNDED_IN_CHAIN):
        got = torch.compile(fn, dynamic=False)(*args)
    ref = fn(*args)
    got = got if isinstance(got, (tuple, list)) else (got,)
    ref = ref if isinstance(ref, (tuple, list)) else (ref,)
    assert len(got) == len(ref)
    for g, r in zip(got, ref):
        assert g.shape == r.shape and g.dtype == r.dtype, (g.shape, r.shape, g.dtype, r.dtype)
        if r.dtype.is_floating_point:
            tol = dict(rtol=2e-2, atol=2e-2) if r.dtype in (torch.bfloat16, torch.float16) else dict(rtol=2e-4, atol=2e-4)
            if name in ROUNDED_IN_CHAIN:
                # a last-bit difference before a 16-bit rounding flips that rounding: one 16-bit ulp
                # per flipped element, however the value is later widened or summed
                tol = dict(rtol=5e-3, atol=5e-3 * max(1.0, float(r.abs().max())))
            torch.testing.assert_close(g, r, equal_nan=True, **tol)
        else:
            assert torch.equal(g, r)


def _compare(got, ref, name=""):
    got = got if isinstance(got, (tuple, list)) else (got,)
    ref = ref if isinstance(ref, (tuple, list)) else (ref,)
    assert len(got) == len(ref)
    for g, r in zip(got, ref):
        assert g.shape == r.shape and g.dtype == r.dtype, (name, g.shape, r.shape, g.dtype, r.dtype)
        if r.dtype.is_floating_point:
            torch.testing.assert_close(g, r, equal_nan=True, rtol=2e-2, atol=2e-2 * max(1.0, float(r.abs().max())))
        else:
            assert torch.equal(g, r), name


@pytest.mark.parametrize("name", sorted(set(CASES) - {"dropout_eval_rand_like_shape"}))
def test_operator_kinds_symbolic_sizes(name):
    """The same graphs with every size symbolic: sizes reach the kernels as arguments
    (reference inductor_x/codegen/wrapper.py:21-38 passes the numels the same way)."""
    announce(f"compile op sweep, dynamic=True: {name}")
    fn, make = CASES[name]
    args = make()
    torch._dynamo.reset()
    got = torch.compile(fn, dynamic=True)(*args)
    _compare(got, fn(*args), name)


def test_dynamic_batch_keeps_vectors():
    """Only the leading size is dynamic: rows of fixed width still move as whole vectors
    (the symbolic element count is provably a multiple of the width), and one artefact
    serves every batch."""
    announce("compile dynamic batch, vector width")
    from torch._inductor.utils import run_and_get_code

    def f(a, b):
        return torch.relu(a) * 2 + b, torch.softmax(a, -1), (a * b).permute(0, 2, 1).contiguous()

    torch._dynamo.reset()
    a, b = _t(24, 40, 256), _t(24, 40, 256, seed=1)
    for t in (a, b):
        torch._dynamo.mark_dynamic(t, 0)
    cf = torch.compile(f)
    got, codes = run_and_get_code(cf, a, b)
    _compare(got, f(a, b))
    import re

    widths = [int(m) for m in re.findall(r"'vec': (\d+)", codes[0])]
    assert widths and min(widths) >= 4, widths
    for batch in (7, 100, 1):
        a, b = _t(batch, 40, 256, seed=2), _t(batch, 40, 256, seed=3)
        _compare(cf(a, b), f(a, b))


def test_layernorm_backward_weight_gradient_is_a_column_sweep():
    """The weight gradient of LayerNorm sums dy * xhat over rows; xhat is rebuilt from per-row
    statistics, whose indices move along the reduced axis only.  Those slivers must not outvote
    the two full tensors when the code shape is chosen: the kernel walks rows with lanes along
    the contiguous kept axis (the reference picks the tiling axis from the low dimension of the
    dominant accesses the same way, reference inductor_x/codegen/split_tiling.py:188-239)."""
    announce("compile layernorm backward, code shapes")
    import re

    from torch._inductor.utils import run_and_get_code

    def ln_bwd(dy, x, w):
        xf = x.float()
        mean = xf.mean(-1, keepdim=True)
        rstd = torch.rsqrt(xf.var(-1, keepdim=True, unbiased=False) + 1e-5)
        return torch.ops.aten.native_layer_norm_backward(dy, x, [x.shape[-1]], mean, rstd, w, None, [True, True, False])

    dy, x = _t(2048, 1024, dtype=torch.bfloat16), _t(2048, 1024, dtype=torch.bfloat16, seed=1)
    w = _t(1024, dtype=torch.bfloat16, seed=2)
    torch._dynamo.reset()
    with torch.no_grad():
        got, codes = run_and_get_code(torch.compile(ln_bwd, dynamic=False), dy, x, w)
        ref = ln_bwd(dy, x, w)
    modes = re.findall(r"meta=\{'mode': '(\w+)'", codes[0])
    assert sorted(modes) == ["col", "row"], modes
    assert "mi::gather" not in codes[0]
    torch.testing.assert_close(got[0], ref[0], rtol=2e-2, atol=2e-2)
    # 2048 bf16-rounded products per column: compare the sums relative to their spread
    torch.testing.assert_close(got[1].float(), ref[1].float(), rtol=2e-2, atol=2e-2 * float(ref[1].float().abs().max()))


def _masked_logits(rows, cols, dtype=torch.float32, seed=0):
    """Scores with -inf holes, one row of nothing but -inf and one NaN: what attention masks and
    padded batches feed a softmax."""
    x = _t(rows, cols, dtype=dtype, seed=seed)
    hole = _t(rows, cols, seed=seed + 1) > 1.0
    x = x.masked_fill(hole, float("-inf"))
    x[1, :] = float("-inf")
    x[2, 5] = float("nan")
    x[3, : cols // 2] = float("-inf")
    return x


SOFTMAX_CASES = {
    # rows too long for registers: maximum and sum in one sweep, the row kept in LDS for the output
    "softmax_long_rows_bf16": (lambda x: torch.softmax(x.float(), -1).to(x.dtype), lambda: (_t(96, 50304, dtype=torch.bfloat16),)),
    "softmax_long_rows_f32": (lambda x: torch.softmax(x, -1), lambda: (_t(64, 32768),)),
    "log_softmax_long_rows": (lambda x: torch.log_softmax(x, -1), lambda: (_t(33, 40000),)),
    "logsumexp_long_rows": (lambda x: torch.logsumexp(x, -1), lambda: (_t(128, 50304),)),
    "softmax_long_rows_holes": (lambda x: torch.softmax(x, -1), lambda: (_masked_logits(16, 20000),)),
    # rows in registers
    "softmax_short_rows_holes": (lambda x: torch.softmax(x, -1), lambda: (_masked_logits(64, 1000),)),
    "softmax_tiny_rows": (lambda x: torch.softmax(x, -1), lambda: (_t(4096, 8),)),
    # the reduced axis strided
    "softmax_dim0": (lambda x: torch.softmax(x, 0), lambda: (_t(2048, 1000),)),
    "softmax_dim0_holes": (lambda x: torch.softmax(x, 0), lambda: (_masked_logits(300, 256).t().contiguous().t(),)),
    "logsumexp_dim0": (lambda x: torch.logsumexp(x, 0), lambda: (_t(65536, 128),)),
    "softmax_middle_axis": (lambda x: torch.softmax(x, 1), lambda: (_t(8, 700, 64),)),
    "cross_entropy_rows": (lambda x, t: F.cross_entropy(x.float(), t), lambda: (_t(512, 50304, dtype=torch.bfloat16), torch.randint(0, 50304, (512,), device=DEV))),
}


@pytest.mark.parametrize("name", sorted(SOFTMAX_CASES))
def test_softmax_family(name):
    """Softmax-shaped graphs reach the generator as one reduction with two results, maximum and
    sum of exponentials (torch/_inductor/lowering.py prepare_softmax_online); the kernels must
    agree with eager to fp32 rounding, -inf holes, all--inf rows (NaN, as eager) and NaN included."""
    announce(f"compile softmax family: {name}")
    fn, make = SOFTMAX_CASES[name]
    args = make()
    torch._dynamo.reset()
    with torch.no_grad():
        got = torch.compile(fn, dynamic=False)(*args)
        ref = fn(*args)
    assert got.shape == ref.shape and got.dtype == ref.dtype
    tol = dict(rtol=2e-2, atol=2e-2) if ref.dtype == torch.bfloat16 else dict(rtol=2e-5, atol=1e-6)
    torch.testing.assert_close(got, ref, equal_nan=True, **tol)


def test_long_softmax_is_one_sweep_plus_lds():
    announce("compile long softmax, code shape")
    import re

    from torch._inductor.utils import run_and_get_code

    x = _t(64, 50304, dtype=torch.bfloat16)
    torch._dynamo.reset()
    with torch.no_grad():
        _, codes = run_and_get_code(torch.compile(lambda x: torch.softmax(x.float(), -1).to(x.dtype), dynamic=False), x)
    code = codes[0]
    assert "mi::softmax_step" in code and "lds_row0" in code, "expected one statistics sweep and an LDS copy of the row"
    assert len(re.findall(r"in_ptr0 \+", code.split("group_merge")[0])) <= 2  # main rounds + the partial round


def _ints(*shape, lo=-(1 << 40), hi=1 << 40, dtype=torch.int64, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return torch.randint(lo, hi, shape, generator=g, dtype=torch.int64).to(dtype).to(DEV)


INTEGER_REDUCTIONS = {
    # values far beyond 2^24: a float accumulator anywhere on the way would show
    "rows_sum_max_min": (lambda a: (a.sum(-1), a.amax(-1), a.amin(-1)), lambda: (_ints(512, 300),)),
    "rows_long": (lambda a: (a.sum(-1), a.amax(-1)), lambda: (_ints(8, 100000),)),
    "columns_split": (lambda a: (a.sum(0), a.amin(0)), lambda: (_ints(70000, 64),)),
    "columns_short": (lambda a: (a.sum(0), a.amax(0)), lambda: (_ints(40, 1000),)),
    "middle_axis_int32": (lambda a: (a.amax(1), a.sum(1)), lambda: (_ints(16, 5000, 8, lo=-(1 << 30), hi=1 << 30, dtype=torch.int32),)),
    "everything": (lambda a: (a.sum(), a.amax(), a.amin()), lambda: (_ints(1000, 1000),)),
    "product_small": (lambda a: a.prod(-1), lambda: (_ints(64, 20, lo=-3, hi=4),)),
    "uint8_int16": (lambda a, b: (a.sum(-1), a.amax(0), b.sum(0), b.amin(-1)),
                    lambda: (_ints(300, 77, lo=0, hi=256, dtype=torch.uint8), _ints(300, 77, lo=-30000, hi=30000, dtype=torch.int16))),
    "count_of_a_mask": (lambda a: ((a > 0).sum(), (a > 0.5).sum(-1), (a < 0).sum(0)), lambda: (_t(777, 333),)),
    "fused_after_arithmetic": (lambda a: ((a * 3 + 7) // 2).sum(-1) - a.amax(-1), lambda: (_ints(128, 4096, lo=-(1 << 20), hi=1 << 20),)),
}


@pytest.mark.parametrize("name", sorted(INTEGER_REDUCTIONS))
def test_integer_reductions_are_exact(name):
    """Sums, products and extrema of integer tensors: 64-bit exact in every code shape (rows in
    registers, looped rows, split and single-sweep columns, the middle axis)."""
    announce(f"compile integer reductions: {name}")
    from torch._inductor.utils import run_and_get_code

    fn, make = INTEGER_REDUCTIONS[name]
    args = make()
    torch._dynamo.reset()
    got, codes = run_and_get_code(torch.compile(fn, dynamic=False), *args)
    ref = fn(*args)
    got = got if isinstance(got, (tuple, list)) else (got,)
    ref = ref if isinstance(ref, (tuple, list)) else (ref,)
    assert "mi::RedInt" in codes[0], "expected generated integer reductions"
    for g, r in zip(got, ref):
        assert g.shape == r.shape and g.dtype == r.dtype, (g.shape, r.shape, g.dtype, r.dtype)
        assert torch.equal(g, r)


FLOAT64_CASES = {
    "elementwise": (lambda a: torch.exp(a) / (1 + a * a) + torch.tanh(a) + torch.erf(a) + torch.sqrt(a.abs())
                    + torch.log1p(a.abs()) + a.pow(3) + torch.sigmoid(a) * torch.sin(a) + torch.atan2(a, a + 2),
                    lambda: (_t(300, 1000, dtype=torch.float64),)),
    "rounding_beyond_2_24": (lambda a: torch.floor(a * 1e9) + torch.round(a * 3e8) + torch.trunc(a * 7e10), lambda: (_t(64, 512, dtype=torch.float64),)),
    "row_and_column_sums": (lambda a: (a.sum(-1), a.sum(0), a.mean(), a.amax(-1), a.amin(0)), lambda: (_t(300, 1000, dtype=torch.float64),)),
    "long_rows_and_split_columns": (lambda a: (a.sum(-1), a.sum(0)), lambda: (_t(16, 70000, dtype=torch.float64),)),
    "mixed_with_fp32": (lambda a, b: (a * b.double() + 1e-9).sum(-1) / b.double().abs().sum(-1), lambda: (_t(128, 2048, dtype=torch.float64), _t(128, 2048, seed=1))),
}


@pytest.mark.parametrize("name", sorted(FLOAT64_CASES))
def test_float64_is_computed_in_float64(name):
    """fp64 tensors keep fp64 arithmetic through generated kernels: elementwise functions and
    sums / extrema agree with eager to 1e-12, far inside what an fp32 detour would give."""
    announce(f"compile float64: {name}")
    fn, make = FLOAT64_CASES[name]
    args = make()
    torch._dynamo.reset()
    got = torch.compile(fn, dynamic=False)(*args)
    ref = fn(*args)
    got = got if isinstance(got, (tuple, list)) else (got,)
    ref = ref if isinstance(ref, (tuple, list)) else (ref,)
    for g, r in zip(got, ref):
        assert g.dtype == torch.float64 and g.shape == r.shape
        torch.testing.assert_close(g, r, rtol=1e-12, atol=1e-12 * max(1.0, float(r.abs().max())))
