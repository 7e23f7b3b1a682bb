"""Seeded random graphs through torch.compile against eager: permuted and sliced views, broadcasts
and reductions over random axes of random (often awkward) shapes.  The generator decides per access
between vector, tile, scalar and gather forms from index arithmetic alone; this sweeps that logic
over many more index shapes than the hand-picked tests do.  Copies must be bit-exact."""
import itertools
import random

import pytest
import torch

from tests.helpers import announce

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SIZES = (1, 2, 3, 5, 8, 16, 24, 33, 64, 72, 128, 200)


@pytest.fixture(scope="module", autouse=True)
def backend():
    import inductor_x_amd  # noqa: F401  registration side effects

    return inductor_x_amd


def _compile_and_compare(fn, args, exact):
    torch._dynamo.reset()
    got = torch.compile(fn, dynamic=False)(*args)
    ref = fn(*args)
    got = got if isinstance(got, (tuple, list)) else (got,)
    ref = ref if isinstance(ref, (tuple, list)) else (ref,)
    for g, r in zip(got, ref):
        assert g.shape == r.shape and g.dtype == r.dtype
        if exact or not r.dtype.is_floating_point:
            assert torch.equal(g, r)
        elif r.dtype == torch.float32:
            # sums over tens of thousands of elements: the bar is relative to the largest entry
            scale = max(r.abs().max().item(), 1.0) if r.numel() else 1.0
            torch.testing.assert_close(g, r, rtol=1e-4, atol=2e-5 * scale)
        else:
            torch.testing.assert_close(g.float(), r.float(), rtol=2e-2, atol=2e-2)


def _random_case(rng: random.Random):
    nd = rng.choice((2, 3, 3, 4))
    shape = tuple(rng.choice(SIZES) for _ in range(nd))
    while 1 in shape and rng.random() < 0.7:
        shape = tuple(rng.choice(SIZES) for _ in range(nd))
    dtype = rng.choice((torch.float32, torch.float32, torch.bfloat16))
    kind = rng.choice(("permute", "permute_add", "slice", "broadcast", "reduce", "reduce_epilogue"))
    perm = list(range(nd))
    rng.shuffle(perm)
    dims = sorted(rng.sample(range(nd), rng.randint(1, max(1, nd - 1))))
    starts = [rng.randint(0, max(0, s // 3)) for s in shape]
    steps = [rng.choice((1, 1, 2)) for _ in shape]
    keep = rng.randrange(nd)
    return shape, dtype, kind, tuple(perm), tuple(dims), tuple(starts), tuple(steps), keep


@pytest.mark.parametrize("seed", range(96))
def test_random_graph(seed):
    rng = random.Random(1000 + seed)
    shape, dtype, kind, perm, dims, starts, steps, keep = _random_case(rng)
    announce(f"random graph seed={seed} {kind} shape={shape} {dtype} perm={perm} dims={dims}")
    torch.manual_seed(seed)
    x = torch.randn(*shape, device=DEV).to(dtype)
    if kind == "permute":
        _compile_and_compare(lambda t: t.permute(*perm).contiguous(), (x,), exact=True)
    elif kind == "permute_add":
        y = torch.randn(*[shape[p] for p in perm], device=DEV).to(dtype)
        _compile_and_compare(lambda t, y: t.permute(*perm) * 2 + y, (x, y), exact=False)
    elif kind == "slice":
        sl = tuple(slice(a, None, st) for a, st in zip(starts, steps))
        _compile_and_compare(lambda t: (t[sl] + 0, t[sl].transpose(0, -1).contiguous()), (x,), exact=True)
    elif kind == "broadcast":
        bshape = [s if i == keep else 1 for i, s in enumerate(shape)]
        b = torch.randn(*bshape, device=DEV).to(dtype)
        _compile_and_compare(lambda t, b: (t + b, (t * b).permute(*perm).contiguous()), (x, b), exact=False)
    elif kind == "reduce":
        xf = x.float()
        _compile_and_compare(lambda t: (t.sum(dims), t.amax(dims), t.argmax(dims[0])), (xf,), exact=False)
        if xf.numel() // max(1, torch.tensor([shape[d] for d in dims]).prod().item()) > 0:
            _compile_and_compare(lambda t: torch.var_mean(t, dims, correction=0), (xf,), exact=False)
    else:
        xf = x.float()
        _compile_and_compare(lambda t: (t - t.mean(dims, keepdim=True)) * torch.rsqrt(t.var(dims, keepdim=True, correction=0) + 1.0),
                             (xf,), exact=False)
