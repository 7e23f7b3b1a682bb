"""Lowering-table patches: which ATen ops reach the HIP code generator, which go
to eager kernels, and the numerics of sum / mean / var.

Counterpart of the reference's lowering module (reference
inductor_x/lowering.py).  What is carried over:
  - make_reduction (:16-45): the Reduction node is tagged with the kept and
    reduced axes and always realized;
  - a list of ops known to generate (GENERATE_LIST, :89-144) and eager
    fallbacks for ops the generator cannot express (:186-198, :327-339);
  - sum accumulates in fp32 (:204-215); mean of a 16-bit tensor is computed in
    fp32 and cast back (:217-233).
What differs, on purpose:
  - the reference sends every op outside its whitelist to eager; here only ops
    whose lowering needs something the HIP generator does not have (scans,
    sorts, atomics, device-side random numbers) are sent there, so sigmoid, pow,
    indexing and embedding - which the reference leaves unfused - stay fused;
  - var / var_mean keep Inductor's single-pass Welford form: it computes the same
    two-pass definition (:270-293) to fp32 accuracy while reading the input once;
  - sum of a 16-bit tensor is rounded back to that type at the end, which keeps
    the output type PyTorch promises; config.sum_returns_fp32 switches to the
    reference's behaviour (the fp32 sum itself is the result);
  - every patch only acts on GPU tensors; CPU compilation in the same process
    keeps Inductor's own lowerings.
"""
from __future__ import annotations

import functools
import logging

import sympy

import torch
import torch._ops
from torch._inductor import config as inductor_config, ir, lowering
from torch._inductor.ir import Reduction
from torch._inductor.lowering import (
    _make_reduction_inner,
    _validate_reduction_axis,
    fallback_handler,
    lowerings,
    to_dtype,
)
from torch._inductor.utils import sympy_product
from torch._inductor.virtualized import V
from torch._prims_common import is_boolean_dtype, is_integer_dtype

from . import config as backend_config

log = logging.getLogger(__name__)
aten = torch.ops.aten
prims = torch.ops.prims

GPU_DEVICE_TYPE = "cuda"


def _is_gpu(x) -> bool:
    try:
        dev = x.get_device()
    except Exception:
        return False
    return dev is not None and getattr(dev, "type", None) == GPU_DEVICE_TYPE


def _any_gpu(args, kwargs) -> bool:
    for a in list(args) + list(kwargs.values()):
        if isinstance(a, (list, tuple)):
            if any(_is_gpu(b) for b in a if hasattr(b, "get_device")):
                return True
        elif hasattr(a, "get_device") and _is_gpu(a):
            return True
    return False


def make_reduction(reduction_type: str, override_return_dtype=None):
    """Reduction lowering that records which axes are kept and which are reduced
    on the IR node and realizes it (reference inductor_x/lowering.py:16-45).  The
    code generator classifies kernels by strides, so the tags are informative."""

    def inner(x, axis=None, keepdims=False, *, dtype=None):
        kwargs = _make_reduction_inner(
            x, axis=axis, keepdims=keepdims, dtype=dtype, override_return_dtype=override_return_dtype
        )
        result = Reduction.create(reduction_type=reduction_type, input_node=x, **kwargs)
        data = getattr(getattr(result, "data", None), "data", None)
        if isinstance(data, Reduction):
            if _is_gpu(x):
                reduced = set(_validate_reduction_axis(x, axis))
                ndim = len(x.get_size())
                # IR nodes are frozen dataclasses: annotate past the freeze
                object.__setattr__(data, "kept_idx", [i for i in range(ndim) if i not in reduced])
                object.__setattr__(data, "reduced_idx", [i for i in range(ndim) if i in reduced])
            result.realize()  # as Inductor's own make_reduction does, for every device
        return result

    return inner


def _init_set(input_list, output_set) -> None:
    for fn in input_list:
        output_set.add(fn)
        if isinstance(fn, torch._ops.OpOverloadPacket):
            for overload in fn.overloads():
                output_set.add(getattr(fn, overload))


# Ops the HIP generator is exercised on (pointwise chains, reductions, views,
# indexing).  Informative: ops outside it still lower through Inductor unless
# they are in FALLBACK_OPS.
GENERATE_LIST = [
    aten.mul, aten.add, aten.sub, aten.div, aten.exp, aten.maximum, aten.minimum, aten.sum, aten.mean,
    aten.var, aten.var_mean, aten.select, aten.unsqueeze, aten.repeat, aten.clone, aten.reshape, aten.where,
    aten.lt, aten.gt, aten.le, aten.ge, aten.eq, aten.ne, aten.ceil, aten.floor, aten.rsqrt, aten.sqrt,
    aten.abs, aten.log, aten.bitwise_xor, aten.amax, aten.amin, prims.convert_element_type, aten.min, aten.max,
    aten.erf, aten.argmax, aten.argmin, aten.clamp_min, aten.clamp_max, aten.clamp, aten.slice, aten.neg,
    aten.cat, aten.arange, aten.expand, aten.scalar_tensor, aten.permute, aten.relu, aten.sigmoid, aten.tanh,
    aten.pow, aten.index, aten.embedding, aten.select_scatter, aten.slice_scatter, prims.broadcast_in_dim,
    prims.maximum,
]

# The members of GENERATE_LIST that lower to a reduction (the rest is pointwise arithmetic, views and indexing).
REDUCING_OPS = [aten.sum, aten.mean, aten.var, aten.var_mean, aten.amax, aten.amin, aten.min, aten.max, aten.argmax,
                aten.argmin]

# Ops whose Inductor lowering needs scans, sorts or device-side random numbers: on GPU tensors
# they run as eager kernels.  Scatters and index_put are generated (plain or atomic stores
# through an indirect index); Inductor itself sends the reducing scatters it cannot express
# (amax / amin / prod, 64-bit and boolean accumulation) to eager.
FALLBACK_OPS = [
    aten.cumsum, aten.cumprod, aten.cummax, aten.cummin, aten.logcumsumexp,
    aten.sort, aten.topk,
    aten.bucketize, aten.searchsorted,
]

FALLBACK_LIST: list = []
# Ops sent to eager kernels after the code generator refused a fused node that came from them
# (filled at compile time by add_runtime_fallback; process-wide, so later graphs skip the retry).
RUNTIME_FALLBACKS: list = []  # ops sent to eager kernels after a refused fused node (process-wide)
_RUNTIME_FALLBACK_ORIGINALS: dict = {}
_registered = False


def _device_aware(op, original, replacement):
    """Use `replacement` when any tensor argument lives on the GPU."""

    @functools.wraps(original)
    def wrapper(*args, **kwargs):
        if _any_gpu(args, kwargs):
            return replacement(*args, **kwargs)
        return original(*args, **kwargs)

    wrapper._inductor_x_amd = True
    return wrapper


def add_runtime_fallback(op) -> bool:
    """Send `op` (an OpOverload with a lowering) to its eager kernel for GPU tensors from now on.
    Returns True when the lowering table changed.  Counterpart of the reference dropping a
    configuration that fails to compile and going on with what is left
    (reference inductor_x/npu_triton_heuristics.py:87-106,194-198): here the unit that is
    dropped is the op's generated lowering, and what is left is its library kernel."""
    if not isinstance(op, torch._ops.OpOverload) or op not in lowerings or op in RUNTIME_FALLBACKS:
        return False
    original = lowerings[op]
    try:
        handler = fallback_handler(op, add_to_fallback_set=False)
    except Exception as e:
        log.debug("no eager fallback for %s: %s", op, e)
        return False
    lowerings[op] = _device_aware(op, original, handler)
    RUNTIME_FALLBACKS.append(op)
    _RUNTIME_FALLBACK_ORIGINALS[op] = original
    return True


def clear_runtime_fallbacks() -> list:
    """Give every op in RUNTIME_FALLBACKS its generated lowering back; returns the ops restored.
    The lowering tables are per process, so a fallback registered while one graph compiled also
    applies to every graph compiled later; a caller that wants the generated lowering tried again
    (after a fix, or for an unrelated model) calls this between compiles."""
    restored = list(RUNTIME_FALLBACKS)
    for op in restored:
        lowerings[op] = _RUNTIME_FALLBACK_ORIGINALS.pop(op)
    RUNTIME_FALLBACKS.clear()
    return restored


def _register_inductor_fallbacks() -> None:
    """Install the patches (idempotent).  Same role and call position as the
    reference's _register_npu_inductor_fallbacks
    (reference inductor_x/lowering.py:173-339, called from
    reference inductor_x/__init__.py:57)."""
    global _registered
    if _registered:
        return
    _registered = True

    # random numbers: generated inside the fused kernels, or ATen's generators as separate kernels
    inductor_config.fallback_random = not backend_config.generate_random

    fb_set: set = set()
    _init_set(FALLBACK_OPS, fb_set)
    for op in list(fb_set):
        if isinstance(op, torch._ops.OpOverload) and op in lowerings:
            original = lowerings[op]
            if getattr(original, "_inductor_x_amd", False):
                continue
            try:
                handler = fallback_handler(op, add_to_fallback_set=False)
            except Exception as e:  # an op Inductor cannot wrap: leave it alone
                log.debug("no eager fallback for %s: %s", op, e)
                continue
            lowerings[op] = _device_aware(op, original, handler)
            FALLBACK_LIST.append(op)

    # ---- numerics of sum / mean on the GPU path
    tagged_sum = make_reduction("sum")

    def sum_gpu(x, axis=None, keepdims=False, *, dtype=None):
        in_dtype = x.get_dtype()
        if (is_integer_dtype(in_dtype) or is_boolean_dtype(in_dtype)) and dtype is None:
            # integer and boolean sums accumulate in int64, as Inductor's own lowering has them
            return make_reduction("sum", override_return_dtype=torch.int64)(x, axis, keepdims, dtype=torch.int64)
        out_dtype = dtype or in_dtype
        if in_dtype in (torch.float16, torch.bfloat16):
            x = to_dtype(x, torch.float32)
        result = tagged_sum(x, axis, keepdims, dtype=torch.float32 if out_dtype != torch.float64 else None)
        if (backend_config.sum_returns_fp32 and dtype is None and in_dtype in (torch.float16, torch.bfloat16)
                and getattr(V.graph, "is_inference", False)):
            return result  # the reference's result type: the fp32 sum, not rounded back
        return to_dtype(result, out_dtype)

    def mean_gpu(x, axis=None, keepdim=False, *, dtype=None):
        if dtype is not None:
            x = to_dtype(x, dtype)
        size = x.get_size()
        axis = _validate_reduction_axis(x, axis)
        out_dtype = x.get_dtype()
        if out_dtype in (torch.float16, torch.bfloat16):
            x = to_dtype(x, torch.float32)
        total = sum_gpu(x, axis, keepdim)
        denom = sympy_product(size[i] for i in axis)
        denom = ir.IndexingConstant(index=denom, dtype=x.get_dtype(), device=x.get_device())
        denom = ir.ExpandView.create(denom, list(total.get_size()))
        return to_dtype(lowering.div(total, denom), out_dtype)

    for op, repl in ((aten.sum, sum_gpu), (prims.sum, sum_gpu), (aten.mean, mean_gpu)):
        for overload in op.overloads():
            fn = getattr(op, overload)
            if fn in lowerings and not getattr(lowerings[fn], "_inductor_x_amd", False):
                lowerings[fn] = _device_aware(fn, lowerings[fn], repl)


# name used by the reference
_register_npu_inductor_fallbacks = _register_inductor_fallbacks
