"""Fused Inductor node -> HIP source for gfx950.

Counterpart of the reference's kernel code generator
(reference inductor_x/codegen/triton.py): where that file prints Triton text
with N-D block indices, this one prints C++ against the hand-written template
library in csrc/mi/codegen.h.  Four code shapes exist:

  pointwise  (reference family F1/F2, triton.py:693-815)    one 16-byte vector per thread; VEC x VEC
                                                            register tiles for transposed operands
  row        (F3/F4/F6, triton.py:1103-1262)                TPR threads per row, DPP + LDS combine
  column     (F5 + the outer-reduce hint, triton.py:1003-1031,
              split_tiling.py:159-165)                      two-pass workgroup partials, or one sweep
                                                            finishing in place when no split is needed
  colloop    (the same strides, short reduced axis or
              values reused after the reduction)            one kernel, lanes along the kept axis, row
                                                            lanes loop over the reduced axis per phase

The shape is chosen from the strides of the accesses (which axis is the
contiguous one), not from tags put on the IR node.

Values are either thread-uniform scalars or mi::V<T, VEC> register vectors
along the contiguous axis.  The generator tracks which is which only where it
must (to choose between a vector load, a scalar load and a gather); the C++
overloads do the rest.
"""
from __future__ import annotations

import dataclasses
import itertools
import math
import os
import re
from typing import Any, Optional, Sequence, Union

import sympy

import torch
from torch._inductor import config as inductor_config, ir
from torch._inductor.codegen.common import (
    CSEVariable,
    DeferredLine,
    IndentedBuffer,
    OpOverrides,
    SizeArg,
    TensorArg,
    WorkspaceArg,
)
from torch._inductor.codegen.simd import (
    DisableReduction,
    EnableReduction,
    IterationRangesEntry,
    SIMDKernel,
)
from torch._inductor.ops_handler import StoreMode
from torch._inductor.utils import sympy_subs
from torch._inductor.virtualized import V
from torch.utils._ordered_set import OrderedSet
from torch._inductor.codegen.triton_utils import should_unwrap_unspec_arg
from torch.utils._sympy.functions import FloorDiv, Identity, ModularIndexing
from torch.utils._sympy.symbol import SymT, symbol_is_type
from torch.utils._sympy.printers import ExprPrinter
from torch.utils._sympy.value_ranges import ValueRanges

from .. import config as backend_config
from ..hip_heuristics import col_fold_all_planes

DTYPE_TO_HIP = {
    torch.float32: "float",
    torch.float64: "double",
    torch.float16: "mi::f16_t",
    torch.bfloat16: "mi::bf16_t",
    torch.int8: "signed char",
    torch.uint8: "unsigned char",
    torch.int16: "short",
    torch.int32: "int",
    torch.int64: "mi::i64",
    torch.bool: "bool",
}

# struct codes for the launcher's argument packing
DTYPE_TO_STRUCT = {torch.int32: "i", torch.int64: "q", torch.float32: "f", torch.float64: "d"}


class VecConstraintError(Exception):
    """The chosen vector width does not fit an index that showed up late."""


class UnsupportedHipCodegen(NotImplementedError):
    pass


def dtype_nbytes(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


# ---------------------------------------------------------------------------
# index expression printer
# ---------------------------------------------------------------------------
class HipExprPrinter(ExprPrinter):
    """sympy index expression -> C++.  Indices are non-negative, so floor
    division and modular indexing are the plain C operators; the same text
    works for scalars and for mi::V<int, N> lane vectors."""

    def _print_FloorDiv(self, expr: sympy.Expr) -> str:
        x, div = expr.args
        return f"(({self.doprint(x)}) / ({self.doprint(div)}))"

    def _print_ModularIndexing(self, expr: sympy.Expr) -> str:
        x, div, mod = expr.args
        xs = self.doprint(x)
        if div != 1:
            xs = f"(({xs}) / ({self.doprint(div)}))"
        return f"(({xs}) % ({self.doprint(mod)}))"

    def _print_Min(self, expr: sympy.Expr) -> str:
        args = [self.doprint(a) for a in expr.args]
        out = args[0]
        for a in args[1:]:
            out = f"mi::minimum({out}, {a})"
        return out

    def _print_Max(self, expr: sympy.Expr) -> str:
        args = [self.doprint(a) for a in expr.args]
        out = args[0]
        for a in args[1:]:
            out = f"mi::maximum({out}, {a})"
        return out

    def _print_Abs(self, expr: sympy.Expr) -> str:
        return f"mi::abs({self.doprint(expr.args[0])})"

    def _print_Where(self, expr: sympy.Expr) -> str:
        c, p, q = (self.doprint(a) for a in expr.args)
        return f"mi::where({c}, {p}, {q})"

    def _print_ToFloat(self, expr: sympy.Expr) -> str:
        return f"mi::cast<float>({self.doprint(expr.args[0])})"

    def _print_Float(self, expr: sympy.Expr) -> str:
        return f"{float(expr)!r}f"

    def _print_PowByNatural(self, expr: sympy.Expr) -> str:
        x, y = expr.args
        if isinstance(y, sympy.Integer) and 0 <= int(y) <= 8:
            xs = self.doprint(x)
            return "(" + " * ".join([f"({xs})"] * int(y)) + ")" if int(y) else "1"
        return f"mi::pow({self.doprint(x)}, {self.doprint(y)})"

    def _print_IntTrueDiv(self, expr: sympy.Expr) -> str:
        a, b = expr.args
        return f"mi::truediv({self.doprint(a)}, {self.doprint(b)})"

    def _print_PythonMod(self, expr: sympy.Expr) -> str:
        # the sign of the result follows the divisor (sizes that are only known at run time keep
        # expressions like (x + s - 3) mod s in this form)
        a, b = expr.args
        return f"mi::pymod({self.doprint(a)}, {self.doprint(b)})"

    def _print_FloorToInt(self, expr: sympy.Expr) -> str:
        return f"mi::cast<mi::i64>(mi::floor({self.doprint(expr.args[0])}))"

    _print_floor = _print_FloorToInt

    def _print_CeilToInt(self, expr: sympy.Expr) -> str:
        return f"mi::cast<mi::i64>(mi::ceil({self.doprint(expr.args[0])}))"

    _print_ceiling = _print_CeilToInt

    def _print_RoundToInt(self, expr: sympy.Expr) -> str:
        return f"mi::cast<mi::i64>(mi::round({self.doprint(expr.args[0])}))"

    def _print_TruncToFloat(self, expr: sympy.Expr) -> str:
        return f"mi::trunc({self.doprint(expr.args[0])})"

    def _print_FloatPow(self, expr: sympy.Expr) -> str:
        x, y = expr.args
        return f"mi::pow({self.doprint(x)}, {self.doprint(y)})"

    def _print_Rational(self, expr: sympy.Expr) -> str:
        return f"({float(expr.p)!r} / {float(expr.q)!r})"

    def _print_TruncToInt(self, expr: sympy.Expr) -> str:
        return f"mi::cast<mi::i64>(mi::trunc({self.doprint(expr.args[0])}))"


hexpr = HipExprPrinter().doprint


def _without_identity(expr: sympy.Expr) -> sympy.Expr:
    """Inductor wraps the shifted index of a concatenated or padded operand in Identity so that
    it is printed as written (it may be negative where the guard is false).  For the analysis
    of how the address moves from lane to lane the wrapper is transparent."""
    if isinstance(expr, sympy.Expr) and expr.has(Identity):
        return expr.replace(Identity, lambda a: a)
    return expr


def value_to_hip(val: Union[float, int, bool, str, CSEVariable], dtype: Optional[torch.dtype] = None) -> str:
    if isinstance(val, bool):
        return "true" if val else "false"
    if isinstance(val, float):
        if math.isinf(val):
            return "__builtin_inff()" if val > 0 else "(-__builtin_inff())"
        if val != val:
            return "__builtin_nanf(\"\")"
        if dtype == torch.float64:
            return repr(val)
        return f"{val!r}f"
    if isinstance(val, int):
        if dtype is not None and dtype.is_floating_point:
            return f"{float(val)!r}" + ("" if dtype == torch.float64 else "f")
        if abs(val) > 2**31 - 1:
            return f"{val}LL"
        return str(val)
    return str(val)


# ---------------------------------------------------------------------------
# op overrides
# ---------------------------------------------------------------------------
class HipOverrides(OpOverrides):
    """One C++ expression per Inductor op.  16-bit floats are computed in fp32
    and only rounded at stores (reference inductor_x/codegen/triton.py:1431-1433),
    so to_dtype to a 16-bit float is a cast to float.  maximum / minimum
    propagate NaN as torch does (the reference's helper drops it,
    reference inductor_x/npu_triton_helpers.py:8-18)."""

    @staticmethod
    def _compute_type(dtype: torch.dtype) -> str:
        if dtype in (torch.float16, torch.bfloat16):
            return "float"
        return DTYPE_TO_HIP[dtype]

    @staticmethod
    def to_dtype(x, dtype: torch.dtype, src_dtype: Optional[torch.dtype] = None, use_compute_types: bool = True) -> str:
        if dtype == torch.bool:
            return f"({x} != 0)"
        if not use_compute_types and dtype in (torch.float16, torch.bfloat16):
            # Asked for when eager's intermediate roundings are to be emulated
            # (torch/_inductor/lowering.py: emulate_precision_casts): round to
            # the 16-bit type, then carry the rounded value in fp32 as usual.
            return f"mi::cast<float>(mi::cast<{DTYPE_TO_HIP[dtype]}>({x}))"
        return f"mi::cast<{HipOverrides._compute_type(dtype)}>({x})"

    @staticmethod
    def to_dtype_bitcast(x, dtype: torch.dtype, src_dtype: torch.dtype) -> str:
        if src_dtype in (torch.float16, torch.bfloat16):
            x = f"mi::cast<{DTYPE_TO_HIP[src_dtype]}>({x})"
        out = f"mi::bitcast<{DTYPE_TO_HIP[dtype]}>({x})"
        if dtype in (torch.float16, torch.bfloat16):
            out = f"mi::cast<float>({out})"
        return out

    @staticmethod
    def constant(val, dtype: torch.dtype) -> str:
        text = value_to_hip(val, dtype)
        if dtype in (torch.int64,) and isinstance(val, int) and not isinstance(val, bool):
            return f"static_cast<mi::i64>({text})"
        return text

    @staticmethod
    def index_expr(expr: sympy.Expr, dtype: torch.dtype) -> str:
        kernel: HipKernel = V.kernel
        idx = kernel.prepare_indexing(expr)
        text = kernel.index_to_vec_str(idx) if kernel.index_is_lane_varying(idx) else kernel.index_to_str(idx)
        var = kernel.cse.generate(kernel.compute, f"mi::cast<{HipOverrides._compute_type(dtype)}>({text})", dtype=dtype)
        var.is_vec = kernel.index_is_lane_varying(idx)
        return var

    @staticmethod
    def masked(mask, body, other):
        # Evaluate the body with loads guarded by the mask, then select.
        kernel: HipKernel = V.kernel
        with kernel.mask_loads(mask, other) as new_mask:
            result = body()
        dtype = result.dtype if isinstance(result, CSEVariable) else None
        if dtype is None:
            dtype = torch.float32 if isinstance(other, float) else (torch.bool if isinstance(other, bool) else torch.int64)
        other_s = value_to_hip(other, dtype)
        # The caller reads dtype off the returned value, so it has to be a
        # variable of the kernel, not an expression string.
        var = kernel.cse.generate(kernel.compute, f"mi::where({new_mask}, {result}, {other_s})", dtype=dtype)
        var.is_vec = any(isinstance(v, HipCSEVariable) and v.is_vec for v in (new_mask, result))
        return var

    @staticmethod
    def where(a, b, c) -> str:
        return f"mi::where({a}, {b}, {c})"

    @staticmethod
    def maximum(a, b) -> str:
        return f"mi::maximum({a}, {b})"

    @staticmethod
    def minimum(a, b) -> str:
        return f"mi::minimum({a}, {b})"

    @staticmethod
    def relu(x) -> str:
        return f"mi::relu({x})"

    @staticmethod
    def sigmoid(x) -> str:
        return f"mi::sigmoid({x})"

    @staticmethod
    def logical_and(a, b) -> str:
        return f"mi::logical_and({a}, {b})"

    @staticmethod
    def logical_or(a, b) -> str:
        return f"mi::logical_or({a}, {b})"

    @staticmethod
    def logical_xor(a, b) -> str:
        return f"mi::logical_xor({a}, {b})"

    @staticmethod
    def logical_not(a) -> str:
        return f"mi::logical_not({a})"

    @staticmethod
    def truediv(a, b) -> str:
        return f"mi::truediv({a}, {b})"

    @staticmethod
    def floordiv(a, b) -> str:
        return f"mi::floordiv({a}, {b})"

    @staticmethod
    def truncdiv(a, b) -> str:
        return f"mi::truncdiv({a}, {b})"

    @staticmethod
    def remainder(a, b) -> str:
        if isinstance(a, CSEVariable) and a.dtype is not None and a.dtype.is_floating_point:
            return f"mi::remainder_f({a}, {b})"
        return f"mi::pymod({a}, {b})"

    @staticmethod
    def mod(a, b) -> str:
        if isinstance(a, CSEVariable) and a.dtype is not None and a.dtype.is_floating_point:
            return f"mi::fmod({a}, {b})"
        return f"({a} % {b})"

    @staticmethod
    def fmod(a, b) -> str:
        return f"mi::fmod({a}, {b})"

    @staticmethod
    def pow(a, b) -> str:
        return f"mi::pow({a}, {b})"

    @staticmethod
    def square(x) -> str:
        return f"({x} * {x})"

    @staticmethod
    def neg(x) -> str:
        return f"(-{x})"

    @staticmethod
    def fma(a, b, c) -> str:
        return f"mi::fma({a}, {b}, {c})"

    @staticmethod
    def isnan(x) -> str:
        return f"mi::isnan({x})"

    @staticmethod
    def isinf(x) -> str:
        return f"mi::isinf({x})"

    @staticmethod
    def signbit(x) -> str:
        return f"mi::signbit({x})"

    @staticmethod
    def sign(x) -> str:
        return f"mi::sign({x})"

    @staticmethod
    def copysign(a, b) -> str:
        return f"mi::copysign({a}, {b})"

    @staticmethod
    def atan2(a, b) -> str:
        return f"mi::atan2({a}, {b})"

    @staticmethod
    def reciprocal(x) -> str:
        return f"mi::reciprocal({x})"

    @staticmethod
    def libdevice_exp(x) -> str:
        return f"mi::exp({x})"

    @staticmethod
    def libdevice_sqrt(x) -> str:
        return f"mi::sqrt({x})"

    @staticmethod
    def libdevice_sigmoid(x) -> str:
        return f"mi::sigmoid({x})"

    @staticmethod
    def libdevice_log(x) -> str:
        return f"mi::log({x})"

    @staticmethod
    def libdevice_abs(x) -> str:
        return f"mi::abs({x})"

    @staticmethod
    def identity(x) -> str:
        return f"{x}"

    # -- random numbers (reference inductor_x/npu_fusion_attention_graph.py:150-164 carries dropout in its
    #    training pattern; Inductor lowers rand / randn / randint / dropout to these three ops and a seed
    #    load when config.fallback_random is off) ------------------------------------------------------
    @staticmethod
    def load_seed(name: str, offset):
        kernel: HipKernel = V.kernel
        var = kernel.args.input(name)
        out = kernel.cse.generate(kernel.compute, f"{var}[{offset}]", dtype=torch.int64)
        out.is_vec = False  # one seed per kernel
        return out

    @staticmethod
    def rand(seed, offset) -> str:
        return f"mi::rand({seed}, {offset})"

    @staticmethod
    def randn(seed, offset) -> str:
        return f"mi::randn({seed}, {offset})"

    @staticmethod
    def randint64(seed, offset, low, high) -> str:
        return f"mi::randint64({seed}, {offset}, {low}, {high})"


def _add_unary(name: str) -> None:
    def fn(x) -> str:
        return f"mi::{name}({x})"

    fn.__name__ = name
    setattr(HipOverrides, name, staticmethod(fn))


for _n in (
    "exp", "exp2", "expm1", "log", "log2", "log10", "log1p", "sqrt", "rsqrt", "sin", "cos", "tan", "tanh",
    "sinh", "cosh", "asin", "acos", "atan", "erf", "erfc", "lgamma", "floor", "ceil", "trunc", "round", "abs",
):
    _add_unary(_n)


# ---------------------------------------------------------------------------
# CSE variable with vector-ness
# ---------------------------------------------------------------------------
class HipCSEVariable(CSEVariable):
    def __init__(self, name: str, bounds: ValueRanges[Any], dtype: Optional[torch.dtype] = None, shape=None):
        super().__init__(name, bounds, dtype, shape=shape)
        # True when the value differs between the lanes of the thread's vector
        self.is_vec = False

    def update_on_args(self, name: str, args: Any, kwargs: Any) -> None:
        def any_vec(a) -> bool:
            if isinstance(a, HipCSEVariable):
                return a.is_vec
            if isinstance(a, (list, tuple)):
                return any(any_vec(b) for b in a)
            return False

        if any_vec(args) or any_vec(list(kwargs.values())):
            self.is_vec = True


# C type and struct code of a scalar kernel argument that stands for a 0-d CPU tensor
SCALAR_ARG = {
    torch.float16: ("float", "f"), torch.bfloat16: ("float", "f"), torch.float32: ("float", "f"),
    torch.float64: ("double", "d"), torch.int64: ("mi::i64", "q"), torch.int32: ("int", "i"),
    torch.int16: ("int", "i"), torch.int8: ("int", "i"), torch.uint8: ("int", "i"), torch.bool: ("int", "i"),
}

REDUCTION_KIND = {
    "sum": "mi::RedSum",
    "prod": "mi::RedProd",
    "max": "mi::RedMax",
    "min": "mi::RedMin",
    "any": "mi::RedAny",
    "argmax": "mi::RedArgMax",
    "argmin": "mi::RedArgMin",
    "welford_reduce": "mi::RedWelford",
    "welford_combine": "mi::RedMoments",
    "online_softmax_reduce": "mi::RedOnlineSoftmax",
}
INT_REDUCTION_OP = {"sum": "Sum", "prod": "Prod", "max": "Max", "min": "Min"}
REDUCTION_WORDS = {"sum": 1, "prod": 1, "max": 1, "min": 1, "any": 1, "argmax": 2, "argmin": 2, "welford_reduce": 3,
                   "online_softmax_reduce": 2}


@dataclasses.dataclass
class ColReduction:
    kind: str  # key of REDUCTION_KIND
    acc: str  # accumulator variable in the partial kernel
    result: str  # merged state variable in the final kernel
    value: str
    ws_offset_words: int  # offset in units of nsplit * xnumel floats
    cxx: str = ""  # reduction class of the template library
    words: int = 1  # floats per state


class HipKernel(SIMDKernel):
    overrides = HipOverrides  # type: ignore[assignment]
    suffix = ";"
    newvar_prefix = "auto "
    kexpr = staticmethod(hexpr)
    sexpr = staticmethod(hexpr)
    allow_block_ptr = False

    MAX_ROW_THREADS = 1024

    def __init__(self, tiling: dict[str, sympy.Expr], force_vec: Optional[int] = None, **kwargs: Any) -> None:
        self.force_vec = force_vec
        self.mode = "pointwise"
        self.vec = 1
        self.block = 256
        self.tpr = 256
        self.col_ct = 128
        self.col_rl = 8
        self.vec_tree_prefix = "x"
        self.lane_syms: OrderedSet[sympy.Symbol] = OrderedSet()
        self.x_entries: list[IterationRangesEntry] = []
        # indices of the non-indirect loads that are contiguous along the vector axis (tile planning)
        self._contiguous_load_indices: list[sympy.Expr] = []
        self.r_entries: list[IterationRangesEntry] = []
        self.r_full = False
        self.prologue = IndentedBuffer()
        self.row_loop_accs: list[str] = []
        # looped row kernels: contiguous loads of the reduced axis seen so far, keyed by buffer and
        # index text; one that comes again in a later pass is served from an LDS copy of the row
        self.row_stash: dict[tuple[str, str], dict] = {}
        # bounds-checked indirect index variable -> (its clamped copy, its in-range predicate)
        self._indirect_bounds: dict[str, tuple] = {}
        self.row_pass = 0
        self.col_reductions: list[ColReduction] = []
        self.partial_body = IndentedBuffer()
        self.final_body = IndentedBuffer()
        self.ws_words = 0
        self.phase_bodies_started = False
        self.acc_ids = itertools.count()
        self.red_stores = IndentedBuffer()
        self._result_defs: list[str] = []
        self._result_defs_col: list[str] = []
        self.mode_decided = False
        # register-tile transposition of loads whose contiguous axis is not the vector axis
        self.tplan: Optional[dict] = None
        self.tile_decls: list[str] = []
        super().__init__(tiling, **kwargs)
        self.n_reduction_phases = self._count_reduction_phases()

    # -- framework hooks --------------------------------------------------
    def create_cse_var(self, *args: Any, **kwargs: Any) -> HipCSEVariable:
        return HipCSEVariable(*args, **kwargs)

    def dtype_to_str(self, dtype: torch.dtype) -> str:
        return DTYPE_TO_HIP[dtype]

    def should_use_persistent_reduction(self) -> bool:
        """Rows that fit one register vector per thread of a single workgroup are
        kept in registers (the reference's limit is 1024 elements,
        reference inductor_x/codegen/triton.py:401-424)."""
        if not self.features.is_reduction():
            return False
        rnumel = self.features.reduction_numel
        if not isinstance(rnumel, (int, sympy.Integer)):
            return False
        return int(rnumel) <= self.MAX_ROW_THREADS * 8 and int(rnumel) <= backend_config.persistent_reduction_max

    def _col_split_ok(self) -> bool:
        """The two-kernel column shape needs everything that follows the (single)
        reduction loop to be a function of the kept axis only: the second kernel
        has no loop over the reduced axis."""
        seen_reduction = False
        xnumel = self.numels.get("x")
        for n in self.features.node_schedule:
            if n is EnableReduction or n is DisableReduction:
                continue
            if getattr(n, "is_reduction", lambda: False)():
                seen_reduction = True
                # merging moments of slices (the second stage of a split variance) exists in the
                # row and column-loop shapes only
                data = getattr(getattr(n, "node", None), "data", None)
                if getattr(data, "reduction_type", None) == "welford_combine":
                    return False
                continue
            if seen_reduction:
                try:
                    numel = n.group[1][0]
                except Exception:
                    return False
                if V.graph.sizevars.simplify(numel - xnumel) != 0:
                    return False
        return seen_reduction

    def _count_reduction_phases(self) -> int:
        phases, inside = 0, False
        for n in self.features.node_schedule:
            if n is EnableReduction or n is DisableReduction:
                inside = False
                continue
            is_red = getattr(n, "is_reduction", lambda: False)()
            if is_red and not inside:
                phases += 1
            inside = is_red
        return phases

    # -- mode / vector width ----------------------------------------------
    def pointwise_unroll(self) -> int:
        """Vectors per thread in a pointwise kernel."""
        forced = os.environ.get("INDUCTOR_X_AMD_PW_UNROLL")
        if forced:
            return max(int(forced), 1)
        # measured on MI355X (permute, gather, a*x+b at 128-512 MiB): 1 vector per
        # thread is fastest; 2 is within 1 %, 4 and 8 lose 5-10 %
        return 1

    def pointwise_tile_plan(self) -> Optional[dict]:
        """Two-dimensional workgroup tiles for a pointwise kernel that reads a tensor with
        its two outer axes swapped relative to the output (a permuted copy).

        With the linear order, a workgroup writes one long run and reads 256-byte pieces a
        large stride apart.  When the output index decomposes as x0 + L0*(x1 + L1*(x2 + ...))
        and some load moves faster along x2 than along x1, a workgroup instead takes T1 values
        of x1 times T2 of x2: its reads come in runs of T2 rows and its writes in runs of T1
        rows.  None when the kernel does not have this shape or the sizes do not divide."""
        if self.mode != "pointwise" or self.vec <= 1 or os.environ.get("INDUCTOR_X_AMD_PW_TILE", "1") == "0":
            return None
        if self.tplan:
            return None
        ents = sorted(
            (e for e in self.x_entries if e.root.prefix == self.vec_tree_prefix), key=lambda e: int(e.divisor)
            if isinstance(e.divisor, (int, sympy.Integer)) else -1
        )
        try:
            ents = [e for e in ents if int(e.divisor) >= 1 and int(e.length) >= 1]
        except (TypeError, ValueError):
            return None
        xnumel = self._static_numel(self.vec_tree_prefix)
        if xnumel is None:
            return None
        # the variable that spans the whole range (the linear index itself) is not an axis
        ents = [e for e in ents if not (int(e.divisor) == 1 and int(e.length) == xnumel)]
        chain = []
        want = 1
        for e in ents:
            if int(e.divisor) == want:
                chain.append(e)
                want *= int(e.length)
        if len(chain) < 3 or len(chain) != len(ents):
            return None
        e0, e1, e2 = chain[0], chain[1], chain[2]
        L0, L1, L2 = int(e0.length), int(e1.length), int(e2.length)
        if L0 % self.vec != 0:
            return None
        cpt = L0 // self.vec  # threads per innermost row
        if cpt > self.block or self.block % cpt != 0:
            return None
        s1, s2 = e1.symbol(), e2.symbol()
        swapped = False
        for index in self._contiguous_load_indices:
            idx = sympy.expand(index)
            try:
                c1, c2 = idx.coeff(s1), idx.coeff(s2)
                rest = sympy.expand(idx - c1 * s1 - c2 * s2)
            except Exception:
                return None
            if rest.has(s1) or rest.has(s2) or not (c1.is_Integer and c2.is_Integer):
                return None  # not affine in the two axes
            if 0 < int(c2) < int(c1):
                swapped = True
        if not swapped:
            return None
        rows_per_iter = self.block // cpt
        unroll = int(os.environ.get("INDUCTOR_X_AMD_PW_TILE_UNROLL", "2"))
        t2_cap = int(os.environ.get("INDUCTOR_X_AMD_PW_TILE_T2", "4"))
        t2 = 1
        while t2 * 2 <= min(L2, t2_cap, rows_per_iter) and L2 % (t2 * 2) == 0:
            t2 *= 2
        t1 = rows_per_iter * unroll // t2
        if t2 < 2 or L1 % t1 != 0 or xnumel % (L0 * L1 * L2) != 0:
            return None
        return {"L0": L0, "L1": L1, "L2": L2, "T1": t1, "T2": t2, "unroll": unroll, "cpt": cpt}

    # -- transposed operands ----------------------------------------------------
    _TPLAN_SHAPES = ((16, 16), (8, 32), (32, 8), (4, 64), (64, 4), (8, 16), (16, 8), (8, 8))

    def _affine_parts(self, index: sympy.Expr) -> Optional[dict]:
        """{symbol: integer coefficient} when the index is an integer-affine function of range
        variables (and nothing else that varies), else None."""
        idx = sympy.expand(index)
        coeffs = {}
        rest = idx
        for s in idx.free_symbols:
            if s not in self.range_tree_nodes:
                return None
            c = idx.coeff(s)
            if not c.is_Integer:
                return None
            coeffs[s] = int(c)
            rest = rest - c * s
        rest = sympy.expand(rest)
        if rest.free_symbols or not rest.is_Integer:
            return None
        return coeffs

    def _transposed_axis(self, index: sympy.Expr) -> Optional[IterationRangesEntry]:
        """For an index that strides along the vector axis but is contiguous along another kept
        axis: the entry of that axis.  None for every other kind of index."""
        coeffs = self._affine_parts(index)
        if not coeffs:
            return None
        lane = [s for s in coeffs if self._is_lane_symbol(s)]
        if len(lane) != 1 or coeffs[lane[0]] <= 1 or coeffs[lane[0]] % self.vec:
            return None
        unit = [s for s in coeffs if coeffs[s] == 1 and not self._is_lane_symbol(s)]
        if len(unit) != 1:
            return None
        entry = self.range_tree_nodes[unit[0]]
        lane_entry = self.range_tree_nodes[lane[0]]
        if entry.root.prefix != self.vec_tree_prefix:
            return None
        try:
            dk, lk, l0 = int(entry.divisor), int(entry.length), int(lane_entry.length)
        except (TypeError, ValueError):
            return None
        if lk % self.vec or dk % l0:
            return None
        # stepping along the axis inside one vector must move no other variable of the index
        for s in coeffs:
            if s in (unit[0], lane[0]):
                continue
            e = self.range_tree_nodes[s]
            try:
                d, n = int(e.divisor), int(e.length)
            except (TypeError, ValueError):
                return None
            if not (d >= dk * lk or d * n <= dk):
                return None
        return entry

    def _transpose_plan(self, prepared: Sequence[sympy.Expr]) -> Optional[dict]:
        """Thread tiles for a pointwise kernel that reads an operand transposed (the operand's
        contiguous axis is another kept axis xk, not the vector axis x0).

        A thread then owns VEC x VEC elements: VEC consecutive x0 times VEC consecutive xk.  The
        transposed operand is read with VEC vector loads along xk (one per x0), everything else is
        read and written with VEC vector accesses along x0 (one per xk), and the transposition is
        register renaming in the fully unrolled loop over xk.  A wavefront covers 8 x 8 such
        threads, so every load and store instruction moves runs of 8 x 16 bytes.  None when no
        load has this shape, when two loads disagree on xk, or when the extents do not divide."""
        if self.vec <= 1 or os.environ.get("INDUCTOR_X_AMD_PW_TRANSPOSE", "1") == "0":
            return None
        xnumel = self._static_numel(self.vec_tree_prefix)
        if xnumel is None:
            return None
        axis = None
        for idx in prepared:
            e = self._transposed_axis(idx)
            if e is None:
                continue
            if axis is not None and e.name != axis.name:
                return None
            axis = e
        if axis is None:
            return None
        lane_lengths = []
        for e in self.range_tree_nodes.values():
            if e.root.prefix == self.vec_tree_prefix and e.divisor == 1:
                try:
                    lane_lengths.append(int(e.length))
                except (TypeError, ValueError):
                    return None
        if not lane_lengths:
            return None
        l0 = min(lane_lengths)
        dk, lk = int(axis.divisor), int(axis.length)
        if any(n % l0 for n in lane_lengths) or dk % l0 or xnumel % (dk * lk) or l0 % self.vec:
            return None
        # The output is contiguous over everything below xk (x0 and the axes between), so the
        # tile's first direction walks that whole flat range, not just x0: a short innermost
        # output axis (16 elements) still gets full 128-byte runs on the store side.
        l0 = dk
        n0, nk = l0 // self.vec, lk // self.vec
        # Workgroup shapes in order of preference (square first); tiles may hang over the end of
        # either direction (threads past the end do nothing): take the shape that wastes the fewest
        # threads, and no plan when even that leaves more than half of them idle (the element-wise
        # fallback is four to eight times slower than a full tile, so a half-empty one still wins).
        best = None
        for ti, tj in self._TPLAN_SHAPES:
            wi = min(ti, 8)
            wj = 64 // wi
            if wj > tj:
                wj = tj
                wi = 64 // wj
            if wi > ti or (ti * tj) % 64:
                continue
            tiles_i, tiles_k = -(-n0 // ti), -(-nk // tj)
            waste = (tiles_i * ti * tiles_k * tj) / float(n0 * nk)
            if best is None or waste < best[0] - 1e-9:
                best = (waste, ti, tj, wi, wj, tiles_i, tiles_k)
        if best is None or best[0] > 2.0:
            return None
        _, ti, tj, wi, wj, tiles_i, tiles_k = best
        rest = xnumel // (dk * lk)
        return {"axis": axis.name, "L0": l0, "DK": dk, "LK": lk, "TI": ti, "TJ": tj, "WI": wi, "WJ": wj,
                "tiles_i": tiles_i, "tiles_k": tiles_k, "grid": tiles_i * tiles_k * rest}

    def _tree(self, prefix: str):
        for t in self.range_trees:
            if t.prefix == prefix:
                return t
        return None

    def _static_numel(self, prefix: str) -> Optional[int]:
        t = self._tree(prefix)
        if t is None:
            return None
        n = V.graph.sizevars.simplify(t.numel)
        return int(n) if isinstance(n, (int, sympy.Integer)) else None

    def _unit_stride_symbols(self, index: sympy.Expr) -> list[sympy.Symbol]:
        out = []
        for s in index.free_symbols:
            if s in self.range_tree_nodes:
                try:
                    c = index.coeff(s)
                except Exception:
                    continue
                if c == 1 and s not in (index - s).free_symbols:
                    out.append(s)
        return out

    def finalize_indexing(self, indices: Sequence[sympy.Expr]) -> None:
        """Choose the code shape and the vector width from every index the fused
        node will use (the reference's find_lowest_dimension / select_tiling_axis
        step, reference inductor_x/codegen/split_tiling.py:85-154,188-239)."""
        prepared = []
        for idx in indices:
            try:
                prepared.append(self.prepare_indexing(idx))
            except Exception:
                continue
        is_red = self.features.is_reduction()
        r_tree = self._tree("r0_")
        if not is_red:
            self.mode = "pointwise"
            self.vec_tree_prefix = "x"
        else:
            r_unit = x_unit = 0
            lane = sympy.Symbol("lane_", integer=True, nonnegative=True)

            def innermost_of(prefix):
                def f(s):
                    e = self.range_tree_nodes.get(s)
                    return e is not None and e.root.prefix == prefix and e.divisor == 1
                return f

            # An index that moves along one of the two axes only (a per-row statistic in a sum
            # over rows, a weight vector in a sum over columns) touches a sliver of what the
            # two-axis indices touch: when both kinds occur, the two-axis ones decide.
            def trees_of(idx):
                return {self.range_tree_nodes[s].root.prefix for s in idx.free_symbols if s in self.range_tree_nodes}

            if any(len(trees_of(idx)) > 1 for idx in prepared):
                deciding = [idx for idx in prepared if len(trees_of(idx)) > 1]
            else:
                deciding = list(prepared)
            for idx in deciding:
                found = False
                for s in self._unit_stride_symbols(idx):
                    entry = self.range_tree_nodes[s]
                    if entry.divisor != 1:
                        continue
                    if entry.root.prefix == "r0_":
                        r_unit += 1
                        found = True
                    elif entry.root.prefix == "x":
                        x_unit += 1
                        found = True
                if not found:
                    # the innermost variable may sit inside a division or a remainder
                    # ((r mod 512) + 32768 * (r div 512)): contiguous in pieces all the same
                    if self._lane_delta(idx, lane, innermost_of("r0_"), 2) == lane:
                        r_unit += 1
                    elif self._lane_delta(idx, lane, innermost_of("x"), 2) == lane:
                        x_unit += 1
            if (
                r_unit == 0
                and x_unit > 0
                and self.n_reduction_phases == 1
                and self._col_split_ok()
                and not self.persistent_reduction_blocks_col()
            ):
                self.mode = "col"
                self.vec_tree_prefix = "x"
                # the reduced axis is always walked in a loop here, and what
                # follows the loop goes to the second kernel
                self.persistent_reduction = False
                for t in self.range_trees:
                    if t.is_reduction:
                        t.is_loop = True
            elif r_unit == 0 and x_unit > 0 and os.environ.get("INDUCTOR_X_AMD_COLLOOP", "1") != "0":
                # the reduced axis is strided and the kept axis contiguous, but the column pair does
                # not apply (values are used again after the reduction, or the reduced axis is
                # short): one kernel, lanes along the kept axis, a loop over the reduced axis per phase
                self.mode = "colloop"
                self.vec_tree_prefix = "x"
                self.persistent_reduction = False
                for t in self.range_trees:
                    if t.is_reduction:
                        t.is_loop = True
            else:
                self.mode = "row"
                self.vec_tree_prefix = "r0_"
        self._choose_vec(prepared)
        self._choose_geometry()
        if self.mode == "pointwise":
            self.tplan = self._transpose_plan(prepared)
            if self.tplan:
                self.block = self.tplan["TI"] * self.tplan["TJ"]
        self.mode_decided = True

    def persistent_reduction_blocks_col(self) -> bool:
        """Column shape is for long reduced axes; a short strided reduction is
        cheaper as a (gathering) row kernel with no workspace round trip."""
        rnumel = self._static_numel("r0_")
        return rnumel is not None and rnumel < 64

    def _buffers_min_itemsize(self) -> int:
        size = 4
        for n in self.features.scheduler_nodes():
            for dep in itertools.chain(n.read_writes.reads, n.read_writes.writes):
                try:
                    size = min(size, dtype_nbytes(V.graph.get_dtype(dep.name)))
                except Exception:
                    pass
        return max(size, 1)

    def _choose_vec(self, prepared: Sequence[sympy.Expr]) -> None:
        vec = max(backend_config.vector_bytes // self._buffers_min_itemsize(), 1)
        if self.force_vec is not None:
            vec = self.force_vec
        numel = self._static_numel(self.vec_tree_prefix)
        if numel is None and self.mode != "pointwise":
            vec = 1
        while vec > 1 and not self._vec_ok(vec, numel):
            vec //= 2
        # A row held in registers by more than 512 threads pays for its workgroup barriers (16
        # wavefronts meet twice per reduction): two 16-byte pieces per thread halve the threads.
        if (
            self.mode == "row" and self.persistent_reduction and self.force_vec is None and numel is not None
            and vec * dtype_nbytes(torch.float32) >= backend_config.vector_bytes // 4
            and numel // max(vec, 1) > 512 and self._vec_ok(vec * 2, numel)
            and os.environ.get("INDUCTOR_X_AMD_ROW_WIDE_VEC", "1") != "0"
        ):
            vec *= 2
        self.vec = vec

    def _vec_ok(self, vec: int, numel: Optional[int]) -> bool:
        if numel is None:
            # a size known only at run time (a dynamic batch of fixed-width rows, say) still
            # takes whole vectors when it is provably a multiple of the width
            tree = self._tree(self.vec_tree_prefix)
            if tree is None or not self._multiple_of(tree.numel, vec):
                return False
        elif numel % vec:
            return False
        for entry in self.range_tree_nodes.values():
            if entry.root.prefix != self.vec_tree_prefix:
                continue
            if not self._entry_fits_vec(entry, vec):
                return False
        return True

    @staticmethod
    def _multiple_of(expr: Any, vec: int) -> bool:
        if isinstance(expr, (int, sympy.Integer)):
            return int(expr) % vec == 0
        try:
            return bool(V.graph.sizevars.statically_known_multiple_of(expr, vec))
        except Exception:
            return False

    @classmethod
    def _entry_fits_vec(cls, entry: IterationRangesEntry, vec: int) -> bool:
        if vec == 1:
            return True
        if isinstance(entry.divisor, (int, sympy.Integer)) and int(entry.divisor) == 1:
            return cls._multiple_of(entry.length, vec)
        return cls._multiple_of(entry.divisor, vec)

    def _choose_geometry(self) -> None:
        from ..hip_heuristics import next_power_of_2

        if self.mode == "row":
            rnumel = self._static_numel("r0_")
            vectors = max(-(-rnumel // self.vec), 1) if rnumel is not None else 256
            if self.persistent_reduction:
                self.tpr = min(max(next_power_of_2(vectors), 1), self.MAX_ROW_THREADS)
                self.r_full = rnumel is not None and self.tpr * self.vec == rnumel
                if self.tpr * self.vec < (rnumel or 0):
                    # cannot hold the row in one vector per thread: walk it instead
                    self.persistent_reduction = False
                    for t in self.range_trees:
                        if t.is_reduction:
                            t.is_loop = True
                    self.tpr = 256
            else:
                self.tpr = min(max(next_power_of_2(vectors), 1), 256)
            self.block = max(256, self.tpr)
        elif self.mode == "colloop":
            xnumel = self._static_numel("x")
            rnumel = self._static_numel("r0_")
            groups = max(-(-(xnumel or 512) // self.vec), 1)
            self.col_ct = min(next_power_of_2(groups), 128)
            rl = max(512 // self.col_ct, 1)
            if rnumel is not None:
                # at least eight rows per row lane: a short reduced axis is cheaper walked by fewer
                # lanes (one lane: no LDS round at all) than folded across many
                while rl > 1 and rl * 8 > rnumel:
                    rl //= 2
            self.col_rl = rl
            self.block = max(self.col_ct * self.col_rl, 64)
            self.col_rl = self.block // self.col_ct
        elif self.mode == "col":
            xnumel = self._static_numel("x")
            groups = max(-(-(xnumel or 512) // self.vec), 1)
            # Narrow column tiles (32 threads x one vector: runs of 512 bytes per row): the kept axis
            # is cut into many tiles and the reduced axis into few splits, and the partials of a
            # column, which the second pass folds, are as many as its splits.  Four wavefronts per
            # workgroup with two batches of four rows in flight per thread (measured at [65536, 512]
            # fp32 with mean, variance and argmax, both passes: 29.8 us; 128 threads across with
            # 512 per workgroup 30.4 us; batches of eight rows 31.9 us).
            self.col_ct = min(next_power_of_2(groups), int(os.environ.get("INDUCTOR_X_AMD_COL_CT", "32")))
            self.col_rl = max(int(os.environ.get("INDUCTOR_X_AMD_COL_THREADS", "256")) // self.col_ct, 1)
            self.block = self.col_ct * self.col_rl
        else:
            self.block = 256

    # -- lane-varying index handling --------------------------------------
    def _is_lane_symbol(self, s: sympy.Symbol) -> bool:
        entry = self.range_tree_nodes.get(s)
        return (
            entry is not None
            and self.vec > 1
            and entry.root.prefix == self.vec_tree_prefix
            and entry.divisor == 1
        )

    def index_is_lane_varying(self, index: sympy.Expr) -> bool:
        if self.vec == 1:
            return False
        for s in index.free_symbols:
            if self._is_lane_symbol(s):
                return True
            v = self.cse.varname_map.get(str(s)) if hasattr(self.cse, "varname_map") else None
            if isinstance(v, HipCSEVariable) and v.is_vec:
                return True
        return False

    def index_to_vec_str(self, index: sympy.Expr) -> str:
        """Index with every lane-varying range variable replaced by its lane
        vector (x0 -> x0_v = x0 + iota)."""
        repl = {s: sympy.Symbol(f"{s}_v", integer=True) for s in index.free_symbols if self._is_lane_symbol(s)}
        return self.index_to_str(sympy_subs(index, repl))

    def classify_index(self, index: sympy.Expr) -> str:
        """'uniform' (same address for all lanes), 'contiguous' (lane i reads
        base + i) or 'gather'."""
        if self.vec == 1:
            return "uniform"
        index = _without_identity(index)
        lane_syms = [s for s in index.free_symbols if self._is_lane_symbol(s)]
        tmp_vec = False
        for s in index.free_symbols:
            v = self.cse.varname_map.get(str(s))
            if isinstance(v, HipCSEVariable) and v.is_vec:
                tmp_vec = True
        if tmp_vec:
            return "gather"
        if not lane_syms:
            return "uniform"
        lane = sympy.Symbol("lane_", integer=True, nonnegative=True)
        delta = self._lane_delta(index, lane)
        if delta is None:
            shifted = sympy_subs(index, {s: s + lane for s in lane_syms})
            delta = sympy.expand(shifted - index)
        if delta == lane:
            return "contiguous"
        if delta == 0:
            return "uniform"
        return "gather"

    def _lane_delta(self, expr: sympy.Expr, lane: sympy.Symbol, is_lane=None, vec: Optional[int] = None) -> Optional[sympy.Expr]:
        """index(lane i) - index(lane 0) as an expression in `lane`, using what symbolic
        expansion cannot see: a lane-varying range variable is a multiple of the vector
        width at lane 0 and 0 <= lane < width, so floor((v + lane) / d) does not depend on the
        lane when the width divides d, and (v + lane) mod m moves with the lane when it
        divides m.  None when the structure is not recognised.  is_lane / vec replace the
        kernel's own lane symbols and vector width (used before those are chosen)."""
        vec = self.vec if vec is None else vec
        is_lane = is_lane or self._is_lane_symbol
        zero = sympy.Integer(0)
        expr = _without_identity(expr)

        def aligned(e: sympy.Expr) -> bool:
            base = sympy.expand(sympy_subs(e, {s: zero for s in e.free_symbols if is_lane(s)}))
            if base == 0:
                return True
            try:
                return bool(V.graph.sizevars.statically_known_multiple_of(base, vec))
            except Exception:
                return False

        def rec(e: sympy.Expr) -> Optional[sympy.Expr]:
            if e.is_Symbol:
                return lane if is_lane(e) else zero
            if e.is_number:
                return zero
            if isinstance(e, sympy.Add):
                parts = [rec(a) for a in e.args]
                return None if any(p is None for p in parts) else sympy.Add(*parts)
            if isinstance(e, sympy.Mul):
                consts = [a for a in e.args if a.is_number]
                rest = [a for a in e.args if not a.is_number]
                if len(rest) == 1:
                    d = rec(rest[0])
                    return None if d is None else sympy.Mul(*consts) * d
                ds = [rec(a) for a in rest]
                return zero if all(d == 0 for d in ds) else None
            if isinstance(e, FloorDiv):
                a, d = e.args
                da = rec(a)
                if da == 0 and rec(d) == 0:
                    return zero
                if da == lane and d.is_Integer and int(d) % vec == 0 and aligned(a):
                    return zero
                return None
            if isinstance(e, ModularIndexing):
                a, d, m = e.args
                da = rec(a)
                if da == 0 and rec(d) == 0 and rec(m) == 0:
                    return zero
                if da == lane and d.is_Integer and aligned(a):
                    if int(d) % vec == 0:
                        return zero
                    if int(d) == 1 and m.is_Integer and int(m) % vec == 0:
                        return lane
                return None
            return None

        try:
            out = rec(expr)
        except Exception:
            return None
        return None if out is None else sympy.expand(out)

    def index_is_aligned(self, index: sympy.Expr) -> bool:
        """True when the address of lane 0 is provably a multiple of the vector
        width (lane-varying variables are multiples of it by construction)."""
        index = _without_identity(index)
        lane_syms = [s for s in index.free_symbols if self._is_lane_symbol(s)]
        base = sympy.expand(sympy_subs(index, {s: sympy.Integer(0) for s in lane_syms}))
        try:
            return bool(V.graph.sizevars.statically_known_multiple_of(base, self.vec))
        except Exception:
            return False

    def _buffer_aligned(self, name: str) -> bool:
        return name not in V.graph.unaligned_buffers

    def _kernel_read_bytes(self) -> int:
        """Bytes of the distinct buffers this kernel reads from memory (buffers it produces itself
        excluded), by size hints; 0 when they cannot be told."""
        cached = getattr(self, "_read_bytes_cache", None)
        if cached is not None:
            return cached
        total = 0
        try:
            reads, made = {}, set()
            for n in self.features.node_schedule:
                rw = getattr(n, "read_writes", None)
                if rw is None:
                    continue
                made.update(d.name for d in rw.writes)
                for d in rw.reads:
                    touched = getattr(d, "get_numel", None)
                    reads.setdefault(d.name, []).append(touched() if touched else None)
            for name, touched in reads.items():
                if name in made:
                    continue
                numel = int(V.graph.sizevars.size_hint(V.graph.get_buffer(name).get_numel()))
                if all(t is not None for t in touched):
                    # a strided slice or a broadcast operand: what the accesses cover, at most the buffer
                    numel = min(numel, max(int(V.graph.sizevars.size_hint(t)) for t in touched))
                nbytes = numel * dtype_nbytes(V.graph.get_dtype(name))
                if nbytes >= (1 << 20):  # weight vectors and the like live in L2 whatever the hint
                    total += nbytes
        except Exception:
            total = 0
        self._read_bytes_cache = total
        return total

    def _reads_stream(self, tiled: bool = False) -> bool:
        """Whether this kernel's aligned contiguous loads carry the non-temporal hint: it reads each
        element once (linear pointwise shape, or a row held in registers; the two-dimensional tiles of
        permuted copies measured slower with the hint) and its read set, small operands aside, is
        larger than half the memory-side cache, so a later kernel would not find the data there."""
        limit = backend_config.streaming_read_bytes()
        if limit <= 0 or tiled or not (self.mode == "pointwise" or (self.mode == "row" and self.persistent_reduction)):
            return False
        return self._kernel_read_bytes() > limit

    # -- range variables ---------------------------------------------------
    def codegen_iteration_ranges_entry(self, entry: IterationRangesEntry) -> None:
        """Range variables are only recorded here; their text is produced when a
        body is assembled, once the code shape and the vector width are known."""
        if self.mode_decided and entry.root.prefix == self.vec_tree_prefix and not self._entry_fits_vec(entry, self.vec):
            raise VecConstraintError(f"{entry.name}: divisor {entry.divisor}, length {entry.length}, vec {self.vec}")
        (self.r_entries if entry.root.is_reduction else self.x_entries).append(entry)

    def _entry_code(self, entries: Sequence[IterationRangesEntry], lane_vectors: bool = True) -> IndentedBuffer:
        buf = IndentedBuffer()
        for entry in entries:
            expr = self.rename_indexing(entry.expr)
            buf.writeline(f"const {self.index_dtype} {entry.name} = {self.kexpr(expr)};")
            if entry.divisor == 1 and entry.root.prefix == self.vec_tree_prefix:
                rhs = f"{entry.name} + mi::iota<VEC>()" if (lane_vectors and self.vec > 1) else entry.name
                buf.writeline(f"const auto {entry.name}_v = {rhs};")
        return buf

    # -- masks ---------------------------------------------------------------
    def _load_mask_for(self, index: sympy.Expr) -> Optional[str]:
        """Guard for a load: the row shape masks accesses that move along the
        reduced axis (the tail of the last vector round); an enclosing
        ops.masked adds its own condition.  Kept-axis indices are clamped into
        range instead of masked, and the column shape only runs live columns."""
        parts = []
        if self.mode == "row" and self.inside_reduction and not self.r_full and self._index_uses_tree(index, "r0_"):
            parts.append("rmask")
        if self._load_mask:
            parts.append(str(self._load_mask))
        if not parts:
            return None
        return parts[0] if len(parts) == 1 else f"({parts[0]} && {parts[1]})"

    # -- loads / stores ------------------------------------------------------
    def load(self, name: str, index: sympy.Expr) -> CSEVariable:
        var = self.args.input(name)
        index, _ = self._bounded_index(index)
        indirect = self.is_indirect_indexing(index)
        index = self.prepare_indexing(index)
        dtype = V.graph.get_dtype(name)
        if should_unwrap_unspec_arg(name):
            # the value itself is the kernel argument
            if dtype in (torch.float16, torch.bfloat16):
                dtype = torch.float32
            text = f"({var} != 0)" if dtype == torch.bool else str(var)
            return self.cse.generate(self.loads, text, dtype=dtype)
        kind = self.classify_index(index)
        mask = self._load_mask_for(index)
        other = value_to_hip(self._load_other if self._load_mask else 0, dtype if dtype.is_floating_point else None)
        if kind == "contiguous":
            if not indirect:
                self._contiguous_load_indices.append(index)
            aligned = self.index_is_aligned(index) and self._buffer_aligned(name)
            ptr = f"{var} + ({self.index_to_str(index)})"
            if mask is None:
                if aligned:
                    # STREAM_READS is a constant of the kernel, defined where its shape is final
                    hinted = not indirect and (self.mode == "pointwise" or (self.mode == "row" and self.persistent_reduction))
                    line = f"mi::vload_x<VEC, STREAM_READS>({ptr})" if hinted else f"mi::vload<VEC>({ptr})"
                else:
                    line = f"mi::vload_u<VEC>({ptr})"
            else:
                line = f"mi::vload_m<VEC{'' if aligned else ', false'}>({ptr}, {mask}, {other})"
            is_vec = True
            if (
                self.mode == "row" and self.inside_reduction and not self.persistent_reduction
                and not indirect and not self._load_mask and self._index_uses_tree(index, "r0_")
            ):
                key = (name, self.index_to_str(index))
                entry = self.row_stash.get(key)
                if entry is None:
                    entry = {"id": len(self.row_stash), "dtype": dtype, "pass": self.row_pass, "reused": False}
                    self.row_stash[key] = entry
                    raw = self.cse.generate(self.loads, line, dtype=dtype)
                    if isinstance(raw, HipCSEVariable):
                        raw.is_vec = True
                    self.loads.writeline(f"MI_ROW_STASH_{entry['id']}({raw});")
                    entry["raw"] = str(raw)
                    line = str(raw)
                elif entry["pass"] == self.row_pass:
                    # the same load again within the pass: the value already in registers
                    line = entry["raw"]
                elif entry["pass"] < self.row_pass:
                    entry["reused"] = True
                    line = f"MI_ROW_RELOAD_{entry['id']}({line})"
        elif kind == "uniform":
            if mask is None:
                line = f"{var}[{self.index_to_str(index)}]"
            else:
                line = f"mi::gather_m({var}, {self.index_to_str(index)}, {mask}, {other})"
            is_vec = False
        elif (
            self.tplan and not indirect and mask is None and not self._load_mask
            and (axis := self._transposed_axis(index)) is not None and axis.name == self.tplan["axis"]
        ):
            # VEC loads along the operand's own contiguous axis at the first step of the tile,
            # one column of the register tile per step
            coeffs = self._affine_parts(index)
            stride = next(c for s_, c in coeffs.items() if self._is_lane_symbol(s_))
            tname = f"tile{len(self.tile_decls)}"
            self.tile_decls.append(f"mi::Tile<{DTYPE_TO_HIP[dtype]}, VEC> {tname};")
            # at the first step the axis variable is a multiple of the vector width, like the lane variable
            base = sympy_subs(index, {s_: sympy.Integer(0) for s_ in coeffs if self._is_lane_symbol(s_) or s_.name == axis.name})
            try:
                aligned = bool(V.graph.sizevars.statically_known_multiple_of(sympy.expand(base), self.vec))
            except Exception:
                aligned = False
            fill = "tile_fill" if (aligned and self._buffer_aligned(name)) else "tile_fill_u"
            self.loads.writeline(f"if (u == 0) mi::{fill}<VEC>({tname}, {var} + ({self.index_to_str(index)}), {stride});")
            line = f"mi::tile_col<VEC>({tname}, u)"
            is_vec = True
        else:
            idx = self.index_to_vec_str(index)
            line = f"mi::gather({var}, {idx})" if mask is None else f"mi::gather_m({var}, {idx}, {mask}, {other})"
            is_vec = True
        if dtype in (torch.float16, torch.bfloat16):
            line = f"mi::cast<float>({line})"
            dtype = torch.float32
        # under a guard that differs between the thread's elements the result differs too, also
        # when every element reads the same address
        if isinstance(self._load_mask, HipCSEVariable) and self._load_mask.is_vec:
            is_vec = True
        # a load whose address or guard is itself computed must follow that computation
        buf = self.compute if (indirect or self._load_mask) else self.loads
        out = self.cse.generate(buf, line, dtype=dtype)
        if isinstance(out, HipCSEVariable):
            out.is_vec = out.is_vec or is_vec
        return out

    STREAMING_BYTES = 32 << 20

    def _is_streaming_buffer(self, name: str) -> bool:
        """Outputs far larger than L2 are written with the non-temporal hint."""
        try:
            buf = V.graph.get_buffer(name)
            numel = V.graph.sizevars.size_hint(buf.get_numel())
            return int(numel) * dtype_nbytes(V.graph.get_dtype(name)) >= self.STREAMING_BYTES
        except Exception:
            return False

    def _index_uses_tree(self, index: sympy.Expr, prefix: str) -> bool:
        for s in index.free_symbols:
            e = self.range_tree_nodes.get(s)
            if e is not None and e.root.prefix == prefix:
                return True
        return False

    def store(self, name: str, index: sympy.Expr, value: CSEVariable, mode: StoreMode = None) -> None:
        var = self.args.output(name)
        index, in_range = self._bounded_index(index)
        index = self.prepare_indexing(index)
        if mode not in (None, "atomic_add"):
            raise UnsupportedHipCodegen(f"store mode {mode}")
        kind = self.classify_index(index)
        if in_range is not None and kind == "contiguous":
            kind = "gather"  # per-element guard: the masked element-wise form
        if self.mode == "row":
            if self.inside_reduction:
                mask = "xmask" if self.r_full else "(rmask && xmask)"
            else:
                mask = "(xmask && rlane == 0)"
        elif self.mode == "col":
            # inside the reduction loop only live columns run; afterwards (final
            # kernel) one of the SL lanes of a column stores
            mask = None if (self.inside_reduction and not self.phase_bodies_started) else "(live && sl == 0)"
        elif self.mode == "colloop":
            # inside a loop every row lane owns its rows; outside, one row lane stores per column
            mask = "xmask" if self.inside_reduction else "(xmask && rl == 0)"
        else:
            mask = None
        if in_range is not None:
            mask = in_range if mask is None else f"mi::logical_and({mask}, {in_range})"
        if mode == "atomic_add":
            # accumulating scatter: several elements may land on one address, each adds atomically
            # (every one of the thread's VEC elements contributes, also when they share an address)
            idx = self.index_to_str(index) if kind == "uniform" else self.index_to_vec_str(index)
            line = f"mi::scatter_add_m<VEC>({var}, {idx}, {value}, {mask or 'true'});"
            self.__dict__.setdefault("accumulated_args", set()).add(str(var))
            self.stores.writeline(DeferredLine(name, line))
            return
        if kind == "contiguous":
            aligned = self.index_is_aligned(index) and self._buffer_aligned(name)
            ptr = f"{var} + ({self.index_to_str(index)})"
            stream = ", true" if self._is_streaming_buffer(name) else ""
            if mask is None:
                line = f"mi::vstore<VEC{stream}>({ptr}, {value});" if aligned else f"mi::vstore_u<VEC>({ptr}, {value});"
            elif aligned:
                line = f"mi::vstore_m<VEC{stream}>({ptr}, {value}, {mask});"
            else:
                line = f"mi::scatter_m<VEC>({var}, {self.index_to_vec_str(index)}, {value}, {mask});"
        elif kind == "uniform":
            line = f"mi::vstore<1>({var} + ({self.index_to_str(index)}), {value});"
            if mask is not None:
                line = f"if ({mask}) {{ {line} }}"
        else:
            idx = self.index_to_vec_str(index)
            line = f"mi::scatter_m<VEC>({var}, {idx}, {value}, {mask or 'true'});"
        self.stores.writeline(DeferredLine(name, line))

    def store_reduction(self, name: str, index: sympy.Expr, value: CSEVariable) -> None:
        """The reduced value is uniform for the row (or column); one thread writes it."""
        var = self.args.output(name)
        index = self.prepare_indexing(index)
        if self.mode == "colloop":
            # one value per column: a vector along the kept axis, written by the first row lane
            if self.classify_index(index) == "contiguous":
                line = f"mi::vstore_m<VEC>({var} + ({self.index_to_str(index)}), {value}, (xmask && rl == 0));"
                if not (self.index_is_aligned(index) and self._buffer_aligned(name)):
                    line = f"mi::scatter_m<VEC>({var}, {self.index_to_vec_str(index)}, {value}, (xmask && rl == 0));"
            else:
                line = f"mi::scatter_m<VEC>({var}, {self.index_to_vec_str(index)}, {value}, (xmask && rl == 0));"
            self.red_stores.writeline(DeferredLine(name, line))
            return
        guard = "(live && sl == 0)" if self.mode == "col" else "(xmask && rlane == 0)"
        line = f"if {guard} {{ mi::vstore<1>({var} + ({self.index_to_str(index)}), {value}); }}"
        self.red_stores.writeline(DeferredLine(name, line))

    def check_bounds(self, expr: sympy.Expr, size: sympy.Expr, lower: bool, upper: bool) -> None:
        """Inductor calls this for every indirect index it would assert on (reference
        inductor_x/npu_triton_heuristics.py:131-133 passes the same switch to Triton as `debug`).
        No device-side assert is generated here; instead (config.indirect_bounds == "clamp") a
        clamped copy of the index is computed next to it, loads through the index use the copy, and
        stores / atomics through it are dropped for elements whose index is out of range."""
        if backend_config.indirect_bounds != "clamp" or not isinstance(expr, sympy.Symbol) or not (lower or upper):
            return
        name = str(expr)
        if name in self._indirect_bounds:
            return
        var = self.cse.varname_map.get(name)
        if var is None:
            return
        size_str = self.index_to_str(size)
        clamped = self.cse.generate(self.compute, f"mi::clamp_index({name}, {size_str})", dtype=getattr(var, "dtype", None))
        inside = self.cse.generate(self.compute, f"mi::index_in_range({name}, {size_str})", dtype=torch.bool)
        for v in (clamped, inside):
            if isinstance(v, HipCSEVariable):
                v.is_vec = bool(getattr(var, "is_vec", False))
        self._indirect_bounds[name] = (sympy.Symbol(str(clamped), integer=True), str(inside))

    def _bounded_index(self, index: sympy.Expr) -> tuple:
        """(index with every bounds-checked indirect symbol replaced by its clamped copy, conjunction
        of their in-range predicates or None)."""
        hits = {s: self._indirect_bounds[str(s)] for s in index.free_symbols if str(s) in self._indirect_bounds}
        if not hits:
            return index, None
        preds = [p for _, p in hits.values()]
        guard = preds[0]
        for p in preds[1:]:
            guard = f"mi::logical_and({guard}, {p})"
        return sympy_subs(index, {s: c for s, (c, _) in hits.items()}), guard

    # -- reductions -----------------------------------------------------------
    def reduction(self, dtype, src_dtype, reduction_type, value):
        cache_key = (src_dtype, reduction_type, value)
        if cache_key in self.cse.reduction_cache:
            return self.cse.reduction_cache[cache_key]
        result = self._reduction_nocache(dtype, src_dtype, reduction_type, value)
        self.cse.reduction_cache[cache_key] = result
        return result

    def _r_index_str(self) -> str:
        return "(r0_index + mi::iota<VEC>())" if (self.mode == "row" and self.vec > 1) else "r0_index"

    def _reduction_nocache(self, dtype, src_dtype, reduction_type, value):
        assert self.inside_reduction
        if reduction_type not in REDUCTION_KIND:
            raise UnsupportedHipCodegen(f"reduction {reduction_type}")
        if isinstance(value, tuple) and reduction_type != "welford_combine":
            raise UnsupportedHipCodegen(f"tuple-valued reduction input for {reduction_type}")
        kind = REDUCTION_KIND[reduction_type]
        words = REDUCTION_WORDS.get(reduction_type, 3)
        # sums, products and extrema of integers are exact 64-bit reductions: their states travel
        # through the same merge machinery as two 32-bit words
        integral = (
            reduction_type in INT_REDUCTION_OP and not src_dtype.is_floating_point
            and (src_dtype != torch.bool or reduction_type in ("sum", "prod"))
        )
        if integral:
            kind = f"mi::RedInt<mi::IntOp::{INT_REDUCTION_OP[reduction_type]}>"
            words = 2
        elif reduction_type in INT_REDUCTION_OP and src_dtype == torch.float64:
            # fp64 tensors reduce in fp64 (moments, arg-extrema and softmax statistics of fp64
            # tensors are still computed in fp32)
            kind = f"mi::RedF64<mi::IntOp::{INT_REDUCTION_OP[reduction_type]}>"
            words = 2
            integral = "f64"
        if self._load_mask:
            raise UnsupportedHipCodegen("reduction under a load mask")
        if self.mode == "row" and self.vec > 1:
            # a value that does not vary over the thread's VEC elements (it was computed from
            # indices a whole vector shares) still counts once per element
            def lanes(v):
                return v if (isinstance(v, HipCSEVariable) and v.is_vec) else f"mi::splat<VEC>({v})"

            value = tuple(lanes(v) for v in value) if isinstance(value, tuple) else lanes(value)
        n = next(self.acc_ids)
        if reduction_type == "welford_combine":
            # inputs are (mean, m2, weight) per element: the second stage of a split variance
            mean, m2, weight = value
            if self.mode == "colloop":
                acc = f"acc{n}"
                self.prologue.writeline(f"mi::ColMomentsAcc<VEC> {acc};")
                self.prologue.writeline(f"{acc}.init();")
                self.compute.writeline(f"{acc}.step({mean}, {m2}, {weight});")
                self.colloop_max_words = max(getattr(self, "colloop_max_words", 1), 3)
                self.row_loop_accs.extend([
                    f"mi::Moments {acc}_m[VEC];",
                    "#pragma unroll",
                    f"for (int i = 0; i < VEC; ++i) {acc}_m[i] = {acc}.finish(i);",
                    f"mi::col_fold<{kind}, VEC, CT, RL>({acc}_m, ct, rl, lds_dyn);",
                    f"mi::col_share<{kind}, VEC, CT, RL>({acc}_m, ct, rl, lds_dyn);",
                ])
                return self._unpack_result(f"{acc}_m", "welford_reduce", dtype)
            if self.mode != "row":
                raise UnsupportedHipCodegen("welford_combine outside the row and column-loop shapes")
            merged_name = f"red{n}"
            if self.persistent_reduction:
                self.compute.writeline(
                    f"const auto {merged_name} = mi::group_merge<{kind}, BLOCK, TPR>("
                    f"mi::moments_step({kind}::init(), {mean}, {m2}, {weight}, rmask), lds_red);"
                )
            else:
                acc = f"acc{n}"
                self.prologue.writeline(f"mi::Moments {acc} = {kind}::init();")
                self.compute.writeline(f"{acc} = mi::moments_step({acc}, {mean}, {m2}, {weight}, rmask);")
                self.row_loop_accs.append(
                    f"const auto {merged_name} = mi::group_merge<{kind}, BLOCK, TPR>({acc}, lds_red);"
                )
            return self._unpack_result(merged_name, reduction_type, dtype)
        if self.mode == "row":
            if self.persistent_reduction:
                if reduction_type == "sum" and not integral:
                    merged = self.cse.generate(
                        self.compute, f"mi::row_sum<BLOCK, TPR>({value}, rmask, lds_red)", dtype=torch.float32
                    )
                    return self._cast_result(merged, dtype)
                if reduction_type == "welford_reduce":
                    # the row is in registers: mean first, then the squared distances from it (the
                    # two-pass definition itself, reference inductor_x/lowering.py:270-293), both as
                    # plain sums
                    mean = self.cse.generate(
                        self.compute, f"mi::row_sum<BLOCK, TPR>({value}, rmask, lds_red) / static_cast<float>(rnumel)",
                        dtype=torch.float32,
                    )
                    m2 = self.cse.generate(
                        self.compute,
                        f"mi::row_sum<BLOCK, TPR>(({value} - {mean}) * ({value} - {mean}), rmask, lds_red)",
                        dtype=torch.float32,
                    )
                    weight = self.cse.generate(self.compute, "static_cast<float>(rnumel)", dtype=torch.float32)
                    return (mean, m2, weight)
                if reduction_type == "online_softmax_reduce":
                    # the row is in registers: the maximum, then the sum against it
                    top = self.cse.generate(
                        self.compute,
                        f"mi::group_merge<mi::RedMax, BLOCK, TPR>(mi::RedMax::finish(mi::thread_step<mi::RedMax>("
                        f"mi::RedMax::init(), {value}, {self._r_index_str()}, rmask)), lds_red)",
                        dtype=torch.float32,
                    )
                    total = self.cse.generate(
                        self.compute, f"mi::row_sum<BLOCK, TPR>(mi::exp({value} - {top}), rmask, lds_red)",
                        dtype=torch.float32,
                    )
                    return (top, total)
                merged_name = f"red{n}"
                self.compute.writeline(
                    f"const auto {merged_name} = mi::group_merge<{kind}, BLOCK, TPR>({kind}::finish("
                    f"mi::thread_step<{kind}>({kind}::init(), {value}, {self._r_index_str()}, rmask)), lds_red);"
                )
            else:
                acc = f"acc{n}"
                self.prologue.writeline(f"typename {kind}::T {acc} = {kind}::init();")
                if reduction_type == "online_softmax_reduce":
                    self.compute.writeline(f"{acc} = mi::softmax_step({acc}, {value}, rmask);")
                else:
                    self.compute.writeline(
                        f"{acc} = mi::thread_step<{kind}>({acc}, {value}, {self._r_index_str()}, rmask);"
                    )
                merged_name = f"red{n}"
                self.row_loop_accs.append(
                    f"const auto {merged_name} = mi::group_merge<{kind}, BLOCK, TPR>({kind}::finish({acc}), lds_red);"
                )
            return self._unpack_result(merged_name, reduction_type, dtype, integral)
        if self.mode == "colloop":
            acc = f"acc{n}"
            self.prologue.writeline(f"mi::ColAcc<{kind}, VEC> {acc};")
            self.prologue.writeline(f"{acc}.init();")
            self.compute.writeline(f"{acc}.step({value}, r0_index, true);")
            self.colloop_max_words = max(getattr(self, "colloop_max_words", 1), words)
            self.row_loop_accs.extend([
                f"typename {kind}::M {acc}_m[VEC];",
                "#pragma unroll",
                f"for (int i = 0; i < VEC; ++i) {acc}_m[i] = {acc}.finish(i);",
                f"mi::col_fold<{kind}, VEC, CT, RL>({acc}_m, ct, rl, lds_dyn);",
                f"mi::col_share<{kind}, VEC, CT, RL>({acc}_m, ct, rl, lds_dyn);",
            ])
            return self._unpack_result(f"{acc}_m", reduction_type, dtype, integral)
        if self.mode == "col":
            acc = f"acc{n}"
            merged_name = f"red{n}"
            self.col_reductions.append(
                ColReduction(reduction_type, acc, merged_name, str(value), self.ws_words, cxx=kind, words=words)
            )
            self.ws_words += words
            self.compute.writeline(f"{acc}.step({value}, r0_index, xmask);")
            return self._unpack_result(merged_name, reduction_type, dtype, integral)
        raise UnsupportedHipCodegen("reduction in a pointwise kernel")

    def _result_var(self, text: str, dtype: torch.dtype) -> CSEVariable:
        """A value that exists once the reduction is complete.  With the whole
        row in registers the code is straight-line, so the definition goes where
        the reduction stands; otherwise it is placed after the loop."""
        name = f"rv{next(self.acc_ids)}"
        var = self.create_cse_var(name, ValueRanges.unknown(), dtype)
        if self.mode == "row" and self.persistent_reduction:
            self.compute.writeline(f"const auto {name} = {text};")
        else:
            self._result_defs.append(f"const auto {name} = {text};")
        return var

    def _cast_result(self, var: CSEVariable, dtype: torch.dtype) -> CSEVariable:
        return var

    def _unpack_result(self, merged: str, reduction_type: str, dtype: torch.dtype, integral: bool = False):
        if integral:
            wide_dtype, getter = (torch.float64, "GetSelfF64") if integral == "f64" else (torch.int64, "GetSelfInt")
            if self.mode == "colloop":
                var = self._result_var(f"mi::col_get<VEC>({merged}, mi::{getter}())", wide_dtype)
                if isinstance(var, HipCSEVariable):
                    var.is_vec = True
                return var
            return self._result_var(f"{merged}", wide_dtype)
        if self.mode == "colloop":
            # `merged` is an array of VEC states, one per column of the thread: results are vectors
            def vec_result(getter: str, dt: torch.dtype) -> CSEVariable:
                var = self._result_var(f"mi::col_get<VEC>({merged}, mi::{getter}())", dt)
                if isinstance(var, HipCSEVariable):
                    var.is_vec = True
                return var

            if reduction_type in ("argmax", "argmin"):
                return vec_result("GetIndex", torch.int64)
            if reduction_type == "welford_reduce":
                return (vec_result("GetMean", torch.float32), vec_result("GetM2", torch.float32),
                        vec_result("GetCount", torch.float32))
            if reduction_type == "online_softmax_reduce":
                return (vec_result("GetSoftmaxMax", torch.float32), vec_result("GetSoftmaxSum", torch.float32))
            if reduction_type == "any":
                return vec_result("GetNonzero", torch.bool)
            return vec_result("GetSelf", torch.float32)
        if reduction_type in ("argmax", "argmin"):
            return self._result_var(f"static_cast<mi::i64>({merged}.i)", torch.int64)
        if reduction_type in ("welford_reduce", "welford_combine"):
            return (
                self._result_var(f"{merged}.mean", torch.float32),
                self._result_var(f"{merged}.m2", torch.float32),
                self._result_var(f"{merged}.n", torch.float32),
            )
        if reduction_type == "online_softmax_reduce":
            return (self._result_var(f"{merged}.m", torch.float32), self._result_var(f"{merged}.s", torch.float32))
        if reduction_type == "any":
            return self._result_var(f"({merged} != 0.f)", torch.bool)
        return self._result_var(f"{merged}", torch.float32)

    # -- body assembly ----------------------------------------------------------
    def _take_result_defs(self) -> list[str]:
        defs = self._result_defs
        self._result_defs = []
        return defs

    def _plan_col_pipeline(self) -> Optional[tuple[str, list[str], str]]:
        """(entry text, loaded variable names, loads text, rest text) when the loop body of a column
        sweep starts with nothing but plain vector loads: those can be issued one batch ahead of
        the folds that use them.  Anything else in the loads (guards, stashes, a load through a
        loaded index) keeps the plain loop."""
        if os.environ.get("INDUCTOR_X_AMD_COL_PIPELINE", "1") == "0":
            return None
        lines = [l.strip() for l in self.loads.getvalue().splitlines() if l.strip()]
        names = []
        for line in lines:
            m = re.fullmatch(r"auto (tmp\d+) = mi::vload(?:_u)?<[^;]*\);", line)
            if m is None or re.search(r"\btmp\d+\b", line.split("=", 1)[1]):
                return None
            names.append(m.group(1))
        if not 1 <= len(names) <= 4:
            return None
        rest = IndentedBuffer()
        rest.splice(self.compute)
        rest.splice(self.stores)
        return (self._entry_code(self.r_entries).getvalue(), names, self.loads.getvalue(), rest.getvalue())

    def codegen_body(self) -> None:
        if not (self.loads or self.compute or self.stores or self.row_loop_accs or self._result_defs or self.red_stores):
            return
        if self.mode == "col":
            if self.inside_reduction and not self.phase_bodies_started:
                # loop body of the partial kernel; what follows belongs to the final kernel
                self.partial_body.splice(self._entry_code(self.r_entries))
                self.partial_body.splice(self.loads)
                self.partial_body.splice(self.compute)
                self.partial_body.splice(self.stores)
                self._col_pipeline = self._plan_col_pipeline()
                self.phase_bodies_started = True
                self._result_defs_col = self._take_result_defs()
                self.final_body.splice(self.red_stores)
                keep = OrderedSet()
                for item in self.cse.reduction_cache.values():
                    for v in item if isinstance(item, tuple) else (item,):
                        keep.add(v)
                self.cse.invalidate(keep)
            else:
                self.final_body.splice(self.loads)
                self.final_body.splice(self.compute)
                self.final_body.splice(self.stores)
                self.final_body.splice(self.red_stores)
        elif self.mode == "colloop" and self.inside_reduction:
            # one pass over the reduced axis, row lanes RL apart; the folds that follow hold
            # barriers, so every thread runs the loop (threads past the end on clamped columns)
            self.body.writeline(f"for ({self.index_dtype} r0_index = rl; r0_index < rnumel; r0_index += RL) {{")
            with self.body.indent():
                self.body.splice(self._entry_code(self.r_entries))
                self.body.splice(self.loads)
                self.body.splice(self.compute)
                self.body.splice(self.stores)
            self.body.writeline("}")
            for line in self.row_loop_accs:
                self.body.writeline(line)
            self.row_loop_accs.clear()
            for line in self._take_result_defs():
                self.body.writeline(line)
            self.body.splice(self.red_stores)
            keep = OrderedSet()
            for item in self.cse.reduction_cache.values():
                for v in item if isinstance(item, tuple) else (item,):
                    keep.add(v)
            self.cse.invalidate(keep)
        elif self.mode == "row" and self.inside_reduction and not self.persistent_reduction:
            # one pass over the reduced axis: whole rounds of TPR * VEC elements run unmasked (the
            # mask is a compile-time true, so loads carry no branch and several rounds' loads can
            # be in flight at once); the last, partial round runs the same body under the mask
            idx_t = self.index_dtype
            unroll = int(os.environ.get("INDUCTOR_X_AMD_ROW_LOOP_UNROLL", "4"))
            split_tail = unroll > 0

            def one_round() -> None:
                self.body.splice(self._entry_code(self.r_entries))
                self.body.splice(self.loads)
                self.body.splice(self.compute)
                self.body.splice(self.stores)

            if split_tail:
                whole = "(rnumel - rnumel % (TPR * VEC))"
                self.body.writeline(f"#pragma unroll {unroll}")
                self.body.writeline(f"for ({idx_t} r0_base = 0; r0_base < {whole}; r0_base += TPR * VEC) {{")
                with self.body.indent():
                    self.body.writeline(f"const {idx_t} r0_index = r0_base + rlane * VEC;")
                    self.body.writeline("constexpr bool rmask = true;")
                    one_round()
                self.body.writeline("}")
                self.body.writeline(f"if ({whole} < rnumel) {{")
                with self.body.indent():
                    self.body.writeline(f"const {idx_t} r0_index = {whole} + rlane * VEC;")
                    self.body.writeline("const bool rmask = r0_index < rnumel;")
                    one_round()
                self.body.writeline("}")
            else:
                self.body.writeline(f"for ({idx_t} r0_base = 0; r0_base < rnumel; r0_base += TPR * VEC) {{")
                with self.body.indent():
                    self.body.writeline(f"const {idx_t} r0_index = r0_base + rlane * VEC;")
                    self.body.writeline("const bool rmask = r0_index < rnumel;")
                    one_round()
                self.body.writeline("}")
            self.row_pass += 1
            for line in self.row_loop_accs:
                self.body.writeline(line)
            self.row_loop_accs.clear()
            for line in self._take_result_defs():
                self.body.writeline(line)
            self.body.splice(self.red_stores)
            # values computed inside the loop die with it; reduction results survive
            keep = OrderedSet()
            for item in self.cse.reduction_cache.values():
                for v in item if isinstance(item, tuple) else (item,):
                    keep.add(v)
            self.cse.invalidate(keep)
        else:
            self.body.splice(self.loads)
            self.body.splice(self.compute)
            for line in self._take_result_defs():
                self.body.writeline(line)
            self.body.splice(self.stores)
            self.body.splice(self.red_stores)
        self.loads.clear()
        self.compute.clear()
        self.stores.clear()
        self.red_stores.clear()

    # -- signature -----------------------------------------------------------------
    def _signature(self):
        """C parameter list, struct codes for packing, python call arguments."""
        _, call_args, signature, _ = self.args.python_argdefs()
        call_args = [str(a) for a in call_args]
        params, codes = [], []
        # buffers a launch both reads and writes (in-place operands, targets of accumulating stores):
        # launching twice is not the same as launching once, so whoever times the kernel must do it on copies
        accumulated = self.__dict__.get("accumulated_args", set())
        self.mutated_arg_positions = [
            pos for pos, arg in enumerate(signature)
            if isinstance(arg, TensorArg) and (arg.name.startswith("in_out_ptr") or arg.name in accumulated)
        ]
        self.written_arg_positions = [
            pos for pos, arg in enumerate(signature)
            if isinstance(arg, TensorArg) and (arg.name.startswith("out_ptr") or arg.name.startswith("in_out_ptr"))
        ]
        for pos, arg in enumerate(signature):
            if isinstance(arg, TensorArg) and should_unwrap_unspec_arg(arg.buffer):
                # a zero-dimensional CPU tensor among GPU operands (a Python number dynamo chose not
                # to bake in, or a CPU scalar tensor): its value is a kernel argument, read on the
                # host at launch (torch/_inductor/codegen/triton_utils.py:24-33, wrapper.py:2743-2747)
                ctype, code = SCALAR_ARG[arg.dtype]
                params.append(f"const {ctype} {arg.name}")
                codes.append(code)
                call_args[pos] = f"{call_args[pos]}.item()"
            elif isinstance(arg, TensorArg):
                const = "" if (arg.name.startswith("out_ptr") or arg.name.startswith("in_out_ptr")) else "const "
                params.append(f"{const}{DTYPE_TO_HIP[arg.dtype]}* __restrict__ {arg.name}")
                codes.append("P")
            elif isinstance(arg, SizeArg):
                expr = getattr(arg, "expr", None)
                is_float = isinstance(expr, (float, sympy.Float)) or (
                    isinstance(expr, sympy.Symbol) and symbol_is_type(expr, (SymT.FLOAT, SymT.UNBACKED_FLOAT))
                )
                if is_float:
                    params.append(f"const double {arg.name}")
                    codes.append("d")
                else:
                    params.append(f"const mi::i64 {arg.name}")
                    codes.append("q")
            elif isinstance(arg, WorkspaceArg):
                raise UnsupportedHipCodegen("Inductor-managed workspace arguments")
            else:
                raise UnsupportedHipCodegen(f"kernel argument {type(arg).__name__}")
        return params, "".join(codes), call_args

    ROW_STASH_BUDGET = 144 * 1024

    def _plan_row_stash(self) -> tuple[list[str], int]:
        """A looped row kernel that reads the same piece of a row in several passes (softmax: the
        maximum, the sum, the output) keeps the row in LDS after the first pass when it fits the
        CU's 160 KB: later passes read LDS instead of going back to memory.  Each thread reads
        back exactly the vectors it stored, so no barrier is involved.  One row per workgroup;
        the workgroup grows with the row so that one or two of them still fill the CU.
        Returns the declarations for the kernel and the dynamic LDS bytes."""
        from ..hip_heuristics import next_power_of_2

        used = [e for e in self.row_stash.values() if e["reused"]]
        if (
            not used or self.mode != "row" or self.persistent_reduction or self.tpr != self.block
            or os.environ.get("INDUCTOR_X_AMD_ROW_STASH", "1") == "0"
        ):
            return [], 0
        rnumel = self._static_numel("r0_")
        if rnumel is None:
            return [], 0
        per_elem = sum(dtype_nbytes(e["dtype"]) for e in used)
        vectors = -(-rnumel // self.vec)
        raw = rnumel * per_elem
        want = 256 if raw <= 40 * 1024 else (512 if raw <= 80 * 1024 else 1024)
        tpr = max(min(want, next_power_of_2(vectors)), 64)
        span = tpr * self.vec
        padded = -(-rnumel // span) * span
        if padded * per_elem > self.ROW_STASH_BUDGET:
            return [], 0
        self.tpr = self.block = tpr
        decls = ["extern __shared__ __align__(16) unsigned char lds_rows[];"]
        offset = 0
        for e in used:
            e["offset"] = offset
            decls.append(
                f"{DTYPE_TO_HIP[e['dtype']]}* const lds_row{e['id']} = "
                f"reinterpret_cast<{DTYPE_TO_HIP[e['dtype']]}*>(lds_rows + {offset});"
            )
            offset += padded * dtype_nbytes(e["dtype"])
        return decls, offset

    def codegen_kernel(self, name: Optional[str] = None) -> str:
        self.codegen_body()
        # Size symbols in the range variables' definitions become kernel
        # arguments the first time they are renamed: do that before the
        # parameter list is taken.
        for entry in (*self.x_entries, *self.r_entries):
            self.rename_indexing(entry.expr)
        params, codes, _ = self._signature()
        idx_t = self.index_dtype
        idx_code = "i" if idx_t == "int" else "q"
        kname = name or "KERNEL_NAME"
        src = IndentedBuffer()
        src.writeline('#include "mi/codegen.h"')
        stash_decls, stash_bytes = self._plan_row_stash()
        for entry in self.row_stash.values():
            k = entry["id"]
            if entry.get("offset") is not None:
                src.writeline(f"#define MI_ROW_STASH_{k}(v) mi::vstore<VEC>(lds_row{k} + r0_index, v)")
                src.writeline(f"#define MI_ROW_RELOAD_{k}(...) mi::vload<VEC>(lds_row{k} + r0_index)")
            else:
                src.writeline(f"#define MI_ROW_STASH_{k}(v)")
                src.writeline(f"#define MI_ROW_RELOAD_{k}(...) (__VA_ARGS__)")
        src.writeline("")
        meta: dict[str, Any] = {"mode": self.mode, "vec": self.vec, "block": self.block, "index_code": idx_code}
        if self.mode == "pointwise":
            plist = ", ".join(params + [f"const {idx_t} xnumel"])
            src.writeline(f'extern "C" __global__ __launch_bounds__({self.block}) void {kname}({plist}) {{')
            tile = self.pointwise_tile_plan()
            tp = self.tplan
            unroll = self.vec if tp else (tile["unroll"] if tile else self.pointwise_unroll())
            with src.indent():
                src.writeline(f"constexpr int VEC = {self.vec};")
                src.writeline(f"constexpr int UNROLL = {unroll};")
                src.writeline(f"constexpr bool STREAM_READS = {'true' if self._reads_stream(tiled=bool(tp or tile)) else 'false'};")
                if tp:
                    # thread -> VEC x VEC elements (x0 times the transposed operands' contiguous axis);
                    # wavefront -> WI x WJ threads; workgroup -> TI x TJ threads; the rest of the index
                    # space is walked by the workgroup id
                    src.writeline(
                        f"constexpr int L0 = {tp['L0']}, DK = {tp['DK']}, LK = {tp['LK']}, TI = {tp['TI']}, "
                        f"TJ = {tp['TJ']}, WI = {tp['WI']}, WJ = {tp['WJ']};"
                    )
                    src.writeline("const int lane_ = threadIdx.x % 64, wave_ = threadIdx.x / 64;")
                    src.writeline("const int tj_ = lane_ % WJ + WJ * (wave_ % (TJ / WJ));")
                    src.writeline("const int ti_ = lane_ / WJ + WI * (wave_ / (TJ / WJ));")
                    src.writeline(f"constexpr int TILES_I = {tp['tiles_i']}, TILES_K = {tp['tiles_k']};")
                    src.writeline(f"const {idx_t} wg_ = static_cast<{idx_t}>(blockIdx.x);")
                    src.writeline(f"const {idx_t} t0_ = wg_ % TILES_I;")
                    src.writeline(f"const {idx_t} tk_ = (wg_ / TILES_I) % TILES_K;")
                    src.writeline(f"const {idx_t} rest_ = wg_ / (TILES_I * TILES_K);")
                    # tiles may hang over the end of either direction
                    src.writeline("if ((t0_ * TI + ti_) * VEC >= L0 || (tk_ * TJ + tj_) * VEC >= LK) return;")
                    src.writeline(
                        f"const {idx_t} xbase = (t0_ * TI + ti_) * VEC + static_cast<{idx_t}>(DK) * ((tk_ * TJ + tj_) * VEC) + "
                        f"(rest_ % (DK / L0)) * L0 + (rest_ / (DK / L0)) * (static_cast<{idx_t}>(DK) * LK);"
                    )
                    for decl in self.tile_decls:
                        src.writeline(decl)
                elif tile:
                    # workgroup -> (T1 x T2) tile of the two axes above the innermost one; within the
                    # tile consecutive threads walk the innermost axis, then axis 2, then axis 1
                    t1, t2, cpt = tile["T1"], tile["T2"], tile["cpt"]
                    src.writeline(f"constexpr int L0 = {tile['L0']}, L1 = {tile['L1']}, L2 = {tile['L2']};")
                    src.writeline(f"constexpr int T1 = {t1}, T2 = {t2}, CPT = {cpt};")
                    src.writeline(f"const {idx_t} tile_ = static_cast<{idx_t}>(blockIdx.x);")
                    src.writeline(f"const {idx_t} tile1 = tile_ % (L1 / T1);")
                    src.writeline(f"const {idx_t} tile2 = (tile_ / (L1 / T1)) % (L2 / T2);")
                    src.writeline(f"const {idx_t} outer_ = tile_ / ((L1 / T1) * (L2 / T2));")
                else:
                    # Workgroup i runs on die i % 8, each die with an L2 of its own.  Die d takes the d-th
                    # eighth of the index space, so neighbouring pieces (which share cache lines when an
                    # operand is broadcast or gathered along the fast axis) meet in one L2; the launch
                    # rounds the workgroup count up to a multiple of 8.  Measured on MI355X: a bf16
                    # output scaled by a per-(row, 128-column group) statistic read with stride 32 bytes
                    # 61 -> 46 us, a plain bf16 add of 96 MiB tensors 42.1 -> 41.0 us.
                    src.writeline(f"const {idx_t} per_die_ = static_cast<{idx_t}>(gridDim.x) >> 3;")
                    src.writeline(
                        f"const {idx_t} wg_ = (gridDim.x & 7) == 0 ? static_cast<{idx_t}>(blockIdx.x & 7) * per_die_ + "
                        f"static_cast<{idx_t}>(blockIdx.x >> 3) : static_cast<{idx_t}>(blockIdx.x);"
                    )
                    src.writeline(f"const {idx_t} xbase = (wg_ * UNROLL * {self.block} + threadIdx.x) * VEC;")
                    meta["grid_multiple"] = 8
                    meta["index_bits"] = 32 if idx_t == "int" else 64
                # each thread handles UNROLL vectors one workgroup-width apart, so a
                # wavefront still touches 1 KiB runs and has UNROLL loads in flight
                src.writeline("#pragma unroll")
                src.writeline("for (int u = 0; u < UNROLL; ++u) {")
                with src.indent():
                    if tp:
                        src.writeline(f"const {idx_t} xindex = xbase + static_cast<{idx_t}>(DK) * u;")
                    elif tile:
                        src.writeline(f"const int e_ = u * {self.block} + static_cast<int>(threadIdx.x);")
                        src.writeline("const int row_ = e_ / CPT;")
                        src.writeline(
                            f"const {idx_t} xindex = (e_ % CPT) * VEC + L0 * ((tile1 * T1 + row_ / T2) + "
                            f"L1 * ((tile2 * T2 + row_ % T2) + static_cast<{idx_t}>(L2) * outer_));"
                        )
                    else:
                        src.writeline(f"const {idx_t} xindex = xbase + static_cast<{idx_t}>(u) * ({self.block} * VEC);")
                        src.writeline("if (xindex >= xnumel) break;")
                    src.splice(self._entry_code(self.x_entries))
                    src.splice(self.body)
                src.writeline("}")
            src.writeline("}")
            sig = codes + idx_code
            meta["unroll"] = unroll
            if tp:
                meta["grid"] = tp["grid"]
        elif self.mode == "row":
            plist = ", ".join(params + [f"const {idx_t} xnumel", f"const {idx_t} rnumel"])
            src.writeline(f'extern "C" __global__ __launch_bounds__({self.block}) void {kname}({plist}) {{')
            with src.indent():
                src.writeline(f"constexpr int VEC = {self.vec};")
                src.writeline(f"constexpr int BLOCK = {self.block};")
                src.writeline(f"constexpr int TPR = {self.tpr};")
                src.writeline(f"constexpr bool STREAM_READS = {'true' if self._reads_stream() else 'false'};")
                src.writeline("__shared__ float lds_red[(BLOCK / 64) * 4];")
                for line in stash_decls:
                    src.writeline(line)
                src.writeline("const int rlane = threadIdx.x % TPR;")
                # a workgroup walks the rows with the stride of the grid, so the launcher can cap the
                # grid when there are many short rows (one workgroup per 4 KiB of input would be
                # bound by the rate at which workgroups are dispatched)
                src.writeline(
                    f"for ({idx_t} xrow0 = static_cast<{idx_t}>(blockIdx.x) * (BLOCK / TPR); xrow0 < xnumel; "
                    f"xrow0 += static_cast<{idx_t}>(gridDim.x) * (BLOCK / TPR)) {{"
                )
                with src.indent():
                    src.writeline(f"const {idx_t} xrow = xrow0 + threadIdx.x / TPR;")
                    src.writeline("const bool xmask = xrow < xnumel;")
                    src.writeline(f"const {idx_t} xindex = xmask ? xrow : xnumel - 1;")
                    if self.persistent_reduction:
                        src.writeline(f"const {idx_t} r0_index = rlane * VEC;")
                        src.writeline("const bool rmask = r0_index < rnumel;")
                    src.splice(self._entry_code(self.x_entries))
                    if self.persistent_reduction:
                        src.splice(self._entry_code(self.r_entries))
                    src.splice(self.prologue)
                    src.splice(self.body)
                src.writeline("}")
            src.writeline("}")
            sig = codes + idx_code + idx_code
            meta.update({"tpr": self.tpr, "persistent": bool(self.persistent_reduction), "block": self.block,
                         "lds_bytes": stash_bytes})
        elif self.mode == "colloop":
            ct, rl = self.col_ct, self.col_rl
            words = getattr(self, "colloop_max_words", 1)
            plist = ", ".join(params + [f"const {idx_t} xnumel", f"const {idx_t} rnumel"])
            src.writeline(f'extern "C" __global__ __launch_bounds__({self.block}) void {kname}({plist}) {{')
            with src.indent():
                src.writeline(f"constexpr int VEC = {self.vec};")
                src.writeline(f"constexpr int CT = {ct};")
                src.writeline(f"constexpr int RL = {rl};")
                src.writeline("extern __shared__ float lds_dyn[];")
                src.writeline("const int ct = threadIdx.x % CT;")
                src.writeline("const int rl = threadIdx.x / CT;")
                src.writeline(f"const {idx_t} xraw = (static_cast<{idx_t}>(blockIdx.x) * CT + ct) * VEC;")
                src.writeline("const bool xmask = xraw < xnumel;")
                src.writeline(f"const {idx_t} xindex = xmask ? xraw : 0;")
                src.splice(self._entry_code(self.x_entries))
                src.splice(self.prologue)
                src.splice(self.body)
            src.writeline("}")
            sig = codes + idx_code + idx_code
            meta.update({"ct": ct, "rl": rl,
                         "lds_bytes": max((rl // 2) * ct * self.vec * words * 4, ct * self.vec * words * 4)})
        else:  # col
            sig = self._codegen_col(src, kname, params, codes, idx_t, idx_code, meta)
        meta["signature"] = sig
        meta["n_buffer_args"] = len(codes)
        meta["mutated_args"] = list(getattr(self, "mutated_arg_positions", []))
        meta["written_args"] = list(getattr(self, "written_arg_positions", []))
        self.meta = meta
        return src.getvalue()

    def _codegen_col(self, src, kname, params, codes, idx_t, idx_code, meta) -> str:
        if not self.col_reductions:
            raise UnsupportedHipCodegen("column kernel without a reduction")
        ct, rl, vec = self.col_ct, self.col_rl, self.vec
        # A plain fp32 sum of a value whose moments the kernel accumulates anyway (mean beside
        # variance) is read off the moments (mean * count) instead of being summed once more.
        alias: dict[str, ColReduction] = {}
        for c in self.col_reductions:
            if c.cxx == "mi::RedSum":
                twin = next((w for w in self.col_reductions if w.kind == "welford_reduce" and w.value == c.value), None)
                if twin is not None:
                    alias[c.acc] = twin
        all_reductions = list(self.col_reductions)
        self.col_reductions = [c for c in all_reductions if c.acc not in alias]
        self.ws_words = 0
        for c in self.col_reductions:
            c.ws_offset_words = self.ws_words
            self.ws_words += c.words
        aliased = [c for c in all_reductions if c.acc in alias]
        max_words = max(c.words for c in self.col_reductions)
        extra = [f"float* __restrict__ ws", f"const {idx_t} xnumel", f"const {idx_t} rnumel", "const int nsplit"]
        # rows handed to a thread between two looks at the loop counter
        unroll = int(os.environ.get("INDUCTOR_X_AMD_COL_UNROLL", "4"))
        plist = ", ".join(params + extra)
        # ---- pass 1, and the same sweep finishing in place ("direct") for launches where one
        # workgroup per column tile already fills the GPU: no workspace, no second kernel
        def sweep(suffix: str, direct: bool) -> None:
            src.writeline(f'extern "C" __global__ __launch_bounds__({ct * rl}) void {kname}{suffix}({plist}) {{')
            with src.indent():
                src.writeline(f"constexpr int VEC = {vec};")
                src.writeline(f"constexpr int CT = {ct};")
                src.writeline(f"constexpr int RL = {rl};")
                src.writeline("extern __shared__ float lds_dyn[];")
                src.writeline("const int ct = threadIdx.x % CT;")
                src.writeline("const int rl = threadIdx.x / CT;")
                src.writeline(f"const {idx_t} xindex = (static_cast<{idx_t}>(blockIdx.x) * CT + ct) * VEC;")
                src.writeline("const int split = blockIdx.y;")
                src.writeline("const bool xmask = xindex < xnumel;")
                # The reduced axis is dealt out in batches of RL * UNR consecutive rows, batch b
                # to split b % nsplit: the workgroups of a column tile read one contiguous
                # stretch between them at any moment, and any split count is valid.
                src.writeline(f"constexpr int UNR = {unroll};")
                src.writeline(f"const {idx_t} batch_ = RL * UNR;")
                src.writeline(f"const {idx_t} full_ = rnumel / batch_;")
                for c in self.col_reductions:
                    kind = c.cxx
                    src.writeline(f"mi::ColAcc<{kind}, VEC> {c.acc};")
                    src.writeline(f"{c.acc}.init();")
                for c in aliased:
                    src.writeline(f"mi::ColAccNone {c.acc};  // read off {alias[c.acc].acc}")
                src.writeline("if (xmask) {")
                with src.indent():
                    src.splice(self._entry_code(self.x_entries))
                    src.writeline(f"{idx_t} b_ = split;")
                    pipe = getattr(self, "_col_pipeline", None)
                    if pipe is not None:
                        # the loads of batch b + nsplit are in flight while batch b is folded
                        entry_text, names, loads_text, rest_text = pipe
                        src.writeline(f"auto ld_ = [&](const {idx_t} r0_index) {{")
                        with src.indent():
                            src.splice(entry_text)
                            src.splice(loads_text)
                            src.writeline(f"return mi::pack({', '.join(names)});")
                        src.writeline("};")
                        src.writeline(f"using L_ = decltype(ld_({idx_t}(0)));")
                        src.writeline("L_ cur_[UNR];")
                        src.writeline("if (b_ < full_) {")
                        with src.indent():
                            src.writeline("#pragma unroll")
                            src.writeline("for (int u_ = 0; u_ < UNR; ++u_) cur_[u_] = ld_(b_ * batch_ + u_ * RL + rl);")
                        src.writeline("}")
                        src.writeline("while (b_ < full_) {")
                        with src.indent():
                            src.writeline(f"const {idx_t} bn_ = b_ + nsplit;")
                            src.writeline("L_ nxt_[UNR];")
                            src.writeline("if (bn_ < full_) {")
                            with src.indent():
                                src.writeline("#pragma unroll")
                                src.writeline("for (int u_ = 0; u_ < UNR; ++u_) nxt_[u_] = ld_(bn_ * batch_ + u_ * RL + rl);")
                            src.writeline("}")
                            src.writeline("#pragma unroll")
                            src.writeline("for (int u_ = 0; u_ < UNR; ++u_) {")
                            with src.indent():
                                src.writeline(f"const {idx_t} r0_index = b_ * batch_ + u_ * RL + rl;")
                                src.splice(entry_text)
                                src.writeline(f"auto [{', '.join(names)}] = cur_[u_];")
                                src.splice(rest_text)
                            src.writeline("}")
                            src.writeline("b_ = bn_;")
                            src.writeline("#pragma unroll")
                            src.writeline("for (int u_ = 0; u_ < UNR; ++u_) cur_[u_] = nxt_[u_];")
                        src.writeline("}")
                    else:
                        src.writeline("for (; b_ < full_; b_ += nsplit) {")
                        with src.indent():
                            src.writeline("#pragma unroll")
                            src.writeline("for (int u_ = 0; u_ < UNR; ++u_) {")
                            with src.indent():
                                src.writeline(f"const {idx_t} r0_index = b_ * batch_ + u_ * RL + rl;")
                                src.splice(self.partial_body)
                            src.writeline("}")
                        src.writeline("}")
                    # the last, partly filled batch
                    src.writeline("if (b_ == full_) {")
                    with src.indent():
                        src.writeline(f"for ({idx_t} r0_index = full_ * batch_ + rl; r0_index < rnumel; r0_index += RL) {{")
                        with src.indent():
                            src.splice(self.partial_body)
                        src.writeline("}")
                    src.writeline("}")
                src.writeline("}")
                for c in self.col_reductions:
                    src.writeline(f"typename {c.cxx}::M {c.acc}_m[VEC];")
                    src.writeline("#pragma unroll")
                    src.writeline(f"for (int i = 0; i < VEC; ++i) {c.acc}_m[i] = {c.acc}.finish(i);")
                # one fold for all reductions: lane exchanges inside a wavefront, one or two LDS rounds
                kinds_ = ", ".join(c.cxx for c in self.col_reductions)
                states_ = ", ".join(f"{c.acc}_m" for c in self.col_reductions)
                src.writeline(f"mi::col_fold_all<VEC, CT, RL, {kinds_}>(lds_dyn, ct, rl, {states_});")
                if not direct:
                    for c in self.col_reductions:
                        src.writeline(
                            f"if (rl == 0) mi::col_store_partial<{c.cxx}, VEC>(ws + {c.ws_offset_words} * "
                            f"static_cast<mi::i64>(nsplit) * xnumel, {c.acc}_m, xindex, xnumel, split, nsplit);"
                        )
                if direct:
                    # the row lane that holds the folded states finishes its VEC columns one by one
                    # with the text of the second kernel (one column per thread there)
                    src.writeline("if (rl == 0 && xmask) {")
                    with src.indent():
                        src.writeline(f"const {idx_t} xfirst_ = xindex;")
                        src.writeline("#pragma unroll")
                        src.writeline("for (int col_ = 0; col_ < VEC; ++col_) {")
                        with src.indent():
                            src.writeline(f"const {idx_t} xindex = xfirst_ + col_;")
                            src.writeline("if (xindex < xnumel) {")
                            with src.indent():
                                src.writeline("constexpr int VEC = 1;")
                                src.writeline("const bool live = true;")
                                src.writeline("const int sl = 0;")
                                for c in self.col_reductions:
                                    src.writeline(f"const auto {c.result} = {c.acc}_m[col_];")
                                for c in aliased:
                                    w = alias[c.acc]
                                    src.writeline(f"const auto {c.result} = {w.acc}_m[col_].mean * {w.acc}_m[col_].n;")
                                for line in self._result_defs_col:
                                    src.writeline(line)
                                src.splice(self._final_indexing_code())
                                src.splice(self.final_body)
                            src.writeline("}")
                        src.writeline("}")
                    src.writeline("}")
            src.writeline("}")
            src.writeline("")

        sweep("_partial", False)
        sweep("_direct", True)
        # ---- pass 2
        # few columns per workgroup, so the second pass runs on hundreds of workgroups of one wavefront
        cpw, sl = (int(t) for t in os.environ.get("INDUCTOR_X_AMD_COL_FINAL", "4,16").split(","))
        src.writeline(f'extern "C" __global__ __launch_bounds__({cpw * sl}) void {kname}_final({plist}) {{')
        with src.indent():
            src.writeline("constexpr int VEC = 1;")
            src.writeline(f"constexpr int CPW = {cpw};")
            src.writeline(f"constexpr int SL = {sl};")
            src.writeline(f"__shared__ float lds_fin[CPW * SL * {sum(c.words for c in self.col_reductions)}];")
            src.writeline("const int slot = threadIdx.x % CPW;")
            src.writeline("const int sl = threadIdx.x / CPW;")
            src.writeline(f"const {idx_t} xraw = static_cast<{idx_t}>(blockIdx.x) * CPW + slot;")
            src.writeline("const bool live = xraw < xnumel;")
            src.writeline(f"const {idx_t} xindex = live ? xraw : xnumel - 1;")
            # the loads of every reduction first, then the folds (each fold holds barriers)
            for c in self.col_reductions:
                kind = c.cxx
                src.writeline(
                    f"const auto {c.result}_g = mi::col_final_gather<{kind}, SL>(ws + {c.ws_offset_words} * "
                    f"static_cast<mi::i64>(nsplit) * xnumel, xindex, xnumel, nsplit, sl, live);"
                )
            for c in self.col_reductions:
                src.writeline(f"auto {c.result} = {c.result}_g;")
            kinds = ", ".join(c.cxx for c in self.col_reductions)
            states = ", ".join(c.result for c in self.col_reductions)
            src.writeline(f"mi::col_final_fold_all<CPW, SL, {kinds}>(lds_fin, slot, sl, {states});")
            for c in aliased:
                src.writeline(f"const auto {c.result} = {alias[c.acc].result}.mean * {alias[c.acc].result}.n;")
            for line in self._result_defs_col:
                src.writeline(line)
            src.splice(self._final_indexing_code())
            src.splice(self.final_body)
        src.writeline("}")
        meta.update({"ct": ct, "rl": rl, "cpw": cpw, "sl": sl, "ws_words": self.ws_words, "col_unroll": unroll,
                     "lds_partial": max((rl // 2) * ct * vec * max_words * 4,
                                        col_fold_all_planes(ct, rl) * ct * vec * sum(c.words for c in self.col_reductions) * 4)})
        return codes + "P" + idx_code + idx_code + "i"

    def _final_indexing_code(self) -> IndentedBuffer:
        """Range variables of the kept axis for the final kernel (one column per
        thread there, so lane vectors collapse to scalars)."""
        return self._entry_code(self.x_entries, lane_vectors=False)

    # -- call ---------------------------------------------------------------------
    def call_kernel(self, name: str, node: Any = None, deallocate_ws: bool = True) -> None:
        wrapper = V.graph.wrapper_code
        for v in self.args.sizevars:
            wrapper.ensure_size_computed(v)
        _, _, call_args = self._signature()
        numels = []
        for tree in self.range_trees:
            if isinstance(tree.numel, (sympy.Integer, int)):
                expr = str(int(tree.numel))
            elif isinstance(tree.numel, sympy.Symbol):
                expr = wrapper.val_to_arg_str(tree.numel) if hasattr(wrapper, "val_to_arg_str") else str(tree.numel)
            else:
                expr = str(wrapper.generate_numel_expr(name, tree).inner)
            numels.append(f"{tree.prefix}numel={expr}")
        device = V.graph.get_current_device_or_throw()
        if device.type == "cpu":
            stream = "0"
        else:
            stream = wrapper.write_get_raw_stream(device.index, V.graph.name)
        args = ", ".join(call_args + numels + [f"stream={stream}"])
        wrapper.writeline(f"{name}.run({args})")
