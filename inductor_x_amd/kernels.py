"""Host entry points of the hand-written kernel families.

Each function checks shapes, dtypes, contiguity and alignment on the host (a
kernel is never launched on operands it was not written for), picks a launch
configuration with the heuristics, and enqueues through the C-ABI launcher on
torch's current stream.  Outputs are allocated with torch; nothing here
computes on the CPU and nothing falls back to eager PyTorch.

The code objects come from csrc/aot/*.hip, compiled ahead of time into the
in-tree store; a missing code object is compiled with hipcc on first use.
"""
from __future__ import annotations

import functools
import math
from typing import Optional

import torch

from . import codecache, config
from .hip_heuristics import (
    CachingLauncher,
    LaunchConfig,
    cdiv,
    col_fold_lds_bytes,
    grid as row_grid,
    next_power_of_2,
    row_reduction_plan,
    split_reduction_plan,
    SplitPlan,
)


def _stream() -> int:
    """Raw hipStream_t of torch's current stream on the current device (the C accessor: building
    a torch.cuda.Stream object for it costs about 8 us per call)."""
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device())


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _aligned(t: torch.Tensor, nbytes: int = 16) -> bool:
    return t.data_ptr() % nbytes == 0


def _check_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        _require(t.is_cuda, "tensor must live on the GPU")
        _require(t.device == tensors[0].device, "tensors must share a device")


# ---------------------------------------------------------------------------
# code objects (one per aot file), loaded lazily
# ---------------------------------------------------------------------------
_ROWSUM_VARIANTS = [(256, 256), (256, 128), (256, 64), (512, 512), (1024, 1024), (512, 256), (512, 128), (128, 128),
                    (64, 64), (128, 64), (512, 64)]
_RMSNORM_VARIANTS = [
    (256, 256, 2),
    (256, 128, 4),
    (256, 64, 8),
    (512, 512, 1),
    (256, 256, 1),
    (256, 256, 4),
    (256, 64, 1),
    (256, 64, 2),
    (256, 64, 4),
    (512, 512, 2),
    (512, 512, 4),
]
_COL_PARTIAL_VARIANTS = [
    (128, 2, 4),
    (128, 2, 8),
    (128, 4, 4),
    (128, 4, 8),
    (128, 8, 4),
    (128, 8, 8),
    (64, 4, 4),
    (64, 4, 8),
    (64, 8, 4),
    (64, 16, 4),
    (64, 1, 8),
    (16, 16, 4),
    (1, 64, 4),
    (16, 64, 4),
    (32, 32, 4),
    (32, 16, 4),
    (16, 32, 4),
    (64, 8, 8),
    (32, 8, 4),
    (32, 8, 8),
    (32, 16, 8),
    (64, 16, 8),
    (64, 4, 16),
    (32, 8, 16),
    (128, 4, 16),
    (128, 2, 16),
    (16, 16, 8),
]
# (ct, rl, unroll, batches held per thread) beyond the default two
_COL_PARTIAL_PF_VARIANTS = [(32, 8, 8, 3), (32, 8, 8, 4), (32, 8, 4, 3), (32, 8, 4, 4), (32, 16, 4, 3), (32, 16, 8, 3),
                            (32, 8, 16, 3), (64, 8, 8, 3)]
_COL_FINAL_VARIANTS = [(16, 16), (16, 32), (8, 64), (8, 32), (4, 64), (64, 4), (4, 16), (4, 32), (2, 64), (2, 32),
                       (8, 16), (8, 8), (16, 4), (16, 8)]
_GATHER_VARIANTS = [(256, 128, 1), (256, 128, 2), (256, 128, 4), (256, 64, 1), (256, 64, 2), (256, 64, 4), (256, 16, 1), (256, 16, 4)]
_PERMUTE_VARIANTS = [
    (256, 16, 32, 8),
    (256, 16, 32, 4),
    (256, 16, 32, 2),
    (256, 16, 16, 8),
    (256, 16, 8, 8),
    (256, 16, 4, 16),
    (256, 16, 1, 64),
    (256, 16, 1, 128),
    (256, 16, 1, 16),
    (256, 16, 2, 8),
    (256, 8, 1, 32),
    (256, 4, 1, 64),
    (256, 64, 1, 4),
    (256, 64, 4, 4),
    (256, 16, 8, 4),
    (256, 16, 16, 4),
    (256, 16, 4, 8),
    (256, 16, 8, 2),
    (256, 16, 4, 4),
]


@functools.lru_cache(maxsize=None)
def _rowsum_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(f"fused_relu_sigmoid_rowsum_f32_b{b}_t{t}", b, meta={"BLOCK": b, "TPR": t, "PER_WG0": b // t})
        for b, t in _ROWSUM_VARIANTS
    ]
    return CachingLauncher(
        "fused_relu_sigmoid_rowsum_f32", codecache.aot_source("row_kernels.hip"), "PPii", cfgs, prefer_intree=True
    )


@functools.lru_cache(maxsize=None)
def _rmsnorm_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(
            f"add_rmsnorm_bf16_b{b}_t{t}_i{i}", b, meta={"BLOCK": b, "TPR": t, "ITERS": i, "PER_WG0": b // t}
        )
        for b, t, i in _RMSNORM_VARIANTS
    ]
    return CachingLauncher(
        "add_rmsnorm_bf16", codecache.aot_source("row_kernels.hip"), "PPPPPiif", cfgs, prefer_intree=True
    )


@functools.lru_cache(maxsize=None)
def _col_partial_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(
            f"col_mean_var_argmax_partial_f32_c{ct}_r{rl}_u{u}",
            ct * rl,
            meta={"CT": ct, "RL": rl, "UNROLL": u},
            lds_bytes=col_fold_lds_bytes(ct, rl),
        )
        for ct, rl, u in _COL_PARTIAL_VARIANTS
    ] + [
        LaunchConfig(
            f"col_mean_var_argmax_partial_f32_c{ct}_r{rl}_u{u}_p{pf}",
            ct * rl,
            meta={"CT": ct, "RL": rl, "UNROLL": u, "PF": pf},
            lds_bytes=col_fold_lds_bytes(ct, rl),
        )
        for ct, rl, u, pf in _COL_PARTIAL_PF_VARIANTS
    ]
    return CachingLauncher(
        "col_mean_var_argmax_partial_f32", codecache.aot_source("col_kernels.hip"), "PPiii", cfgs, prefer_intree=True
    )


@functools.lru_cache(maxsize=None)
def _col_final_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(f"col_mean_var_argmax_final_f32_c{c}_s{s}", c * s, meta={"CPW": c, "SL": s})
        for c, s in _COL_FINAL_VARIANTS
    ]
    return CachingLauncher(
        "col_mean_var_argmax_final_f32", codecache.aot_source("col_kernels.hip"), "PPPPiiiif", cfgs, prefer_intree=True
    )


@functools.lru_cache(maxsize=None)
def _gather_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(f"gather_rows_b16_b{b}_t{t}_r{r}", b, meta={"BLOCK": b, "TPR": t, "RPT": r})
        for b, t, r in _GATHER_VARIANTS
    ]
    cfgs.append(LaunchConfig("gather_rows_b32_b256_t64_r2", 256, meta={"BLOCK": 256, "TPR": 64, "RPT": 2, "ELEM": 4}))
    return CachingLauncher("gather_rows", codecache.aot_source("copy_kernels.hip"), "PPPiii", cfgs, prefer_intree=True)


@functools.lru_cache(maxsize=None)
def _permute_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(
            f"permute_copy_b16_b{b}_p{p}_t{t1}x{t2}", b, meta={"BLOCK": b, "TPC": p, "T1": t1, "T2": t2}
        )
        for b, p, t1, t2 in _PERMUTE_VARIANTS
    ]
    cfgs.append(
        LaunchConfig("permute_copy_b32_b256_p16_t8x8", 256, meta={"BLOCK": 256, "TPC": 16, "T1": 8, "T2": 8, "ELEM": 4})
    )
    return CachingLauncher(
        "permute_copy", codecache.aot_source("copy_kernels.hip"), "PPiiiiqqq", cfgs, prefer_intree=True
    )


@functools.lru_cache(maxsize=None)
def _copy_launcher() -> CachingLauncher:
    return CachingLauncher(
        "copy_b128", codecache.aot_source("copy_kernels.hip"), "PPq", [LaunchConfig("copy_b128", 256)],
        prefer_intree=True,
    )


def copy_bytes(dst: torch.Tensor, src: torch.Tensor) -> None:
    """dst <- src for two contiguous tensors of equal byte size (a multiple of
    16).  A known-size streaming kernel: the probe that calibrates HBM byte
    counters when profiling."""
    _check_cuda(dst, src)
    nbytes = src.numel() * src.element_size()
    _require(dst.numel() * dst.element_size() == nbytes, "size mismatch")
    _require(nbytes % 16 == 0 and dst.is_contiguous() and src.is_contiguous(), "contiguous, multiple of 16 bytes")
    _require(_aligned(dst) and _aligned(src), "16-byte alignment")
    if nbytes == 0:
        return
    n_vec = nbytes // 16
    l = _copy_launcher()
    l.precompile()
    l._launch(0, (src.data_ptr(), dst.data_ptr(), n_vec), (cdiv(n_vec, 256), 1, 1), _stream())


def _find(l: CachingLauncher, symbol: str) -> int:
    index = l.__dict__.get("_symbol_index")
    if index is None:
        l.precompile()
        index = {cfg.symbol: i for i, (cfg, _) in enumerate(l.launchers)}
        l.__dict__["_symbol_index"] = index
    try:
        return index[symbol]
    except KeyError:
        raise KeyError(f"{l.name}: no variant {symbol}") from None


# ---------------------------------------------------------------------------
# graph 1: y = sum(relu(2x+1) * sigmoid(x), -1), fp32
# ---------------------------------------------------------------------------
def fused_relu_sigmoid_rowsum(x: torch.Tensor, variant: Optional[tuple] = None) -> torch.Tensor:
    _check_cuda(x)
    _require(x.dtype == torch.float32 and x.dim() >= 1, "x must be fp32 with at least one dim")
    _require(x.is_contiguous(), "x must be contiguous")
    rnumel = x.shape[-1]
    xnumel = x.numel() // max(rnumel, 1) if rnumel else 0
    out = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    if xnumel == 0:
        return out
    if rnumel == 0:
        return out.zero_()
    _require(rnumel % 4 == 0 and _aligned(x), "row length must be a multiple of 4 and x 16-byte aligned")
    _require(x.numel() < 2**31, "numel must fit int32 indexing")
    l = _rowsum_launcher()
    args = (x.data_ptr(), out.data_ptr(), xnumel, rnumel)
    if variant is None:
        plan = row_reduction_plan(xnumel, rnumel, 4, persistent=False)
        b, t = plan.block, max(plan.tpr, 64)  # instantiated shapes start at one wavefront per row
        idx = _find(l, f"fused_relu_sigmoid_rowsum_f32_b{b}_t{t}")
        # every instantiated shape loops over any row length: all are candidates when tuning
        if config.autotune:
            idx = l.pick(f"{xnumel}x{rnumel}", idx, range(len(l.launchers)), args, row_grid(xnumel), _stream())
    else:
        b, t = variant
        idx = _find(l, f"fused_relu_sigmoid_rowsum_f32_b{b}_t{t}")
    l._launch(idx, args, (cdiv(xnumel, l.launchers[idx][0].meta["PER_WG0"]), 1, 1), _stream())
    return out


# ---------------------------------------------------------------------------
# graph 2: s = h + r; out = s * rsqrt(mean(s^2, -1) + eps) * w   (bf16)
# ---------------------------------------------------------------------------
def add_rmsnorm(
    h: torch.Tensor, r: torch.Tensor, w: torch.Tensor, eps: float = 1e-6, variant: Optional[tuple] = None
) -> tuple[torch.Tensor, torch.Tensor]:
    """Returns (normed, h + r), both bf16."""
    _check_cuda(h, r, w)
    _require(h.dtype == r.dtype == w.dtype == torch.bfloat16, "h, r, w must be bf16")
    _require(h.shape == r.shape and h.dim() >= 1, "h and r must have the same shape")
    cols = h.shape[-1]
    _require(w.shape == (cols,), "w must be a vector of the row length")
    _require(h.is_contiguous() and r.is_contiguous() and w.is_contiguous(), "operands must be contiguous")
    rows = h.numel() // max(cols, 1) if cols else 0
    out = torch.empty_like(h)
    s = torch.empty_like(h)
    if rows == 0 or cols == 0:
        return out, s
    _require(cols % 8 == 0, "row length must be a multiple of 8")
    _require(all(_aligned(t) for t in (h, r, w, out, s)), "operands must be 16-byte aligned")
    l = _rmsnorm_launcher()
    if variant is None:
        plan = row_reduction_plan(rows, cols, 2, persistent=True)
        tpr = max(plan.tpr, 64)  # instantiated shapes start at one wavefront per row
        iters = next_power_of_2(cdiv(cdiv(cols, 8), tpr))
        variant = (max(256, tpr), tpr, iters)
        have = set(_RMSNORM_VARIANTS)
        while variant not in have and variant[2] < 8:
            variant = (variant[0], variant[1], variant[2] * 2)
        _require(variant in have, f"row length {cols} exceeds the persistent kernel's reach")
        tuned = True
    else:
        tuned = False
    b, t, i = variant
    _require(cols <= t * 8 * i, "variant too small for the row length")
    idx = _find(l, f"add_rmsnorm_bf16_b{b}_t{t}_i{i}")
    args = (h.data_ptr(), r.data_ptr(), w.data_ptr(), out.data_ptr(), s.data_ptr(), rows, cols, float(eps))
    if tuned and config.autotune:
        # candidates when tuning: the register-resident shapes that hold a whole row
        fits = [k for k, (cfg, _) in enumerate(l.launchers) if cols <= cfg.meta["TPR"] * 8 * cfg.meta["ITERS"]]
        idx = l.pick(f"{rows}x{cols}", idx, fits, args, row_grid(rows), _stream())
    l._launch(idx, args, (cdiv(rows, l.launchers[idx][0].meta["PER_WG0"]), 1, 1), _stream())
    return out, s


def _snap_split_plan(plan: SplitPlan, rows: int, cols: int) -> SplitPlan:
    """Map a heuristic plan onto the nearest instantiated partial-kernel shape
    (threads beyond the matrix edge idle, so a wider shape is always valid)."""
    if (plan.ct, plan.rl, plan.unroll) in set(_COL_PARTIAL_VARIANTS):
        return plan
    avail_ct = sorted({v[0] for v in _COL_PARTIAL_VARIANTS})
    ct = next((c for c in avail_ct if c >= plan.ct), avail_ct[-1])
    cands = [v for v in _COL_PARTIAL_VARIANTS if v[0] == ct]
    _, rl, u = min(cands, key=lambda v: (abs(v[1] - plan.rl), abs(v[2] - plan.unroll)))
    batch = rl * u
    rps = cdiv(max(plan.rows_per_split, 1), batch) * batch
    return SplitPlan(ct, rl, u, cdiv(rows, rps), rps, cdiv(cols, ct * 4))



# ---------------------------------------------------------------------------
# graph 3: per-column mean, var, argmax over dim 0 (fp32 matrix)
# ---------------------------------------------------------------------------
def col_mean_var_argmax(
    x: torch.Tensor,
    correction: float = 0.0,
    plan: Optional[SplitPlan] = None,
    final_variant: Optional[tuple] = None,
    workspace=None,
    out: Optional[tuple] = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (mean, var, argmax) over dim 0 of a [rows, cols] fp32 matrix.

    workspace: a fp32 tensor for the per-split partials (allocated when None), or the string
    "library": both kernels then run on the launcher library's fixed per-GPU scratch array
    (mi_launch_packed_scratch), and with `out=(mean, var, argmax)` given the call allocates no
    device memory at all.  Calls on the library scratch must not overlap on one GPU."""
    _check_cuda(x)
    _require(x.dtype == torch.float32 and x.dim() == 2, "x must be a 2-D fp32 matrix")
    _require(x.is_contiguous(), "x must be contiguous")
    rows, cols = x.shape
    _require(rows > 0, "argmax over an empty axis is undefined")
    if out is not None:
        mean, var, arg = out
        _check_cuda(x, mean, var, arg)
        _require(mean.dtype == var.dtype == torch.float32 and arg.dtype == torch.int64, "out must be (fp32, fp32, int64)")
        _require(mean.shape == var.shape == arg.shape == (cols,), "out tensors must have one element per column")
        _require(mean.is_contiguous() and var.is_contiguous() and arg.is_contiguous(), "out tensors must be contiguous")
    else:
        mean = torch.empty(cols, dtype=torch.float32, device=x.device)
        var = torch.empty(cols, dtype=torch.float32, device=x.device)
        arg = torch.empty(cols, dtype=torch.int64, device=x.device)
    if cols == 0:
        return mean, var, arg
    _require(cols % 4 == 0 and _aligned(x), "cols must be a multiple of 4 and x 16-byte aligned")
    _require(x.numel() < 2**31, "numel must fit int32 indexing")
    if plan is None:
        plan = _snap_split_plan(split_reduction_plan(rows, cols, 4), rows, cols)
    _require(plan.rows_per_split * plan.nsplit >= rows, "split plan does not cover all rows")
    _require(plan.col_tiles * plan.ct * 4 >= cols, "split plan does not cover all columns")
    need = plan.workspace_floats(cols)
    lp, lf = _col_partial_launcher(), _col_final_launcher()
    pf = "" if plan.prefetch == 2 else f"_p{plan.prefetch}"
    ip = _find(lp, f"col_mean_var_argmax_partial_f32_c{plan.ct}_r{plan.rl}_u{plan.unroll}{pf}")
    if final_variant is None:
        # few columns per workgroup so that the second pass has hundreds of workgroups, and as many
        # split lanes as there are splits up to 16 (measured at 512 columns x 64 splits: (4, 16) 25.3 us
        # for both passes, (16, 16) 25.6, (16, 32) 26.1, (64, 4) 28.1)
        final_variant = (4, 16) if cols >= 256 else (8, 8)
    cpw, sl = final_variant
    jf = _find(lf, f"col_mean_var_argmax_final_f32_c{cpw}_s{sl}")
    st = _stream()
    if isinstance(workspace, str):
        _require(workspace == "library", "workspace must be a tensor, None or 'library'")
        # every partial word the second kernel reads is written by the first: nothing to clear
        lp._launch_on_library_scratch(
            ip, (x.data_ptr(), 0, rows, cols, plan.nsplit), 1, need * 4, (plan.col_tiles, plan.nsplit, 1), st
        )
        lf._launch_on_library_scratch(
            jf, (0, mean.data_ptr(), var.data_ptr(), arg.data_ptr(), cols, plan.nsplit, rows, plan.rl * plan.unroll,
                 float(correction)), 0,
            need * 4, (cdiv(cols, cpw), 1, 1), st,
        )
        return mean, var, arg
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.float32, device=x.device)
    _require(workspace.numel() >= need and workspace.dtype == torch.float32, "workspace too small")
    lp._launch(
        ip,
        (x.data_ptr(), workspace.data_ptr(), rows, cols, plan.nsplit),
        (plan.col_tiles, plan.nsplit, 1),
        st,
    )
    lf._launch(
        jf,
        (workspace.data_ptr(), mean.data_ptr(), var.data_ptr(), arg.data_ptr(), cols, plan.nsplit, rows,
         plan.rl * plan.unroll, float(correction)),
        (cdiv(cols, cpw), 1, 1),
        st,
    )
    return mean, var, arg


# ---------------------------------------------------------------------------
# graph 4a: out = table[idx]
# ---------------------------------------------------------------------------
def gather_rows(table: torch.Tensor, idx: torch.Tensor, variant: Optional[tuple] = None) -> torch.Tensor:
    _check_cuda(table, idx)
    _require(table.dim() == 2 and table.is_contiguous(), "table must be a contiguous matrix")
    _require(idx.dtype == torch.int64 and idx.is_contiguous(), "idx must be contiguous int64")
    _require(table.element_size() in (2, 4), "gather kernels exist for 2- and 4-byte elements")
    nrows, width = table.shape
    out = torch.empty(idx.shape + (width,), dtype=table.dtype, device=table.device)
    n = idx.numel()
    if n == 0 or width == 0:
        return out
    _require(nrows > 0, "cannot gather from an empty table")
    vec = 16 // table.element_size()
    _require(width % vec == 0 and _aligned(table) and _aligned(out), "row bytes must be a multiple of 16")
    _require(out.numel() < 2**31, "numel must fit int32 indexing")
    l = _gather_launcher()
    if table.element_size() == 4:
        sym, (b, t, r) = "gather_rows_b32_b256_t64_r2", (256, 64, 2)
    else:
        if variant is None:
            t = min(max(next_power_of_2(width // vec), 16), 128)
            t = 128 if t > 64 else (64 if t > 16 else 16)
            variant = (256, t, 2 if t >= 64 else 4)
        b, t, r = variant
        sym = f"gather_rows_b16_b{b}_t{t}_r{r}"
    i = _find(l, sym)
    rows_per_wg = (b // t) * r
    l._launch(i, (table.data_ptr(), idx.data_ptr(), out.data_ptr(), n, width, nrows), (cdiv(n, rows_per_wg), 1, 1), _stream())
    return out


# ---------------------------------------------------------------------------
# graph 4b: t.permute(0, 2, 1, 3).contiguous()
# ---------------------------------------------------------------------------
def permute_0213_contiguous(t: torch.Tensor, variant: Optional[tuple] = None) -> torch.Tensor:
    """Contiguous copy of t.permute(0, 2, 1, 3) for a contiguous 4-D tensor."""
    _check_cuda(t)
    _require(t.dim() == 4 and t.is_contiguous(), "t must be a contiguous 4-D tensor")
    _require(t.element_size() in (2, 4), "permute kernels exist for 2- and 4-byte elements")
    n0, n2, n1, inner = t.shape  # output dims are (n0, n1, n2, inner)
    out = torch.empty((n0, n1, n2, inner), dtype=t.dtype, device=t.device)
    if out.numel() == 0:
        return out
    vec = 16 // t.element_size()
    _require(inner % vec == 0 and _aligned(t) and _aligned(out), "inner run must be a multiple of 16 bytes")
    _require(out.numel() < 2**31, "numel must fit int32 indexing")
    s0, s2, s1, _ = t.stride()  # input strides of output axes a, b, c
    l = _permute_launcher()
    if t.element_size() == 4:
        sym, (b, p, t1, t2) = "permute_copy_b32_b256_p16_t8x8", (256, 16, 8, 8)
        _require(inner // vec <= 16, "inner run too long for the fp32 permute variant")
    else:
        if variant is None:
            # 8 x 2 rows of the two swapped axes per workgroup: one 16-byte vector per thread.  Measured
            # on MI355X at [16,2048,32,128] bf16, one input replayed / four inputs in turn: 76.6 / 86.9 us
            # against 78.3 / 95.9 us for 32 x 4 and 76.1 / 90.0 us for 4 x 8.
            variant = (256, 16, 8, 2)
        b, p, t1, t2 = variant
        _require(inner // vec <= p, "inner run too long for this permute variant")
        sym = f"permute_copy_b16_b{b}_p{p}_t{t1}x{t2}"
    i = _find(l, sym)
    tiles = n0 * cdiv(n1, t1) * cdiv(n2, t2)
    l._launch(i, (t.data_ptr(), out.data_ptr(), n0, n1, n2, inner, s0, s1, s2), (tiles, 1, 1), _stream())
    return out


# ---------------------------------------------------------------------------
# ring-attention merge step: (prev_out, prev_max, prev_sum) + (cur_out, cur_max, cur_sum)
# ---------------------------------------------------------------------------
_RING_DTYPES = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}
_RING_VARIANTS = [("bf16", 128, 8), ("bf16", 128, 16), ("f16", 128, 8), ("f32", 128, 8), ("bf16", 64, 8), ("f16", 64, 8), ("f32", 64, 8)]


@functools.lru_cache(maxsize=None)
def _ring_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(f"ring_forward_update_{t}_d{d}_s{st}{'_nt' if nt else ''}", 256,
                     meta={"DTYPE": t, "D": d, "ST": st, "STREAM": nt})
        for t, d, st in _RING_VARIANTS for nt in (0, 1)
    ]
    return CachingLauncher(
        "ring_forward_update", codecache.aot_source("ring_kernels.hip"), "PPPPPPPPPiiiqq", cfgs, prefer_intree=True
    )


def ring_forward_update(
    prev_attn_out: torch.Tensor, prev_softmax_max: torch.Tensor, prev_softmax_sum: torch.Tensor,
    cur_attn_out: torch.Tensor, cur_softmax_max: torch.Tensor, cur_softmax_sum: torch.Tensor,
    variant: Optional[tuple] = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """One merge step of ring attention in a single kernel: returns (attn_out, softmax_max,
    softmax_sum) of the union of the two key sets.  Attention outputs are [S, B, H] (bf16, fp16 or
    fp32, H = N * D with D 64 or 128), statistics fp32 [B, N, S, 8] whose head stride may differ
    between the two steps (a slice of a larger buffer); the returned statistics take the current
    step's strides.  Argument order, layouts and result as the reference's hand-written
    forward_update_triton (reference test/npu_indexing/written/attn_cp_triton_kernel_3d.py:88-139).
    variant = (ST, streaming loads) overrides the launch choice."""
    stats = (prev_softmax_max, prev_softmax_sum, cur_softmax_max, cur_softmax_sum)
    _check_cuda(prev_attn_out, cur_attn_out, *stats)
    _require(prev_attn_out.dtype == cur_attn_out.dtype and prev_attn_out.dtype in _RING_DTYPES,
             "attention outputs must share one of bf16, fp16, fp32")
    _require(prev_attn_out.dim() == 3 and prev_attn_out.shape == cur_attn_out.shape, "attention outputs must share an [S, B, H] shape")
    _require(prev_attn_out.is_contiguous() and cur_attn_out.is_contiguous(), "attention outputs must be contiguous")
    S, B, H = cur_attn_out.shape
    for t in stats:
        _require(t.dtype == torch.float32 and t.dim() == 4 and t.shape == cur_softmax_max.shape, "statistics must share a fp32 [B, N, S, 8] shape")
    _require(cur_softmax_max.shape[0] == B and cur_softmax_max.shape[2] == S and cur_softmax_max.shape[3] == 8,
             "statistics must be [B, N, S, 8] for [S, B, H] outputs")
    N = cur_softmax_max.shape[1]
    _require(N > 0 and H % N == 0, "H must be a multiple of the head count")
    D = H // N
    _require(prev_softmax_max.stride() == prev_softmax_sum.stride() and cur_softmax_max.stride() == cur_softmax_sum.stride(),
             "maximum and sum of one step must share their strides")
    for t in (prev_softmax_max, cur_softmax_max):
        _require(t.stride(3) == 1 and t.stride(2) == 8, "statistics must be contiguous along their last two axes")
        _require(B == 1 or t.stride(0) == N * t.stride(1), "the batch stride must be N head strides (no slice along N)")
        _require(t.stride(1) % 4 == 0, "the head stride must be a multiple of 16 bytes")
    out = torch.empty_like(cur_attn_out)
    smax = torch.empty_strided(cur_softmax_max.shape, cur_softmax_max.stride(), dtype=torch.float32, device=cur_attn_out.device)
    ssum = torch.empty_strided(cur_softmax_sum.shape, cur_softmax_sum.stride(), dtype=torch.float32, device=cur_attn_out.device)
    if S * B * H == 0:
        return out, smax, ssum
    _require(all(_aligned(t) for t in (prev_attn_out, cur_attn_out, out, smax, ssum) + stats), "operands must be 16-byte aligned")
    _require(out.numel() < 2**31 and B * N < 2**31 // max(S, 1), "extents must fit int32 indexing")
    name = _RING_DTYPES[cur_attn_out.dtype]
    shapes = [(d, st) for t, d, st in _RING_VARIANTS if t == name]
    _require(any(d == D for d, _ in shapes), f"no forward_update kernel for head dimension {D} in {name}")
    if variant is None:
        # eight sequence positions per workgroup, plain loads: measured best at the reference's shape
        # (377 MB per call) also against non-temporal loads (58 us against 65 us replayed)
        variant = (8, False)
    st, stream = variant
    _require((D, st) in shapes, f"no forward_update kernel with {st} sequence positions per workgroup")
    l = _ring_launcher()
    i = _find(l, f"ring_forward_update_{name}_d{D}_s{st}{'_nt' if stream else ''}")
    nt = 256 // (D * out.element_size() // 16)  # heads per workgroup
    l._launch(
        i,
        (prev_attn_out.data_ptr(), prev_softmax_max.data_ptr(), prev_softmax_sum.data_ptr(), cur_attn_out.data_ptr(),
         cur_softmax_max.data_ptr(), cur_softmax_sum.data_ptr(), out.data_ptr(), smax.data_ptr(), ssum.data_ptr(),
         S, B, N, prev_softmax_max.stride(1), cur_softmax_max.stride(1)),
        (cdiv(S, st), cdiv(N, nt), B),
        _stream(),
    )
    return out, smax, ssum


# ---------------------------------------------------------------------------
# graph 5: fused attention forward (bf16 / fp16, head dim 128)
# ---------------------------------------------------------------------------
_ATTN_DTYPES = {torch.bfloat16: "bf16", torch.float16: "f16"}
_ATTN_LDS_BYTES = 4 * 64 * 128 * 2  # two K and two V tiles of [64, 128] 16-bit elements
_ATTN_BLOCK_QUERIES = 256


@functools.lru_cache(maxsize=None)
def _attention_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(
            f"fused_attention_fwd_{t}_d128_{'causal' if c else 'full'}_v5{'_ragged' if r else ''}",
            512,
            meta={"DTYPE": t, "CAUSAL": c, "RAGGED": r, "WAVES": 8},
            lds_bytes=_ATTN_LDS_BYTES,
        )
        for t in ("bf16", "f16")
        for c in (1, 0)
        for r in (0, 1)
    ] + [
        LaunchConfig(
            f"fused_attention_fwd_{t}_d64_{'causal' if c else 'full'}_v5",
            512,
            meta={"DTYPE": t, "CAUSAL": c, "RAGGED": 1, "WAVES": 8, "DATA_COLUMNS": 64},
            lds_bytes=_ATTN_LDS_BYTES,
        )
        for t in ("bf16", "f16")
        for c in (1, 0)
    ]
    return CachingLauncher(
        "fused_attention_fwd_d128",
        codecache.aot_source("attention_kernels.hip"),
        "PPPPPPiiif",
        cfgs,
        prefer_intree=True,
    )


@functools.lru_cache(maxsize=None)
def _attention_masked_launcher() -> CachingLauncher:
    cfgs = [
        LaunchConfig(
            f"fused_attention_fwd_{t}_d128_{'causal' if c else 'full'}_v5_masked",
            512,
            meta={"DTYPE": t, "CAUSAL": c, "RAGGED": 1, "WAVES": 8, "MASKED": 1},
            lds_bytes=_ATTN_LDS_BYTES,
        )
        for t in ("bf16", "f16")
        for c in (1, 0)
    ]
    return CachingLauncher(
        "fused_attention_fwd_d128_masked",
        codecache.aot_source("attention_kernels.hip"),
        "PPPPPPiiifPqqiPii",
        cfgs,
        prefer_intree=True,
    )


def attention_mask_bits(mask: torch.Tensor, B: int, N: int, Sq: int, Sk: int) -> torch.Tensor:
    """A mask given as [Sq, Sk] or as a 4-D tensor that broadcasts to [B, N, Sq, Sk] (any type; non-zero =
    the key is hidden from the query) packed for the masked attention kernel: bytes
    [B or 1, N or 1, Sq, 8 * ceil(Sk / 64)], i.e. one little-endian 64-bit word per query and 64-key tile
    whose bit j is set when key 64 * tile + j is hidden (bits past Sk are clear)."""
    if mask.dim() == 2:
        mask = mask.view(1, 1, *mask.shape)
    _require(mask.dim() == 4 and tuple(mask.shape[2:]) == (Sq, Sk) and mask.shape[0] in (1, B) and mask.shape[1] in (1, N),
             f"mask of shape {tuple(mask.shape)} does not broadcast to [{B}, {N}, {Sq}, {Sk}]")
    hide = mask if mask.dtype == torch.bool else mask != 0
    tiles = cdiv(Sk, 64)
    if tiles * 64 != Sk:
        hide = torch.nn.functional.pad(hide, (0, tiles * 64 - Sk))
    # 1, 2, 4, ... 128 made on the device (no host copy, so the packing can be captured in a HIP graph)
    weights = torch.bitwise_left_shift(torch.ones(8, dtype=torch.uint8, device=mask.device),
                                       torch.arange(8, dtype=torch.uint8, device=mask.device))
    groups = hide.reshape(hide.shape[0], hide.shape[1], Sq, tiles * 8, 8).to(torch.uint8)
    return (groups * weights).sum(-1, dtype=torch.uint8).contiguous()


def attention_mask_tile_ranges(packed: torch.Tensor, Sq: int, Sk: int, causal: bool = False,
                               transposed: bool = False) -> torch.Tensor:
    """For a packed mask (attention_mask_bits) the key tiles each block of 256 queries has to visit: int32
    [B or 1, N or 1, ceil(Sq / 256), 2] holding the first and the last 64-key tile in which some query of the
    block sees a key (under `causal` only tiles up to the block's diagonal count); (0, 0) for a block that sees
    nothing.  The masked kernels leave the tiles outside the range alone, so a sliding window or a block-sparse
    mask costs what it shows.  transposed: `packed` is the packing of the transposed mask (rows = keys, tiles of
    queries, what the dK and dV kernels read), for which `causal` keeps the tiles from the block's diagonal on.
    Device work only (no host copy)."""
    tiles = cdiv(Sk, 64)
    dev = packed.device
    words = packed.view(torch.int64)  # [b, n, Sq, tiles]
    # bits a fully hidden tile has set: all 64, in the last tile only those of existing keys
    full = torch.full((tiles,), -1, dtype=torch.int64, device=dev)
    if Sk % 64:
        full[tiles - 1] = (1 << (Sk % 64)) - 1
    seen = (words & full) != full  # [b, n, Sq, tiles]: the query sees a key of the tile
    blocks = cdiv(Sq, _ATTN_BLOCK_QUERIES)
    if blocks * _ATTN_BLOCK_QUERIES != Sq:
        seen = torch.nn.functional.pad(seen, (0, 0, 0, blocks * _ATTN_BLOCK_QUERIES - Sq))
    seen = seen.view(seen.shape[0], seen.shape[1], blocks, _ATTN_BLOCK_QUERIES, tiles).any(dim=3)  # [b, n, blocks, tiles]
    t = torch.arange(tiles, device=dev)
    if causal and transposed:
        first_visible = (torch.arange(blocks, device=dev) * _ATTN_BLOCK_QUERIES) // 64
        seen = seen & (t.view(1, 1, 1, tiles) >= first_visible.view(1, 1, blocks, 1))
    elif causal:
        last_visible = (torch.arange(blocks, device=dev) * _ATTN_BLOCK_QUERIES + _ATTN_BLOCK_QUERIES - 1) // 64
        seen = seen & (t.view(1, 1, 1, tiles) <= last_visible.view(1, 1, blocks, 1))
    lo = torch.where(seen, t, tiles).amin(dim=-1)
    hi = torch.where(seen, t, -1).amax(dim=-1)
    none = hi < 0
    lo = torch.where(none, 0, lo)
    hi = torch.where(none, 0, hi)
    return torch.stack((lo, hi), dim=-1).to(torch.int32).contiguous()


def fused_attention(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, causal: bool, data_columns: int = 128,
    mask: Optional[torch.Tensor] = None, mask_is_packed: bool = False, tile_ranges: Optional[torch.Tensor] = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """softmax(q k^T * scale [+ causal mask]) v for q [B, N, Sq, 128] and k, v [B, N, Sk, 128], bf16
    or fp16, any positive sequence lengths (a causal mask needs Sq == Sk).

    Returns (out [B,N,Sq,128] in the input type, softmax_max fp32 [B,N,Sq,8], softmax_sum fp32
    [B,N,Sq,8]); the statistics are the row maximum of the scaled scores and the row sum of
    exp(score - max), each repeated over the trailing axis.  Lengths that are multiples of 256
    (queries) and 128 (keys) run the kernel without bounds handling, all others the instantiation
    that masks the ragged end.
    data_columns (128, or at most 64): how many leading columns of the 128-wide heads carry data; the
    caller vouches that the others are zero in q, k and v (a smaller head padded to 128).  With at most 64
    the kernel skips the matrix work on the zero half and leaves columns 64.. of `out` undefined.
    mask ([Sq, Sk] or broadcastable to [B, N, Sq, Sk], any type, non-zero = the key is hidden from the
    query) is applied besides the causal mask (it is packed to one bit per key first; a caller that uses
    one mask many times packs it once with attention_mask_bits and passes mask_is_packed=True, best together with
    tile_ranges=attention_mask_tile_ranges(packed, ...), without which a packed mask visits every key tile); a
    query with every key hidden gets a zero output row, maximum 0 and sum 1."""
    _check_cuda(q, k, v)
    _require(q.dtype == k.dtype == v.dtype and q.dtype in _ATTN_DTYPES, "q, k, v must share bf16 or fp16")
    _require(q.dim() == 4 and k.dim() == 4 and k.shape == v.shape, "q [B, N, Sq, D]; k and v one [B, N, Sk, D] shape")
    B, N, Sq, D = q.shape
    Sk = k.shape[2]
    _require(k.shape[0] == B and k.shape[1] == N and k.shape[3] == D, "q, k, v must share batch, heads and head dimension")
    _require(D == 128, "head dimension must be 128")
    _require(0 < data_columns <= 128, "data_columns must lie in 1..128")
    _require(Sq > 0 and Sk > 0, "sequence lengths must be positive")
    _require(not causal or Sq == Sk, "a causal mask needs equal query and key lengths")
    _require(q.is_contiguous() and k.is_contiguous() and v.is_contiguous(), "q, k, v must be contiguous (BNSD)")
    _require(all(_aligned(t) for t in (q, k, v)), "q, k, v must be 16-byte aligned")
    _require(scale > 0 and math.isfinite(scale), "scale must be positive and finite")
    _require(B * N * max(Sq, Sk) * D < 2**31, "numel must fit int32 indexing")
    out = torch.empty_like(q)
    smax = torch.empty((B, N, Sq, 8), dtype=torch.float32, device=q.device)
    ssum = torch.empty((B, N, Sq, 8), dtype=torch.float32, device=q.device)
    heads = B * N
    if heads == 0:
        return out, smax, ssum
    n_qb = cdiv(Sq, _ATTN_BLOCK_QUERIES)
    per_head = (n_qb + 1) // 2 if causal else n_qb  # causal: query blocks (b, n - 1 - b) are one work item
    items = 8 * cdiv(heads, 8) * per_head
    # persistent launch: at most one workgroup per CU, a multiple of 8 (one per die in turn); every
    # workgroup walks items blockIdx.x, blockIdx.x + gridDim.x, ...
    grid = min(items, max(config.hardware().cu_count // 8, 1) * 8)
    if mask is not None:
        _check_cuda(mask)
        if mask_is_packed:
            mb = mask
            _require(mb.dtype == torch.uint8 and mb.dim() == 4 and mb.is_contiguous() and mb.shape[0] in (1, B)
                     and mb.shape[1] in (1, N) and tuple(mb.shape[2:]) == (Sq, 8 * cdiv(Sk, 64)),
                     "a packed mask is what attention_mask_bits returns for these lengths")
        else:
            mb = attention_mask_bits(mask, B, N, Sq, Sk)
            tile_ranges = attention_mask_tile_ranges(mb, Sq, Sk, causal)
        if tile_ranges is not None:
            _check_cuda(tile_ranges)
            _require(tile_ranges.dtype == torch.int32 and tile_ranges.is_contiguous()
                     and tuple(tile_ranges.shape) == (mb.shape[0], mb.shape[1], cdiv(Sq, _ATTN_BLOCK_QUERIES), 2),
                     "tile_ranges is what attention_mask_tile_ranges returns for this packed mask")
        tr = tile_ranges
        lm = _attention_masked_launcher()
        lm._launch(
            _find(lm, f"fused_attention_fwd_{_ATTN_DTYPES[q.dtype]}_d128_{'causal' if causal else 'full'}_v5_masked"),
            (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), smax.data_ptr(), ssum.data_ptr(), heads, Sq, Sk,
             float(scale) * 1.4426950408889634, mb.data_ptr(), mb.stride(0) if mb.shape[0] > 1 else 0,
             mb.stride(1) if mb.shape[1] > 1 else 0, N, tr.data_ptr() if tr is not None else 0,
             (tr.stride(0) if tr.shape[0] > 1 else 0) if tr is not None else 0,
             (tr.stride(1) if tr.shape[1] > 1 else 0) if tr is not None else 0),
            (grid, 1, 1),
            _stream(),
        )
        return out, smax, ssum
    ragged = Sq % _ATTN_BLOCK_QUERIES != 0 or Sk % 128 != 0
    l = _attention_launcher()
    if data_columns <= 64:
        i = _find(l, f"fused_attention_fwd_{_ATTN_DTYPES[q.dtype]}_d64_{'causal' if causal else 'full'}_v5")
    else:
        i = _find(l, f"fused_attention_fwd_{_ATTN_DTYPES[q.dtype]}_d128_{'causal' if causal else 'full'}_v5"
                     f"{'_ragged' if ragged else ''}")
    l._launch(
        i,
        (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), smax.data_ptr(), ssum.data_ptr(), heads, Sq, Sk,
         float(scale) * 1.4426950408889634),
        (grid, 1, 1),
        _stream(),
    )
    return out, smax, ssum


# ---------------------------------------------------------------------------
# fused attention backward (bf16, head dim 128): row statistics, then dQ, dK and dV kernels
# ---------------------------------------------------------------------------
# two buffers of two [64][128] tiles as they lie in memory (dQ: K, V; dK and dV: Q, dO, with the 64 (offset, D)
# pairs of the query tile behind them); the row staging of the result at the end uses the first 64 KiB
_ATTN_BWD8_DQ_LDS = 2 * (2 * 64 * 128 * 2)
_ATTN_BWD8_DK_LDS = 2 * (2 * 64 * 128 * 2 + 64 * 2 * 4)
_ATTN_BWD8_DV_LDS = 2 * (2 * 64 * 128 * 2 + 64 * 2 * 4)


@functools.lru_cache(maxsize=None)
def _attention_bwd_launchers() -> dict:
    src = codecache.aot_source("attention_bwd_kernels.hip")
    mk = lambda name, sig, cfgs: CachingLauncher(name, src, sig, cfgs, prefer_intree=True)  # noqa: E731
    types = tuple(_ATTN_DTYPES.values())
    return {
        "stats": mk("attention_bwd_stats_d128", "PPPPPi", [LaunchConfig(f"attention_bwd_stats_{t}_d128", 256) for t in types]),
        **{
            which: mk(
                f"attention_bwd8_{which[:2]}_d128", "PPPPPPiif",
                [LaunchConfig(f"attention_bwd8_{which[:2]}_{t}_d{d}_{c}", 512, meta={"CAUSAL": c == "causal", "DATA_COLUMNS": d},
                              lds_bytes=lds)
                 for t in types for d in (128, 64) for c in ("causal", "full")],
            )
            for which, lds in (("dq8", _ATTN_BWD8_DQ_LDS), ("dk8", _ATTN_BWD8_DK_LDS), ("dv8", _ATTN_BWD8_DV_LDS))
        },
    }


@functools.lru_cache(maxsize=None)
def _attention_bwd_masked_launchers() -> dict:
    src = codecache.aot_source("attention_bwd_kernels.hip")
    return {
        which: CachingLauncher(
            f"attention_bwd8_{which[:2]}_d128_masked", src, "PPPPPPiifPqqiPii",
            [LaunchConfig(f"attention_bwd8_{which[:2]}_{t}_d128_{c}_masked", 512, meta={"CAUSAL": c == "causal", "MASKED": 1},
                          lds_bytes=lds)
             for t in _ATTN_DTYPES.values() for c in ("causal", "full")],
            prefer_intree=True,
        )
        for which, lds in (("dq8", _ATTN_BWD8_DQ_LDS), ("dk8", _ATTN_BWD8_DK_LDS), ("dv8", _ATTN_BWD8_DV_LDS))
    }


def fused_attention_backward(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, dout: torch.Tensor,
    softmax_max: torch.Tensor, softmax_sum: torch.Tensor, scale: float, causal: bool, data_columns: int = 128,
    mask: Optional[torch.Tensor] = None, packed_masks: Optional[tuple] = None, tile_ranges: Optional[tuple] = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gradients (dq, dk, dv) of fused_attention for [B, N, S, 128] bf16 or fp16 tensors; softmax_max /
    softmax_sum are the forward's [B, N, S, 8] fp32 statistics.  Workgroups of eight wavefronts on
    256 rows, a statistics pass and separate dQ, dK and dV kernels; S a positive multiple of 64.
    data_columns (128, or at most 64): how many leading columns of the 128-wide heads carry data, the
    others being zero in q, k, v, out and dout (a smaller head padded to 128): with at most 64 the
    kernels skip the matrix work on the zero half and leave columns 64.. of the gradients undefined.
    mask: the forward's mask ([S, S] or broadcastable to [B, N, S, S], non-zero = hidden); it is packed to
    bits, once as it stands for dQ and once transposed for dK and dV.  packed_masks: those two packings
    (attention_mask_bits of the mask and of its transpose), for a caller that holds them already; tile_ranges:
    attention_mask_tile_ranges of the two (the second with transposed=True), computed here when a mask is
    given unpacked; without them packed masks visit every tile."""
    _check_cuda(q, k, v, out, dout, softmax_max, softmax_sum)
    for t in (q, k, v, out, dout):
        _require(t.dtype == q.dtype and t.dtype in _ATTN_DTYPES and t.dim() == 4 and t.shape == q.shape,
                 "q, k, v, out, dout: one [B, N, S, D] shape in bf16 or fp16")
        _require(t.is_contiguous() and _aligned(t), "q, k, v, out, dout must be contiguous and 16-byte aligned")
    B, N, S, D = q.shape
    _require(D == 128, "head dimension must be 128")
    _require(S % 64 == 0 and S > 0, "sequence length must be a positive multiple of 64")
    for t in (softmax_max, softmax_sum):
        _require(t.dtype == torch.float32 and t.shape == (B, N, S, 8) and t.is_contiguous(), "statistics must be contiguous fp32 [B, N, S, 8]")
    _require(scale > 0 and math.isfinite(scale), "scale must be positive and finite")
    _require(B * N * S * D < 2**31, "numel must fit int32 indexing")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    heads = B * N
    if heads == 0:
        return dq, dk, dv
    ls = _attention_bwd_launchers()
    st = _stream()
    which = "causal" if causal else "full"
    stats = torch.empty(heads * S, 2, dtype=torch.float32, device=q.device)
    ty = _ATTN_DTYPES[q.dtype]
    _require(0 < data_columns <= 128, "data_columns must lie in 1..128")
    dcols = 64 if data_columns <= 64 else 128
    ls["stats"]._launch(
        _find(ls["stats"], f"attention_bwd_stats_{ty}_d128"),
        (out.data_ptr(), dout.data_ptr(), softmax_max.data_ptr(), softmax_sum.data_ptr(), stats.data_ptr(), heads * S),
        (cdiv(heads * S * 16, 256), 1, 1), st,
    )
    blocks = cdiv(S, 256)
    grid = (8 * cdiv(heads, 8) * (cdiv(blocks, 2) if causal else blocks), 1, 1)  # causal: pairs of blocks
    if mask is not None or packed_masks is not None:
        if packed_masks is not None:
            rows, cols = packed_masks
            for w in (rows, cols):
                _check_cuda(w)
                _require(w.dtype == torch.uint8 and w.dim() == 4 and w.is_contiguous() and w.shape[0] in (1, B)
                         and w.shape[1] in (1, N) and tuple(w.shape[2:]) == (S, S // 8),
                         "packed masks are what attention_mask_bits returns for this length")
        else:
            _check_cuda(mask)
            m4 = mask.view(1, 1, *mask.shape) if mask.dim() == 2 else mask
            rows = attention_mask_bits(m4, B, N, S, S)                     # [.., query, key tiles]
            cols = attention_mask_bits(m4.transpose(-1, -2), B, N, S, S)   # [.., key, query tiles]
            tile_ranges = (attention_mask_tile_ranges(rows, S, S, causal),
                           attention_mask_tile_ranges(cols, S, S, causal, transposed=True))
        if tile_ranges is not None:
            for r, w in zip(tile_ranges, (rows, cols)):
                _check_cuda(r)
                _require(r.dtype == torch.int32 and r.is_contiguous() and tuple(r.shape) == (w.shape[0], w.shape[1], cdiv(S, 256), 2),
                         "tile_ranges are what attention_mask_tile_ranges returns for the two packed masks")
        rr, rc = tile_ranges if tile_ranges is not None else (None, None)
        lm = _attention_bwd_masked_launchers()
        for name, dst, words, tr in (("dk8", dk, cols, rc), ("dv8", dv, cols, rc), ("dq8", dq, rows, rr)):
            l = lm[name]
            l._launch(
                _find(l, f"attention_bwd8_{name[:2]}_{ty}_d128_{which}_masked"),
                (q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), stats.data_ptr(), dst.data_ptr(), heads, S,
                 float(scale), words.data_ptr(), words.stride(0) if words.shape[0] > 1 else 0,
                 words.stride(1) if words.shape[1] > 1 else 0, N, tr.data_ptr() if tr is not None else 0,
                 (tr.stride(0) if tr.shape[0] > 1 else 0) if tr is not None else 0,
                 (tr.stride(1) if tr.shape[1] > 1 else 0) if tr is not None else 0),
                grid, st,
            )
        return dq, dk, dv
    for name, dst in (("dk8", dk), ("dv8", dv), ("dq8", dq)):
        l = ls[name]
        l._launch(
            _find(l, f"attention_bwd8_{name[:2]}_{ty}_d{dcols}_{which}"),
            (q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), stats.data_ptr(), dst.data_ptr(), heads, S, float(scale)),
            grid, st,
        )
    return dq, dk, dv
