"""IR-level adjustments.

The reference replaces Reduction.num_splits by a stub returning (DEFAULT, 1) so
that Inductor never splits a reduction into two IR nodes
(reference inductor_x/codegen/ir.py:13-24, installed at
reference inductor_x/codegen/__init__.py:23); cutting a long reduced axis is left
to the kernel.  Here the replacement does the same for most reductions (scans keep
Inductor's behaviour), with one exception the reference does not make: a reduction
with fewer outputs than the GPU has compute units over a long range keeps
Inductor's two-stage split (whether the range is contiguous or strided), because a
single kernel would occupy a handful of workgroups.  It only acts for GPU devices, so CPU compilation in the same process
is untouched.
"""
from __future__ import annotations

from torch._inductor.ir import Reduction, ReductionHint

_installed = False


def num_splits(device, dst_dtype, src_dtype, inner_fn, ranges, reduction_ranges, reduction_type, reduction_numel,
               input_node=None):
    if device is not None and getattr(device, "type", None) in _DEVICE_TYPES and reduction_type != "scan":
        if not _few_long_rows(ranges, reduction_numel):
            return ReductionHint.DEFAULT, 1
        hint, split = _original_num_splits(
            device, dst_dtype, src_dtype, inner_fn, ranges, reduction_ranges, reduction_type, reduction_numel, input_node
        )
        # contiguous rows and strided ones alike: a strided range whose values are used again
        # after the reduction (batch statistics of a channels-last tensor) becomes one
        # column-loop kernel, which does not cut the range across workgroups
        if __import__("os").environ.get("INDUCTOR_X_AMD_SPLIT_OUTER", "1") == "0" and hint != ReductionHint.INNER:
            return ReductionHint.DEFAULT, 1
        return hint, split
    return _original_num_splits(
        device, dst_dtype, src_dtype, inner_fn, ranges, reduction_ranges, reduction_type, reduction_numel, input_node
    )


_original_num_splits = Reduction.num_splits
# the dry-run mode of the code generator (no GPU, kernels registered for the cpu device) takes
# the same decisions
_DEVICE_TYPES = ("cuda", "cpu") if __import__("os").environ.get("INDUCTOR_X_AMD_DRYRUN") == "1" else ("cuda",)

# A reduction with fewer outputs than the GPU has compute units, each over a long range, would
# run on a handful of workgroups: those keep Inductor's two-stage split (partials per slice of the
# range, then a short second reduction), both stages being ordinary kernels of this backend.
_FEW_OUTPUTS = 256
_LONG_RANGE = 1 << 16


def _few_long_rows(ranges, reduction_numel) -> bool:
    import os

    if os.environ.get("INDUCTOR_X_AMD_SPLIT_REDUCTIONS", "1") == "0":
        return False
    try:
        outputs = 1
        for r in ranges:
            outputs *= int(r)
        return outputs < _FEW_OUTPUTS and int(reduction_numel) >= _LONG_RANGE
    except (TypeError, ValueError):
        return False


def install_num_splits_stub() -> None:
    global _installed
    if not _installed:
        Reduction.num_splits = staticmethod(num_splits)
        _installed = True
