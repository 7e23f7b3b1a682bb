"""IR-level adjustments.

The reference replaces Reduction.num_splits by a stub returning (DEFAULT, 1) so
that Inductor never splits a reduction into two IR nodes
(reference inductor_x/codegen/ir.py:13-24, installed at
reference inductor_x/codegen/__init__.py:23); cutting a long reduced axis is left
to the kernel.  Here the backend declares BackendFeature.REDUCE_TO_SINGLE_ELEMENT
for the same effect on most reductions, and this stub covers what the feature
flag does not (scans keep Inductor's behaviour).  It only acts for GPU devices,
so CPU compilation in the same process is untouched.
"""
from __future__ import annotations

from torch._inductor.ir import Reduction, ReductionHint

_installed = False


def num_splits(device, dst_dtype, src_dtype, inner_fn, ranges, reduction_ranges, reduction_type, reduction_numel,
               input_node=None):
    if device is not None and getattr(device, "type", None) == "cuda" and reduction_type != "scan":
        return ReductionHint.DEFAULT, 1
    return _original_num_splits(
        device, dst_dtype, src_dtype, inner_fn, ranges, reduction_ranges, reduction_type, reduction_numel, input_node
    )


_original_num_splits = Reduction.num_splits


def install_num_splits_stub() -> None:
    global _installed
    if not _installed:
        Reduction.num_splits = staticmethod(num_splits)
        _installed = True
