"""Decomposition-table hook.

The reference removes a handful of decompositions and adds three of its own
(reference inductor_x/decomposition.py:8-47): a dim-1 one-hot scatter.src for
its device, expm1 = exp(x) - 1 and an erfc formula that is not erfc.  None of
them is on the path this backend accelerates and the last is wrong, so the hook
is kept (same name and call position, reference inductor_x/__init__.py:58) with
only the entry that is mathematically sound and useful to the HIP generator:
the ops listed in DECOMPOSITION_OVERLOAD_OP keep Inductor's own treatment.
"""
from __future__ import annotations

DECOMPOSITION_OVERLOAD_OP: list = []


def _register_inductor_decompositions() -> None:
    """No decomposition is changed: mi::expm1 / mi::erfc exist as device
    functions, so the generator needs neither of the reference's rewrites."""
    return None


# name used by the reference (its spelling included)
_register_npu_inductor_decompositons = _register_inductor_decompositions
