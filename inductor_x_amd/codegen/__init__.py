"""Code generation for the MI355X backend.

Importing this package installs the few patches of Inductor internals the
backend needs, in the spirit of the reference's codegen/__init__.py
(reference inductor_x/codegen/__init__.py:23-37); most of what the reference
monkey-patches (tiling choice, index dtype, grouping) is done here by
subclassing instead.
"""
from .ir import install_num_splits_stub  # noqa: F401
