"""Wrapper (host-side call sequence) code generation.

Counterpart of the reference's NPUWrapperCodeGen
(reference inductor_x/codegen/wrapper.py:3-47).  The generated module imports
the kernel factory and the raw-stream getter of this package.  Unlike the
reference, buffers are freed as soon as Inductor says they are dead and input
size asserts stay on: the reference disables both to work around problems of
its own generator.
"""
from __future__ import annotations

from torch._inductor.codegen.wrapper import PythonWrapperCodegen
from torch._inductor.virtualized import V


class HipWrapperCodegen(PythonWrapperCodegen):
    @staticmethod
    def create(is_subgraph, subgraph_name, parent_wrapper, partition_signatures=None):
        if is_subgraph:
            return PythonWrapperCodegen.create(is_subgraph, subgraph_name, parent_wrapper, partition_signatures)
        return HipWrapperCodegen()

    def write_header(self) -> None:
        super().write_header()
        self.header.splice(
            """
            from inductor_x_amd.hip_heuristics import generated_kernel, grid
            """
        )
        self._inductor_x_amd_header = True
