"""Scheduling backend: fused Inductor nodes -> generated HIP kernels.

Counterpart of the reference's NPUTritonScheduling
(reference inductor_x/codegen/schduling.py:17-163).  Fusion decisions, node
ordering and reduction-loop placement come from Inductor's SIMD scheduling;
this class supplies the kernel type, disables 2-D pointwise tiling (the
reference does the same: select_tiling -> (numel, rnumel),
reference inductor_x/codegen/triton.py:175-177), retries a kernel with scalar
accesses when a late index does not fit the chosen vector width, and writes the
kernel definition into the generated wrapper.
"""
from __future__ import annotations

import logging
from typing import Any, Optional

import sympy

import torch
from torch._inductor.codegen.common import BackendFeature
from torch._inductor.codegen.simd import SIMDScheduling
from torch._inductor.codegen.simd_kernel_features import SIMDKernelFeatures
from torch._inductor.utils import get_kernel_metadata
from torch._inductor.virtualized import V
from torch.utils._ordered_set import OrderedSet

from .hip_kernel import HipKernel, UnsupportedHipCodegen, VecConstraintError

log = logging.getLogger(__name__)

KERNEL_PLACEHOLDER = "KERNEL_NAME"


class HipScheduling(SIMDScheduling):
    kernel_type = HipKernel  # type: ignore[assignment]

    def __init__(self, scheduler: Optional[Any]) -> None:
        super().__init__(scheduler)
        wrapper = V.graph.wrapper_code
        if wrapper is not None and not getattr(wrapper, "_inductor_x_amd_header", False):
            wrapper.header.splice("from inductor_x_amd.hip_heuristics import generated_kernel")
            wrapper._inductor_x_amd_header = True

    @classmethod
    def get_backend_features(cls, device: torch.device) -> OrderedSet[BackendFeature]:
        # Whether a long reduction is split at the IR level is decided by the num_splits
        # replacement in codegen/ir.py (only for a few outputs over a long range; the column
        # kernel cuts the reduced axis across workgroups itself), so REDUCE_TO_SINGLE_ELEMENT,
        # which would switch the split off everywhere, is not declared.
        return OrderedSet([BackendFeature.TUPLE_REDUCTION])

    @classmethod
    def get_tiling_and_scores(cls, node_schedule, numel, reduction_numel=sympy.S.One, coalesce_analysis=None):
        """One flat kept axis and one flat reduced axis; strided and permuted
        accesses are recovered from the index expressions instead of from tiles."""
        if reduction_numel == 1 or reduction_numel is sympy.S.One:
            return {"x": numel, "r0_": sympy.S.One}, None
        return {"x": numel, "r0_": reduction_numel}, None

    def codegen_node_schedule_with_kernel(self, node_schedule, kernel):
        try:
            return super().codegen_node_schedule_with_kernel(node_schedule, kernel)
        except VecConstraintError as e:
            log.debug("retrying kernel with scalar accesses: %s", e)
            features = kernel.features
            tiling = kernel.tiling
            kernel.__init__(tiling, force_vec=1, features=features)
            return super().codegen_node_schedule_with_kernel(node_schedule, kernel)

    def codegen_node(self, node):
        """A fused node the generator cannot express ends compilation with ONE error that names the
        node, the ATen ops it came from and the reason; the ops travel on the exception so that the
        compile wrapper (inductor_x_amd.install_unsupported_retry) can send them to their eager kernels
        and compile the graph again.  The reference drops a failing configuration and goes on
        (reference inductor_x/npu_triton_heuristics.py:87-106,194-198)."""
        try:
            return super().codegen_node(node)
        except UnsupportedHipCodegen as e:
            if getattr(e, "node_names", None):
                raise
            nodes = list(node.get_nodes()) if hasattr(node, "get_nodes") else [node]
            culprits = [n for n in nodes if n.is_reduction()] or nodes
            ops: list = []
            for n in culprits:
                for fx in getattr(n.node, "origins", ()) or ():
                    tgt = getattr(fx, "target", None)
                    if isinstance(tgt, torch._ops.OpOverload) and tgt not in ops:
                        ops.append(tgt)
            # ops the generator is exercised on every day (pointwise arithmetic fused into the node)
            # are not what it refused: keep them generated unless they are all there is
            from ..lowering import GENERATE_LIST, REDUCING_OPS

            everyday = {p for p in GENERATE_LIST if p not in REDUCING_OPS}
            narrowed = [o for o in ops if getattr(o, "overloadpacket", None) not in everyday]
            ops = narrowed or ops
            names = [n.get_name() for n in nodes]
            err = UnsupportedHipCodegen(
                f"inductor_x_amd cannot generate a HIP kernel for fused node {'+'.join(names)} "
                f"(from {', '.join(str(o) for o in ops) or 'unknown ops'}): {e}"
            )
            err.node_names = names
            err.ops = ops
            raise err from e

    def define_kernel(self, src_code: str, node_schedule, kernel: HipKernel) -> str:
        wrapper = V.graph.wrapper_code
        if src_code in wrapper.src_to_kernel:
            return wrapper.src_to_kernel[src_code]
        kernel_name = f"hip_{kernel.mode}_{wrapper.next_kernel_suffix()}"
        wrapper.src_to_kernel[src_code] = kernel_name
        source = src_code.replace(KERNEL_PLACEHOLDER, kernel_name)
        origins, detailed = get_kernel_metadata(node_schedule, wrapper)
        body = (
            f"generated_kernel(\n    name={kernel_name!r},\n    meta={kernel.meta!r},\n"
            f"    source='''\n{source}''',\n)"
        )
        wrapper.define_kernel(kernel_name, body, f"{origins}\n{detailed}", gpu=False)
        return kernel_name

    def codegen_sync(self) -> None:
        V.graph.wrapper_code.writeline(V.graph.device_ops.synchronize())

    def benchmark_fused_nodes(self, nodes):
        raise NotImplementedError("fusion benchmarking is not used by this backend")
