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

    # -- fusion benchmarking ----------------------------------------------------
    def generate_kernel_code_from_nodes(self, nodes, benchmark_kernel=False, hint_override=None):
        """Python source of a module that holds the kernel for `nodes` (under the attribute name
        Inductor's scheduler looks up, `triton_`), random operands of the graph's hinted sizes
        (`get_args`) and one launch (`call`): what Inductor's scheduler compiles and times when
        `benchmark_fusion` asks whether fusing two nodes pays (the reference inherits Triton's
        form of it, reference inductor_x/codegen/triton.py:525-526,550-553,613-614)."""
        from torch._inductor import config as inductor_config
        from torch._inductor.codegen.common import SizeArg, TensorArg, WorkspaceArg
        from torch._inductor.utils import IndentedBuffer

        if any(n.is_template() for n in nodes):
            raise NotImplementedError("this backend has no template kernels")
        _, (numel, rnumel) = max(nodes, key=lambda x: int(x.is_reduction())).group
        node_schedule = self.generate_node_schedule(nodes, numel, rnumel)
        tiling = self.select_tiling(node_schedule, numel, rnumel)
        kernel = self.kernel_type(tiling, features=SIMDKernelFeatures(node_schedule, numel, rnumel))
        self.codegen_node_schedule_with_kernel(node_schedule, kernel)
        with V.set_kernel_handler(kernel):
            src_code = kernel.codegen_kernel()
        name = "hip_bench"
        device = V.graph.get_current_device_or_throw()
        hint = lambda e: V.graph.sizevars.size_hint(e, fallback=inductor_config.unbacked_symint_fallback)  # noqa: E731
        hints = lambda es: [hint(e) for e in es]  # noqa: E731
        out = IndentedBuffer()
        out.splice(
            "import torch\nfrom torch._dynamo.testing import rand_strided\n"
            "from inductor_x_amd.hip_heuristics import generated_kernel\n\n"
        )
        out.writeline(f"triton_ = generated_kernel(\n    name={name!r},\n    meta={kernel.meta!r},\n    source='''")
        out.splice(src_code.replace(KERNEL_PLACEHOLDER, name))
        out.writeline("''',\n)")
        out.writelines(["", "", "def get_args():"])
        _argdefs, call_args, signature, _ = kernel.args.python_argdefs()
        with out.indent():
            names = []
            for i, (arg_name, sig) in enumerate(zip(call_args, signature)):
                arg_name, var = str(arg_name), f"arg_{i}"
                buf = V.graph.try_get_buffer(arg_name) if isinstance(sig, TensorArg) else None
                if buf is not None:
                    line = (f"{var} = rand_strided({hints(buf.get_size())}, {hints(buf.get_stride())}, "
                            f"device='{buf.get_device()}', dtype={buf.get_dtype()})")
                    # a zero-dimensional CPU tensor among GPU operands is a scalar kernel argument
                    if buf.get_device().type == "cpu" and len(buf.get_size()) == 0:
                        line += ".item()"
                    out.writeline(line)
                elif arg_name in V.graph.constants:
                    c = V.graph.constants[arg_name]
                    out.writeline(f"{var} = rand_strided({hints(c.size())}, {hints(c.stride())}, device='{device}', dtype={c.dtype})")
                elif isinstance(sig, SizeArg):
                    out.writeline(f"{var} = {0 if 'seed_offset' in sig.name else hint(sig.expr)}")
                elif isinstance(sig, WorkspaceArg):
                    out.writeline(f"{var} = torch.zeros({hint(sig.count)}, device='{device}', dtype={sig.dtype})")
                else:
                    raise KeyError(f"no buffer or constant behind kernel argument {arg_name}")
                names.append(var)
            extents = {f"{tree.prefix}numel": hint(tree.numel) for tree in kernel.range_trees}
            out.writeline(f"return ({', '.join(names)}{',' if names else ''}), {extents!r}")
        out.writelines(["", "", "def call(args):"])
        with out.indent():
            out.writeline("operands, extents = args")
            out.writeline(f"with torch.cuda.device({device.index or 0}):")
            with out.indent():
                out.writeline(f"triton_.run(*operands, **extents, stream=torch._C._cuda_getCurrentRawStream({device.index or 0}))")
        return out.getvalue()

    def benchmark_codegened_module(self, mod, n_spills_threshold=8, node_names=None) -> tuple[float, str]:
        """Milliseconds per launch of a module made by generate_kernel_code_from_nodes, and its path."""
        args = mod.get_args()
        for _ in range(3):
            mod.call(args)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(10):
            mod.call(args)
        end.record()
        end.synchronize()
        ms = start.elapsed_time(end) / 10
        log.debug("kernel for %s: %.4f ms (%s)", node_names, ms, mod.__file__)
        return ms, mod.__file__

    def benchmark_fused_nodes(self, nodes, n_spills_threshold=8) -> tuple[float, str]:
        """Milliseconds one launch of the kernel for `nodes` takes on random operands."""
        from torch._inductor.codecache import PyCodeCache

        mod = PyCodeCache.load(self.generate_kernel_code_from_nodes(nodes, benchmark_kernel=True))
        return self.benchmark_codegened_module(mod, n_spills_threshold, OrderedSet(n.get_name() for n in nodes))
