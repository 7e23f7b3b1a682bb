"""MI355X-native TorchInductor backend (gfx950).

Importing the package has side effects only, like the reference's import hook
(reference inductor_x/__init__.py:1-63): it registers the HIP scheduling and a
wrapper code generator for the GPU device type, a device-op override whose
generated wrappers fetch the raw stream from this package, a device interface,
the lowering / decomposition table patches and the fused-attention graph
pattern.  After `import inductor_x_amd`, `torch.compile(fn)` on PyTorch-ROCm
emits hand-templated HIP kernels launched through the C-ABI launcher; no Triton
is generated.
"""
from __future__ import annotations

__version__ = "0.1.0"

import torch

from . import config  # noqa: F401

DEVICE_TYPE = "cuda"  # PyTorch-ROCm exposes AMD GPUs under this device type


def get_current_raw_stream(device) -> int:
    """Raw hipStream_t of torch's current stream as an integer
    (reference inductor_x/__init__.py:26-27)."""
    index = device if isinstance(device, int) else torch.device(device).index
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if index is None else index)


def _backend_fingerprint() -> str:
    """Hash of everything that decides what this backend generates: its Python sources, the
    device headers and ahead-of-time kernel sources, and the INDUCTOR_X_AMD_* switches."""
    import hashlib
    import os

    here = os.path.dirname(os.path.abspath(__file__))
    h = hashlib.sha256()
    for root, dirs, files in os.walk(here):
        dirs[:] = sorted(d for d in dirs if not d.startswith(("_hsaco", "__pycache__")))
        for name in sorted(files):
            if name.endswith((".py", ".h", ".hip", ".cpp")):
                path = os.path.join(root, name)
                h.update(os.path.relpath(path, here).encode())
                with open(path, "rb") as f:
                    h.update(f.read())
    for key in sorted(os.environ):
        if key.startswith("INDUCTOR_X_AMD_") and key not in ("INDUCTOR_X_AMD_CACHE",):
            h.update(f"{key}={os.environ[key]}".encode())
    return h.hexdigest()


def _inductor_register_backend_for_device() -> None:
    from torch._inductor.codegen.common import register_backend_for_device
    from torch._inductor.custom_graph_pass import CustomGraphModulePass

    from .codegen.scheduling import HipScheduling
    from .codegen.wrapper import HipWrapperCodegen

    class BackendFingerprint(CustomGraphModulePass):
        """Changes no graph.  Inductor folds the uuid of a backend's custom pass into the keys of its
        on-disk caches (compiled graphs, AOTAutograd artefacts), so entries written by other
        sources of this package, or under other switches, are not served."""

        def __call__(self, gm) -> None:
            return None

        def uuid(self):
            return _backend_fingerprint()

    register_backend_for_device(DEVICE_TYPE, HipScheduling, HipWrapperCodegen, device_custom_pass=BackendFingerprint())


def _inductor_register_device_op_overrides() -> None:
    from torch._inductor.codegen.common import get_device_op_overrides, register_device_op_overrides

    # Inductor fills its table of per-device overrides lazily and only while the
    # table is empty (importing any one device's module makes it non-empty); ask
    # for an entry first so the CPU and other defaults are in place before the
    # GPU entry is replaced.
    get_device_op_overrides("cpu")
    from torch._inductor.codegen.cuda.device_op_overrides import CUDADeviceOpOverrides

    class HipDeviceOpOverrides(CUDADeviceOpOverrides):
        def import_get_raw_stream_as(self, name: str) -> str:
            return f"from inductor_x_amd import get_current_raw_stream as {name}"

    register_device_op_overrides(DEVICE_TYPE, HipDeviceOpOverrides())


def _register_device_interface() -> None:
    from torch._dynamo.device_interface import CudaInterface, register_interface_for_device

    class HipInterface(CudaInterface):
        """reference inductor_x/__init__.py:40-52"""

        @staticmethod
        def is_available() -> bool:
            return torch.cuda.device_count() > 0

        @staticmethod
        def get_compute_capability(device=None):
            # the code object target, e.g. "gfx950"
            if torch.cuda.device_count() == 0:
                return "gfx950"
            return torch.cuda.get_device_properties(device).gcnArchName.split(":")[0]

    register_interface_for_device(DEVICE_TYPE, HipInterface)


def _find_unsupported(exc: BaseException):
    """The UnsupportedHipCodegen in the cause / context chain of `exc`, if any."""
    from .codegen.hip_kernel import UnsupportedHipCodegen

    seen = set()
    while exc is not None and id(exc) not in seen:
        seen.add(id(exc))
        if isinstance(exc, UnsupportedHipCodegen):
            return exc
        inner = getattr(exc, "inner_exception", None)
        exc = inner or exc.__cause__ or exc.__context__
    return None


def install_unsupported_retry() -> None:
    """Wrap Inductor's in-process graph compile: when the HIP generator refuses a fused node, the ATen
    ops that node came from are sent to their eager kernels (lowering.add_runtime_fallback) and the
    graph is lowered again, instead of torch.compile failing.  When nothing is left to fall back on,
    the generator's error, which names the node and the ops, ends the compilation.  Switch:
    config.retry_unsupported_with_eager."""
    import copy
    import logging

    from torch._inductor import compile_fx as cfx

    cls = getattr(cfx, "_InProcessFxCompile", None)
    if cls is None or getattr(cls.codegen_and_compile, "_inductor_x_amd", False):
        return
    original = cls.codegen_and_compile
    log = logging.getLogger(__name__)

    def codegen_and_compile(self, gm, example_inputs, inputs_to_check, graph_kwargs):
        from .lowering import add_runtime_fallback

        if not config.retry_unsupported_with_eager:
            return original(self, gm, example_inputs, inputs_to_check, graph_kwargs)
        try:
            pristine = copy.deepcopy(gm)  # the post-grad passes rewrite gm in place
        except Exception as e:  # a graph that cannot be copied compiles without the retry
            log.debug("graph module cannot be copied (%s): no eager retry for this compile", e)
            return original(self, gm, example_inputs, inputs_to_check, graph_kwargs)
        for _ in range(4):
            try:
                return original(self, gm, example_inputs, inputs_to_check, graph_kwargs)
            except Exception as e:
                unsupported = _find_unsupported(e)
                # The fallbacks registered here stay for the rest of the process (lowering tables are
                # process-wide): later graphs run these ops as eager kernels too.
                # lowering.RUNTIME_FALLBACKS lists them, lowering.clear_runtime_fallbacks() undoes them.
                changed = [op for op in getattr(unsupported, "ops", ()) if add_runtime_fallback(op)]
                if unsupported is None or not changed:
                    raise
                log.warning("%s; compiling again with %s as eager kernels", unsupported, ", ".join(map(str, changed)))
                gm = copy.deepcopy(pristine)
        return original(self, gm, example_inputs, inputs_to_check, graph_kwargs)

    codegen_and_compile._inductor_x_amd = True
    cls.codegen_and_compile = codegen_and_compile


_registered = False


def _register() -> None:
    global _registered
    if _registered:
        return
    _registered = True
    from torch._inductor import lowering as inductor_lowering

    from . import codegen  # noqa: F401  (installs the Reduction.num_splits stub)
    from .codegen.ir import install_num_splits_stub
    from .decomposition import _register_inductor_decompositions
    from .lowering import _register_inductor_fallbacks, make_reduction

    config.apply_inductor_settings()
    _inductor_register_backend_for_device()
    _inductor_register_device_op_overrides()
    _register_device_interface()
    install_num_splits_stub()
    inductor_lowering.make_reduction = make_reduction
    _register_inductor_fallbacks()
    _register_inductor_decompositions()
    install_unsupported_retry()
    from . import fusion_attention_graph

    fusion_attention_graph.register_fx_pass()


_register()
