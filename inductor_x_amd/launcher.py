"""ctypes binding of the C-ABI launcher declared in include/mi355_launcher.h.

Stands where the reference builds a per-kernel Python closure around the Triton
binary (reference inductor_x/npu_triton_heuristics.py:239-253).  There is no
fallback: if the shared library is missing or a call fails, a RuntimeError with
the kernel name and the HIP error text is raised.
"""
from __future__ import annotations

import ctypes
import os
import struct
import threading
from typing import Optional, Sequence

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libmi355_launcher.so"
LIB_PATH = os.path.join(_HERE, LIB_NAME)

EXPORTS = (
    "mi_abi_version",
    "mi_module_load",
    "mi_module_unload",
    "mi_module_get_function",
    "mi_function_get_attrs",
    "mi_launch",
    "mi_launch_packed",
    "mi_launch_packed_scratch",
    "mi_scratch_capacity",
    "mi_device_props_get",
    "mi_device_count",
    "mi_error_string",
)


class DeviceProps(ctypes.Structure):
    _fields_ = [
        ("cu_count", ctypes.c_int32),
        ("xcd_count", ctypes.c_int32),
        ("wave_size", ctypes.c_int32),
        ("lds_bytes", ctypes.c_int32),
        ("max_threads_per_cu", ctypes.c_int32),
        ("max_waves_per_cu", ctypes.c_int32),
        ("regs_per_cu", ctypes.c_int32),
        ("clock_khz", ctypes.c_int32),
        ("mem_clock_khz", ctypes.c_int32),
        ("mem_bus_bits", ctypes.c_int32),
        ("l2_bytes", ctypes.c_int64),
        ("hbm_bytes", ctypes.c_int64),
        ("mall_bytes", ctypes.c_int64),
        ("arch", ctypes.c_char * 64),
    ]


class FunctionAttrs(ctypes.Structure):
    _fields_ = [
        ("num_regs", ctypes.c_int32),
        ("static_lds_bytes", ctypes.c_int32),
        ("scratch_bytes", ctypes.c_int32),
        ("max_threads_per_block", ctypes.c_int32),
    ]


ABI_VERSION = 2
SCRATCH_TOO_LARGE = 100001  # MI_ERROR_SCRATCH_TOO_LARGE

_lib_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None


class LauncherError(RuntimeError):
    pass


def load_library(path: str = LIB_PATH) -> ctypes.CDLL:
    """Load the launcher library (once) and declare its prototypes."""
    global _lib
    with _lib_lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(path):
            raise LauncherError(
                f"{path} not found: build it first (python -c 'import __graft_entry__ as g; g.build()')"
            )
        lib = ctypes.CDLL(path)
        vp, u32, sz = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_size_t
        lib.mi_abi_version.restype = ctypes.c_int
        lib.mi_abi_version.argtypes = []
        lib.mi_module_load.restype = ctypes.c_int
        lib.mi_module_load.argtypes = [vp, sz, ctypes.POINTER(vp)]
        lib.mi_module_unload.restype = ctypes.c_int
        lib.mi_module_unload.argtypes = [vp]
        lib.mi_module_get_function.restype = ctypes.c_int
        lib.mi_module_get_function.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(vp)]
        lib.mi_function_get_attrs.restype = ctypes.c_int
        lib.mi_function_get_attrs.argtypes = [vp, ctypes.POINTER(FunctionAttrs)]
        lib.mi_launch.restype = ctypes.c_int
        lib.mi_launch.argtypes = [vp, u32, u32, u32, u32, u32, u32, u32, vp, ctypes.POINTER(vp)]
        lib.mi_launch_packed.restype = ctypes.c_int
        lib.mi_launch_packed.argtypes = [vp, u32, u32, u32, u32, u32, u32, u32, vp, ctypes.c_char_p, sz]
        lib.mi_launch_packed_scratch.restype = ctypes.c_int
        lib.mi_launch_packed_scratch.argtypes = [vp, u32, u32, u32, u32, u32, u32, u32, vp, ctypes.c_char_p, sz, sz, sz]
        lib.mi_scratch_capacity.restype = ctypes.c_int
        lib.mi_scratch_capacity.argtypes = [ctypes.POINTER(sz)]
        lib.mi_device_props_get.restype = ctypes.c_int
        lib.mi_device_props_get.argtypes = [ctypes.c_int, ctypes.POINTER(DeviceProps)]
        lib.mi_device_count.restype = ctypes.c_int
        lib.mi_device_count.argtypes = [ctypes.POINTER(ctypes.c_int)]
        lib.mi_error_string.restype = ctypes.c_char_p
        lib.mi_error_string.argtypes = [ctypes.c_int]
        if lib.mi_abi_version() != ABI_VERSION:
            raise LauncherError(f"{path}: unexpected ABI version {lib.mi_abi_version()}")
        _lib = lib
        _load_fastcall(lib)
        return lib


FASTCALL_PATH = os.path.join(_HERE, "_mi_fastcall.so")
_fast = None


def _load_fastcall(lib: ctypes.CDLL):
    """The vectorcall entry to mi_launch_packed (csrc/mi_fastcall.c), bound to the loaded library.
    Optional: without it every launch goes through ctypes, which is the same C ABI call with more
    Python objects on the way."""
    global _fast
    if _fast is not None or not os.path.exists(FASTCALL_PATH):
        return _fast
    import importlib.machinery
    import importlib.util

    try:
        loader = importlib.machinery.ExtensionFileLoader("_mi_fastcall", FASTCALL_PATH)
        spec = importlib.util.spec_from_loader("_mi_fastcall", loader)
        mod = importlib.util.module_from_spec(spec)
        loader.exec_module(mod)
        mod.bind(ctypes.cast(lib.mi_launch_packed, ctypes.c_void_p).value)
        _fast = mod
    except Exception:  # built for another interpreter: ctypes carries on
        _fast = None
    return _fast


def error_string(err: int) -> str:
    return load_library().mi_error_string(err).decode()


def _check(err: int, what: str) -> None:
    if err != 0:
        raise LauncherError(f"{what}: HIP error {err} ({error_string(err)})")


def device_count() -> int:
    n = ctypes.c_int(0)
    err = load_library().mi_device_count(ctypes.byref(n))
    return n.value if err == 0 else 0


def device_props(device: int = 0) -> DeviceProps:
    p = DeviceProps()
    _check(load_library().mi_device_props_get(device, ctypes.byref(p)), f"mi_device_props_get({device})")
    return p


class Module:
    """A loaded gfx950 code object."""

    def __init__(self, hsaco: bytes, label: str = "<hsaco>"):
        self.label = label
        self._handle = ctypes.c_void_p()
        self._functions: dict[str, "Function"] = {}
        buf = ctypes.create_string_buffer(hsaco, len(hsaco))
        _check(
            load_library().mi_module_load(ctypes.cast(buf, ctypes.c_void_p), len(hsaco), ctypes.byref(self._handle)),
            f"mi_module_load({label})",
        )

    def function(self, name: str) -> "Function":
        fn = self._functions.get(name)
        if fn is None:
            h = ctypes.c_void_p()
            _check(
                load_library().mi_module_get_function(self._handle, name.encode(), ctypes.byref(h)),
                f"mi_module_get_function({self.label}:{name})",
            )
            fn = Function(self, name, h)
            self._functions[name] = fn
        return fn

    def unload(self) -> None:
        if self._handle:
            _check(load_library().mi_module_unload(self._handle), f"mi_module_unload({self.label})")
            self._handle = ctypes.c_void_p()
            self._functions.clear()


# When set to a list, every enqueue appends the kernel's symbol to it (measurement harnesses use
# this to report which code object symbols a call really launched).
launch_log: Optional[list] = None


# struct-module codes for the kernel-parameter signature strings used below:
#   P pointer, i int32, I uint32, q int64, Q uint64, f float, d double
_VALID = set("PiIqQfd")


class Function:
    """One kernel of a module, launched through mi_launch_packed."""

    def __init__(self, module: Module, name: str, handle: ctypes.c_void_p):
        self.module = module
        self.name = name
        self._handle = handle
        self._lib = load_library()
        self._fast = _fast
        self._raw_handle = handle.value
        self._packers: dict[str, struct.Struct] = {}

    def attrs(self) -> FunctionAttrs:
        a = FunctionAttrs()
        _check(self._lib.mi_function_get_attrs(self._handle, ctypes.byref(a)), f"mi_function_get_attrs({self.name})")
        return a

    def launch(
        self,
        signature: str,
        args: Sequence,
        grid: Sequence[int],
        block: Sequence[int],
        stream: int,
        lds_bytes: int = 0,
    ) -> None:
        """Enqueue the kernel.  `signature` has one struct code per parameter;
        the values are packed with native alignment, which is the layout of the
        kernel's argument segment."""
        packer = self._packers.get(signature)
        if packer is None:
            bad = set(signature) - _VALID
            if bad:
                raise LauncherError(f"{self.name}: bad signature codes {sorted(bad)}")
            packer = struct.Struct("@" + signature)
            self._packers[signature] = packer
        if len(args) != len(signature):
            raise LauncherError(f"{self.name}: expected {len(signature)} kernel arguments, got {len(args)}")
        seg = packer.pack(*args)
        gx, gy, gz = (tuple(grid) + (1, 1))[:3]
        bx, by, bz = (tuple(block) + (1, 1))[:3]
        if launch_log is not None:
            launch_log.append(self.name)
        if self._fast is not None:
            err = self._fast.launch(self._raw_handle, gx, gy, gz, bx, by, bz, lds_bytes, stream, seg)
        else:
            err = self._lib.mi_launch_packed(
                self._handle, gx, gy, gz, bx, by, bz, lds_bytes, ctypes.c_void_p(stream), seg, len(seg)
            )
        if err != 0:
            raise LauncherError(
                f"launch of {self.name} grid=({gx},{gy},{gz}) block=({bx},{by},{bz}) lds={lds_bytes} failed: "
                f"HIP error {err} ({error_string(err)})"
            )

    def launch_with_library_scratch(
        self,
        signature: str,
        args: Sequence,
        scratch_arg: int,
        scratch_bytes: int,
        grid: Sequence[int],
        block: Sequence[int],
        stream: int,
        lds_bytes: int = 0,
    ) -> None:
        """Enqueue through mi_launch_packed_scratch: parameter number `scratch_arg` (a pointer) is
        filled in by the library with its fixed per-GPU scratch array, of which the kernel uses
        `scratch_bytes`.  Nothing is allocated on the way."""
        if signature[scratch_arg] != "P":
            raise LauncherError(f"{self.name}: parameter {scratch_arg} is not a pointer")
        packer = self._packers.get(signature)
        if packer is None:
            packer = struct.Struct("@" + signature)
            self._packers[signature] = packer
        seg = packer.pack(*args)
        offset = struct.calcsize("@" + signature[:scratch_arg] + "P") - 8
        gx, gy, gz = (tuple(grid) + (1, 1))[:3]
        bx, by, bz = (tuple(block) + (1, 1))[:3]
        err = self._lib.mi_launch_packed_scratch(
            self._handle, gx, gy, gz, bx, by, bz, lds_bytes, ctypes.c_void_p(stream), seg, len(seg), offset,
            scratch_bytes,
        )
        if err != 0:
            raise LauncherError(f"launch of {self.name} on the library scratch failed: error {err} ({error_string(err)})")

    def launch_pointers(self, ctypes_values: Sequence, grid, block, stream: int, lds_bytes: int = 0) -> None:
        """Enqueue through mi_launch (array of pointers to ctypes values)."""
        n = len(ctypes_values)
        arr = (ctypes.c_void_p * n)(*[ctypes.cast(ctypes.pointer(v), ctypes.c_void_p) for v in ctypes_values])
        gx, gy, gz = (tuple(grid) + (1, 1))[:3]
        bx, by, bz = (tuple(block) + (1, 1))[:3]
        err = self._lib.mi_launch(self._handle, gx, gy, gz, bx, by, bz, lds_bytes, ctypes.c_void_p(stream), arr)
        if err != 0:
            raise LauncherError(f"launch of {self.name} failed: HIP error {err} ({error_string(err)})")
