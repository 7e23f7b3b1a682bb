"""hipcc -> gfx950 code-object cache.

Stands where the reference calls triton.compile on generated source and keeps
the result next to the source file (reference
inductor_x/npu_triton_heuristics.py:111-199, 302-393).  A code object is keyed
by a hash of the translation unit, the device headers it includes and the
compiler flags.  Lookups go first to the in-tree store that ships with the
package (filled ahead of time), then to a per-user store; a miss runs hipcc
under a per-key file lock so concurrent compile workers do not race.
"""
from __future__ import annotations

import fcntl
import hashlib
import os
import re
import shutil
import subprocess
import tempfile
import threading
from typing import Iterable, Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(_HERE, "csrc")
HEADER_DIR = os.path.join(CSRC_DIR, "mi")
AOT_DIR = os.path.join(CSRC_DIR, "aot")
PROBE_DIR = os.path.join(CSRC_DIR, "probes")
INTREE_STORE = os.path.join(_HERE, "_hsaco")
# Code objects of generated (torch.compile) kernels that ship with the tree, so a
# machine that has seen a graph before does not invoke hipcc for it again.
GENERATED_STORE = os.path.join(_HERE, "_hsaco_gen")

ARCH = "gfx950"
# Packed-fp32 instruction selection is switched off for every device compile.
HIPCC_FLAGS = (
    "-O3",
    f"--offload-arch={ARCH}",
    "--genco",
    "-std=c++17",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
)


# second attempt after an internal compiler error (see compile_source)
BACKEND_ERROR_RETRY_FLAGS = ("-fno-slp-vectorize",)


class CompileError(RuntimeError):
    pass


def _first_lines(stderr: str, n: int = 3) -> str:
    """The head of a long compiler message (the tail alone loses the line that names the error)."""
    if len(stderr) <= 4000:
        return ""
    return "\n".join(stderr.splitlines()[:n]) + "\n[...]\n"


def hipcc_path() -> str:
    cand = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(cand):
        raise CompileError("hipcc not found; cannot build gfx950 code objects")
    return cand


def toolchain_version() -> str:
    """ROCm release the code objects are built with (part of every cache key: an object built by
    another compiler release is never reused).  Read from the installation's version file; running
    the compiler for its banner would cost more than most cache hits save."""
    root = os.path.dirname(os.path.dirname(os.path.realpath(hipcc_path())))
    for rel in (".info/version", ".info/version-dev"):
        try:
            with open(os.path.join(root, rel)) as f:
                return f.read().strip()
        except OSError:
            continue
    return "unknown"


_INCLUDE = re.compile(r'^\s*#\s*include\s+"(?:\.\./)?(?:mi/)?([A-Za-z0-9_.]+\.h)"', re.M)
_header_text_cache: dict[str, str] = {}


def _header_text(name: str) -> Optional[str]:
    if name not in _header_text_cache:
        try:
            with open(os.path.join(HEADER_DIR, name)) as f:
                _header_text_cache[name] = f.read()
        except OSError:
            _header_text_cache[name] = ""
    return _header_text_cache[name] or None


def reachable_headers(source: str) -> list[str]:
    """Names of the device headers (csrc/mi/*.h) a translation unit includes, directly or through
    other headers, sorted.  Only these enter its cache key: editing the attention kernels does not
    invalidate the code objects of generated row or column kernels."""
    seen: set[str] = set()
    todo = list(_INCLUDE.findall(source))
    while todo:
        name = todo.pop()
        if name in seen:
            continue
        text = _header_text(name)
        if text is None:
            continue
        seen.add(name)
        todo.extend(_INCLUDE.findall(text))
    return sorted(seen)


def _headers_digest(source: str) -> str:
    h = hashlib.sha256()
    h.update(toolchain_version().encode())
    for name in reachable_headers(source):
        h.update(name.encode())
        h.update(_header_text(name).encode())
    return h.hexdigest()


def source_key(source: str, extra_flags: Iterable[str] = ()) -> str:
    h = hashlib.sha256()
    h.update(_headers_digest(source).encode())
    h.update("\0".join(HIPCC_FLAGS + tuple(extra_flags)).encode())
    h.update(source.encode())
    return h.hexdigest()[:32]


def user_store() -> str:
    base = os.environ.get("INDUCTOR_X_AMD_CACHE") or os.path.join(
        os.environ.get("XDG_CACHE_HOME", os.path.join(os.path.expanduser("~"), ".cache")), "inductor_x_amd"
    )
    return base


def _stores() -> list[str]:
    return [INTREE_STORE, GENERATED_STORE, user_store()]


def lookup(key: str) -> Optional[str]:
    for d in _stores():
        p = os.path.join(d, key + ".hsaco")
        if os.path.exists(p) and os.path.getsize(p) > 0:
            return p
    return None


def _writable_store(prefer_intree: bool) -> str:
    order = [INTREE_STORE, user_store()] if prefer_intree else [user_store(), INTREE_STORE]
    for d in order:
        try:
            os.makedirs(d, exist_ok=True)
            # one probe name per thread: the compile pool's threads run this concurrently
            probe = os.path.join(d, f".w{os.getpid()}.{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.unlink(probe)
            return d
        except OSError:
            continue
    return tempfile.mkdtemp(prefix="inductor_x_amd_")


def compile_source(
    source: str,
    label: str = "kernel",
    extra_flags: Iterable[str] = (),
    prefer_intree: bool = False,
    force: bool = False,
    include_dir: Optional[str] = None,
) -> str:
    """Return the path of the code object for `source`, compiling on a miss.

    `source` may #include "mi/<header>.h".  Raises CompileError with the
    compiler's stderr when hipcc fails.
    """
    extra_flags = tuple(extra_flags)
    key = source_key(source, extra_flags)
    if not force:
        hit = lookup(key)
        if hit:
            return hit
    store = _writable_store(prefer_intree)
    out = os.path.join(store, key + ".hsaco")
    lock_path = os.path.join(store, key + ".lock")
    with open(lock_path, "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        try:
            if not force and os.path.exists(out) and os.path.getsize(out) > 0:
                return out
            with tempfile.TemporaryDirectory(prefix="mi_hipcc_") as tmp:
                src = os.path.join(tmp, f"{label}.hip")
                with open(src, "w") as f:
                    f.write(source)
                tmp_out = os.path.join(tmp, "out.hsaco")
                cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-I", include_dir or CSRC_DIR, "-o", tmp_out, src]
                proc = subprocess.run(cmd, capture_output=True, text=True)
                if proc.returncode != 0 and "error in backend" in proc.stderr:
                    # The compiler itself gave up, not the source: with packed fp32 instructions switched off,
                    # this release cannot select some two-element float vectors that its SLP vectorizer forms
                    # ("Cannot select: v2f32 = bitcast", seen on a generated pointwise kernel with a negated
                    # select beside an erf).  Without that vectorizer the same source compiles; the code object
                    # is stored under the key of the request.
                    first = proc.stderr
                    proc = subprocess.run(cmd[:-1] + list(BACKEND_ERROR_RETRY_FLAGS) + [src], capture_output=True, text=True)
                    if proc.returncode != 0:
                        proc.stderr = _first_lines(first) + proc.stderr
                if proc.returncode != 0 or not os.path.exists(tmp_out):
                    raise CompileError(f"hipcc failed for {label} (key {key}):\n{_first_lines(proc.stderr)}{proc.stderr[-4000:]}")
                final_tmp = out + f".tmp{os.getpid()}"
                shutil.copyfile(tmp_out, final_tmp)
                os.replace(final_tmp, out)
            with open(os.path.join(store, key + ".txt"), "w") as f:
                f.write(label + "\n")
            return out
        finally:
            fcntl.flock(lock, fcntl.LOCK_UN)


def harvest(source_dir: Optional[str] = None) -> int:
    """Copy the code objects of `source_dir` (default: the per-user store) into the package's
    store of generated kernels, so that a tree shipped to a machine without a warm per-user store
    starts with them.  Returns the number of objects copied."""
    source_dir = source_dir or user_store()
    os.makedirs(GENERATED_STORE, exist_ok=True)
    copied = 0
    for name in sorted(os.listdir(source_dir)) if os.path.isdir(source_dir) else ():
        dst = os.path.join(GENERATED_STORE, name)
        if name.endswith(".hsaco") and not os.path.exists(dst) and not os.path.exists(os.path.join(INTREE_STORE, name)):
            tmp = dst + f".tmp{os.getpid()}"
            shutil.copyfile(os.path.join(source_dir, name), tmp)
            os.replace(tmp, dst)
            copied += 1
    return copied


def aot_source(name: str) -> str:
    """Text of one of the hand-written instantiation files under csrc/aot,
    with its relative includes rewritten to the include root."""
    with open(os.path.join(AOT_DIR, name)) as f:
        return f.read().replace('#include "../mi/', '#include "mi/')


def probe_source(name: str) -> str:
    """Text of a measurement kernel file under csrc/probes (resource probes that no graph launches;
    they are compiled for the benchmark program only and are not part of the ahead-of-time set)."""
    with open(os.path.join(PROBE_DIR, name)) as f:
        return f.read().replace('#include "../mi/', '#include "mi/')


def build_probes(force: bool = True) -> dict[str, str]:
    """Compile the measurement kernels of csrc/probes into the in-tree store."""
    out = {}
    for name in sorted(n for n in os.listdir(PROBE_DIR) if n.endswith(".hip")):
        out[name] = compile_source(probe_source(name), label=name[:-4], prefer_intree=True, force=force)
    return out


def aot_files() -> list[str]:
    return sorted(n for n in os.listdir(AOT_DIR) if n.endswith(".hip"))


def build_aot(force: bool = True) -> dict[str, str]:
    """Compile every file of csrc/aot into the in-tree store."""
    out = {}
    for name in aot_files():
        out[name] = compile_source(aot_source(name), label=name[:-4], prefer_intree=True, force=force)
    return out
