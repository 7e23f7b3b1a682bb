"""Host-side logic that needs no GPU: the C-ABI library and its header, the
code-object cache, the launch heuristics, the launcher's error handling, and
the code generator (graphs are compiled with the HIP scheduling registered for
the CPU device in dry-run mode: HIP source is generated and cross-compiled for
gfx950, nothing is launched)."""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def built():
    from inductor_x_amd import launcher

    if not os.path.exists(launcher.LIB_PATH):
        import __graft_entry__

        __graft_entry__.build()
    return launcher


def test_header_symbols_are_exported(built):
    header = open(os.path.join(ROOT, "include", "mi355_launcher.h")).read()
    declared = set(re.findall(r"\b(mi_[a-z_]+)\s*\(", header))
    assert declared == set(built.EXPORTS)
    lib = ctypes.CDLL(built.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert built.load_library().mi_abi_version() == 2


def test_scratch_array_is_resolvable_by_the_runtime(built, tmp_path):
    """The HIP runtime finds a registered device variable by name in the library's gfx950 code
    object; a symbol with local binding there aborts the process at hipGetSymbolAddress."""
    import subprocess

    llvm = "/opt/rocm/llvm/bin"
    if not os.path.exists(os.path.join(llvm, "clang-offload-bundler")):
        pytest.skip("ROCm LLVM tools not installed")
    fat, co = str(tmp_path / "fat.bin"), str(tmp_path / "dev.co")
    subprocess.run(["objcopy", "-O", "binary", "--only-section=.hip_fatbin", built.LIB_PATH, fat], check=True)
    subprocess.run([os.path.join(llvm, "clang-offload-bundler"), "--type=o", "--unbundle", f"--input={fat}",
                    "--targets=hipv4-amdgcn-amd-amdhsa--gfx950", f"--output={co}"], check=True)
    syms = subprocess.run([os.path.join(llvm, "llvm-readelf"), "-sW", co], check=True, capture_output=True, text=True).stdout
    rows = [ln.split() for ln in syms.splitlines() if ln.strip().endswith("scratch")]
    assert rows, "no scratch array in the device code object"
    assert all(r[4] == "GLOBAL" and int(r[2]) == 8 << 20 for r in rows), rows
    # nothing above the capacity is accepted, and the refusal has a text of its own
    assert lib_refuses_oversize(built)


def lib_refuses_oversize(built) -> bool:
    lib = built.load_library()
    seg = bytes(16)
    err = lib.mi_launch_packed_scratch(ctypes.c_void_p(1), 1, 1, 1, 64, 1, 1, 0, None, seg, len(seg), 0, (8 << 20) + 1)
    return err == built.SCRATCH_TOO_LARGE and "scratch" in built.error_string(err)


def test_fastcall_entry_reaches_the_same_c_abi(built):
    """The vectorcall entry hands its arguments to mi_launch_packed unchanged: the library's own
    argument checks answer (no GPU needed), and wrong Python types are refused before the call."""
    if not os.path.exists(built.FASTCALL_PATH):
        import __graft_entry__

        __graft_entry__.build_fastcall()
    built.load_library()
    fast = built._load_fastcall(built.load_library())
    assert fast is not None
    assert fast.launch(0, 1, 1, 1, 64, 1, 1, 0, 0, b"") != 0  # null function handle: hipErrorInvalidValue
    assert fast.launch(1, 0, 1, 1, 64, 1, 1, 0, 0, b"") != 0  # empty grid: hipErrorInvalidConfiguration
    with pytest.raises(TypeError):
        fast.launch(1, 1, 1, 1, 64, 1, 1, 0, 0, "not bytes")
    with pytest.raises(TypeError):
        fast.launch(1, 1, 1)
    with pytest.raises(OverflowError):
        fast.launch(1, 1 << 40, 1, 1, 64, 1, 1, 0, 0, b"")


def test_launcher_error_paths_without_gpu(built):
    lib = built.load_library()
    assert lib.mi_module_load(None, 0, None) != 0  # invalid arguments never crash
    assert lib.mi_module_get_function(None, b"x", None) != 0
    assert lib.mi_launch_packed(None, 1, 1, 1, 64, 1, 1, 0, None, None, 0) != 0
    assert isinstance(built.error_string(1), str) and built.error_string(1)
    if not torch.cuda.is_available():
        assert built.device_count() == 0
        with pytest.raises(built.LauncherError):
            built.Module(b"\x7fELF-not-a-code-object", label="bogus")


def test_codecache_compile_hit_and_error(tmp_path, monkeypatch):
    from inductor_x_amd import codecache

    monkeypatch.setenv("INDUCTOR_X_AMD_CACHE", str(tmp_path))
    src = '#include "mi/common.h"\nextern "C" __global__ void k(float* p) { p[threadIdx.x] = mi::sigmoid_f32(1.f); }\n'
    p1 = codecache.compile_source(src, label="t")
    assert p1.startswith(str(tmp_path)) and os.path.getsize(p1) > 0
    mtime = os.path.getmtime(p1)
    assert codecache.compile_source(src, label="t") == p1 and os.path.getmtime(p1) == mtime  # cache hit
    assert codecache.source_key(src) != codecache.source_key(src, ("-DX=1",))
    with pytest.raises(codecache.CompileError) as e:
        codecache.compile_source('extern "C" __global__ void k() { not_a_symbol(); }', label="bad")
    assert "not_a_symbol" in str(e.value)


BACKEND_ERROR_KERNEL = r'''
#include "mi/codegen.h"
// a generated pointwise kernel (negated select beside an erf, a second output with atan2 / expm1) on which
// this compiler release stops with "Cannot select: v2f32 = bitcast" when packed fp32 instructions are off
extern "C" __global__ __launch_bounds__(256) void hip_pointwise_0(const mi::bf16_t* __restrict__ in_ptr0, mi::bf16_t* __restrict__ out_ptr0, mi::bf16_t* __restrict__ out_ptr1, const int xnumel) {
    constexpr int VEC = 8;
    const int x0 = (static_cast<int>(blockIdx.x) * 256 + threadIdx.x) * VEC;
    if (x0 >= xnumel) return;
    auto tmp0 = mi::cast<float>(mi::vload_u<VEC>(in_ptr0 + (x0)));
    auto tmp1 = mi::sin(tmp0);
    auto tmp3 = 0.5f;
    auto tmp10 = (tmp0 * tmp3) * (mi::erf(tmp0 * 0.7071067811865476f) + 1.0f);
    auto tmp14 = mi::where(tmp1 > tmp10, tmp1, tmp10 * tmp3);
    auto tmp15 = (-tmp14);
    auto tmp16 = mi::abs(tmp0);
    auto tmp19 = mi::reciprocal(tmp16 + tmp3) * 1.0f;
    auto tmp21 = tmp19 * tmp19 * tmp19;
    auto tmp26 = mi::atan2(tmp0, tmp16 + 0.1f) + (tmp0 + tmp0);
    auto tmp29 = mi::truediv(tmp21, mi::abs(tmp26) + tmp3);
    auto tmp33 = mi::truediv(tmp0, mi::abs(mi::maximum(tmp0, tmp0)) + tmp3);
    auto tmp37 = mi::cast<float>(tmp0 > 0.0f) + tmp0;
    auto tmp44 = mi::expm1(mi::minimum(mi::maximum(tmp37, -5.0f), 5.0f));
    mi::vstore<VEC>(out_ptr0 + (x0), tmp15);
    mi::vstore<VEC>(out_ptr1 + (x0), mi::maximum(tmp29, mi::maximum(tmp33, tmp44)));
}
'''


def test_codecache_retries_an_internal_compiler_error(tmp_path, monkeypatch):
    """A source on which the compiler's backend gives up is compiled once more without the SLP
    vectorizer and stored under the key of the request; a source that is wrong still fails."""
    from inductor_x_amd import codecache

    monkeypatch.setenv("INDUCTOR_X_AMD_CACHE", str(tmp_path))
    path = codecache.compile_source(BACKEND_ERROR_KERNEL, label="ice")
    assert os.path.getsize(path) > 0 and os.path.basename(path) == codecache.source_key(BACKEND_ERROR_KERNEL) + ".hsaco"
    assert codecache.lookup(codecache.source_key(BACKEND_ERROR_KERNEL)) == path


def test_aot_code_objects_are_built_for_gfx950(built):
    from inductor_x_amd import codecache

    for name in codecache.aot_files():
        key = codecache.source_key(codecache.aot_source(name))
        path = codecache.lookup(key)
        assert path is not None, f"{name} has no ahead-of-time code object (run build())"
        blob = open(path, "rb").read()
        # hipcc --genco wraps the gfx950 ELF in a clang offload bundle
        assert blob[:4] in (b"\x7fELF", b"__CL") and b"gfx950" in blob


def test_split_heuristic_properties():
    from inductor_x_amd import config
    from inductor_x_amd.hip_heuristics import split_factor, split_reduction_plan

    hw = config.Hardware()
    for rows, cols in [(65536, 512), (4096, 512), (513, 1024), (100000, 8), (1, 4), (70000, 2048), (40000, 12)]:
        p = split_reduction_plan(rows, cols, hw=hw)
        assert p.nsplit >= 1 and p.rows_per_split * p.nsplit >= rows  # every row covered
        assert p.rows_per_split * (p.nsplit - 1) < rows  # no empty split
        assert p.col_tiles * p.ct * 4 >= cols
        assert p.block <= 1024 and p.lds_bytes <= hw.lds_bytes
        if rows * cols * 4 >= 1 << 20:
            assert 2 * p.workspace_floats(cols) * 4 <= 0.06 * rows * cols * 4 + 40 * cols  # partial traffic cap
    big = split_reduction_plan(65536, 512, hw=hw)
    assert (big.ct, big.rl, big.col_tiles) == (32, 8, 4)  # narrow column tiles: few partials per column
    assert big.nsplit == 64 and big.rows_per_split == 1024 and big.block == 256 and big.unroll == 8
    # more CUs never means fewer splits
    import dataclasses

    small = dataclasses.replace(hw, cu_count=64)
    assert split_reduction_plan(1 << 20, 512, hw=small).nsplit <= split_reduction_plan(1 << 20, 512, hw=hw).nsplit
    n, rps = split_factor(65536, 512, 128, 8, 4, hw=hw)
    assert n * rps >= 65536 and rps % (8 * 4) == 0


def test_row_plan_and_vector_width():
    from inductor_x_amd.hip_heuristics import row_reduction_plan, vector_width

    assert vector_width(4, 4096) == 4 and vector_width(2, 4096) == 8 and vector_width(2, 4100) == 4
    assert vector_width(4, 7) == 1
    p = row_reduction_plan(1024, 4096, 4, persistent=False)
    assert (p.block, p.tpr, p.vec) == (256, 256, 4)
    p = row_reduction_plan(8192, 4096, 2, persistent=True)
    assert (p.block, p.tpr, p.iters) == (512, 512, 1)
    p = row_reduction_plan(10, 64, 4, persistent=True)
    assert p.tpr == 16 and p.rows_per_wg == 16  # short rows share a workgroup


def test_grid_helper():
    from inductor_x_amd.hip_heuristics import grid

    assert grid(1000)({"PER_WG0": 256}) == (4, 1, 1)
    assert grid(10, 7)({}) == (10, 7, 1)


def test_kernels_fail_loudly_without_gpu(built):
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from inductor_x_amd import kernels

    with pytest.raises(ValueError):
        kernels.add_rmsnorm(torch.zeros(2, 8).bfloat16(), torch.zeros(2, 8).bfloat16(), torch.ones(8).bfloat16())


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode != 0 and "one GPU" in proc.stderr


DRY = r'''
import os, sys
os.environ["INDUCTOR_X_AMD_DRYRUN"] = "1"
os.environ["INDUCTOR_X_AMD_CACHE"] = sys.argv[1]
sys.path.insert(0, sys.argv[2])
import torch
import inductor_x_amd
from torch._inductor.codegen.common import register_backend_for_device
from torch._inductor.codegen.wrapper import PythonWrapperCodegen
from inductor_x_amd.codegen.scheduling import HipScheduling
from torch._inductor.utils import run_and_get_code
register_backend_for_device("cpu", HipScheduling, PythonWrapperCodegen)
def rms(h, r, w):
    s = h + r; sf = s.float()
    return (sf * torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + 1e-6) * w.float()).to(torch.bfloat16), s
cases = {
  "rowsum": (lambda x: (torch.relu(2*x+1)*torch.sigmoid(x)).sum(-1), (torch.randn(64, 4096),)),
  "rms": (rms, (torch.randn(16, 4096).bfloat16(), torch.randn(16, 4096).bfloat16(), torch.randn(4096).bfloat16())),
  "col": (lambda x: (x.mean(0), x.var(0, unbiased=False), x.argmax(0)), (torch.randn(65536, 64),)),
  "gather": (lambda t, i: t[i], (torch.randn(100, 1024).bfloat16(), torch.randint(0, 100, (64,)))),
  "permute": (lambda t: t.permute(0, 2, 1, 3).contiguous(), (torch.randn(2, 16, 4, 128).bfloat16(),)),
  "looped": (lambda x: torch.softmax(x, -1), (torch.randn(8, 40000),)),
  "odd": (lambda a, b: (a + b).sum(-1), (torch.randn(7, 9, 13), torch.randn(7, 9, 13))),
}
for name, (fn, args) in cases.items():
    torch._dynamo.reset()
    _, codes = run_and_get_code(torch.compile(fn), *args)
    code = "\n".join(codes)
    modes = sorted(set(m for m in ("pointwise", "row", "col") if f"'mode': '{m}'" in code))
    print("CASE", name, ",".join(modes), "vload" in code, "triton" in code.lower().replace("triton_", ""))
'''


def test_codegen_dry_run(tmp_path, built):
    """Generated source for the benchmark graphs compiles for gfx950 and takes
    the expected code shape."""
    script = tmp_path / "dry.py"
    script.write_text(DRY)
    proc = subprocess.run([sys.executable, str(script), str(tmp_path / "cache"), ROOT], capture_output=True, text=True,
                          timeout=900)
    assert proc.returncode == 0, proc.stderr[-3000:]
    got = {l.split()[1]: l.split()[2:] for l in proc.stdout.splitlines() if l.startswith("CASE")}
    assert got["rowsum"][0] == "row" and got["rms"][0] == "row" and got["looped"][0] == "row"
    assert got["col"][0] == "col"
    assert got["gather"][0] == "pointwise" and got["permute"][0] == "pointwise"
    assert all(v[1] == "True" for k, v in got.items() if k != "odd")  # vector accesses
    built_objs = [f for f in os.listdir(tmp_path / "cache") if f.endswith(".hsaco")]
    assert len(built_objs) >= len(got)


DRY_HEAD = r'''
import os, sys
os.environ["INDUCTOR_X_AMD_DRYRUN"] = "1"
os.environ["INDUCTOR_X_AMD_CACHE"] = sys.argv[1]
os.environ["TORCHINDUCTOR_FORCE_DISABLE_CACHES"] = "1"  # every graph is lowered here, never served from disk
sys.path.insert(0, sys.argv[2])
import torch
import inductor_x_amd
from inductor_x_amd import lowering, config
from inductor_x_amd.codegen import hip_kernel
lowering.GPU_DEVICE_TYPE = "cpu"  # the device-aware patches then act on the CPU tensors of the dry run
from torch._inductor.codegen.common import register_backend_for_device
from torch._inductor.codegen.wrapper import PythonWrapperCodegen
from inductor_x_amd.codegen.scheduling import HipScheduling
from torch._inductor.utils import run_and_get_code
register_backend_for_device("cpu", HipScheduling, PythonWrapperCodegen)
'''

DRY_UNSUPPORTED = DRY_HEAD + r'''
hip_kernel.REDUCTION_KIND.pop("prod")  # force the generator to refuse a product reduction
x = torch.rand(8, 256) + 0.5
_, codes = run_and_get_code(torch.compile(lambda x: (x * 2).prod(-1) + 1), x)
code = "\n".join(codes)
print("RETRY", "aten.prod" in code, "generated_kernel(" in code, ",".join(str(o) for o in lowering.RUNTIME_FALLBACKS))
config.retry_unsupported_with_eager = False
hip_kernel.REDUCTION_KIND.pop("max")
torch._dynamo.reset()
try:
    torch.compile(lambda x: x.amax(-1))(x)
    print("ERROR none")
except Exception as e:
    msg = str(e)
    print("ERROR", "cannot generate a HIP kernel for fused node" in msg, "aten.amax" in msg, "reduction max" in msg)
'''

DRY_BOUNDS = DRY_HEAD + r'''
cases = {
  "embedding": (lambda t, i: torch.nn.functional.embedding(i, t) * 2, (torch.randn(100, 1024).bfloat16(), torch.randint(0, 100, (64,)))),
  "index": (lambda t, i: t[i], (torch.randn(100, 64), torch.randint(0, 100, (7, 5)))),
  "index_put": (lambda t, i, v: t.index_put((i,), v, accumulate=True), (torch.zeros(100, 64), torch.randint(0, 100, (32,)), torch.randn(32, 64))),
  "scatter": (lambda t, i, v: t.scatter(1, i, v), (torch.zeros(16, 64), torch.randint(0, 64, (16, 8)), torch.randn(16, 8))),
  "gather": (lambda t, i: torch.gather(t, 1, i), (torch.randn(16, 64), torch.randint(0, 64, (16, 8)))),
}
import re
for name, (fn, args) in cases.items():
    torch._dynamo.reset()
    _, codes = run_and_get_code(torch.compile(fn), *args)
    code = "\n".join(codes)
    clamp = re.search(r"auto (tmp\d+) = mi::clamp_index\((tmp\d+), (\d+)\)", code)
    inside = re.search(r"auto (tmp\d+) = mi::index_in_range\((tmp\d+), (\d+)\)", code)
    raw, safe, ok = clamp.group(2), clamp.group(1), inside.group(1)
    accesses = [l for l in code.splitlines() if re.search(r"mi::(gather|vload|scatter)", l) and (raw in re.findall(r"tmp\d+", l) or safe in l)]
    uses_raw = any(raw in re.findall(r"tmp\d+", l.split("=", 1)[-1]) for l in accesses)
    guarded = all(ok in l for l in accesses if "scatter" in l)
    print("CASE", name, clamp.group(3), bool(accesses), uses_raw, guarded)
'''


DRY_SHAPES = DRY_HEAD + r'''
import re
def code_of(fn, *args):
    torch._dynamo.reset()
    _, codes = run_and_get_code(torch.compile(fn), *args)
    return "\n".join(codes)
# read set above / below half of the 256 MiB memory-side cache; a weight vector does not count
big = code_of(lambda a, b: a + b, torch.zeros(36 << 20, dtype=torch.bfloat16), torch.zeros(36 << 20, dtype=torch.bfloat16))
small = code_of(lambda a, b, w: (a + b) * w, torch.zeros(8192, 4096, dtype=torch.bfloat16), torch.zeros(8192, 4096, dtype=torch.bfloat16),
                torch.zeros(4096, dtype=torch.bfloat16))
flag = lambda c: re.findall(r"constexpr bool STREAM_READS = (\w+);", c)
print("STREAM", flag(big), flag(small))
print("ORDER", "blockIdx.x & 7" in big and "gridDim.x & 7" in big, re.search(r"'grid_multiple': (\d+)", big).group(1))
col = code_of(lambda x: (x.mean(0), x.var(0, unbiased=False), x.argmax(0)), torch.randn(65536, 512))
print("COL", "mi::ColAccNone acc0" in col, re.search(r"'ws_words': (\d+)", col).group(1),
      len(re.findall(r"mi::col_fold_all<VEC, CT, RL, mi::RedWelford, mi::RedArgMax>", col)),
      "red2.mean * red2.n" in col, re.search(r"'lds_partial': (\d+)", col).group(1))
'''


def _run_dry(tmp_path, text):
    script = tmp_path / "dry_case.py"
    script.write_text(text)
    proc = subprocess.run([sys.executable, str(script), str(tmp_path / "cache"), ROOT], capture_output=True, text=True,
                          timeout=900)
    assert proc.returncode == 0, proc.stderr[-3000:]
    return proc.stdout


def test_unsupported_node_falls_back_to_eager_or_names_the_node(tmp_path, built):
    """A fused node the generator refuses: by default its ops are sent to their eager kernels and the
    graph compiles on the second attempt; with the retry off compilation ends with one error naming
    the node, the ATen op and the reason (reference inductor_x/npu_triton_heuristics.py:87-106)."""
    out = _run_dry(tmp_path, DRY_UNSUPPORTED)
    retry = next(l.split() for l in out.splitlines() if l.startswith("RETRY"))
    assert retry[1:3] == ["True", "True"] and "aten.prod" in retry[3] and "aten.mul" not in retry[3]
    assert next(l for l in out.splitlines() if l.startswith("ERROR")).split()[1:] == ["True", "True", "True"]


def test_indirect_accesses_stay_inside_their_buffer(tmp_path, built):
    """Generated embedding / index / gather loads read through a clamped copy of the index, and
    index_put / scatter stores carry the in-range predicate, so an out-of-range index cannot touch
    memory outside the buffer (the emitted source is checked; nothing is launched)."""
    out = _run_dry(tmp_path, DRY_BOUNDS)
    got = {l.split()[1]: l.split()[2:] for l in out.splitlines() if l.startswith("CASE")}
    assert set(got) == {"embedding", "index", "index_put", "scatter", "gather"}
    assert got["embedding"][0] == "100" and got["scatter"][0] == "64"
    for name, (size, found, uses_raw, guarded) in got.items():
        assert found == "True" and uses_raw == "False" and guarded == "True", (name, got[name])


def test_generated_kernel_shapes_follow_read_set_and_reduction_set(tmp_path, built):
    """Emitted source of three graphs (nothing launched): a pointwise kernel reads with the
    non-temporal hint only when its large operands exceed half the memory-side cache, it deals
    workgroups to the dies in eighths with a grid that is a multiple of 8, and the column pair of the
    third benchmark graph folds its two states in one call, takes the mean's sum from the moments
    (five partial words) and sizes its LDS for three planes of 32 x 4 columns x 5 words."""
    from inductor_x_amd.hip_heuristics import col_fold_all_planes

    out = _run_dry(tmp_path, DRY_SHAPES)
    line = {l.split()[0]: l.split(None, 1)[1] for l in out.splitlines() if l.split() and l.split()[0] in ("STREAM", "ORDER", "COL")}
    assert line["STREAM"] == "['true'] ['false']"
    assert line["ORDER"] == "True 8"
    assert line["COL"].split() == ["True", "5", "2", "True", str(col_fold_all_planes(32, 8) * 32 * 4 * 5 * 4)]
    assert [col_fold_all_planes(ct, rl) for ct, rl in ((32, 8), (64, 8), (16, 16), (64, 1), (128, 2), (32, 2))] == [3, 4, 3, 0, 1, 0]


def test_code_object_key_follows_only_the_headers_a_source_includes(monkeypatch):
    """A generated kernel includes mi/codegen.h (and through it common.h): its key moves with those
    and not with the attention headers; the compiler flags and the source text move it as well."""
    from inductor_x_amd import codecache

    gen = '#include "mi/codegen.h"\nextern "C" __global__ void k() {}\n'
    assert codecache.reachable_headers(gen) == ["codegen.h", "common.h"]
    assert "attention_v5.h" in codecache.reachable_headers(codecache.aot_source("attention_kernels.hip"))
    key = codecache.source_key(gen)
    assert key == codecache.source_key(gen) and key != codecache.source_key(gen, ("-DX=1",)) and key != codecache.source_key(gen + " ")
    real = codecache._header_text
    monkeypatch.setattr(codecache, "_header_text", lambda n: real(n) + "// edited" if n == "attention_v5.h" else real(n))
    assert codecache.source_key(gen) == key
    monkeypatch.setattr(codecache, "_header_text", lambda n: real(n) + "// edited" if n == "common.h" else real(n))
    assert codecache.source_key(gen) != key


def test_import_hook_keeps_cpu_inductor_working():
    """The table patches only act on GPU tensors: CPU compilation in the same
    process still goes through Inductor's C++ backend and matches eager."""
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "import torch, inductor_x_amd\n"
        "from torch._inductor.codegen.common import get_scheduling_for_device\n"
        "assert get_scheduling_for_device('cuda').__name__ == 'HipScheduling'\n"
        "f = torch.compile(lambda x: (x.sum(-1), x.mean(0), torch.cumsum(x, 1)))\n"
        "x = torch.randn(17, 33)\n"
        "a, b, c = f(x)\n"
        "torch.testing.assert_close(a, x.sum(-1)); torch.testing.assert_close(b, x.mean(0))\n"
        "torch.testing.assert_close(c, torch.cumsum(x, 1)); print('ok')\n" % ROOT
    )
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0 and "ok" in proc.stdout, proc.stderr[-2000:]


def test_backend_fingerprint_enters_inductor_cache_keys(monkeypatch):
    """Inductor's on-disk caches are keyed on the uuid of the backend's custom pass: it must be
    stable for unchanged sources and switches, and move with a code-generation switch."""
    import inductor_x_amd
    from torch._inductor.codegen.common import custom_backend_passes

    p = custom_backend_passes.get(inductor_x_amd.DEVICE_TYPE)
    assert p is not None
    a = p.uuid()
    assert a == p.uuid() and len(a) == 64
    monkeypatch.setenv("INDUCTOR_X_AMD_PW_TRANSPOSE", "0")
    assert p.uuid() != a
    monkeypatch.delenv("INDUCTOR_X_AMD_PW_TRANSPOSE")
    monkeypatch.setenv("INDUCTOR_X_AMD_CACHE", "/tmp/elsewhere")  # where code objects go does not change them
    assert p.uuid() == a
