"""Launch-time side of the backend: launch configurations, the caching
launcher, grid computation and the CU/occupancy-aware split heuristic.

Counterpart of the reference's launch heuristics module
(reference inductor_x/npu_triton_heuristics.py):
  NPUCachingAutotuner.precompile / _precompile_config (:71-266) -> CachingLauncher
  cached_autotune + .best_config file (:302-435)                -> CachingLauncher.autotune
  NPUDebugAutotuner bandwidth print (:268-299)                  -> config.profile_bandwidth
  grid(*numels) (:444-464)                                      -> grid()
  triton_config_npu_index (:467-544)                            -> *_configs()
and of the split / tile choosers
(reference inductor_x/codegen/split_tiling.py:46-182,
 reference inductor_x/codegen/tile_generator.py:24-130)        -> split_reduction_plan(),
                                                                   row_reduction_plan(), ...
The reference sizes everything for `num_vector_core` persistent programs of one
"warp"; here the unit is a 64-lane wavefront, a CU holds many of them, and the
aim is enough 16-byte loads in flight per CU to cover HBM latency.
"""
from __future__ import annotations

import dataclasses
import functools
import hashlib
import json
import logging
import os
from typing import Callable, Optional, Sequence

from . import codecache, config, launcher

log = logging.getLogger(__name__)


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def next_power_of_2(n: int) -> int:
    n = max(int(n), 1)
    return 1 << (n - 1).bit_length()


def prev_power_of_2(n: int) -> int:
    n = max(int(n), 1)
    return 1 << (n.bit_length() - 1)


# ---------------------------------------------------------------------------
# Launch configuration and caching launcher
# ---------------------------------------------------------------------------
@dataclasses.dataclass
class LaunchConfig:
    """One way to run a kernel: which symbol, workgroup shape, how the grid and
    the dynamic LDS size follow from the call's numels.  `meta` carries the
    compile-time parameters the symbol was instantiated with (the analogue of a
    Triton Config's kwargs, e.g. XBLOCK / RBLOCK in the reference)."""

    symbol: str
    block: int
    meta: dict = dataclasses.field(default_factory=dict)
    defines: dict = dataclasses.field(default_factory=dict)
    lds_bytes: int = 0

    def key(self) -> str:
        return json.dumps([self.symbol, self.block, self.meta, self.defines, self.lds_bytes], sort_keys=True)


def grid(*numels: int) -> Callable[[dict], tuple]:
    """grid(numel0[, numel1[, numel2]]) -> fn(meta) -> (g0, g1, g2).

    Same call shape as the reference's helper
    (reference inductor_x/npu_triton_heuristics.py:444-464).  Axis k is covered
    by cdiv(numel_k, meta["PER_WG<k>"]) workgroups (PER_WG defaults to 1)."""

    def fn(meta: dict) -> tuple:
        g = [1, 1, 1]
        for k, n in enumerate(numels[:3]):
            per = int(meta.get(f"PER_WG{k}", 1))
            g[k] = max(cdiv(int(n), per), 1)
        return tuple(g)

    return fn


class CachingLauncher:
    """Compiles (or fetches) a kernel's code object, keeps the usable launch
    configurations, optionally times them once, and launches the chosen one.

    Behaviour carried over from the reference's NPUCachingAutotuner:
      - configs are tried in order and those that fail to build or resolve are
        dropped; it is an error only if none survive (:71-107);
      - with more than one survivor and autotuning on, each is timed on the
        first call and the winner is remembered in a `.best_config` JSON next to
        the code object (:372-390);
      - run(*args, grid=, stream=) enqueues on the given raw stream and never
        synchronises (:239-253).
    """

    def __init__(
        self,
        name: str,
        source: str,
        signature: str,
        configs: Sequence[LaunchConfig],
        bytes_fn: Optional[Callable[..., int]] = None,
        prefer_intree: bool = False,
    ):
        self.name = name
        self.source = source
        self.signature = signature
        self.configs = list(configs)
        self.bytes_fn = bytes_fn
        self.prefer_intree = prefer_intree
        self.launchers: list[tuple[LaunchConfig, launcher.Function]] = []
        self._best: Optional[int] = None
        self._modules: dict[str, launcher.Module] = {}
        self._hsaco_path: Optional[str] = None

    # -- compile / load ----------------------------------------------------
    def _module_for(self, cfg: LaunchConfig) -> launcher.Module:
        flags = tuple(f"-D{k}={v}" for k, v in sorted(cfg.defines.items()))
        key = "|".join(flags)
        mod = self._modules.get(key)
        if mod is None:
            path = codecache.compile_source(
                self.source, label=self.name, extra_flags=flags, prefer_intree=self.prefer_intree
            )
            self._hsaco_path = path
            with open(path, "rb") as f:
                mod = launcher.Module(f.read(), label=f"{self.name}[{os.path.basename(path)}]")
            self._modules[key] = mod
        return mod

    def precompile(self) -> None:
        if self.launchers:
            return
        errors = []
        for cfg in self.configs:
            try:
                fn = self._module_for(cfg).function(cfg.symbol)
            except (codecache.CompileError, launcher.LauncherError) as e:
                errors.append(f"{cfg.symbol}: {e}")
                log.debug("dropping launch config %s of %s: %s", cfg.symbol, self.name, e)
                continue
            self.launchers.append((cfg, fn))
        if not self.launchers:
            raise RuntimeError(f"No valid launch configuration for kernel {self.name}:\n" + "\n".join(errors))
        if len(self.launchers) == 1:
            self._best = 0
        else:
            self._best = self._load_best()

    # -- best-config persistence ------------------------------------------
    def _configs_hash(self) -> str:
        h = hashlib.sha256()
        for cfg in self.configs:
            h.update(cfg.key().encode())
        return h.hexdigest()[:16]

    def _best_path(self) -> Optional[str]:
        return (self._hsaco_path[: -len(".hsaco")] + ".best_config") if self._hsaco_path else None

    def _load_best(self) -> Optional[int]:
        p = self._best_path()
        if not p or not os.path.exists(p):
            return None
        try:
            with open(p) as f:
                rec = json.load(f)
        except (OSError, ValueError):
            return None
        if rec.get("configs_hash") != self._configs_hash():
            return None
        for i, (cfg, _) in enumerate(self.launchers):
            if cfg.symbol == rec.get("symbol") and cfg.defines == rec.get("defines", {}):
                return i
        return None

    def _save_best(self, idx: int, timings_ms: dict) -> None:
        p = self._best_path()
        if not p:
            return
        cfg = self.launchers[idx][0]
        rec = {
            "symbol": cfg.symbol,
            "block": cfg.block,
            "defines": cfg.defines,
            **cfg.meta,
            "configs_hash": self._configs_hash(),
            "timings_ms": timings_ms,
        }
        try:
            with open(p, "w") as f:
                json.dump(rec, f)
        except OSError:
            pass

    # -- launch -------------------------------------------------------------
    def _launch(self, idx: int, args, grid_arg, stream: int) -> None:
        cfg, fn = self.launchers[idx]
        g = grid_arg(cfg.meta) if callable(grid_arg) else grid_arg
        fn.launch(self.signature, args, g, (cfg.block,), stream, cfg.lds_bytes)

    def _launch_on_library_scratch(self, idx: int, args, scratch_arg: int, scratch_bytes: int, grid_arg, stream: int) -> None:
        """_launch with pointer parameter `scratch_arg` supplied by the launcher library's fixed
        per-GPU scratch array (nothing is allocated)."""
        cfg, fn = self.launchers[idx]
        g = grid_arg(cfg.meta) if callable(grid_arg) else grid_arg
        fn.launch_with_library_scratch(self.signature, args, scratch_arg, scratch_bytes, g, (cfg.block,), stream, cfg.lds_bytes)

    def bench(self, idx: int, args, grid_arg, stream: int, warmup: int = 3, rep: int = 10) -> float:
        """Average milliseconds per launch of configuration idx, timed with
        events on torch's current stream (which must be `stream`)."""
        import torch

        for _ in range(warmup):
            self._launch(idx, args, grid_arg, stream)
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(rep):
            self._launch(idx, args, grid_arg, stream)
        end.record()
        end.synchronize()
        return start.elapsed_time(end) / rep

    def autotune(self, args, grid_arg, stream: int) -> int:
        timings = {}
        best, best_ms = 0, float("inf")
        for i, (cfg, _) in enumerate(self.launchers):
            try:
                ms = self.bench(i, args, grid_arg, stream)
            except launcher.LauncherError as e:
                log.debug("config %s of %s failed to launch: %s", cfg.symbol, self.name, e)
                continue
            timings[cfg.symbol] = ms
            if ms < best_ms:
                best, best_ms = i, ms
        self._save_best(best, timings)
        return best

    def pick(self, shape_key: str, default_idx: int, eligible: Sequence[int], args, grid_arg, stream: int) -> int:
        """Configuration for one problem shape of a kernel family whose best variant depends on the
        extents: the heuristic's `default_idx` unless config.autotune is on; then the fastest of
        `eligible`, timed once per shape (outputs are overwritten with the same values by every
        variant) and remembered in `<code object>.<shape_key>.best_config` for later processes."""
        if not config.autotune or len(eligible) < 2:
            return default_idx
        tuned = self.__dict__.setdefault("_tuned", {})
        idx = tuned.get(shape_key)
        if idx is not None:
            return idx
        import torch

        if torch.cuda.is_current_stream_capturing():
            return default_idx
        path = (self._hsaco_path[: -len(".hsaco")] + f".{shape_key}.best_config") if self._hsaco_path else None
        symbols = {cfg.symbol: i for i, (cfg, _) in enumerate(self.launchers)}
        if path and os.path.exists(path):
            try:
                with open(path) as f:
                    rec = json.load(f)
                if rec.get("symbol") in symbols and symbols[rec["symbol"]] in eligible:
                    tuned[shape_key] = symbols[rec["symbol"]]
                    return tuned[shape_key]
            except (OSError, ValueError):
                pass
        timings, best, best_ms = {}, default_idx, float("inf")
        for i in eligible:
            try:
                ms = self.bench(i, args, grid_arg, stream, warmup=5, rep=20)
            except launcher.LauncherError as e:
                log.debug("config %s of %s failed to launch: %s", self.launchers[i][0].symbol, self.name, e)
                continue
            timings[self.launchers[i][0].symbol] = ms
            if ms < best_ms:
                best, best_ms = i, ms
        tuned[shape_key] = best
        if path:
            try:
                with open(path, "w") as f:
                    json.dump({"symbol": self.launchers[best][0].symbol, "shape": shape_key, "timings_ms": timings}, f)
            except OSError:
                pass
        return best

    def run(self, *args, grid, stream: int) -> None:
        if not self.launchers:
            self.precompile()
        if self._best is None:
            self._best = self.autotune(args, grid, stream) if config.autotune else 0
        self._launch(self._best, args, grid, stream)
        if config.profile_bandwidth and self.bytes_fn is not None:
            ms = self.bench(self._best, args, grid, stream, warmup=1, rep=5)
            nbytes = self.bytes_fn(*args)
            print(f"{self.name}: {ms:.4f} ms  {nbytes / 1e9:.4f} GB  {nbytes / 1e6 / ms:.1f} GB/s")

    def select(self, symbol: str) -> None:
        """Pin the configuration with the given symbol (used by sweeps and tests)."""
        if not self.launchers:
            self.precompile()
        for i, (cfg, _) in enumerate(self.launchers):
            if cfg.symbol == symbol:
                self._best = i
                return
        raise KeyError(f"{self.name}: no launch configuration {symbol}")

    def best_config(self) -> LaunchConfig:
        if not self.launchers:
            self.precompile()
        return self.launchers[self._best or 0][0]


# ---------------------------------------------------------------------------
# Heuristics
# ---------------------------------------------------------------------------
def vector_width(elem_bytes: int, *extents_and_strides: int) -> int:
    """Largest element count per lane access (<= 16 bytes) that divides every
    given extent/stride/offset, so every vector stays aligned and in range.
    Counterpart of the reference's 32-byte block alignment rule
    (reference inductor_x/codegen/triton_utils.py:22-27)."""
    vec = max(config.vector_bytes // elem_bytes, 1)
    while vec > 1 and any(int(e) % vec for e in extents_and_strides):
        vec //= 2
    return vec


# Bytes a CU wants in flight to cover HBM latency at full bandwidth:
# 8 TB/s * ~2 us / 256 CUs.
_BYTES_IN_FLIGHT_PER_CU = 64 * 1024


def waves_per_cu_target(unroll: int, vgprs: int = 64, hw: Optional[config.Hardware] = None) -> int:
    """Resident wavefronts per CU needed so that waves * 64 lanes * 16 B * unroll
    covers the in-flight byte target, capped by what the register file allows."""
    hw = hw or config.hardware()
    need = cdiv(_BYTES_IN_FLIGHT_PER_CU, hw.wave_size * config.vector_bytes * max(unroll, 1))
    reg_limit = max(hw.regs_per_simd // max(vgprs, 1), 1) * hw.simds_per_cu
    return max(min(need, reg_limit, hw.max_waves_per_cu), 1)


@dataclasses.dataclass(frozen=True)
class RowPlan:
    block: int  # threads per workgroup
    tpr: int  # threads cooperating on one row
    vec: int  # elements per lane access
    iters: int  # vectors per thread (persistent form) or 0 (looped form)
    rows_per_wg: int


@functools.lru_cache(maxsize=4096)
def row_reduction_plan(xnumel: int, rnumel: int, elem_bytes: int, persistent: bool) -> RowPlan:
    """Thread mapping for a last-dimension reduction.

    One row gets as many threads as it has 16-byte vectors, up to a whole
    256-thread workgroup; shorter rows share a workgroup so wavefronts stay
    full.  Replaces the reference's XBLOCK / XBLOCK_SUB / RBLOCK sweep
    (reference inductor_x/codegen/tile_generator.py:38-130)."""
    vec = vector_width(elem_bytes, rnumel)
    vectors = cdiv(rnumel, vec)
    block = 256
    if persistent:
        # one vector per thread while a row fits 512 threads (measured fastest on
        # MI355X: most loads in flight per byte of register state), more beyond
        tpr = min(next_power_of_2(vectors), 512)
        block = max(block, tpr)
        iters = cdiv(vectors, tpr)
    else:
        tpr = min(next_power_of_2(vectors), block)
        iters = 0
    return RowPlan(block=block, tpr=tpr, vec=vec, iters=iters, rows_per_wg=block // tpr)


def col_fold_all_planes(ct: int, rl: int, wave: int = 64) -> int:
    """LDS planes of the generated column sweep's fold over row lanes (mi::col_fold_all computes
    the same number on the device): row lanes that share a wavefront meet through lane exchanges,
    the remaining groups are halved through LDS while more than four are left, then collected in
    one round.  One plane is CT * VEC * (words of all reduction states) floats."""
    in_wave = min(wave // ct, rl) if ct < wave else 1
    groups = rl // max(in_wave, 1)
    if groups <= 1:
        return 0
    tree = groups // 2 if groups > 4 else 0
    last = min(groups, 4) - 1
    return max(tree, last)


def col_fold_lds_bytes(ct: int, rl: int, wave: int = 64) -> int:
    """Dynamic LDS of the hand-written column sweep's fold over row lanes: row lanes that share a
    wavefront meet through lane exchanges, the remaining groups are halved through LDS while more than
    four are left and then collected in one round (the device side computes the same number,
    col_fold_planes in csrc/mi/col.h)."""
    in_wave = min(wave // ct, rl) if ct < wave else 1
    groups = rl // max(in_wave, 1)
    if groups <= 1:
        return 0
    tree = groups // 2 if groups > 4 else 0
    last = min(groups, 4) - 1
    return max(tree, last) * ct * 4 * 5 * 4


@dataclasses.dataclass(frozen=True)
class SplitPlan:
    ct: int  # threads across the kept (contiguous) axis, 4 elements each
    rl: int  # row lanes per workgroup
    unroll: int
    nsplit: int  # workgroups along the reduced axis
    rows_per_split: int
    col_tiles: int
    prefetch: int = 2  # batches of `unroll` loads a thread holds (one being folded, the others in flight)

    @property
    def block(self) -> int:
        return self.ct * self.rl

    @property
    def lds_bytes(self) -> int:
        return col_fold_lds_bytes(self.ct, self.rl)

    def workspace_floats(self, cols: int) -> int:
        # mean, M2, best value, best row per (split, column); the row count is implied by the geometry
        return 4 * self.nsplit * cols


def split_reduction_plan(
    rows: int,
    cols: int,
    elem_bytes: int = 4,
    vgprs: int = 48,
    unroll: int = 8,
    hw: Optional[config.Hardware] = None,
    max_workspace_frac: float = 0.05,
) -> SplitPlan:
    """CU/occupancy-aware split factor for a column reduction (rows reduced,
    cols kept and contiguous).

    The reference cuts the reduced axis only above 32768 elements and then into
    about one slice per vector core (reference
    inductor_x/codegen/split_tiling.py:159-182).  Here:
      1. the number of wavefronts wanted per CU comes from the in-flight-bytes
         target and the kernel's register budget (waves_per_cu_target); measured
         on MI355X at [65536, 512], first pass alone: the same bytes in flight from
         half as many wavefronts with twice the unrolled batch (4 per CU, 2 x 8
         loads each: 22.3 us) do as well as 8 per CU with 2 x 4 loads (22.3 us) and
         better than 16 per CU (25.3 us), and fewer wavefronts mean fewer partials;
      2. a workgroup spans only 128 kept elements (32 threads x float4, runs of
         512 bytes per row) and as many row lanes as make up those wavefronts, so
         the kept axis is cut into many column tiles and the reduced axis into few
         splits: the partials a column has are what the second pass must fold, and
         their number is the workgroup count divided by the column tiles.  Measured
         at [65536, 512], both passes: 32 x 8 threads in 4 tiles x 64 splits 25.3 us,
         64 x 4 in 2 x 128 26.0 us, 128 x 2 in 1 x 256 27.1 us (at 2 KiB rows the
         narrower tiles cost the sweep nothing);
      3. nsplit is the smallest count that gives every CU that many wavefronts,
         rounded to a multiple of the CU count so the last round of workgroups
         is full, then capped so that writing and re-reading the partials stays
         below `max_workspace_frac` of the input bytes and every thread keeps at
         least one unrolled batch of rows;
      4. rows_per_split is rounded up to a whole number of unrolled batches.
    """
    hw = hw or config.hardware()
    vec = 4
    ct = min(next_power_of_2(cdiv(cols, vec)), 32)
    col_tiles = cdiv(cols, ct * vec)
    # the kernel keeps two batches of `unroll` loads in flight (software pipeline)
    waves_cu = waves_per_cu_target(2 * unroll, vgprs, hw)
    wg_threads = min(max(waves_cu * hw.wave_size, ct), 1024)
    rl = max(min(wg_threads // ct, prev_power_of_2(max(rows // unroll, 1))), 1)
    waves_per_wg = max(ct * rl // hw.wave_size, 1)
    want_waves = hw.cu_count * waves_cu
    nsplit = cdiv(want_waves, waves_per_wg * col_tiles)
    if nsplit * col_tiles > hw.cu_count:
        per = max(hw.cu_count // col_tiles, 1)
        nsplit = cdiv(nsplit, per) * per
    # workspace traffic cap: 2 * nsplit * cols * 16 B <= frac * rows * cols * elem_bytes
    cap_ws = int(max_workspace_frac * rows * elem_bytes / 32)
    # every thread should own at least one unrolled batch
    cap_rows = rows // (rl * unroll)
    nsplit = max(min(nsplit, max(cap_ws, 1), max(cap_rows, 1)), 1)
    batch = rl * unroll
    rows_per_split = cdiv(cdiv(rows, nsplit), batch) * batch
    nsplit = cdiv(rows, rows_per_split)
    return SplitPlan(ct=ct, rl=rl, unroll=unroll, nsplit=nsplit, rows_per_split=rows_per_split, col_tiles=col_tiles)


def pointwise_plan(numel: int, elem_bytes: int, inner_extent: int) -> tuple[int, int]:
    """(block, vec) for a flat pointwise kernel whose innermost contiguous run is
    `inner_extent` elements long."""
    vec = vector_width(elem_bytes, inner_extent, numel)
    return 256, vec


# ---------------------------------------------------------------------------
# Kernels emitted by the Inductor code generator
# ---------------------------------------------------------------------------
def split_factor(rows: int, cols: int, ct: int, rl: int, vec: int, elem_bytes: int = 4, unroll: int = 4,
                 words: int = 5, hw: Optional[config.Hardware] = None) -> tuple[int, int]:
    """(nsplit, rows_per_split) for a generated column kernel whose workgroup
    shape (ct x rl threads, vec columns per thread) is already fixed.  Same
    rules as split_reduction_plan."""
    hw = hw or config.hardware()
    col_tiles = cdiv(cols, ct * vec)
    waves_per_wg = max(ct * rl // hw.wave_size, 1)
    want_waves = hw.cu_count * waves_per_cu_target(2 * unroll, 64, hw)
    nsplit = cdiv(want_waves, waves_per_wg * col_tiles)
    if nsplit * col_tiles > hw.cu_count:
        per = max(hw.cu_count // col_tiles, 1)
        nsplit = cdiv(nsplit, per) * per
    cap_ws = int(0.05 * rows * elem_bytes / (8 * max(words, 1)))
    cap_rows = rows // (rl * unroll)
    nsplit = max(min(nsplit, max(cap_ws, 1), max(cap_rows, 1)), 1)
    batch = rl * unroll
    rows_per_split = cdiv(cdiv(rows, nsplit), batch) * batch
    return cdiv(rows, rows_per_split), rows_per_split


_DRYRUN = os.environ.get("INDUCTOR_X_AMD_DRYRUN", "0") == "1"


# Row kernels walk the rows with the stride of the grid, so any grid is valid.  One workgroup per
# round of rows is the rule: measured on MI355X, capping the grid (workgroups looping over rounds
# far apart) gains under 5 % on plain short-row reductions and loses 25-50 % where the kernel also
# writes a permuted output, because rows written close in time are then far apart in memory.  The
# cap only keeps the grid dimension in range.
_ROW_GRID_FREE = 1 << 22
_ROW_GRID_WAVES_OF_WORKGROUPS = 4


def row_grid(rounds: int) -> int:
    if rounds <= _ROW_GRID_FREE or os.environ.get("INDUCTOR_X_AMD_ROW_GRID_CAP", "1") == "0":
        return max(rounds, 1)
    hw = config.hardware()
    return min(rounds, hw.cu_count * 8 * int(os.environ.get("INDUCTOR_X_AMD_ROW_GRID_WAVES", _ROW_GRID_WAVES_OF_WORKGROUPS)))


_pool = None


def _compile_pool():
    global _pool
    if _pool is None:
        from concurrent.futures import ThreadPoolExecutor

        workers = int(os.environ.get("INDUCTOR_X_AMD_COMPILE_THREADS", "0")) or min(16, os.cpu_count() or 4)
        _pool = ThreadPoolExecutor(max_workers=workers, thread_name_prefix="mi-hipcc")
    return _pool


class LaunchPlan:
    """Everything one (kernel, extents) pair needs at launch, computed once: which entry points,
    their grids, the split of a column reduction and its workspace size."""

    __slots__ = ("steps", "ws_floats", "candidate")

    def __init__(self, steps, ws_floats: int, candidate: dict):
        self.steps = steps  # [(function key, grid, block, lds bytes, tail of scalar arguments, takes workspace)]
        self.ws_floats = ws_floats
        self.candidate = candidate


class GeneratedKernel:
    """Run-time side of one generated kernel: compiles (or fetches) its code
    object on first use and launches it through the C-ABI launcher.  This is the
    object the generated wrapper calls, in the place of the reference's
    `kernel.run(*args, grid=grid(...), stream=stream0)`
    (reference test/npu_indexing/issue61_test.py:62).

    Per extents the launch geometry is planned once and kept (grids, the split of a column
    reduction, its workspace).  Where the geometry is a run-time choice there are a few candidates
    (the grid of a row kernel, which walks its rows with the stride of the grid; the split count of
    a column pair): the first is the heuristic's, and with config.autotune on all are timed on the
    first call and the winner is written next to the code object as
    `<code object>.<xnumel>x<rnumel>.best_config`, which later objects and processes read instead
    of timing again (reference inductor_x/npu_triton_heuristics.py:302-435).  With
    config.profile_bandwidth on, every planned launch is timed once more and
    `name: ms  GB  GB/s` is printed (reference :268-299)."""

    def __init__(self, name: str, meta: dict, source: str):
        self.name = name
        self.meta = dict(meta)
        self.source = source
        self.mode = meta["mode"]
        self._fns: Optional[dict] = None
        self._plans: dict = {}
        self.hsaco_path: Optional[str] = None
        # hipcc starts as soon as the wrapper module defines the kernel, in a worker thread (the
        # compiler is a subprocess), so the kernels of a graph build side by side instead of one
        # after the other at their first launches (the reference compiles inside precompile(),
        # reference inductor_x/npu_triton_heuristics.py:71-109, which Inductor's AsyncCompile
        # calls from its worker pool)
        self._pending = _compile_pool().submit(codecache.compile_source, source, label=name)

    # -- what Inductor's AsyncCompile asks of a kernel object (its worker pool compiles the kernels of
    #    a benchmark module and sends the objects back pickled; reference
    #    inductor_x/npu_triton_heuristics.py:53-109 is the same protocol on the reference's side) ------
    autotune_cache_info = None

    def set_compile_info(self, compile_id=None, is_backward: bool = False) -> None:
        self.compile_id, self.is_backward = compile_id, is_backward

    def prepare_for_pickle(self):
        return None

    def restore_after_unpickle(self, old_values=None) -> None:
        return None

    def __getstate__(self):
        # the code object is on disk by now; module handles and the pending compile stay behind
        self._pending.result()
        return {"name": self.name, "meta": self.meta, "source": self.source}

    def __setstate__(self, state):
        self.__init__(state["name"], state["meta"], state["source"])

    def precompile(self, warm_cache_only: bool = False, **_unused) -> None:
        if self._fns is not None:
            return
        path = self._pending.result()
        self.hsaco_path = path
        if warm_cache_only:  # a compile worker: the code object is in the store, nothing to load
            return
        if _DRYRUN:
            self._fns = {}
            return
        with open(path, "rb") as f:
            mod = launcher.Module(f.read(), label=self.name)
        if self.mode == "col":
            self._fns = {"partial": mod.function(self.name + "_partial"), "final": mod.function(self.name + "_final"),
                         "direct": mod.function(self.name + "_direct")}
        else:
            self._fns = {"main": mod.function(self.name)}
        self._module = mod

    @staticmethod
    def _raw(a):
        if hasattr(a, "data_ptr"):
            return a.data_ptr()
        # numbers that are kernel arguments themselves (sizes, values of 0-d CPU tensors)
        return a if isinstance(a, float) else int(a)

    # -- launch geometry ------------------------------------------------------
    def candidates(self, xnumel: int, rnumel: int) -> list:
        """Run-time choices for these extents, the heuristic's first."""
        m = self.mode
        if m == "row":
            rounds = cdiv(xnumel, self.meta["block"] // self.meta["tpr"])
            cu = config.hardware().cu_count
            caps = [None] + [c for c in (cu * 16, cu * 8) if c < rounds]
            return [{"grid_cap": c} for c in caps]
        if m == "col":
            mm = self.meta
            base, _ = split_factor(rnumel, xnumel, mm["ct"], mm["rl"], mm["vec"], unroll=mm.get("col_unroll", 4),
                                   words=mm["ws_words"])
            out = []
            for n in (base, max(base // 2, 1), base * 2):
                n = min(n, max(rnumel // (mm["rl"] * mm.get("col_unroll", 4)), 1))
                if n >= 1 and {"nsplit": n} not in out:
                    out.append({"nsplit": n})
            return out
        return [{}]

    def _plan(self, xnumel: int, rnumel: int, cand: dict) -> LaunchPlan:
        m = self.meta
        if self.mode == "pointwise":
            # a tiled kernel (static shapes) carries its own workgroup count
            g = m["grid"] if "grid" in m else cdiv(xnumel, m["block"] * m["vec"] * m.get("unroll", 1))
            mult = int(m.get("grid_multiple", 1))  # the kernel deals workgroups out to the dies itself
            padded = cdiv(g, mult) * mult
            # up to mult - 1 extra workgroups compute a start index before their bounds check: keep the
            # exact count (the kernel then takes the plain workgroup order) when that index would
            # leave the kernel's index type
            if padded * m["block"] * m["vec"] * m.get("unroll", 1) >= 2 ** (int(m.get("index_bits", 64)) - 1):
                padded = g
            grid = (padded, 1, 1)
            return LaunchPlan([("main", grid, (m["block"],), 0, (xnumel,), False)], 0, cand)
        if self.mode == "row":
            rounds = cdiv(xnumel, m["block"] // m["tpr"])
            g = row_grid(rounds)
            if cand.get("grid_cap"):
                g = min(g, int(cand["grid_cap"]))
            return LaunchPlan([("main", (g, 1, 1), (m["block"],), m.get("lds_bytes", 0), (xnumel, rnumel), False)], 0, cand)
        if self.mode == "colloop":
            grid = (cdiv(xnumel, m["ct"] * m["vec"]), 1, 1)
            return LaunchPlan([("main", grid, (m["block"],), m["lds_bytes"], (xnumel, rnumel), False)], 0, cand)
        nsplit = int(cand["nsplit"])
        tiles = cdiv(xnumel, m["ct"] * m["vec"])
        if nsplit == 1:
            # one sweep that finishes in place: no workspace, no second kernel
            return LaunchPlan([("direct", (tiles, 1, 1), (m["block"],), m["lds_partial"], (0, xnumel, rnumel, 1), False)], 0, cand)
        tail = (xnumel, rnumel, nsplit)
        return LaunchPlan(
            [("partial", (tiles, nsplit, 1), (m["block"],), m["lds_partial"], tail, True),
             ("final", (cdiv(xnumel, m["cpw"]), 1, 1), (m["cpw"] * m["sl"],), 0, tail, True)],
            m["ws_words"] * nsplit * xnumel, cand,
        )

    def _workspace(self, args, floats: int):
        """fp32 workspace of a column pair, from torch's caching allocator on every call (a block
        handed back by the previous call as a rule).  A buffer kept across calls would outlive the
        memory pools that HIP-graph capture of a compiled module (mode="reduce-overhead") checks for
        stray live storage."""
        import torch

        dev = next(a.device for a in args if hasattr(a, "device"))
        return torch.empty(floats, dtype=torch.float32, device=dev)

    def _launch_plan(self, plan: LaunchPlan, args, raw, stream: int) -> None:
        sig = self.meta["signature"]
        ws = self._workspace(args, plan.ws_floats) if plan.ws_floats else None
        ws_ptr = ws.data_ptr() if ws is not None else None
        for key, grid, block, lds, tail, takes_ws in plan.steps:
            full = raw + ((ws_ptr,) if takes_ws else ()) + tail
            self._fns[key].launch(sig, full, grid, block, stream, lds)

    # -- best-configuration record ------------------------------------------
    def _best_path(self, xnumel: int, rnumel: int) -> Optional[str]:
        if not self.hsaco_path:
            return None
        return f"{self.hsaco_path[:-len('.hsaco')]}.{xnumel}x{rnumel}.best_config"

    def _load_best(self, xnumel: int, rnumel: int, cands: list) -> Optional[dict]:
        p = self._best_path(xnumel, rnumel)
        if not p or not os.path.exists(p):
            return None
        try:
            with open(p) as f:
                rec = json.load(f)
        except (OSError, ValueError):
            return None
        if rec.get("candidates") != cands or rec.get("best") not in cands:
            return None
        return rec["best"]

    def _autotune(self, xnumel: int, rnumel: int, cands: list, args, raw, stream: int) -> dict:
        timings = []
        for cand in cands:
            plan = self._plan(xnumel, rnumel, cand)
            try:
                timings.append(self._time(plan, args, raw, stream, warmup=2, rep=5))
            except launcher.LauncherError as e:
                log.debug("candidate %s of %s failed to launch: %s", cand, self.name, e)
                timings.append(float("inf"))
        best = cands[timings.index(min(timings))]
        p = self._best_path(xnumel, rnumel)
        if p:
            try:
                with open(p, "w") as f:
                    json.dump({"kernel": self.name, "mode": self.mode, "xnumel": xnumel, "rnumel": rnumel,
                               "candidates": cands, "timings_ms": timings, "best": best}, f)
            except OSError:
                pass
        return best

    def _time(self, plan: LaunchPlan, args, raw, stream: int, warmup: int, rep: int) -> float:
        """Milliseconds per call of the plan, with events on torch's current stream (which the
        wrapper's raw stream is)."""
        import torch

        private = self._args_to_copy(args)
        if private:
            # in-place operands, targets of accumulating stores and outputs that share memory with an
            # input (a mutated graph input arrives as both): time on copies, the caller's buffers see
            # exactly one launch (reference inductor_x/npu_triton_heuristics.py:395-429 hands its
            # tuner the mutated argument names for the same reason)
            args = list(args)
            for i in private:
                t = args[i]  # same sizes and strides as the original: the kernel's index arithmetic is baked in
                args[i] = torch.empty_strided(t.size(), t.stride(), dtype=t.dtype, device=t.device).copy_(t)
            args = tuple(args)
            raw = tuple(self._raw(a) for a in args)
        for _ in range(warmup):
            self._launch_plan(plan, args, raw, stream)
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(rep):
            self._launch_plan(plan, args, raw, stream)
        end.record()
        end.synchronize()
        return start.elapsed_time(end) / rep

    def _args_to_copy(self, args) -> list:
        """Positions of the tensor arguments a repeated launch would change the result of: buffers
        the kernel reads and writes (in-place operands, accumulation targets), and written buffers
        whose memory overlaps another argument's."""
        is_t = lambda a: hasattr(a, "data_ptr") and hasattr(a, "untyped_storage")  # noqa: E731
        out = {i for i in self.meta.get("mutated_args", ()) if i < len(args) and is_t(args[i])}
        span = {}
        for i, a in enumerate(args):
            if is_t(a) and a.numel() > 0:
                st = a.untyped_storage()
                span[i] = (st.data_ptr(), st.data_ptr() + st.nbytes())
        for i in self.meta.get("written_args", ()):
            if i in span and any(j != i and span[j][0] < span[i][1] and span[i][0] < span[j][1] for j in span):
                out.add(i)
        return sorted(out)

    def num_bytes(self, args) -> int:
        """Bytes of every tensor argument, read or written once: the figure the reference's
        bandwidth print divides by (reference inductor_x/npu_triton_heuristics.py:282-299)."""
        return sum(a.numel() * a.element_size() for a in args if hasattr(a, "data_ptr"))

    def run(self, *args, xnumel: int, r0_numel: int = 1, stream: int = 0) -> None:
        self.precompile()
        if _DRYRUN:
            return
        xnumel, rnumel = int(xnumel), int(r0_numel)
        if xnumel == 0:
            return
        raw = tuple(self._raw(a) for a in args)
        key = (xnumel, rnumel)
        plan = self._plans.get(key)
        if plan is None:
            import torch

            cands = self.candidates(xnumel, rnumel)
            best = cands[0]
            if len(cands) > 1:
                best = self._load_best(xnumel, rnumel, cands) or best
                if config.autotune and best is cands[0] and not torch.cuda.is_current_stream_capturing() \
                        and self._load_best(xnumel, rnumel, cands) is None:
                    best = self._autotune(xnumel, rnumel, cands, args, raw, stream)
            plan = self._plan(xnumel, rnumel, best)
            self._plans[key] = plan
            if config.profile_bandwidth and not torch.cuda.is_current_stream_capturing():
                ms = self._time(plan, args, raw, stream, warmup=1, rep=5)
                nbytes = self.num_bytes(args)
                print(f"{self.name}: {ms:.4f} ms  {nbytes / 1e9:.4f} GB  {nbytes / 1e6 / ms:.1f} GB/s")
        self._launch_plan(plan, args, raw, stream)


def generated_kernel(name: str, meta: dict, source: str) -> GeneratedKernel:
    return GeneratedKernel(name, meta, source)
