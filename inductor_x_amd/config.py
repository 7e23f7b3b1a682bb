"""Backend knobs and the hardware numbers every split / tiling decision reads.

Mirrors the role of the reference's config module (reference
inductor_x/config.py:6-28): a switch the tests flip, a few forced Inductor
settings, and the core count taken from the device.  The Ascend quantities are
replaced by their CDNA4 counterparts: compute units for `num_vector_core`,
the 16-byte vector access for the 32-byte `npu_block`, plus wavefront width,
LDS size and resident-wave limits that the occupancy-aware heuristic needs.
"""
from __future__ import annotations

import dataclasses
import os

# Switch kept for interface parity; the reference's tests set it
# (reference test/npu_indexing/pointwise_test.py:8) and nothing reads it.
enable_npu_indexing = True

# Bytes moved by one lane in one global access; vector widths are derived
# from it (16 B -> 4 x fp32, 8 x bf16).
vector_bytes = 16

# Benchmark every candidate launch configuration of a kernel on first use and
# remember the fastest (analogue of the reference's cached_autotune,
# reference inductor_x/npu_triton_heuristics.py:302-435).
autotune = os.environ.get("INDUCTOR_X_AMD_AUTOTUNE", "0") == "1"

# Print per-kernel ms / GB / GB/s after each launch is timed (analogue of the
# reference's NPUDebugAutotuner, reference inductor_x/npu_triton_heuristics.py:268-299).
profile_bandwidth = os.environ.get("INDUCTOR_X_AMD_PROFILE_BANDWIDTH", "0") == "1"

# A fused node the HIP generator cannot express: send the ATen ops it came from to their eager
# kernels and lower the graph again (True), or end compilation with the generator's error (False).
retry_unsupported_with_eager = os.environ.get("INDUCTOR_X_AMD_RETRY_UNSUPPORTED", "1") == "1"

# sum of a 16-bit floating-point tensor: accumulate in fp32 and round the result back to the input
# type, which is the type eager PyTorch returns (False), or return the fp32 sum itself as the
# reference's lowering does (True; reference inductor_x/lowering.py:204-215).  True is for inference
# graphs that compare against the reference's outputs only: the buffer's type then differs from the
# type dynamo and AOTAutograd traced for the node, so a graph output, a guard or a backward pass that
# relies on the traced type can see a mismatch; the lowering applies it to inference graphs only
# (no backward graph is compiled for the function).
sum_returns_fp32 = os.environ.get("INDUCTOR_X_AMD_SUM_FP32", "0") == "1"

# Random numbers in compiled graphs (rand, randn, randint, dropout): True generates them inside the
# fused kernels with a counter-based Philox generator keyed by the graph's seed (what Inductor does
# on its own GPU backends and what the reference's Triton path does; the values then differ from
# eager's for one torch.manual_seed, and a backward pass regenerates the forward's dropout mask from
# the same seed), False calls the ATen generators as separate kernels (eager's stream, bit for bit).
generate_random = os.environ.get("INDUCTOR_X_AMD_GENERATE_RANDOM", "1") == "1"

# Generated indirect accesses (embedding, index, gather, index_put, scatter): "clamp" keeps every
# index inside its buffer (loads read the nearest valid element, stores and atomics outside the
# range are dropped), "none" uses the index as it comes, as the reference's generated code does
# unless assert_indirect_indexing is on.
indirect_bounds = os.environ.get("INDUCTOR_X_AMD_INDIRECT_BOUNDS", "clamp")

# Persistent (row held in registers) reductions are used up to this many
# elements per row (the reference's limit is 1024,
# reference inductor_x/codegen/triton.py:401-424; registers allow more here).
persistent_reduction_max = 16384

# Reduced axes longer than this, with a contiguous kept axis, are cut across
# workgroups (reference inductor_x/codegen/split_tiling.py:159-165).
outer_reduce_threshold = 32768

# Published peaks used for roofline fractions.
hbm_peak_bytes_per_s = 8.0e12
mfma_bf16_peak_flops = 2.5e15


@dataclasses.dataclass(frozen=True)
class Hardware:
    cu_count: int = 256
    xcd_count: int = 8
    wave_size: int = 64
    lds_bytes: int = 65536
    lds_bytes_per_cu: int = 160 * 1024
    max_waves_per_cu: int = 32
    max_threads_per_cu: int = 2048
    regs_per_simd: int = 512
    simds_per_cu: int = 4
    clock_khz: int = 2400000
    l2_bytes: int = 4 * 1024 * 1024
    mall_bytes: int = 256 * 1024 * 1024
    hbm_bytes: int = 288 * 1024**3
    arch: str = "gfx950"
    probed: bool = False


_hardware: Hardware | None = None


def hardware(device: int = 0) -> Hardware:
    """Device numbers from the launcher when a GPU is present, otherwise the
    MI355X data-sheet values (so heuristics stay testable on a host without one)."""
    global _hardware
    if _hardware is not None:
        return _hardware
    hw = Hardware()
    try:
        from . import launcher

        if launcher.device_count() > device:
            p = launcher.device_props(device)
            hw = dataclasses.replace(
                hw,
                cu_count=p.cu_count or hw.cu_count,
                xcd_count=p.xcd_count or hw.xcd_count,
                wave_size=p.wave_size or hw.wave_size,
                lds_bytes=p.lds_bytes or hw.lds_bytes,
                max_waves_per_cu=p.max_waves_per_cu or hw.max_waves_per_cu,
                max_threads_per_cu=p.max_threads_per_cu or hw.max_threads_per_cu,
                clock_khz=p.clock_khz or hw.clock_khz,
                l2_bytes=p.l2_bytes or hw.l2_bytes,
                mall_bytes=p.mall_bytes or hw.mall_bytes,
                hbm_bytes=p.hbm_bytes or hw.hbm_bytes,
                arch=p.arch.decode() or hw.arch,
                probed=True,
            )
    except Exception:  # no library / no device: keep data-sheet values
        pass
    _hardware = hw
    return hw


def num_compute_units() -> int:
    """Counterpart of the reference's num_vector_core (reference inductor_x/config.py:15-28)."""
    return hardware().cu_count


def apply_inductor_settings() -> None:
    """Inductor settings the reference forces at import
    (reference inductor_x/config.py:8-12).  unique_kernel_names keeps kernel
    symbols readable in profiles.  Buffer reuse stays at Inductor's default:
    the reference disables it to sidestep an aliasing issue of its own code
    generator, which does not apply here."""
    from torch._inductor import config as inductor_config

    inductor_config.triton.unique_kernel_names = True
    # one kernel that reduces the same tile along rows and along columns at once is a Triton
    # code shape (torch/_inductor/codegen/simd.py codegen_mix_order_reduction); here the row
    # reduction and the column reduction stay two kernels
    if hasattr(inductor_config.triton, "mix_order_reduction"):
        inductor_config.triton.mix_order_reduction = False


def streaming_read_bytes() -> int:
    """A generated kernel whose read set exceeds this many bytes loads with the non-temporal hint
    (it reads each element once, and a set of more than half the memory-side cache is not found
    there again by the next kernel).  INDUCTOR_X_AMD_STREAM_READS overrides the limit in bytes;
    0 switches the hint off."""
    forced = os.environ.get("INDUCTOR_X_AMD_STREAM_READS")
    if forced is not None:
        return int(forced)
    return hardware().mall_bytes // 2
