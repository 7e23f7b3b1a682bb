/*
 * mi355_launcher.h -- C ABI of the MI355X (gfx950) kernel launcher.
 *
 * This is the process->device boundary of the backend.  The reference has no
 * FFI of its own: its boundary is a Python closure generated per kernel,
 *     launcher(*args, grid, stream):  bin[g0, g1, g2](*args, stream=stream)
 * (reference inductor_x/npu_triton_heuristics.py:239-253), fed by
 * triton.compile + binary._init_handles() (:195-199) and by the raw stream
 * handle returned from get_current_raw_stream (inductor_x/__init__.py:26-27).
 * The functions below are what an FFI for that closure binds to on ROCm:
 * load a code object, look a kernel up, enqueue it on a raw hipStream_t.
 *
 * Conventions
 *   - Every function returns a hipError_t value as int (0 == hipSuccess),
 *     except mi_error_string / mi_abi_version.  Nothing throws across the ABI.
 *   - Handles are opaque pointers owned by the library's caller; a module
 *     handle stays valid until mi_module_unload.  Code-object bytes are copied
 *     by the HIP runtime during mi_module_load and may be freed afterwards.
 *   - Device buffers are borrowed for the duration of the enqueue only; the
 *     caller keeps them alive until the stream has run the kernel.
 *   - mi_launch* never synchronise the stream or the device and take no
 *     library-wide lock; they may be called from any thread.
 */
#ifndef MI355_LAUNCHER_H
#define MI355_LAUNCHER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_ABI_VERSION 2

/* Hardware numbers the split/tiling heuristics consume.  Replaces the
 * reference's num_aicore / num_vector_core / npu_block knobs
 * (reference inductor_x/config.py:15-28). */
typedef struct mi_device_props {
  int32_t cu_count;          /* compute units (256 on MI355X)                  */
  int32_t xcd_count;         /* accelerator dies; each has its own L2          */
  int32_t wave_size;         /* lanes per wavefront (64)                        */
  int32_t lds_bytes;         /* LDS per workgroup, bytes                        */
  int32_t max_threads_per_cu;/* resident threads per CU                         */
  int32_t max_waves_per_cu;  /* max_threads_per_cu / wave_size                  */
  int32_t regs_per_cu;       /* 32-bit VGPR entries per CU                      */
  int32_t clock_khz;         /* peak shader clock                               */
  int32_t mem_clock_khz;     /* peak memory clock                               */
  int32_t mem_bus_bits;      /* memory bus width                                */
  int64_t l2_bytes;          /* L2 size as reported by the runtime              */
  int64_t hbm_bytes;         /* total device memory                             */
  int64_t mall_bytes;        /* memory-side cache (Infinity Cache) in front of
                                HBM: summed level-3 entries of the device's KFD
                                topology node, 0 when the topology is unreadable */
  char    arch[64];          /* gcnArchName, e.g. "gfx950:sramecc+:xnack-"      */
} mi_device_props;

/* Per-kernel resource usage, read back after load; feeds the occupancy-aware
 * part of the split heuristic. */
typedef struct mi_function_attrs {
  int32_t num_regs;           /* VGPRs per lane                                 */
  int32_t static_lds_bytes;   /* LDS the kernel declares statically             */
  int32_t scratch_bytes;      /* per-lane private (spill) bytes                 */
  int32_t max_threads_per_block;
} mi_function_attrs;

int mi_abi_version(void);

/* Replaces triton.compile(...)+binary._init_handles()
 * (reference inductor_x/npu_triton_heuristics.py:195-199): take a finished
 * gfx950 code object in memory and make it launchable. */
int mi_module_load(const void* hsaco, size_t nbytes, void** module_out);
int mi_module_unload(void* module);

/* Replaces the `bin` lookup of the generated launcher
 * (reference inductor_x/npu_triton_heuristics.py:239-253). */
int mi_module_get_function(void* module, const char* name, void** function_out);
int mi_function_get_attrs(void* function, mi_function_attrs* out);

/* Replaces `bin[g0, g1, g2](*args, stream=stream)`
 * (reference inductor_x/npu_triton_heuristics.py:247-249).  grid is given in
 * workgroups, block in threads.  kernel_args is an array with one pointer per
 * kernel parameter, each pointing at that parameter's value. */
int mi_launch(void* function,
              uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
              uint32_t block_x, uint32_t block_y, uint32_t block_z,
              uint32_t dynamic_lds_bytes, void* hip_stream,
              void** kernel_args);

/* Same launch, but the parameters arrive already laid out as the kernel's
 * argument segment (natural alignment of each member, as in a C struct).
 * Lets a caller pack arguments once and re-launch without per-argument work. */
int mi_launch_packed(void* function,
                     uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                     uint32_t block_x, uint32_t block_y, uint32_t block_z,
                     uint32_t dynamic_lds_bytes, void* hip_stream,
                     const void* arg_segment, size_t arg_segment_bytes);

/* No counterpart in the reference.  For callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): mi_launch_packed for a kernel that takes a workspace
 * pointer among its parameters, with that workspace supplied by the library.
 * The 8-byte pointer parameter at byte `scratch_arg_offset` of the argument
 * segment (whatever the caller put there is ignored) is replaced by the address
 * of a fixed MI355_SCRATCH_BYTES array in device memory that the library holds,
 * one copy per GPU, until the process ends; the kernel must need no more than
 * `scratch_bytes_needed` bytes of it.  The call allocates and frees nothing.
 *   - scratch_bytes_needed > MI355_SCRATCH_BYTES returns
 *     MI_ERROR_SCRATCH_TOO_LARGE and launches nothing.
 *   - The array keeps the previous call's contents: a kernel that needs zeroed
 *     workspace must clear it itself.  Launches that share the array must be
 *     ordered on one stream; calls that overlap on one GPU race.
 *   - The device is the calling thread's current device, which must be the
 *     stream's device. */
#define MI355_SCRATCH_BYTES (8u << 20)
#define MI_ERROR_SCRATCH_TOO_LARGE 100001
int mi_launch_packed_scratch(void* function,
                             uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                             uint32_t block_x, uint32_t block_y, uint32_t block_z,
                             uint32_t dynamic_lds_bytes, void* hip_stream,
                             const void* arg_segment, size_t arg_segment_bytes,
                             size_t scratch_arg_offset, size_t scratch_bytes_needed);
int mi_scratch_capacity(size_t* bytes_out);

/* Hardware query used where the reference reads the Triton driver's device
 * properties (reference inductor_x/config.py:15-20). */
int mi_device_props_get(int device, mi_device_props* out);
int mi_device_count(int* count_out);

/* Text for an error code returned by any function above. */
const char* mi_error_string(int err);

#ifdef __cplusplus
}
#endif
#endif /* MI355_LAUNCHER_H */
