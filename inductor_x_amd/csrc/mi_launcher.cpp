// C-ABI kernel launcher for gfx950: code-object load, kernel lookup and
// hipModuleLaunchKernel enqueue on a caller-supplied raw stream.  The declared
// interface and the reference call sites it stands in for are in
// include/mi355_launcher.h.  Host code only: no kernels live in this library.
#include <hip/hip_runtime.h>

#include <cstring>

#include "mi355_launcher.h"

namespace {

inline int rc(hipError_t e) { return static_cast<int>(e); }

}  // namespace

extern "C" {

int mi_abi_version(void) { return MI355_ABI_VERSION; }

int mi_module_load(const void* hsaco, size_t nbytes, void** module_out) {
  if (hsaco == nullptr || nbytes == 0 || module_out == nullptr) return rc(hipErrorInvalidValue);
  hipModule_t mod = nullptr;
  hipError_t e = hipModuleLoadData(&mod, hsaco);
  if (e != hipSuccess) return rc(e);
  *module_out = reinterpret_cast<void*>(mod);
  return rc(hipSuccess);
}

int mi_module_unload(void* module) {
  if (module == nullptr) return rc(hipErrorInvalidValue);
  return rc(hipModuleUnload(reinterpret_cast<hipModule_t>(module)));
}

int mi_module_get_function(void* module, const char* name, void** function_out) {
  if (module == nullptr || name == nullptr || function_out == nullptr) return rc(hipErrorInvalidValue);
  hipFunction_t fn = nullptr;
  hipError_t e = hipModuleGetFunction(&fn, reinterpret_cast<hipModule_t>(module), name);
  if (e != hipSuccess) return rc(e);
  *function_out = reinterpret_cast<void*>(fn);
  return rc(hipSuccess);
}

int mi_function_get_attrs(void* function, mi_function_attrs* out) {
  if (function == nullptr || out == nullptr) return rc(hipErrorInvalidValue);
  hipFunction_t fn = reinterpret_cast<hipFunction_t>(function);
  int v = 0;
  hipError_t e = hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, fn);
  if (e != hipSuccess) return rc(e);
  out->num_regs = v;
  e = hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, fn);
  if (e != hipSuccess) return rc(e);
  out->static_lds_bytes = v;
  e = hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, fn);
  if (e != hipSuccess) return rc(e);
  out->scratch_bytes = v;
  e = hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, fn);
  if (e != hipSuccess) return rc(e);
  out->max_threads_per_block = v;
  return rc(hipSuccess);
}

int mi_launch(void* function, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z, uint32_t block_x,
              uint32_t block_y, uint32_t block_z, uint32_t dynamic_lds_bytes, void* hip_stream,
              void** kernel_args) {
  if (function == nullptr) return rc(hipErrorInvalidValue);
  if (grid_x == 0 || grid_y == 0 || grid_z == 0 || block_x == 0 || block_y == 0 || block_z == 0)
    return rc(hipErrorInvalidConfiguration);
  if (static_cast<uint64_t>(block_x) * block_y * block_z > 1024u) return rc(hipErrorInvalidConfiguration);
  return rc(hipModuleLaunchKernel(reinterpret_cast<hipFunction_t>(function), grid_x, grid_y, grid_z,
                                  block_x, block_y, block_z, dynamic_lds_bytes,
                                  reinterpret_cast<hipStream_t>(hip_stream), kernel_args, nullptr));
}

int mi_launch_packed(void* function, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                     uint32_t block_x, uint32_t block_y, uint32_t block_z,
                     uint32_t dynamic_lds_bytes, void* hip_stream, const void* arg_segment,
                     size_t arg_segment_bytes) {
  if (function == nullptr) return rc(hipErrorInvalidValue);
  if (arg_segment == nullptr && arg_segment_bytes != 0) return rc(hipErrorInvalidValue);
  if (grid_x == 0 || grid_y == 0 || grid_z == 0 || block_x == 0 || block_y == 0 || block_z == 0)
    return rc(hipErrorInvalidConfiguration);
  if (static_cast<uint64_t>(block_x) * block_y * block_z > 1024u) return rc(hipErrorInvalidConfiguration);
  size_t nbytes = arg_segment_bytes;
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(arg_segment),
                   HIP_LAUNCH_PARAM_BUFFER_SIZE, &nbytes, HIP_LAUNCH_PARAM_END};
  return rc(hipModuleLaunchKernel(reinterpret_cast<hipFunction_t>(function), grid_x, grid_y, grid_z,
                                  block_x, block_y, block_z, dynamic_lds_bytes,
                                  reinterpret_cast<hipStream_t>(hip_stream), nullptr, extra));
}

int mi_device_count(int* count_out) {
  if (count_out == nullptr) return rc(hipErrorInvalidValue);
  return rc(hipGetDeviceCount(count_out));
}

int mi_device_props_get(int device, mi_device_props* out) {
  if (out == nullptr) return rc(hipErrorInvalidValue);
  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, device);
  if (e != hipSuccess) return rc(e);
  std::memset(out, 0, sizeof(*out));
  out->cu_count = p.multiProcessorCount;
  out->wave_size = p.warpSize;
  out->lds_bytes = static_cast<int32_t>(p.sharedMemPerBlock);
  out->max_threads_per_cu = p.maxThreadsPerMultiProcessor;
  out->max_waves_per_cu = p.warpSize > 0 ? p.maxThreadsPerMultiProcessor / p.warpSize : 0;
  out->regs_per_cu = p.regsPerMultiprocessor;
  out->clock_khz = p.clockRate;
  out->mem_clock_khz = p.memoryClockRate;
  out->mem_bus_bits = p.memoryBusWidth;
  out->l2_bytes = p.l2CacheSize;
  out->hbm_bytes = static_cast<int64_t>(p.totalGlobalMem);
  // MI300/MI350-class parts expose 32 CUs per accelerator die (XCD).
  out->xcd_count = p.multiProcessorCount >= 32 ? (p.multiProcessorCount + 31) / 32 : 1;
  std::strncpy(out->arch, p.gcnArchName, sizeof(out->arch) - 1);
  return rc(hipSuccess);
}

const char* mi_error_string(int err) { return hipGetErrorString(static_cast<hipError_t>(err)); }

}  // extern "C"
