// C-ABI kernel launcher for gfx950: code-object load, kernel lookup and
// hipModuleLaunchKernel enqueue on a caller-supplied raw stream.  The declared
// interface and the reference call sites it stands in for are in
// include/mi355_launcher.h.  No kernels live in this library; the only device
// object is the fixed scratch array behind mi_launch_packed_scratch.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "mi355_launcher.h"

// Device memory for kernels that need a workspace when the caller may not
// allocate one.  Each GPU the library runs on holds its own copy of the array,
// at its own address, until the process ends.  On the host the name below is
// only a handle for hipGetSymbolAddress: the device address is looked up once
// per device (scratch_pointer) and that pointer is what kernels receive.
// No `used` attribute here: with it clang emits the device-side symbol with local binding, the
// runtime then cannot resolve the registered variable by name and aborts the process at the
// lookup.  The host-side reference in scratch_pointer is what makes the compiler emit the
// array and give it global binding in the device code object.
static __device__ __align__(256) unsigned char scratch[MI355_SCRATCH_BYTES];

namespace {

inline int rc(hipError_t e) { return static_cast<int>(e); }

constexpr int kMaxDevices = 64;
constexpr size_t kMaxArgSegment = 4096;  // the HSA kernel-argument segment never exceeds this here
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Address of the current device's copy of `scratch`; looked up on the first call per device
// (two racing first calls read the same value).
hipError_t scratch_pointer(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (p == nullptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return hipSuccess;
}

// Bytes of memory-side (level 3) cache of the GPU at the given PCI location, from the KFD
// topology files; 0 when they cannot be read.
int64_t mall_bytes_from_topology(int domain, int bus, int dev) {
  const long want_location = (static_cast<long>(bus) << 8) | (static_cast<long>(dev) << 3);
  for (int node = 0; node < 256; ++node) {
    char path[160];
    std::snprintf(path, sizeof(path), "/sys/class/kfd/kfd/topology/nodes/%d/properties", node);
    std::FILE* f = std::fopen(path, "r");
    if (f == nullptr) {
      if (node > 16) break;
      continue;
    }
    long location = -1, dom = 0, simd = 0;
    char key[64];
    long long val;
    while (std::fscanf(f, "%63s %lld", key, &val) == 2) {
      if (std::strcmp(key, "location_id") == 0) location = static_cast<long>(val);
      else if (std::strcmp(key, "domain") == 0) dom = static_cast<long>(val);
      else if (std::strcmp(key, "simd_count") == 0) simd = static_cast<long>(val);
    }
    std::fclose(f);
    if (simd == 0 || (location & ~7L) != want_location || dom != domain) continue;
    int64_t total = 0;
    for (int c = 0; c < 4096; ++c) {
      std::snprintf(path, sizeof(path), "/sys/class/kfd/kfd/topology/nodes/%d/caches/%d/properties", node, c);
      f = std::fopen(path, "r");
      if (f == nullptr) break;
      long level = 0;
      long long size_kib = 0;
      while (std::fscanf(f, "%63s %lld", key, &val) == 2) {
        if (std::strcmp(key, "level") == 0) level = static_cast<long>(val);
        else if (std::strcmp(key, "size") == 0) size_kib = val;
      }
      std::fclose(f);
      if (level == 3) total += static_cast<int64_t>(size_kib) * 1024;
    }
    return total;
  }
  return 0;
}

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

int mi_scratch_capacity(size_t* bytes_out) {
  if (bytes_out == nullptr) return rc(hipErrorInvalidValue);
  *bytes_out = MI355_SCRATCH_BYTES;
  return rc(hipSuccess);
}

int mi_launch_packed_scratch(void* function, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                             uint32_t block_x, uint32_t block_y, uint32_t block_z,
                             uint32_t dynamic_lds_bytes, void* hip_stream, const void* arg_segment,
                             size_t arg_segment_bytes, size_t scratch_arg_offset,
                             size_t scratch_bytes_needed) {
  if (function == nullptr || arg_segment == nullptr) return rc(hipErrorInvalidValue);
  if (scratch_bytes_needed > MI355_SCRATCH_BYTES) return MI_ERROR_SCRATCH_TOO_LARGE;
  if (arg_segment_bytes > kMaxArgSegment) return rc(hipErrorInvalidValue);
  // written so that an offset near SIZE_MAX cannot wrap past the check
  if (scratch_arg_offset % sizeof(void*) != 0 || arg_segment_bytes < sizeof(void*) ||
      scratch_arg_offset > arg_segment_bytes - sizeof(void*))
    return rc(hipErrorInvalidValue);
  if (grid_x == 0 || grid_y == 0 || grid_z == 0 || block_x == 0 || block_y == 0 || block_z == 0)
    return rc(hipErrorInvalidConfiguration);
  if (static_cast<uint64_t>(block_x) * block_y * block_z > 1024u) return rc(hipErrorInvalidConfiguration);
  void* ws = nullptr;
  hipError_t e = scratch_pointer(&ws);
  if (e != hipSuccess) return rc(e);
  // the caller's segment with the workspace parameter replaced, on the stack (no allocation)
  alignas(16) unsigned char seg[kMaxArgSegment];
  std::memcpy(seg, arg_segment, arg_segment_bytes);
  std::memcpy(seg + scratch_arg_offset, &ws, sizeof(void*));
  size_t nbytes = arg_segment_bytes;
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, seg, HIP_LAUNCH_PARAM_BUFFER_SIZE, &nbytes,
                   HIP_LAUNCH_PARAM_END};
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
  out->mall_bytes = mall_bytes_from_topology(p.pciDomainID, p.pciBusID, p.pciDeviceID);
  // MI300/MI350-class parts expose 32 CUs per accelerator die (XCD).
  out->xcd_count = p.multiProcessorCount >= 32 ? (p.multiProcessorCount + 31) / 32 : 1;
  std::strncpy(out->arch, p.gcnArchName, sizeof(out->arch) - 1);
  return rc(hipSuccess);
}

const char* mi_error_string(int err) {
  if (err == MI_ERROR_SCRATCH_TOO_LARGE)
    return "workspace request exceeds the library's fixed scratch array (MI355_SCRATCH_BYTES)";
  return hipGetErrorString(static_cast<hipError_t>(err));
}

}  // extern "C"
