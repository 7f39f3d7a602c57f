// libdeca_hip.so: loads gfx950 code objects and launches their kernels.
// The C ABI is declared in include/deca_hip.h; every entry point returns a
// hipError_t value as int and never lets a C++ exception cross the boundary.
#include "deca_hip.h"

#include <hip/hip_runtime.h>

#include <cstring>

namespace {

constexpr unsigned kMaxArgs = 16;

inline int rc(hipError_t e) { return static_cast<int>(e); }

// Host-side sanity checks shared by the two launch entry points.  A bad
// geometry is rejected here instead of being handed to the runtime.
inline bool geometry_ok(unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
                        unsigned bz, unsigned nargs) {
  if (gx == 0 || gy == 0 || gz == 0 || bx == 0 || by == 0 || bz == 0) return false;
  if (static_cast<unsigned long long>(bx) * by * bz > 1024ull) return false;
  if (nargs == 0 || nargs > kMaxArgs) return false;
  return true;
}

}  // namespace

extern "C" {

int deca_init(int dev) {
  hipError_t e = hipSetDevice(dev);
  if (e != hipSuccess) return rc(e);
  return rc(hipFree(nullptr));  // forces context creation
}

int deca_device_count(int* count) {
  if (!count) return rc(hipErrorInvalidValue);
  return rc(hipGetDeviceCount(count));
}

int deca_device_info(int dev, deca_devinfo* info) {
  if (!info) return rc(hipErrorInvalidValue);
  hipDeviceProp_t p;
  hipError_t e = hipGetDeviceProperties(&p, dev);
  if (e != hipSuccess) return rc(e);
  std::memset(info, 0, sizeof(*info));
  std::strncpy(info->name, p.name, sizeof(info->name) - 1);
  std::strncpy(info->gcn_arch, p.gcnArchName, sizeof(info->gcn_arch) - 1);
  info->cu_count = p.multiProcessorCount;
  info->clock_khz = p.clockRate;
  info->mem_clock_khz = p.memoryClockRate;
  info->mem_bus_bits = p.memoryBusWidth;
  info->wave_size = p.warpSize;
  info->l2_bytes = p.l2CacheSize;
  info->max_threads_per_block = p.maxThreadsPerBlock;
  info->max_threads_per_cu = p.maxThreadsPerMultiProcessor;
  info->regs_per_block = p.regsPerBlock;
  info->lds_per_block = p.sharedMemPerBlock;
  info->lds_per_cu = p.maxSharedMemoryPerMultiProcessor;
  info->total_mem = p.totalGlobalMem;
  return rc(hipSuccess);
}

int deca_module_load(const char* path, void** mod) {
  if (!path || !mod) return rc(hipErrorInvalidValue);
  hipModule_t m = nullptr;
  hipError_t e = hipModuleLoad(&m, path);
  *mod = (e == hipSuccess) ? m : nullptr;
  return rc(e);
}

int deca_module_load_data(const void* image, size_t size, void** mod) {
  if (!image || !mod || size == 0) return rc(hipErrorInvalidValue);
  hipModule_t m = nullptr;
  hipError_t e = hipModuleLoadData(&m, image);
  *mod = (e == hipSuccess) ? m : nullptr;
  return rc(e);
}

int deca_module_unload(void* mod) {
  if (!mod) return rc(hipErrorInvalidValue);
  return rc(hipModuleUnload(static_cast<hipModule_t>(mod)));
}

int deca_get_function(void* mod, const char* sym, void** fn) {
  if (!mod || !sym || !fn) return rc(hipErrorInvalidValue);
  hipFunction_t f = nullptr;
  hipError_t e = hipModuleGetFunction(&f, static_cast<hipModule_t>(mod), sym);
  *fn = (e == hipSuccess) ? f : nullptr;
  return rc(e);
}

int deca_function_info(void* fn, deca_funcinfo* info) {
  if (!fn || !info) return rc(hipErrorInvalidValue);
  hipFunction_t f = static_cast<hipFunction_t>(fn);
  std::memset(info, 0, sizeof(*info));
  hipError_t e;
  if ((e = hipFuncGetAttribute(&info->num_regs, HIP_FUNC_ATTRIBUTE_NUM_REGS, f)) != hipSuccess)
    return rc(e);
  if ((e = hipFuncGetAttribute(&info->static_lds_bytes, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES,
                               f)) != hipSuccess)
    return rc(e);
  if ((e = hipFuncGetAttribute(&info->scratch_bytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, f)) !=
      hipSuccess)
    return rc(e);
  if ((e = hipFuncGetAttribute(&info->max_threads_per_block,
                               HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, f)) != hipSuccess)
    return rc(e);
  if ((e = hipFuncGetAttribute(&info->const_bytes, HIP_FUNC_ATTRIBUTE_CONST_SIZE_BYTES, f)) !=
      hipSuccess)
    return rc(e);
  return rc(hipSuccess);
}

int deca_set_max_dynamic_lds(void* fn, unsigned bytes) {
  if (!fn) return rc(hipErrorInvalidValue);
  return rc(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(bytes)));
}

int deca_launch(void* fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
                unsigned bz, unsigned lds_bytes, void* stream, void* const* args,
                unsigned nargs) {
  if (!fn || !args || !geometry_ok(gx, gy, gz, bx, by, bz, nargs))
    return rc(hipErrorInvalidValue);
  void* values[kMaxArgs];
  void* params[kMaxArgs];
  for (unsigned i = 0; i < nargs; ++i) {
    values[i] = args[i];
    params[i] = &values[i];
  }
  return rc(hipModuleLaunchKernel(static_cast<hipFunction_t>(fn), gx, gy, gz, bx, by, bz,
                                  lds_bytes, static_cast<hipStream_t>(stream), params, nullptr));
}

int deca_launch_timed(void* fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
                      unsigned bz, unsigned lds_bytes, void* stream, void* const* args,
                      unsigned nargs, unsigned nsets, unsigned iters, float* ms_total) {
  if (!fn || !args || !ms_total || nsets == 0 || iters == 0 ||
      !geometry_ok(gx, gy, gz, bx, by, bz, nargs))
    return rc(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipFunction_t f = static_cast<hipFunction_t>(fn);
  hipEvent_t start = nullptr, stop = nullptr;
  hipError_t e = hipEventCreate(&start);
  if (e != hipSuccess) return rc(e);
  e = hipEventCreate(&stop);
  if (e != hipSuccess) {
    (void)hipEventDestroy(start);
    return rc(e);
  }
  // The launch reads each argument's value through params[a] before it returns,
  // so the slots of the caller's array serve as the argument storage: no copy,
  // no allocation, nothing that could throw across the C boundary.
  void* params[kMaxArgs];
  e = hipEventRecord(start, s);
  for (unsigned i = 0; e == hipSuccess && i < iters; ++i) {
    void* const* set = args + static_cast<size_t>(i % nsets) * nargs;
    for (unsigned a = 0; a < nargs; ++a) params[a] = const_cast<void**>(&set[a]);
    e = hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, lds_bytes, s, params, nullptr);
  }
  if (e == hipSuccess) e = hipEventRecord(stop, s);
  if (e == hipSuccess) e = hipEventSynchronize(stop);
  if (e == hipSuccess) e = hipEventElapsedTime(ms_total, start, stop);
  (void)hipEventDestroy(start);
  (void)hipEventDestroy(stop);
  return rc(e);
}

int deca_launch_between(void* fn, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
                        unsigned bz, unsigned lds_bytes, void* stream, void* const* args,
                        unsigned nargs, unsigned nsets, unsigned iters, void* start_event,
                        void* stop_event) {
  if (!fn || !args || nsets == 0 || iters == 0 || !geometry_ok(gx, gy, gz, bx, by, bz, nargs))
    return rc(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipFunction_t f = static_cast<hipFunction_t>(fn);
  void* params[kMaxArgs];
  hipError_t e = hipSuccess;
  if (start_event) e = hipEventRecord(static_cast<hipEvent_t>(start_event), s);
  for (unsigned i = 0; e == hipSuccess && i < iters; ++i) {
    void* const* set = args + static_cast<size_t>(i % nsets) * nargs;
    for (unsigned a = 0; a < nargs; ++a) params[a] = const_cast<void**>(&set[a]);
    e = hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, lds_bytes, s, params, nullptr);
  }
  if (e == hipSuccess && stop_event) e = hipEventRecord(static_cast<hipEvent_t>(stop_event), s);
  return rc(e);
}

int deca_synchronize(void* stream) {
  if (stream) return rc(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return rc(hipDeviceSynchronize());
}

const char* deca_error_string(int code) {
  const char* s = hipGetErrorString(static_cast<hipError_t>(code));
  return s ? s : "unknown error";
}

}  // extern "C"
