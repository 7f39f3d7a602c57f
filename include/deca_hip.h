/*
 * deca_hip.h -- C ABI of libdeca_hip.so, the kernel loader / launcher of the
 * MI355X (gfx950) build of DeCA.
 *
 * The reference runs every tuned kernel through TVM's runtime:
 *   tvm.runtime.load_module(path)["main"](dlpack tensors...)
 * (src/RuntimeMod.py:104-109 loads, :204-208 and :165-169 call, and
 * test_gemm_tc.py:146-150 / test_rowwise.py:120-124 / test_flash_attn.py
 * re-load the finalists).  The launch geometry lives in TVM's generated host
 * stub.  Here the artefact produced by build_*_to_file is a HIP code object
 * (.hsaco, `hipcc --genco --offload-arch=gfx950`), and the functions below are
 * what a binding needs to load one and launch its `deca_main` kernel.
 *
 * Conventions
 *  - every function returns a hipError_t value as int (0 == success) and never
 *    throws; deca_error_string() turns the code into text;
 *  - the library owns no tensor memory: kernel arguments are raw device
 *    pointers, handed over as an array of pointer VALUES (kernels of this
 *    project take pointers only -- shapes and tile configs are compile-time
 *    constants of the code object, as in src/kernels/gemm_tir.py:123-156);
 *  - launches are asynchronous on the caller's stream (`stream` is a
 *    hipStream_t, NULL == the default stream);
 *  - nothing touches the GPU at dlopen time, so compile workers may import
 *    the binding without creating a device context.
 */
#ifndef DECA_HIP_H
#define DECA_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Device attributes read by the hardware model.  Replaces the tvm.cuda(0)
 * attribute reads of arch/H20.py:69-82 (configure_device) and
 * src/utils/helper.py:64-71 (GPUDetector.detect_gpu). */
typedef struct deca_devinfo {
  char name[256];          /* marketing name, e.g. "AMD Instinct MI355X" */
  char gcn_arch[256];      /* e.g. "gfx950:sramecc+:xnack-" */
  int cu_count;            /* compute units */
  int clock_khz;           /* peak shader clock */
  int mem_clock_khz;       /* peak memory clock */
  int mem_bus_bits;        /* memory bus width */
  int wave_size;           /* lanes per wavefront */
  int l2_bytes;            /* L2 size reported by the runtime */
  int max_threads_per_block;
  int max_threads_per_cu;
  int regs_per_block;      /* 32-bit registers available to one workgroup */
  int reserved;
  size_t lds_per_block;    /* LDS bytes one workgroup may use */
  size_t lds_per_cu;       /* LDS bytes per compute unit */
  size_t total_mem;        /* device memory in bytes */
} deca_devinfo;

/* Resource usage of a loaded kernel, as recorded in the code object.  The
 * reference estimates these (src/kernels/gemm_tir.py:91-98,
 * rowwise_tir.py:68-85, flash_attn_tir.py:59-67); here they can be read back. */
typedef struct deca_funcinfo {
  int num_regs;            /* VGPRs (arch + accumulation) per lane */
  int static_lds_bytes;
  int scratch_bytes;       /* private (spill) bytes per lane */
  int max_threads_per_block;
  int const_bytes;
  int reserved;
} deca_funcinfo;

/* Selects device `dev` for the calling thread and creates its context.
 * Replaces the implicit tvm.cuda(0) of src/RuntimeMod.py:146. */
int deca_init(int dev);

/* Number of visible devices. */
int deca_device_count(int* count);

/* Fills `info` for device `dev` (see deca_devinfo). */
int deca_device_info(int dev, deca_devinfo* info);

/* Loads the code object at `path`; replaces tvm.runtime.load_module
 * (src/RuntimeMod.py:109). */
int deca_module_load(const char* path, void** mod);

/* Same, from an in-memory image of `size` bytes (`size` is only checked to be
 * non-zero; the image is self-describing). */
int deca_module_load_data(const void* image, size_t size, void** mod);

/* Unloads a module; every function handle obtained from it becomes invalid. */
int deca_module_unload(void* mod);

/* Looks up kernel `sym` (this project exports "deca_main"; the reference's
 * symbol is "main", src/kernels/gemm_tir.py:145-146, src/RuntimeMod.py:205). */
int deca_get_function(void* mod, const char* sym, void** fn);

/* Reads the kernel's recorded resource usage. */
int deca_function_info(void* fn, deca_funcinfo* info);

/* Raises the dynamic-LDS limit of `fn` to `bytes` (needed above 64 KiB).
 * Counterpart of the opt-in dynamic shared memory the reference's host stub
 * requests for its `shared.dyn` buffers (src/kernels/gemm_tir.py:170-173). */
int deca_set_max_dynamic_lds(void* fn, unsigned bytes);

/* Launches `fn` with grid (gx,gy,gz) workgroups of (bx,by,bz) work-items and
 * `lds_bytes` of dynamic LDS on `stream`.  `args[0..nargs)` are the device
 * pointers in the operator's kernel_args order: a,b,c / x[,w],y / q,k,v,o
 * (src/operators/GEMMTC.py:105-107, Rowwise.py:66-68, RuntimeMod.py:167).
 * Replaces the PackedFunc call of src/RuntimeMod.py:208. */
int deca_launch(void* fn, unsigned gx, unsigned gy, unsigned gz,
                unsigned bx, unsigned by, unsigned bz, unsigned lds_bytes,
                void* stream, void* const* args, unsigned nargs);

/* Launches `fn` `iters` times back to back on `stream` between two events and
 * stores the elapsed milliseconds of the whole batch in `*ms_total`; blocks
 * until the batch has finished.  Launch i uses the argument set
 * args[(i % nsets) * nargs .. +nargs), so that callers can rotate buffers that
 * together exceed the last-level cache.  Replaces the event loop of
 * bench_cuda (src/kernels/attn_bench.py:35-70) for back-to-back averages. */
int deca_launch_timed(void* fn, unsigned gx, unsigned gy, unsigned gz,
                      unsigned bx, unsigned by, unsigned bz, unsigned lds_bytes,
                      void* stream, void* const* args, unsigned nargs,
                      unsigned nsets, unsigned iters, float* ms_total);

/* Enqueues the same batch as deca_launch_timed between two events of the caller
 * (hipEvent_t handles, e.g. torch.cuda.Event.cuda_event; either may be NULL) and
 * returns without waiting: the events are recorded on `stream` directly before
 * the first and directly after the last launch, so that a caller who reads its
 * own clock around the call gets event and host time over the same launches.
 * The events stay the caller's.  Replaces the start.record() ... end.record()
 * pair around the launches in bench_cuda (src/kernels/attn_bench.py:58-66). */
int deca_launch_between(void* fn, unsigned gx, unsigned gy, unsigned gz,
                        unsigned bx, unsigned by, unsigned bz, unsigned lds_bytes,
                        void* stream, void* const* args, unsigned nargs,
                        unsigned nsets, unsigned iters, void* start_event,
                        void* stop_event);

/* Blocks until `stream` is idle (NULL: the whole device). */
int deca_synchronize(void* stream);

/* Text of a code returned by any function above (never NULL). */
const char* deca_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* DECA_HIP_H */
