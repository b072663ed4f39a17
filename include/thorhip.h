/*
 * thorhip.h -- the device-side C ABI of the MI355X (gfx950) backend for Thor's Expression / reduction / TypeConverter
 * hot path.
 *
 * This is the seam the reference keeps behind `CudaDriverApi` (a dlopen'd function table over the CUDA driver,
 * Utilities/CudaDriver/CudaDrivertApi.h:9-158), `EquationCompiler::{compileToLtoIr, linkToCubin, loadCubin}`
 * (Utilities/Expression/EquationCompiler.h:39-47), `EquationRunner::run`'s final `cuLaunchKernel`
 * (Utilities/Expression/EquationRunner.cpp:263-289) and `TypeConverter::gpuConvertType`
 * (Utilities/TensorOperations/DataTypeConversions/TypeConverter.h:61-66).  Host code above this header never includes
 * a HIP header: it sees plain pointers, sizes and integer codes only.
 *
 * Conventions
 *   - every function returns 0 on success and a negative value on failure; `thorhip_last_error()` then returns a
 *     thread-local, NUL-terminated description (HIP / hipRTC error name, file:line, compile log);
 *   - `stream` arguments are opaque stream handles created by `thorhip_stream_create` (NULL = the null stream);
 *   - dtype codes are the reference's `DataType` enum values (DeepLearning/Implementation/Tensor/DataType.h:7-27);
 *   - nothing here allocates behind the caller's back except `thorhip_compile` (host memory for the code object,
 *     released with `thorhip_code_free`).
 */
#ifndef THORHIP_H
#define THORHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define THORHIP_ABI_VERSION 1

/* DataType.h:7-27 */
enum thorhip_dtype {
    THORHIP_FP16 = 10,
    THORHIP_FP32 = 11,
    THORHIP_FP64 = 12,
    THORHIP_INT8 = 13,
    THORHIP_INT16 = 14,
    THORHIP_INT32 = 15,
    THORHIP_INT64 = 16,
    THORHIP_UINT8 = 17,
    THORHIP_UINT16 = 18,
    THORHIP_UINT32 = 19,
    THORHIP_UINT64 = 20,
    THORHIP_BOOLEAN = 21,
    THORHIP_FP8_E4M3 = 22,
    THORHIP_FP8_E5M2 = 23,
    THORHIP_BF16 = 24
};

enum thorhip_memcpy_kind { THORHIP_H2D = 1, THORHIP_D2H = 2, THORHIP_D2D = 3 };

typedef struct thorhip_device_info {
    int compute_units;          /* 256 on MI355X */
    int wavefront_size;         /* 64 */
    int max_threads_per_block;  /* 1024 */
    int lds_bytes_per_block;    /* 65536 default opt-out limit, 160 KiB per CU physical */
    int l2_bytes;
    int clock_khz;
    int memory_clock_khz;
    int memory_bus_width_bits;
    size_t total_global_mem;
    char arch_name[64];         /* "gfx950:sramecc+:xnack-" */
    char name[128];
} thorhip_device_info;

/* ---- errors / library ------------------------------------------------------------------------------------------- */
int thorhip_abi_version(void);
const char* thorhip_last_error(void);

/* ---- devices (CudaDrivertApi.h: cuDeviceGet / cuCtx*; Utilities/Common/ScopedGpu.h) ------------------------------- */
int thorhip_device_count(int* count);
int thorhip_set_device(int device);
int thorhip_get_device(int* device);
int thorhip_device_get_info(int device, thorhip_device_info* info);
int thorhip_device_synchronize(void);

/* ---- memory (Tensor::allocateMemory, DeepLearning/Implementation/Tensor/Tensor.cpp:221-299) ----------------------- */
int thorhip_malloc(void** ptr, size_t bytes);
int thorhip_free(void* ptr);
int thorhip_host_malloc(void** ptr, size_t bytes); /* pinned host memory */
int thorhip_host_free(void* ptr);
int thorhip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream);
int thorhip_memset_async(void* dst, int byte_value, size_t bytes, void* stream);
int thorhip_mem_get_info(size_t* free_bytes, size_t* total_bytes);

/* ---- streams / events (Utilities/Common/Stream.h:35-116, Event.h) -------------------------------------------------- */
int thorhip_stream_create(void** stream); /* default priority, non-blocking w.r.t. the null stream */
int thorhip_stream_destroy(void* stream);
int thorhip_stream_synchronize(void* stream);
int thorhip_stream_wait_event(void* stream, void* event);
typedef void (*thorhip_host_fn)(void* user_data);
int thorhip_stream_enqueue_host_function(void* stream, thorhip_host_fn fn, void* user_data);
int thorhip_event_create(void** event, int enable_timing);
int thorhip_event_destroy(void* event);
int thorhip_event_record(void* event, void* stream);
int thorhip_event_synchronize(void* event);
int thorhip_event_elapsed_ms(float* ms, void* start, void* stop);

/* ---- run-time compilation (replaces NVRTC -> nvJitLink -> cuModuleLoadData; EquationCompiler.cpp:1756-1908) ------- */
/* Compiles HIP source for `arch` (NULL = the current device's gcnArchName, "gfx950" when no device is present) with
 * hipRTC.  `options` are appended after the library's fixed flags.  On success *code / *code_size describe a code
 * object owned by the caller (thorhip_code_free).  The compile log (possibly empty) is copied into `log`. */
int thorhip_compile(const char* source, const char* program_name, const char* arch, const char* const* options,
                    int num_options, void** code, size_t* code_size, char* log, size_t log_capacity);
int thorhip_code_free(void* code);
/* Compile isolation.  With it on, thorhip_compile runs the compiler in a child process of its own (the worker program next to
 * the library, started with posix_spawn; it links the run-time compiler only and never touches a GPU) and gets the code object
 * or the log back over a pipe, so that a compiler that aborts - an internal compiler error ends in abort() - fails that one
 * compilation with an error instead of ending the calling process.  Costs a process start per compilation (compiled kernels
 * are cached by the host layer).  Off by default; THORHIP_COMPILE_ISOLATION=1 in the environment turns it on.  Returns the
 * previous setting.  No counterpart in the reference, whose NVRTC calls are in-process (EquationCompiler.cpp:1864-1908). */
int thorhip_set_compile_isolation(int enabled);
int thorhip_module_load(void** module, const void* code, size_t code_size);
int thorhip_module_unload(void* module);
int thorhip_module_get_function(void** function, void* module, const char* kernel_name);
int thorhip_function_get_attributes(void* function, int* num_vgprs_hint, int* static_lds_bytes, int* max_threads_per_block);

/* cuLaunchKernel shape: args is an array of pointers to the individual kernel arguments (EquationRunner.cpp:153-166). */
int thorhip_launch(void* function, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z, uint32_t block_x, uint32_t block_y,
                   uint32_t block_z, uint32_t dynamic_lds_bytes, void* stream, void** args);

/* ---- type conversion (TypeConverter::gpuConvertType, TypeConverterKernels.cu:39-823,906-936,1340-1433) ------------- */
/* dst[i] = static_cast<dst_dtype>(src[i]) for i in [0, num_elements), every pair of the 15 storage dtypes; ->fp8 e4m3
 * and e5m2 saturate to the largest finite value; fp16/bf16 narrowing is round-to-nearest-even with +-Inf on overflow
 * and gradual underflow.  src == dst (in place) is supported; any other overlap is rejected.  Unlike the reference's
 * kernels nothing past num_elements is ever read or written. */
int thorhip_convert(const void* src, void* dst, int src_dtype, int dst_dtype, int64_t num_elements, void* stream);
int thorhip_dtype_size(int dtype);

#ifdef __cplusplus
}
#endif
#endif /* THORHIP_H */
