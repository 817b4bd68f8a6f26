/*
 * spio_hip.h -- C ABI of libspio_hip.so, the native boundary under the
 * conv2d_gw8 operator on AMD CDNA4 (gfx950).
 *
 * The reference project reaches its GPU through two foreign-function layers:
 * a Cython binding of the CUDA driver API (spio/cuda/driver.pyx) and a ctypes
 * binding of NVRTC (spio/cuda/nvrtc_ctypes.py).  This header declares the
 * entry points that replace both, on top of hipRTC and the HIP module API.
 * Every entry point takes plain pointers, sizes and integers; there are no
 * torch types at this boundary.
 *
 * Conventions
 *   - Every function returning int returns 0 on success and a non-zero code
 *     on failure.  After a failure spio_hip_last_error() returns a
 *     thread-local, NUL-terminated description (valid until the next call on
 *     the same thread).  The Python binding turns it into ValueError, the
 *     exception type the reference raises (driver.pyx:118-123).
 *   - Handles (module, function) are opaque pointers owned by the caller.
 *   - Buffers returned through out-pointers (code objects, logs) are released
 *     with spio_hip_free().
 *   - The library is re-entrant; it keeps no state besides the resolved HIP /
 *     hipRTC entry points.  It resolves them at run time (spio_hip_init) from
 *     the copies of libamdhip64 / libhiprtc already mapped into the process,
 *     so device pointers and streams made by PyTorch stay valid.
 */
#ifndef SPIO_HIP_H
#define SPIO_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes of this layer (HIP and hipRTC codes are passed through with an
 * offset so the origin stays visible). */
enum {
    SPIO_HIP_OK = 0,
    SPIO_HIP_ERR_NOT_INITIALIZED = 1,
    SPIO_HIP_ERR_DLOPEN = 2,
    SPIO_HIP_ERR_SYMBOL = 3,
    SPIO_HIP_ERR_ARGUMENT = 4,
    SPIO_HIP_ERR_COMPILE = 5,
    SPIO_HIP_ERR_HIP_BASE = 1000,   /* 1000 + hipError_t   */
    SPIO_HIP_ERR_HIPRTC_BASE = 2000 /* 2000 + hiprtcResult */
};

/* Device description.  Replaces DeviceAttributes / get_device_attributes
 * (spio/cuda/driver.pyx:98-108, 360-369). */
typedef struct spio_hip_device_attrs {
    int compute_unit_count;      /* multiprocessor_count in the reference */
    int l2_cache_bytes;
    int max_lds_bytes_per_block; /* max_shared_memory_per_block */
    int wavefront_size;
    int clock_khz;
    int memory_clock_khz;
    int memory_bus_width_bits;
    int max_threads_per_block;
    char name[128];              /* marketing name                */
    char arch[64];               /* gcnArchName, e.g. gfx950:...  */
} spio_hip_device_attrs_t;

/* Replaces init() (driver.pyx:276-281): binds the HIP runtime and hipRTC.
 * Either path may be NULL; then the copies already loaded in the process are
 * used, else the default sonames.  Safe to call more than once. */
int spio_hip_init(const char* hip_library_path, const char* hiprtc_library_path);

/* Last error text of the calling thread. */
const char* spio_hip_last_error(void);

/* Releases a buffer returned by this library. */
void spio_hip_free(void* ptr);

/* Replaces Program(...).compile(options) / .cubin() / .log()
 * (spio/cuda/nvrtc_ctypes.py:152-217; options built in
 * spio/compiler/compile.py:46-62).  Compiles one translation unit given as
 * text, with in-memory headers, to a gfx950 code object.  *log is set whenever
 * the compiler produced any output, also on failure. */
int spio_hip_compile(const char* source, const char* name,
                     int num_headers, const char* const* header_sources,
                     const char* const* header_names,
                     int num_options, const char* const* options,
                     void** code, size_t* code_size, char** log);

/* Replace Module.load_data / get_function / unload (driver.pyx:210-242). */
int spio_hip_module_load(const void* code, void** module);
int spio_hip_module_unload(void* module);
int spio_hip_get_function(void* module, const char* kernel_name, void** function);

/* Replaces Function.set_attributes (driver.pyx:157-169): raises the dynamic
 * LDS limit of one kernel. */
int spio_hip_func_set_max_dynamic_lds(void* function, int bytes);

/* Replaces Function.launch (driver.pyx:171-208).  Asynchronous launch on
 * `stream` (NULL = the null stream).  `params` is an array of num_params
 * pointers, each to the storage of one kernel argument; at most 16 arguments
 * (driver.pyx:178-179). */
int spio_hip_launch(void* function,
                    unsigned grid_x, unsigned grid_y, unsigned grid_z,
                    unsigned block_x, unsigned block_y, unsigned block_z,
                    unsigned dynamic_lds_bytes, void* stream,
                    void** params, int num_params);

/* Timing helper for the on-device configuration sweep and the benchmark (the
 * reference times kernels with torch.profiler, scripts/profile_block.py:
 * 646-668).  Launches the kernel `warmup` times untimed, then `iters` times
 * between two HIP events recorded on `stream`, cycling through `num_sets`
 * argument sets (param_sets[i] is a `params` array as in spio_hip_launch), and
 * returns the elapsed milliseconds of the timed region.  Synchronises the
 * stream before returning. */
int spio_hip_launch_timed(void* function,
                          unsigned grid_x, unsigned grid_y, unsigned grid_z,
                          unsigned block_x, unsigned block_y, unsigned block_z,
                          unsigned dynamic_lds_bytes, void* stream,
                          void*** param_sets, int num_sets, int num_params,
                          int warmup, int iters, float* elapsed_ms);

/* One launch of a multi-kernel sequence (same fields as spio_hip_launch). */
typedef struct spio_hip_launch_desc {
    void* function;
    unsigned grid[3];
    unsigned block[3];
    unsigned dynamic_lds_bytes;
    int num_params;
    void** params;
} spio_hip_launch_desc_t;

/* Like spio_hip_launch_timed for operators made of several kernels run back
 * to back (the two-stage weight gradient).  `descs` holds num_sets * stages
 * descriptors; iteration i launches the `stages` descriptors of set
 * i % num_sets in order.  No counterpart in the reference, whose operators
 * are single kernels. */
int spio_hip_launch_sequence_timed(const spio_hip_launch_desc_t* descs, int stages, int num_sets,
                                   void* stream, int warmup, int iters, float* elapsed_ms);

/* Size of the library's static device workspace (one copy per GPU). */
#define SPIO_HIP_SCRATCH_BYTES (32u * 1024u * 1024u)

/* Like spio_hip_launch, for kernels that need a workspace in device memory
 * (the two-stage weight gradient: the main kernel stores per-workgroup partial
 * sums into it, its `_reduce` kernel reads them back), for callers that cannot
 * allocate: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  No counterpart in the reference, whose kernels need no
 * workspace.  Kernel argument number `scratch_param` (a device pointer) is
 * replaced by the address of a fixed SPIO_HIP_SCRATCH_BYTES array that lives
 * in the library's own device code, of which the kernel may use the first
 * `scratch_bytes`; more than SPIO_HIP_SCRATCH_BYTES is rejected with
 * SPIO_HIP_ERR_ARGUMENT.  The call allocates and frees nothing.  Every call on
 * one GPU shares that GPU's array: it keeps the last call's contents, and
 * calls that overlap on one GPU (different streams or threads) race on it. */
int spio_hip_launch_scratch(void* function,
                            unsigned grid_x, unsigned grid_y, unsigned grid_z,
                            unsigned block_x, unsigned block_y, unsigned block_z,
                            unsigned dynamic_lds_bytes, void* stream,
                            void** params, int num_params,
                            int scratch_param, size_t scratch_bytes);

/* Asynchronous fill of a device buffer with zero bytes on `stream`, for the
 * pre-zeroed weight-gradient contract
 * (spio/functional/conv2d_gw8_function.py:124-127) by callers without torch.
 * A fill kernel is launched, not a runtime memset, so the call may be recorded
 * under HIP graph capture like any other kernel launch. */
int spio_hip_zero_fill_async(void* device_ptr, size_t bytes, void* stream);

/* Replace get_device_attributes, ctx_synchronize, get_driver_version
 * (driver.pyx:284-303, 360-369) and PrimaryContextGuard.set_device (259-265). */
int spio_hip_device_count(int* count);
int spio_hip_device_attrs(int ordinal, spio_hip_device_attrs_t* attrs);
int spio_hip_set_device(int ordinal);
int spio_hip_synchronize(void);
int spio_hip_stream_synchronize(void* stream);
int spio_hip_driver_version(int* version);
int spio_hip_runtime_version(int* version);
int spio_hiprtc_version(int* major, int* minor);

#ifdef __cplusplus
}
#endif
#endif /* SPIO_HIP_H */
