// libspio_hip.so -- the C ABI declared in include/spio_hip.h.
//
// A thin, re-entrant layer over hipRTC and the HIP module API.  It takes the
// place of the reference's Cython driver binding (spio/cuda/driver.pyx) and its
// ctypes NVRTC binding (spio/cuda/nvrtc_ctypes.py).  The HIP entry points are
// resolved with dlopen/dlsym at run time, preferring the copies of the
// libraries that the process has already mapped (PyTorch ships its own), so
// that device pointers and streams created by the host framework are valid
// for the launches issued here.

#include "spio_hip.h"
#include "spio_hip_internal.h"

#include <dlfcn.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

// Table of the runtime entry points this layer uses.
struct Api {
    void* hip_handle = nullptr;
    void* rtc_handle = nullptr;

    hipError_t (*hipInit)(unsigned) = nullptr;
    hipError_t (*hipGetDeviceCount)(int*) = nullptr;
    hipError_t (*hipSetDevice)(int) = nullptr;
    hipError_t (*hipDeviceGetAttribute)(int*, hipDeviceAttribute_t, int) = nullptr;
    hipError_t (*hipDeviceGetName)(char*, int, hipDevice_t) = nullptr;
    hipError_t (*hipDeviceSynchronize)() = nullptr;
    hipError_t (*hipStreamSynchronize)(hipStream_t) = nullptr;
    hipError_t (*hipDriverGetVersion)(int*) = nullptr;
    hipError_t (*hipRuntimeGetVersion)(int*) = nullptr;
    hipError_t (*hipModuleLoadData)(hipModule_t*, const void*) = nullptr;
    hipError_t (*hipModuleUnload)(hipModule_t) = nullptr;
    hipError_t (*hipModuleGetFunction)(hipFunction_t*, hipModule_t, const char*) = nullptr;
    hipError_t (*hipFuncSetAttribute)(const void*, hipFuncAttribute, int) = nullptr;
    hipError_t (*hipModuleLaunchKernel)(hipFunction_t, unsigned, unsigned, unsigned, unsigned,
                                        unsigned, unsigned, unsigned, hipStream_t, void**,
                                        void**) = nullptr;
    hipError_t (*hipEventCreate)(hipEvent_t*) = nullptr;
    hipError_t (*hipEventDestroy)(hipEvent_t) = nullptr;
    hipError_t (*hipEventRecord)(hipEvent_t, hipStream_t) = nullptr;
    hipError_t (*hipEventSynchronize)(hipEvent_t) = nullptr;
    hipError_t (*hipEventElapsedTime)(float*, hipEvent_t, hipEvent_t) = nullptr;
    const char* (*hipGetErrorString)(hipError_t) = nullptr;

    hiprtcResult (*hiprtcCreateProgram)(hiprtcProgram*, const char*, const char*, int,
                                        const char**, const char**) = nullptr;
    hiprtcResult (*hiprtcDestroyProgram)(hiprtcProgram*) = nullptr;
    hiprtcResult (*hiprtcCompileProgram)(hiprtcProgram, int, const char**) = nullptr;
    hiprtcResult (*hiprtcGetProgramLogSize)(hiprtcProgram, size_t*) = nullptr;
    hiprtcResult (*hiprtcGetProgramLog)(hiprtcProgram, char*) = nullptr;
    hiprtcResult (*hiprtcGetCodeSize)(hiprtcProgram, size_t*) = nullptr;
    hiprtcResult (*hiprtcGetCode)(hiprtcProgram, char*) = nullptr;
    const char* (*hiprtcGetErrorString)(hiprtcResult) = nullptr;
    hiprtcResult (*hiprtcVersion)(int*, int*) = nullptr;

    bool ready = false;
};

Api g_api;
std::mutex g_init_mutex;

// Opens `explicit_path` when given; otherwise tries each soname first without
// loading (picking up a copy that is already mapped) and then normally.
void* open_library(const char* explicit_path, const char* const* sonames, std::string* tried) {
    if (explicit_path && explicit_path[0]) {
        void* h = dlopen(explicit_path, RTLD_NOW | RTLD_LOCAL);
        if (!h) *tried += std::string(explicit_path) + ": " + dlerror() + "; ";
        return h;
    }
    for (const char* const* s = sonames; *s; ++s) {
        void* h = dlopen(*s, RTLD_NOW | RTLD_LOCAL | RTLD_NOLOAD);
        if (h) return h;
    }
    for (const char* const* s = sonames; *s; ++s) {
        void* h = dlopen(*s, RTLD_NOW | RTLD_LOCAL);
        if (h) return h;
        *tried += std::string(*s) + ": " + dlerror() + "; ";
    }
    return nullptr;
}

template <typename F>
bool bind(void* handle, const char* name, F* slot, std::string* missing) {
    *slot = reinterpret_cast<F>(dlsym(handle, name));
    if (!*slot) {
        *missing += name;
        *missing += " ";
        return false;
    }
    return true;
}

int hip_fail(hipError_t e, const char* what) {
    const char* s = g_api.hipGetErrorString ? g_api.hipGetErrorString(e) : "?";
    return fail(SPIO_HIP_ERR_HIP_BASE + static_cast<int>(e), "HIP error: %s failed: %s (%d)", what,
                s, static_cast<int>(e));
}

int rtc_fail(hiprtcResult e, const char* what) {
    const char* s = g_api.hiprtcGetErrorString ? g_api.hiprtcGetErrorString(e) : "?";
    return fail(SPIO_HIP_ERR_HIPRTC_BASE + static_cast<int>(e), "hipRTC error: %s failed: %s (%d)",
                what, s, static_cast<int>(e));
}

#define REQUIRE_READY()                                                                        \
    do {                                                                                       \
        if (!g_api.ready)                                                                      \
            return fail(SPIO_HIP_ERR_NOT_INITIALIZED, "spio_hip_init has not been called");    \
    } while (0)

#define HIP_TRY(expr)                                  \
    do {                                               \
        hipError_t e_ = g_api.expr;                    \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

char* dup_string(const std::string& s) {
    char* p = static_cast<char*>(malloc(s.size() + 1));
    if (p) memcpy(p, s.c_str(), s.size() + 1);
    return p;
}

}  // namespace

extern "C" {

const char* spio_hip_last_error(void) { return g_last_error.c_str(); }

void spio_hip_free(void* ptr) { free(ptr); }

int spio_hip_init(const char* hip_library_path, const char* hiprtc_library_path) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_api.ready) return SPIO_HIP_OK;

    static const char* const hip_names[] = {"libamdhip64.so.7", "libamdhip64.so.6",
                                            "libamdhip64.so", "/opt/rocm/lib/libamdhip64.so",
                                            nullptr};
    static const char* const rtc_names[] = {"libhiprtc.so.7", "libhiprtc.so.6", "libhiprtc.so",
                                            "/opt/rocm/lib/libhiprtc.so", nullptr};
    std::string tried;
    Api api;
    api.hip_handle = open_library(hip_library_path, hip_names, &tried);
    if (!api.hip_handle)
        return fail(SPIO_HIP_ERR_DLOPEN, "cannot load the HIP runtime: %s", tried.c_str());
    api.rtc_handle = open_library(hiprtc_library_path, rtc_names, &tried);
    if (!api.rtc_handle)
        return fail(SPIO_HIP_ERR_DLOPEN, "cannot load hipRTC: %s", tried.c_str());

    std::string missing;
    void* h = api.hip_handle;
    bind(h, "hipInit", &api.hipInit, &missing);
    bind(h, "hipGetDeviceCount", &api.hipGetDeviceCount, &missing);
    bind(h, "hipSetDevice", &api.hipSetDevice, &missing);
    bind(h, "hipDeviceGetAttribute", &api.hipDeviceGetAttribute, &missing);
    bind(h, "hipDeviceGetName", &api.hipDeviceGetName, &missing);
    bind(h, "hipDeviceSynchronize", &api.hipDeviceSynchronize, &missing);
    bind(h, "hipStreamSynchronize", &api.hipStreamSynchronize, &missing);
    bind(h, "hipDriverGetVersion", &api.hipDriverGetVersion, &missing);
    bind(h, "hipRuntimeGetVersion", &api.hipRuntimeGetVersion, &missing);
    bind(h, "hipModuleLoadData", &api.hipModuleLoadData, &missing);
    bind(h, "hipModuleUnload", &api.hipModuleUnload, &missing);
    bind(h, "hipModuleGetFunction", &api.hipModuleGetFunction, &missing);
    bind(h, "hipFuncSetAttribute", &api.hipFuncSetAttribute, &missing);
    bind(h, "hipModuleLaunchKernel", &api.hipModuleLaunchKernel, &missing);
    bind(h, "hipEventCreate", &api.hipEventCreate, &missing);
    bind(h, "hipEventDestroy", &api.hipEventDestroy, &missing);
    bind(h, "hipEventRecord", &api.hipEventRecord, &missing);
    bind(h, "hipEventSynchronize", &api.hipEventSynchronize, &missing);
    bind(h, "hipEventElapsedTime", &api.hipEventElapsedTime, &missing);
    bind(h, "hipGetErrorString", &api.hipGetErrorString, &missing);
    void* r = api.rtc_handle;
    bind(r, "hiprtcCreateProgram", &api.hiprtcCreateProgram, &missing);
    bind(r, "hiprtcDestroyProgram", &api.hiprtcDestroyProgram, &missing);
    bind(r, "hiprtcCompileProgram", &api.hiprtcCompileProgram, &missing);
    bind(r, "hiprtcGetProgramLogSize", &api.hiprtcGetProgramLogSize, &missing);
    bind(r, "hiprtcGetProgramLog", &api.hiprtcGetProgramLog, &missing);
    bind(r, "hiprtcGetCodeSize", &api.hiprtcGetCodeSize, &missing);
    bind(r, "hiprtcGetCode", &api.hiprtcGetCode, &missing);
    bind(r, "hiprtcGetErrorString", &api.hiprtcGetErrorString, &missing);
    bind(r, "hiprtcVersion", &api.hiprtcVersion, &missing);
    if (!missing.empty())
        return fail(SPIO_HIP_ERR_SYMBOL, "missing runtime symbols: %s", missing.c_str());

    api.ready = true;
    g_api = api;
    return SPIO_HIP_OK;
}

int spio_hip_compile(const char* source, const char* name, int num_headers,
                     const char* const* header_sources, const char* const* header_names,
                     int num_options, const char* const* options, void** code, size_t* code_size,
                     char** log) {
    REQUIRE_READY();
    if (!source || !code || !code_size || num_headers < 0 || num_options < 0)
        return fail(SPIO_HIP_ERR_ARGUMENT, "spio_hip_compile: bad argument");
    *code = nullptr;
    *code_size = 0;
    if (log) *log = nullptr;

    hiprtcProgram prog = nullptr;
    hiprtcResult r = g_api.hiprtcCreateProgram(
        &prog, source, name ? name : "kernel.hip", num_headers,
        num_headers ? const_cast<const char**>(header_sources) : nullptr,
        num_headers ? const_cast<const char**>(header_names) : nullptr);
    if (r != HIPRTC_SUCCESS) return rtc_fail(r, "hiprtcCreateProgram");

    hiprtcResult cr =
        g_api.hiprtcCompileProgram(prog, num_options, const_cast<const char**>(options));

    std::string log_text;
    size_t log_size = 0;
    if (g_api.hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        log_text.resize(log_size);
        if (g_api.hiprtcGetProgramLog(prog, &log_text[0]) != HIPRTC_SUCCESS) log_text.clear();
        while (!log_text.empty() && log_text.back() == '\0') log_text.pop_back();
    }
    if (log && !log_text.empty()) *log = dup_string(log_text);

    if (cr != HIPRTC_SUCCESS) {
        g_api.hiprtcDestroyProgram(&prog);
        const char* s = g_api.hiprtcGetErrorString(cr);
        return fail(SPIO_HIP_ERR_COMPILE, "hipRTC compilation of %s failed: %s (%d)\n%s",
                    name ? name : "kernel.hip", s, static_cast<int>(cr), log_text.c_str());
    }

    size_t size = 0;
    r = g_api.hiprtcGetCodeSize(prog, &size);
    if (r != HIPRTC_SUCCESS || size == 0) {
        g_api.hiprtcDestroyProgram(&prog);
        return rtc_fail(r, "hiprtcGetCodeSize");
    }
    char* buf = static_cast<char*>(malloc(size));
    if (!buf) {
        g_api.hiprtcDestroyProgram(&prog);
        return fail(SPIO_HIP_ERR_ARGUMENT, "out of host memory for %zu byte code object", size);
    }
    r = g_api.hiprtcGetCode(prog, buf);
    g_api.hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) {
        free(buf);
        return rtc_fail(r, "hiprtcGetCode");
    }
    *code = buf;
    *code_size = size;
    return SPIO_HIP_OK;
}

int spio_hip_module_load(const void* code, void** module) {
    REQUIRE_READY();
    if (!code || !module) return fail(SPIO_HIP_ERR_ARGUMENT, "spio_hip_module_load: null argument");
    hipModule_t m = nullptr;
    HIP_TRY(hipModuleLoadData(&m, code));
    *module = m;
    return SPIO_HIP_OK;
}

int spio_hip_module_unload(void* module) {
    REQUIRE_READY();
    if (!module) return SPIO_HIP_OK;
    HIP_TRY(hipModuleUnload(static_cast<hipModule_t>(module)));
    return SPIO_HIP_OK;
}

int spio_hip_get_function(void* module, const char* kernel_name, void** function) {
    REQUIRE_READY();
    if (!module || !kernel_name || !function)
        return fail(SPIO_HIP_ERR_ARGUMENT, "spio_hip_get_function: null argument");
    hipFunction_t f = nullptr;
    HIP_TRY(hipModuleGetFunction(&f, static_cast<hipModule_t>(module), kernel_name));
    *function = f;
    return SPIO_HIP_OK;
}

int spio_hip_func_set_max_dynamic_lds(void* function, int bytes) {
    REQUIRE_READY();
    if (!function || bytes < 0)
        return fail(SPIO_HIP_ERR_ARGUMENT, "spio_hip_func_set_max_dynamic_lds: bad argument");
    HIP_TRY(hipFuncSetAttribute(function, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    return SPIO_HIP_OK;
}

}  // extern "C"

int spio_hip_set_error(int code, const char* text) {
    g_last_error = text ? text : "";
    return code;
}

int spio_hip_check_launch_args(void* function, unsigned gx, unsigned gy, unsigned gz, unsigned bx,
                               unsigned by, unsigned bz, int num_params) {
    if (!function) return fail(SPIO_HIP_ERR_ARGUMENT, "launch: null function handle");
    if (num_params < 0 || num_params > 16)
        return fail(SPIO_HIP_ERR_ARGUMENT, "launch: %d kernel arguments, at most 16 are supported",
                    num_params);
    if (!gx || !gy || !gz || !bx || !by || !bz)
        return fail(SPIO_HIP_ERR_ARGUMENT, "launch: zero-sized grid (%u,%u,%u) or block (%u,%u,%u)",
                    gx, gy, gz, bx, by, bz);
    if (static_cast<unsigned long long>(bx) * by * bz > 1024ull)
        return fail(SPIO_HIP_ERR_ARGUMENT, "launch: block of %llu threads exceeds 1024",
                    static_cast<unsigned long long>(bx) * by * bz);
    return SPIO_HIP_OK;
}

extern "C" {

int spio_hip_launch(void* function, unsigned grid_x, unsigned grid_y, unsigned grid_z,
                    unsigned block_x, unsigned block_y, unsigned block_z,
                    unsigned dynamic_lds_bytes, void* stream, void** params, int num_params) {
    REQUIRE_READY();
    int rc = spio_hip_check_launch_args(function, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                               num_params);
    if (rc) return rc;
    if (num_params > 0 && !params) return fail(SPIO_HIP_ERR_ARGUMENT, "launch: null params");
    HIP_TRY(hipModuleLaunchKernel(static_cast<hipFunction_t>(function), grid_x, grid_y, grid_z,
                                  block_x, block_y, block_z, dynamic_lds_bytes,
                                  static_cast<hipStream_t>(stream), params, nullptr));
    return SPIO_HIP_OK;
}

int spio_hip_launch_timed(void* function, unsigned grid_x, unsigned grid_y, unsigned grid_z,
                          unsigned block_x, unsigned block_y, unsigned block_z,
                          unsigned dynamic_lds_bytes, void* stream, void*** param_sets,
                          int num_sets, int num_params, int warmup, int iters,
                          float* elapsed_ms) {
    REQUIRE_READY();
    int rc = spio_hip_check_launch_args(function, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                               num_params);
    if (rc) return rc;
    if (!param_sets || num_sets < 1 || warmup < 0 || iters < 1 || !elapsed_ms)
        return fail(SPIO_HIP_ERR_ARGUMENT, "spio_hip_launch_timed: bad argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipFunction_t f = static_cast<hipFunction_t>(function);

    hipEvent_t start = nullptr, stop = nullptr;
    HIP_TRY(hipEventCreate(&start));
    hipError_t e = g_api.hipEventCreate(&stop);
    if (e != hipSuccess) {
        (void)g_api.hipEventDestroy(start);
        return hip_fail(e, "hipEventCreate");
    }
    int set = 0;
    e = hipSuccess;
    for (int i = 0; i < warmup && e == hipSuccess; ++i) {
        e = g_api.hipModuleLaunchKernel(f, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                                        dynamic_lds_bytes, s, param_sets[set], nullptr);
        set = (set + 1) % num_sets;
    }
    if (e == hipSuccess) e = g_api.hipEventRecord(start, s);
    for (int i = 0; i < iters && e == hipSuccess; ++i) {
        e = g_api.hipModuleLaunchKernel(f, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                                        dynamic_lds_bytes, s, param_sets[set], nullptr);
        set = (set + 1) % num_sets;
    }
    if (e == hipSuccess) e = g_api.hipEventRecord(stop, s);
    if (e == hipSuccess) e = g_api.hipEventSynchronize(stop);
    if (e == hipSuccess) e = g_api.hipEventElapsedTime(elapsed_ms, start, stop);
    (void)g_api.hipEventDestroy(start);
    (void)g_api.hipEventDestroy(stop);
    if (e != hipSuccess) return hip_fail(e, "timed launch");
    return SPIO_HIP_OK;
}

int spio_hip_launch_sequence_timed(const spio_hip_launch_desc_t* descs, int stages, int num_sets,
                                   void* stream, int warmup, int iters, float* elapsed_ms) {
    REQUIRE_READY();
    if (!descs || stages < 1 || num_sets < 1 || warmup < 0 || iters < 1 || !elapsed_ms)
        return fail(SPIO_HIP_ERR_ARGUMENT, "spio_hip_launch_sequence_timed: bad argument");
    for (int i = 0; i < stages * num_sets; ++i) {
        const spio_hip_launch_desc_t& d = descs[i];
        int rc = spio_hip_check_launch_args(d.function, d.grid[0], d.grid[1], d.grid[2], d.block[0],
                                   d.block[1], d.block[2], d.num_params);
        if (rc) return rc;
        if (d.num_params > 0 && !d.params)
            return fail(SPIO_HIP_ERR_ARGUMENT, "launch sequence: null params");
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipEvent_t start = nullptr, stop = nullptr;
    HIP_TRY(hipEventCreate(&start));
    hipError_t e = g_api.hipEventCreate(&stop);
    if (e != hipSuccess) {
        (void)g_api.hipEventDestroy(start);
        return hip_fail(e, "hipEventCreate");
    }
    auto run = [&](int set) {
        hipError_t err = hipSuccess;
        for (int st = 0; st < stages && err == hipSuccess; ++st) {
            const spio_hip_launch_desc_t& d = descs[set * stages + st];
            err = g_api.hipModuleLaunchKernel(static_cast<hipFunction_t>(d.function), d.grid[0],
                                              d.grid[1], d.grid[2], d.block[0], d.block[1],
                                              d.block[2], d.dynamic_lds_bytes, s, d.params, nullptr);
        }
        return err;
    };
    int set = 0;
    e = hipSuccess;
    for (int i = 0; i < warmup && e == hipSuccess; ++i, set = (set + 1) % num_sets) e = run(set);
    if (e == hipSuccess) e = g_api.hipEventRecord(start, s);
    for (int i = 0; i < iters && e == hipSuccess; ++i, set = (set + 1) % num_sets) e = run(set);
    if (e == hipSuccess) e = g_api.hipEventRecord(stop, s);
    if (e == hipSuccess) e = g_api.hipEventSynchronize(stop);
    if (e == hipSuccess) e = g_api.hipEventElapsedTime(elapsed_ms, start, stop);
    (void)g_api.hipEventDestroy(start);
    (void)g_api.hipEventDestroy(stop);
    if (e != hipSuccess) return hip_fail(e, "timed launch sequence");
    return SPIO_HIP_OK;
}

int spio_hip_device_count(int* count) {
    REQUIRE_READY();
    if (!count) return fail(SPIO_HIP_ERR_ARGUMENT, "null argument");
    HIP_TRY(hipGetDeviceCount(count));
    return SPIO_HIP_OK;
}

int spio_hip_device_attrs(int ordinal, spio_hip_device_attrs_t* attrs) {
    REQUIRE_READY();
    if (!attrs) return fail(SPIO_HIP_ERR_ARGUMENT, "null argument");
    memset(attrs, 0, sizeof(*attrs));
    HIP_TRY(hipDeviceGetAttribute(&attrs->compute_unit_count,
                                  hipDeviceAttributeMultiprocessorCount, ordinal));
    HIP_TRY(hipDeviceGetAttribute(&attrs->l2_cache_bytes, hipDeviceAttributeL2CacheSize, ordinal));
    HIP_TRY(hipDeviceGetAttribute(&attrs->max_lds_bytes_per_block,
                                  hipDeviceAttributeMaxSharedMemoryPerBlock, ordinal));
    HIP_TRY(hipDeviceGetAttribute(&attrs->wavefront_size, hipDeviceAttributeWarpSize, ordinal));
    HIP_TRY(hipDeviceGetAttribute(&attrs->clock_khz, hipDeviceAttributeClockRate, ordinal));
    HIP_TRY(hipDeviceGetAttribute(&attrs->memory_clock_khz, hipDeviceAttributeMemoryClockRate,
                                  ordinal));
    HIP_TRY(hipDeviceGetAttribute(&attrs->memory_bus_width_bits,
                                  hipDeviceAttributeMemoryBusWidth, ordinal));
    HIP_TRY(hipDeviceGetAttribute(&attrs->max_threads_per_block,
                                  hipDeviceAttributeMaxThreadsPerBlock, ordinal));
    HIP_TRY(hipDeviceGetName(attrs->name, static_cast<int>(sizeof(attrs->name)), ordinal));
    // The architecture string is only available through the properties
    // struct, whose layout differs between runtime releases; the versioned
    // symbol keeps the layout matching the header this file was built with.
    typedef hipError_t (*props_fn)(hipDeviceProp_t*, int);
    props_fn get_props =
        reinterpret_cast<props_fn>(dlsym(g_api.hip_handle, "hipGetDevicePropertiesR0600"));
    if (get_props) {
        hipDeviceProp_t* p = static_cast<hipDeviceProp_t*>(calloc(1, sizeof(hipDeviceProp_t) + 4096));
        if (p && get_props(p, ordinal) == hipSuccess) {
            strncpy(attrs->arch, p->gcnArchName, sizeof(attrs->arch) - 1);
        }
        free(p);
    }
    return SPIO_HIP_OK;
}

int spio_hip_set_device(int ordinal) {
    REQUIRE_READY();
    HIP_TRY(hipSetDevice(ordinal));
    return SPIO_HIP_OK;
}

int spio_hip_synchronize(void) {
    REQUIRE_READY();
    HIP_TRY(hipDeviceSynchronize());
    return SPIO_HIP_OK;
}

int spio_hip_stream_synchronize(void* stream) {
    REQUIRE_READY();
    HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return SPIO_HIP_OK;
}

int spio_hip_driver_version(int* version) {
    REQUIRE_READY();
    if (!version) return fail(SPIO_HIP_ERR_ARGUMENT, "null argument");
    HIP_TRY(hipDriverGetVersion(version));
    return SPIO_HIP_OK;
}

int spio_hip_runtime_version(int* version) {
    REQUIRE_READY();
    if (!version) return fail(SPIO_HIP_ERR_ARGUMENT, "null argument");
    HIP_TRY(hipRuntimeGetVersion(version));
    return SPIO_HIP_OK;
}

int spio_hiprtc_version(int* major, int* minor) {
    REQUIRE_READY();
    if (!major || !minor) return fail(SPIO_HIP_ERR_ARGUMENT, "null argument");
    hiprtcResult r = g_api.hiprtcVersion(major, minor);
    if (r != HIPRTC_SUCCESS) return rtc_fail(r, "hiprtcVersion");
    return SPIO_HIP_OK;
}

}  // extern "C"
