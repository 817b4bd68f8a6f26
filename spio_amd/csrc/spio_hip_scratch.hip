// spio_hip_launch_scratch -- a launch that brings its own workspace.
//
// Two-stage kernels (the weight gradient that stores per-workgroup partial
// sums and folds them in a second kernel) need device memory beyond their
// inputs and outputs.  Through spio_hip_launch the caller allocates it and
// passes it as a kernel argument.  Callers that must not allocate -- code
// under HIP graph capture, tight serving loops -- use this entry point
// instead: the workspace is a fixed array in device memory that belongs to the
// library, and the entry point puts its address into the argument slot the
// caller names.  Nothing is allocated here or in anything this file calls.
//
// The array exists once per GPU (each device that loads this library's code
// object holds its own copy at its own address) and is shared by every call on
// that GPU: it keeps the previous call's contents, and calls that overlap on
// one GPU (two streams, two threads) race on it.  The two-stage weight
// gradient writes every partial sum it later reads, so nothing needs clearing
// between calls.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <mutex>

#include "spio_hip.h"
#include "spio_hip_internal.h"

namespace {

// The workspace.  In host code this name is only a handle for
// hipGetSymbolAddress; the device address is looked up once per device below
// and that pointer is what kernels receive.
static __device__ __align__(256) unsigned char scratch[SPIO_HIP_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int fail(int code, const char* what, hipError_t e) {
    char buf[512];
    snprintf(buf, sizeof(buf), "HIP error: %s failed: %s (%d)", what, hipGetErrorString(e),
             static_cast<int>(e));
    return spio_hip_set_error(code, buf);
}

// Device address of `scratch` on the current device (looked up on first use).
int scratch_address(void** out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return fail(SPIO_HIP_ERR_HIP_BASE + static_cast<int>(e), "hipGetDevice", e);
    if (device < 0 || device >= kMaxDevices)
        return spio_hip_set_error(SPIO_HIP_ERR_ARGUMENT, "spio_hip_launch_scratch: device ordinal out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(SPIO_HIP_ERR_HIP_BASE + static_cast<int>(e), "hipGetSymbolAddress(scratch)", e);
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return SPIO_HIP_OK;
}

}  // namespace

extern "C" int spio_hip_launch_scratch(void* function, unsigned grid_x, unsigned grid_y, unsigned grid_z,
                                       unsigned block_x, unsigned block_y, unsigned block_z,
                                       unsigned dynamic_lds_bytes, void* stream, void** params,
                                       int num_params, int scratch_param, size_t scratch_bytes) {
    int rc = spio_hip_check_launch_args(function, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                                        num_params);
    if (rc) return rc;
    if (!params || scratch_param < 0 || scratch_param >= num_params)
        return spio_hip_set_error(SPIO_HIP_ERR_ARGUMENT,
                                  "spio_hip_launch_scratch: scratch_param does not name a kernel argument");
    if (scratch_bytes > static_cast<size_t>(SPIO_HIP_SCRATCH_BYTES)) {
        char buf[256];
        snprintf(buf, sizeof(buf),
                 "spio_hip_launch_scratch: %zu bytes of workspace requested, the static workspace holds %zu",
                 scratch_bytes, static_cast<size_t>(SPIO_HIP_SCRATCH_BYTES));
        return spio_hip_set_error(SPIO_HIP_ERR_ARGUMENT, buf);
    }
    void* workspace = nullptr;
    rc = scratch_address(&workspace);
    if (rc) return rc;

    // A private copy of the argument table with the workspace in its slot; the caller's table
    // and slot storage are left untouched.
    void* args[16];
    for (int i = 0; i < num_params; ++i) args[i] = params[i];
    args[scratch_param] = &workspace;
    hipError_t e = hipModuleLaunchKernel(static_cast<hipFunction_t>(function), grid_x, grid_y, grid_z,
                                         block_x, block_y, block_z, dynamic_lds_bytes,
                                         static_cast<hipStream_t>(stream), args, nullptr);
    if (e != hipSuccess)
        return fail(SPIO_HIP_ERR_HIP_BASE + static_cast<int>(e), "hipModuleLaunchKernel", e);
    return SPIO_HIP_OK;
}
