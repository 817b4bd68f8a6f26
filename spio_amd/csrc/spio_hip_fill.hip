// spio_hip_zero_fill_async -- clear a device buffer with a kernel.
//
// The weight-gradient kernels add into grad_weight, so the buffer has to hold
// zeros when they start.  Callers without a tensor library clear it through
// this entry point.  It launches a small fill kernel rather than a runtime
// memset: a kernel node behaves the same eagerly and under HIP graph capture,
// so the call may sit inside a captured region.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

#include "spio_hip.h"
#include "spio_hip_internal.h"

namespace {

constexpr int kFillThreads = 256;
constexpr unsigned kMaxFillBlocks = 2048;  // 8 workgroups per CU; the kernel strides over the rest

// Bytes before the first and after the last 16-byte boundary are written one by one (by the
// first lanes of block 0); everything between as 16-byte vectors, grid-strided.
__global__ void __launch_bounds__(kFillThreads)
zero_fill_kernel(unsigned char* ptr, size_t bytes, size_t head, size_t vectors) {
    const size_t tid = static_cast<size_t>(blockIdx.x) * kFillThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kFillThreads;
    uint4* body = reinterpret_cast<uint4*>(ptr + head);
    for (size_t i = tid; i < vectors; i += stride) body[i] = uint4{0u, 0u, 0u, 0u};
    const size_t tail_begin = head + vectors * 16;
    if (tid < head) ptr[tid] = 0;
    if (tid < bytes - tail_begin) ptr[tail_begin + tid] = 0;
}

}  // namespace

extern "C" int spio_hip_zero_fill_async(void* device_ptr, size_t bytes, void* stream) {
    if (!device_ptr && bytes) return spio_hip_set_error(SPIO_HIP_ERR_ARGUMENT, "zero fill: null pointer");
    if (!bytes) return SPIO_HIP_OK;
    const uintptr_t address = reinterpret_cast<uintptr_t>(device_ptr);
    size_t head = static_cast<size_t>((16 - address % 16) % 16);
    if (head > bytes) head = bytes;
    const size_t vectors = (bytes - head) / 16;
    // head and tail are shorter than 16 bytes each: the first 16 threads cover them
    size_t blocks = (vectors + kFillThreads - 1) / kFillThreads;
    if (blocks < 1) blocks = 1;
    if (blocks > kMaxFillBlocks) blocks = kMaxFillBlocks;
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kFillThreads), 0,
                       static_cast<hipStream_t>(stream), static_cast<unsigned char*>(device_ptr), bytes,
                       head, vectors);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        char buf[256];
        snprintf(buf, sizeof(buf), "HIP error: zero-fill launch failed: %s (%d)", hipGetErrorString(e),
                 static_cast<int>(e));
        return spio_hip_set_error(SPIO_HIP_ERR_HIP_BASE + static_cast<int>(e), buf);
    }
    return SPIO_HIP_OK;
}
