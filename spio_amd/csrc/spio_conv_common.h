// Shared definitions for the grouped-width-8 convolution kernels (gfx950).
//
// Every kernel of this directory is specialised at compile time: the shape of
// one convolution and the tile configuration arrive as SPIO_* macros, either
// from hipRTC options at run time or from -D flags of an offline hipcc build.
// Kernels therefore take only pointers, as the reference's kernels do
// (spio/src/conv2d_gw8.cu:10-12, spio/src/conv2d_gw8_wgrad.cu:10-12).
//
// Memory layouts (physical):
//   activations  [N][H][W][C]      fp16   (NCHW tensors with channels_last strides)
//   weights      [K][R][S][8]      fp16   ([K,8,R,S] tensors with channels_last strides)
//   bias         [K]               fp32
//   grad_weight  [K][R][S][8]      fp32
// A group is 8 consecutive channels: 16 bytes of one pixel.
#ifndef SPIO_CONV_COMMON_H
#define SPIO_CONV_COMMON_H

#ifndef SPIO_N
#error "shape macros (SPIO_N, SPIO_C, SPIO_H, SPIO_W, SPIO_R, SPIO_S, SPIO_PY, SPIO_PX) are required"
#endif

typedef _Float16 spio_half;
typedef _Float16 spio_half2 __attribute__((ext_vector_type(2)));
typedef _Float16 spio_half4 __attribute__((ext_vector_type(4)));
typedef _Float16 spio_half8 __attribute__((ext_vector_type(8)));
typedef float spio_float4 __attribute__((ext_vector_type(4)));
typedef unsigned int spio_uint2 __attribute__((ext_vector_type(2)));
typedef unsigned int spio_uint4 __attribute__((ext_vector_type(4)));
typedef short spio_short4 __attribute__((ext_vector_type(4)));

namespace spio {

// The convolution as the user states it (forward orientation).
constexpr int kN = SPIO_N;
constexpr int kC = SPIO_C;
constexpr int kH = SPIO_H;
constexpr int kW = SPIO_W;
constexpr int kR = SPIO_R;
constexpr int kS = SPIO_S;
constexpr int kPadY = SPIO_PY;
constexpr int kPadX = SPIO_PX;
constexpr int kP = kH + 2 * kPadY - kR + 1;
constexpr int kQ = kW + 2 * kPadX - kS + 1;
constexpr int kGroups = kC / 8;

static_assert(kC % 8 == 0, "channels must be a multiple of the group width 8");
static_assert(kP > 0 && kQ > 0, "empty output");

// The kernels use compiler builtins only, so they compile identically under
// hipRTC and under an offline hipcc build without any runtime header.
#define SPIO_DEVICE __device__ inline __attribute__((always_inline))
#define SPIO_LAUNCH_BOUNDS(threads) __attribute__((amdgpu_flat_work_group_size(threads, threads)))

SPIO_DEVICE int imin(int a, int b) { return a < b ? a : b; }
SPIO_DEVICE int imax(int a, int b) { return a > b ? a : b; }
SPIO_DEVICE int thread_id() { return (int)__builtin_amdgcn_workitem_id_x(); }
SPIO_DEVICE int block_id() { return (int)__builtin_amdgcn_workgroup_id_x(); }

// Workgroup barrier with LDS/global visibility among the waves of the group.
SPIO_DEVICE void block_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Orders the LDS accesses of the lanes of one wave: what some lanes stored before it is what
// other lanes of the same wave load after it.  The hardware executes the LDS operations of a
// wave in order anyway; this keeps the compiler from moving them across (the store and the load
// sit under disjoint lane masks, so nothing else tells it they depend on each other).
SPIO_DEVICE void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Streaming accesses: activations are touched once per kernel, so they are
// loaded and stored with the non-temporal hint (measured on MI355X: a plain
// 16-byte-per-lane copy gains about 10% from it).
#ifndef SPIO_NT
#define SPIO_NT 1
#endif
SPIO_DEVICE spio_uint4 load_stream(const spio_uint4* p) {
#if SPIO_NT
    return __builtin_nontemporal_load(p);
#else
    return *p;
#endif
}
SPIO_DEVICE void store_stream(spio_uint4 v, spio_uint4* p) {
#if SPIO_NT
    __builtin_nontemporal_store(v, p);
#else
    *p = v;
#endif
}

// Closes a group of 16-byte buffer stores.  Such a store reads its data registers for a few
// cycles after it issues; an instruction that writes one of them in the very next slot can have
// its value stored instead (seen on gfx950 as stray values in the first two channels of some
// pixels).  The compiler keeps that slot free only for some operand forms of the store, so the
// kernels do not rely on it: nothing is scheduled across this point, and the wait state between
// the last store and whatever follows is explicit.
#ifndef SPIO_STORE_GUARD
#define SPIO_STORE_GUARD 1
#endif
SPIO_DEVICE void store_group_end() {
#if SPIO_STORE_GUARD
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 0");
    __builtin_amdgcn_sched_barrier(0);
#endif
}

// Device-scope fp32 add without a return value.
SPIO_DEVICE void atomic_add_f32(float* address, float value) {
    __hip_atomic_fetch_add(address, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Bit-cast helpers between the 16-byte vector views of one (pixel, group).
union Pack16 {
    spio_uint4 u;
    spio_uint4 i;  // the buffer builtins' 128-bit operand type
    spio_half8 h;
    spio_half4 h4[2];
};

union Pack8 {
    spio_uint2 u;
    spio_half4 h;
    spio_short4 s;
};

}  // namespace spio

#endif  // SPIO_CONV_COMMON_H
