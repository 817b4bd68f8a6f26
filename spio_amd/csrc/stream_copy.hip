// Streaming copies: yardsticks, not part of the convolution path.
//
// Their measured rate is the HBM bandwidth that a kernel which reads X bytes and
// writes X bytes can reach on this device, and the HBM traffic counters of the
// profiler are scaled by what they report for the plain kernel, whose traffic is
// known exactly (n * 16 bytes read, n * 16 bytes written).
//
//   spio_stream_copy          one 16-byte non-temporal load and store per lane,
//                             one workgroup of 256 lanes per 4 KiB.
//   spio_stream_copy_strided  a fixed grid of workgroups walks the buffer in
//                             chunks of SPIO_COPY_THREADS * SPIO_COPY_UNROLL
//                             16-byte units (workgroup g takes chunks g, g + grid,
//                             ...), with SPIO_COPY_UNROLL independent loads in
//                             flight per lane.  The benchmark tries a few (lanes,
//                             unroll, grid) combinations and quotes the best as
//                             the ceiling.  The number of workgroups is a kernel
//                             argument: reading it from the dispatch packet costs a
//                             fetch from host memory in every wave (measured: +10 us
//                             on a 17 us kernel).
//   spio_stream_combine_strided  the same walk with two sources and one destination
//                             (dst = a ^ b): the mix of the fused backward kernel,
//                             which reads two activation tensors and writes one.
typedef unsigned int spio_copy_u4 __attribute__((ext_vector_type(4)));

#ifndef SPIO_COPY_THREADS
#define SPIO_COPY_THREADS 256
#endif
#ifndef SPIO_COPY_UNROLL
#define SPIO_COPY_UNROLL 4
#endif

extern "C" __global__ void __attribute__((amdgpu_flat_work_group_size(256, 256)))
spio_stream_copy(spio_copy_u4* __restrict__ dst, const spio_copy_u4* __restrict__ src, long long n) {
    const long long i = (long long)__builtin_amdgcn_workgroup_id_x() * 256 + __builtin_amdgcn_workitem_id_x();
    if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

extern "C" __global__ void __attribute__((amdgpu_flat_work_group_size(SPIO_COPY_THREADS, SPIO_COPY_THREADS)))
spio_stream_copy_strided(spio_copy_u4* __restrict__ dst, const spio_copy_u4* __restrict__ src, long long n,
                         long long num_workgroups) {
    constexpr long long CHUNK = (long long)SPIO_COPY_THREADS * SPIO_COPY_UNROLL;
    const long long chunks = (n + CHUNK - 1) / CHUNK;
    const int tid = __builtin_amdgcn_workitem_id_x();
    for (long long c = __builtin_amdgcn_workgroup_id_x(); c < chunks; c += num_workgroups) {
        const long long base = c * CHUNK + tid;
        spio_copy_u4 v[SPIO_COPY_UNROLL];
#pragma unroll
        for (int u = 0; u < SPIO_COPY_UNROLL; ++u) {
            const long long i = base + (long long)u * SPIO_COPY_THREADS;
            v[u] = __builtin_nontemporal_load(src + (i < n ? i : n - 1));
        }
#pragma unroll
        for (int u = 0; u < SPIO_COPY_UNROLL; ++u) {
            const long long i = base + (long long)u * SPIO_COPY_THREADS;
            if (i < n) __builtin_nontemporal_store(v[u], dst + i);
        }
    }
}

extern "C" __global__ void __attribute__((amdgpu_flat_work_group_size(SPIO_COPY_THREADS, SPIO_COPY_THREADS)))
spio_stream_combine_strided(spio_copy_u4* __restrict__ dst, const spio_copy_u4* __restrict__ a,
                            const spio_copy_u4* __restrict__ b, long long n, long long num_workgroups) {
    constexpr long long CHUNK = (long long)SPIO_COPY_THREADS * SPIO_COPY_UNROLL;
    const long long chunks = (n + CHUNK - 1) / CHUNK;
    const int tid = __builtin_amdgcn_workitem_id_x();
    for (long long c = __builtin_amdgcn_workgroup_id_x(); c < chunks; c += num_workgroups) {
        const long long base = c * CHUNK + tid;
        spio_copy_u4 va[SPIO_COPY_UNROLL], vb[SPIO_COPY_UNROLL];
#pragma unroll
        for (int u = 0; u < SPIO_COPY_UNROLL; ++u) {
            const long long i = base + (long long)u * SPIO_COPY_THREADS;
            va[u] = __builtin_nontemporal_load(a + (i < n ? i : n - 1));
            vb[u] = __builtin_nontemporal_load(b + (i < n ? i : n - 1));
        }
#pragma unroll
        for (int u = 0; u < SPIO_COPY_UNROLL; ++u) {
            const long long i = base + (long long)u * SPIO_COPY_THREADS;
            if (i < n) __builtin_nontemporal_store(va[u] ^ vb[u], dst + i);
        }
    }
}
