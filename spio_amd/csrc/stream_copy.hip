// Plain streaming copy: one 16-byte non-temporal load and store per lane.
//
// Not part of the convolution path.  It is the yardstick the benchmark and the
// profiles use: its measured rate is the HBM bandwidth a kernel that reads X
// bytes and writes X bytes can reach on this device, and the HBM traffic
// counters of the profiler are scaled by what they report for this kernel,
// whose traffic is known exactly (n * 16 bytes read, n * 16 bytes written).
typedef unsigned int spio_copy_u4 __attribute__((ext_vector_type(4)));

extern "C" __global__ void __attribute__((amdgpu_flat_work_group_size(256, 256)))
spio_stream_copy(spio_copy_u4* __restrict__ dst, const spio_copy_u4* __restrict__ src, long long n) {
    const long long i = (long long)__builtin_amdgcn_workgroup_id_x() * 256 + __builtin_amdgcn_workitem_id_x();
    if (i < n) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}
