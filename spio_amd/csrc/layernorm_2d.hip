// LayerNorm over the channels of every pixel of an NHWC fp16 tensor (gfx950).
//
// Contract (reference kernel: spio/src/layernorm_2d.cu:81-222):
//   mean[x]  = sum_c in[x][c] / C                       (fp32)
//   var[x]   = sum_c (in[x][c] - mean[x])^2 / C          (fp32, two passes over registers)
//   out[x][c] = rn16((in[x][c] - mean[x]) * rsqrt(var[x] + eps) * weight[c] + bias[c])
// for every pixel x of the [N*H*W][C] matrix; weight and bias are fp32 and optional.
//
// Design: the operator is HBM-bound (2 bytes in, 2 bytes out per element), so what matters is
// that every load and store is a full 16-byte unit of contiguous pixels.  A pixel's C/8 units
// are spread over LPP = 2^k >= C/8 adjacent lanes (UPL units per lane when C/8 > 64), so a wave
// covers 64/LPP consecutive pixels with one load instruction per unit and the two sums of a
// pixel are xor-butterflies inside its LPP lanes.  A lane keeps the same channels for all its
// pixels, so weight and bias stay in registers.  Loads of SPIO_LN_UNROLL pixel groups are in
// flight per lane; buffer instructions predicate the tail (out-of-range loads give zeros,
// stores are dropped).
#ifndef SPIO_LN_C
#error "SPIO_LN_C, SPIO_LN_PIXELS, SPIO_LN_LPP, SPIO_LN_THREADS, SPIO_LN_GRID are required"
#endif
#ifndef SPIO_LN_UNROLL
#define SPIO_LN_UNROLL 4
#endif
#ifndef SPIO_LN_HAS_WEIGHT
#define SPIO_LN_HAS_WEIGHT 1
#endif
#ifndef SPIO_LN_HAS_BIAS
#define SPIO_LN_HAS_BIAS 1
#endif
#ifndef SPIO_LN_EPS
#define SPIO_LN_EPS 1e-6f
#endif

typedef _Float16 ln_half8 __attribute__((ext_vector_type(8)));
typedef unsigned int ln_uint4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t ln_rsrc;

namespace {

constexpr int C = SPIO_LN_C;
constexpr long long PIXELS = SPIO_LN_PIXELS;
constexpr int UNITS = C / 8;              // 16-byte units per pixel
constexpr int LPP = SPIO_LN_LPP;          // lanes per pixel (power of two, <= 64)
constexpr int UPL = (UNITS + LPP - 1) / LPP;  // units per lane
constexpr int THREADS = SPIO_LN_THREADS;
constexpr int PPW = 64 / LPP;             // pixels per wave and pass
constexpr int PPB = PPW * (THREADS / 64);     // pixels per workgroup and pass
constexpr int UN = SPIO_LN_UNROLL;
constexpr unsigned OOB = 0x80000000u;
static_assert(C % 8 == 0 && (LPP & (LPP - 1)) == 0 && LPP <= 64 && LPP * UPL >= UNITS, "bad geometry");

union Pack {
    ln_uint4 u;
    ln_half8 h;
};

// Sum over the LPP lanes of a pixel; every lane ends up with the total.  Inside a row of 16
// lanes the partner's value comes through the data-parallel-primitive operand path (swap inside
// pairs, swap the pairs of a quad, mirror the halves of 8, mirror the row); beyond a row through
// the LDS crossbar.
template <int CTRL>
__device__ inline float dpp_add(float v) {
    const int other = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
    return v + __builtin_bit_cast(float, other);
}
__device__ inline float pixel_sum(float v) {
    if (LPP >= 2) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    if (LPP >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    if (LPP >= 8) v = dpp_add<0x141>(v);  // row_half_mirror: lane i of 8 <-> lane 7-i
    if (LPP >= 16) v = dpp_add<0x140>(v); // row_mirror: lane i of 16 <-> lane 15-i
    const int lane = (int)__builtin_amdgcn_workitem_id_x() & 63;
#pragma unroll
    for (int m = 16; m < LPP; m <<= 1) {
        const int other = __builtin_amdgcn_ds_bpermute(((lane ^ m) << 2), __builtin_bit_cast(int, v));
        v += __builtin_bit_cast(float, other);
    }
    return v;
}

}  // namespace

extern "C" __global__ void __attribute__((amdgpu_flat_work_group_size(THREADS, THREADS)))
SPIO_KERNEL_NAME(ln_uint4* __restrict__ out, const ln_uint4* __restrict__ in,
                 const float* __restrict__ weight, const float* __restrict__ bias) {
    // the launch grid is a compile-time constant (reading it from the dispatch packet would cost
    // every wave a fetch from host memory)
    constexpr long long num_workgroups = SPIO_LN_GRID;
    const int tid = (int)__builtin_amdgcn_workitem_id_x();
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int sub = lane % LPP;                         // this lane's place among its pixel's lanes
    const int pix_in_pass = wave * PPW + lane / LPP;    // this lane's pixel within a workgroup pass

    // 32-bit buffer offsets cover 2 GiB: the descriptor is rebased per workgroup iteration below
    float w[UPL][8], b[UPL][8];
    bool live[UPL];
#pragma unroll
    for (int k = 0; k < UPL; ++k) {
        const int unit = sub + k * LPP;
        live[k] = unit < UNITS;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            w[k][e] = (SPIO_LN_HAS_WEIGHT && live[k]) ? weight[unit * 8 + e] : 1.f;
            b[k][e] = (SPIO_LN_HAS_BIAS && live[k]) ? bias[unit * 8 + e] : 0.f;
        }
    }

    constexpr long long PASS_PIXELS = (long long)PPB * UN;  // pixels a workgroup takes per iteration
    const long long passes = (PIXELS + PASS_PIXELS - 1) / PASS_PIXELS;
    for (long long it = (long long)__builtin_amdgcn_workgroup_id_x(); it < passes; it += num_workgroups) {
        const long long first = it * PASS_PIXELS;
        const long long left = PIXELS - first;
        const int npix = (int)(left < PASS_PIXELS ? left : PASS_PIXELS);
        const ln_rsrc rs_in = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<unsigned char*>(reinterpret_cast<const unsigned char*>(in)) + first * C * 2, 0, npix * C * 2,
            0x00020000);
        const ln_rsrc rs_out = __builtin_amdgcn_make_buffer_rsrc(
            reinterpret_cast<unsigned char*>(out) + first * C * 2, 0, npix * C * 2, 0x00020000);

        Pack v[UN][UPL];
        unsigned off[UN][UPL];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int pix = u * PPB + pix_in_pass;
#pragma unroll
            for (int k = 0; k < UPL; ++k) {
                off[u][k] = live[k] ? (unsigned)((pix * UNITS + sub + k * LPP) * 16) : OOB;
                v[u][k].u = __builtin_amdgcn_raw_buffer_load_b128(rs_in, (int)off[u][k], 0, 2);
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            float x[UPL][8];
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < UPL; ++k)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[k][e] = (float)v[u][k].h[e];  // dead units loaded zeros
                    s += x[k][e];
                }
            const float mean = pixel_sum(s) * (1.0f / C);
            float d2 = 0.f;
#pragma unroll
            for (int k = 0; k < UPL; ++k)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float d = x[k][e] - mean;
                    d2 += live[k] ? d * d : 0.f;
                }
            const float var = pixel_sum(d2) * (1.0f / C);
            const float rstd = __builtin_amdgcn_rsqf(var + SPIO_LN_EPS);
#pragma unroll
            for (int k = 0; k < UPL; ++k) {
                Pack o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o.h[e] = (_Float16)((x[k][e] - mean) * (rstd * w[k][e]) + b[k][e]);
                __builtin_amdgcn_raw_buffer_store_b128(o.u, rs_out, (int)off[u][k], 0, 2);
            }
        }
    }
}
