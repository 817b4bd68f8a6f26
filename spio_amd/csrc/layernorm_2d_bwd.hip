// Backward of the channel LayerNorm of layernorm_2d.hip (NHWC fp16 tensors, gfx950).
//
// The reference ships the forward device source only (spio/src/layernorm_2d.cu:81-222); this is
// the gradient of that contract, with the statistics recomputed from the input:
//   xhat[x][c] = (in[x][c] - mean[x]) * rstd[x]              mean, rstd as in the forward kernel
//   g[x][c]    = dout[x][c] * weight[c]                       (weight = 1 without one)
//   din[x][c]  = rn16(rstd[x] * (g - mean_c(g) - xhat * mean_c(g * xhat)))
//   dweight[c] = sum_x dout[x][c] * xhat[x][c]                fp32
//   dbias[c]   = sum_x dout[x][c]                             fp32
//
// Design: the lane mapping of the forward kernel (LPP lanes share a pixel, a lane keeps the same
// channels for all its pixels), so the per-channel sums stay in registers over the whole
// workgroup loop.  At the end the lanes of a wave that hold the same channels are added by an
// xor butterfly, the waves through LDS, and the workgroup writes one row of
// `partials[workgroup][2][C]` with plain stores: every row is written completely, so the
// workspace needs no zeroing and nothing is atomic (with atomics every workgroup would add to the
// same C addresses, one after the other).  The small <name>_reduce kernel below adds the rows
// into `sums[2][C]` (0 = grad_weight, 1 = grad_bias), which it overwrites.  HBM-bound: 4 bytes in,
// 2 bytes out per element.
#ifndef SPIO_LN_C
#error "SPIO_LN_C, SPIO_LN_PIXELS, SPIO_LN_LPP, SPIO_LN_THREADS, SPIO_LN_GRID are required"
#endif
#ifndef SPIO_LN_UNROLL
#define SPIO_LN_UNROLL 2
#endif
#ifndef SPIO_LN_HAS_WEIGHT
#define SPIO_LN_HAS_WEIGHT 1
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
constexpr int WAVES = THREADS / 64;
constexpr int PPW = 64 / LPP;             // pixels per wave and pass
constexpr int PPB = PPW * WAVES;          // pixels per workgroup and pass
constexpr int UN = SPIO_LN_UNROLL;
constexpr unsigned OOB = 0x80000000u;
static_assert(C % 8 == 0 && (LPP & (LPP - 1)) == 0 && LPP <= 64 && LPP * UPL >= UNITS, "bad geometry");

union Pack {
    ln_uint4 u;
    ln_half8 h;
};

template <int CTRL>
__device__ inline float dpp_add(float v) {
    const int other = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
    return v + __builtin_bit_cast(float, other);
}
__device__ inline float lane_xor_add(float v, int m) {
    const int lane = (int)__builtin_amdgcn_workitem_id_x() & 63;
    const int other = __builtin_amdgcn_ds_bpermute(((lane ^ m) << 2), __builtin_bit_cast(int, v));
    return v + __builtin_bit_cast(float, other);
}
// Sum over the LPP lanes of a pixel; every lane ends up with the total (as in the forward kernel).
__device__ inline float pixel_sum(float v) {
    if (LPP >= 2) v = dpp_add<0xB1>(v);    // quad_perm [1,0,3,2]
    if (LPP >= 4) v = dpp_add<0x4E>(v);    // quad_perm [2,3,0,1]
    if (LPP >= 8) v = dpp_add<0x141>(v);   // row_half_mirror
    if (LPP >= 16) v = dpp_add<0x140>(v);  // row_mirror
#pragma unroll
    for (int m = 16; m < LPP; m <<= 1) v = lane_xor_add(v, m);
    return v;
}
// Sum over the PPW lanes of a wave that hold the same channels (lanes sub, sub + LPP, ...).
__device__ inline float channel_sum(float v) {
#pragma unroll
    for (int m = LPP; m < 64; m <<= 1) v = lane_xor_add(v, m);
    return v;
}

}  // namespace

extern "C" __global__ void __attribute__((amdgpu_flat_work_group_size(THREADS, THREADS)))
SPIO_KERNEL_NAME(float* __restrict__ partials, ln_uint4* __restrict__ din, const ln_uint4* __restrict__ in,
                 const ln_uint4* __restrict__ dout, const float* __restrict__ weight) {
    constexpr long long num_workgroups = SPIO_LN_GRID;
    __shared__ float red[WAVES][2][LPP * UPL * 8];
    const int tid = (int)__builtin_amdgcn_workitem_id_x();
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int sub = lane % LPP;
    const int pix_in_pass = wave * PPW + lane / LPP;

    float w[UPL][8];
    bool live[UPL];
#pragma unroll
    for (int k = 0; k < UPL; ++k) {
        const int unit = sub + k * LPP;
        live[k] = unit < UNITS;
#pragma unroll
        for (int e = 0; e < 8; ++e) w[k][e] = (SPIO_LN_HAS_WEIGHT && live[k]) ? weight[unit * 8 + e] : 1.f;
    }
    float dw[UPL][8], db[UPL][8];
#pragma unroll
    for (int k = 0; k < UPL; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) dw[k][e] = db[k][e] = 0.f;

    constexpr long long PASS_PIXELS = (long long)PPB * UN;
    const long long passes = (PIXELS + PASS_PIXELS - 1) / PASS_PIXELS;
    for (long long it = (long long)__builtin_amdgcn_workgroup_id_x(); it < passes; it += num_workgroups) {
        const long long first = it * PASS_PIXELS;
        const long long left = PIXELS - first;
        const int npix = (int)(left < PASS_PIXELS ? left : PASS_PIXELS);
        // 32-bit buffer offsets cover 2 GiB: the descriptors are rebased per iteration
        const ln_rsrc rs_in = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<unsigned char*>(reinterpret_cast<const unsigned char*>(in)) + first * C * 2, 0, npix * C * 2,
            0x00020000);
        const ln_rsrc rs_dout = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<unsigned char*>(reinterpret_cast<const unsigned char*>(dout)) + first * C * 2, 0, npix * C * 2,
            0x00020000);
        const ln_rsrc rs_din = __builtin_amdgcn_make_buffer_rsrc(
            reinterpret_cast<unsigned char*>(din) + first * C * 2, 0, npix * C * 2, 0x00020000);

        Pack vx[UN][UPL], vd[UN][UPL];
        unsigned off[UN][UPL];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int pix = u * PPB + pix_in_pass;
#pragma unroll
            for (int k = 0; k < UPL; ++k) {
                off[u][k] = live[k] ? (unsigned)((pix * UNITS + sub + k * LPP) * 16) : OOB;
                vx[u][k].u = __builtin_amdgcn_raw_buffer_load_b128(rs_in, (int)off[u][k], 0, 2);
                vd[u][k].u = __builtin_amdgcn_raw_buffer_load_b128(rs_dout, (int)off[u][k], 0, 2);
            }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            // statistics as in the forward kernel (pixels past the end load zeros: rstd is finite,
            // every product below is zero, their stores are dropped)
            float x[UPL][8];
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < UPL; ++k)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[k][e] = (float)vx[u][k].h[e];
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
            const float rstd = __builtin_amdgcn_rsqf(pixel_sum(d2) * (1.0f / C) + SPIO_LN_EPS);
            // xhat (in place of x), g = dy * w, the two means, the channel sums
            float g[UPL][8];
            float sg = 0.f, sgx = 0.f;
#pragma unroll
            for (int k = 0; k < UPL; ++k)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float dy = (float)vd[u][k].h[e];  // dead units loaded zeros
                    x[k][e] = live[k] ? (x[k][e] - mean) * rstd : 0.f;
                    g[k][e] = dy * w[k][e];
                    sg += g[k][e];
                    sgx += g[k][e] * x[k][e];
                    dw[k][e] += dy * x[k][e];
                    db[k][e] += dy;
                }
            const float m1 = pixel_sum(sg) * (1.0f / C);
            const float m2 = pixel_sum(sgx) * (1.0f / C);
#pragma unroll
            for (int k = 0; k < UPL; ++k) {
                Pack o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o.h[e] = (_Float16)(rstd * (g[k][e] - m1 - x[k][e] * m2));
                __builtin_amdgcn_raw_buffer_store_b128(o.u, rs_din, (int)off[u][k], 0, 2);
            }
        }
    }

    // ---- the workgroup's row of partial sums: lanes with the same channels, then the waves ----
#pragma unroll
    for (int k = 0; k < UPL; ++k)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            dw[k][e] = channel_sum(dw[k][e]);
            db[k][e] = channel_sum(db[k][e]);
        }
    if (lane < LPP) {
#pragma unroll
        for (int k = 0; k < UPL; ++k)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                red[wave][0][(sub + k * LPP) * 8 + e] = dw[k][e];
                red[wave][1][(sub + k * LPP) * 8 + e] = db[k][e];
            }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    float* row = partials + (long long)__builtin_amdgcn_workgroup_id_x() * 2 * C;
    for (int i = tid; i < 2 * C; i += THREADS) {
        const int which = i / C;
        const int c = i % C;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) v += red[wv][which][c];
        row[i] = v;
    }
}

// Second stage: sums[i] = sum over the workgroups' rows of partials[row][i], i < 2*C.  A workgroup
// owns 32 columns; its 8 slices each add the rows r = slice, slice + 8, ... with up to 32 loads
// in flight, and meet in LDS.  Every element has one owner: no atomics, no dependence on timing.
#define SPIO_LN_CONCAT2(a, b) a##b
#define SPIO_LN_CONCAT(a, b) SPIO_LN_CONCAT2(a, b)
extern "C" __global__ void __attribute__((amdgpu_flat_work_group_size(256, 256)))
SPIO_LN_CONCAT(SPIO_KERNEL_NAME, _reduce)(float* __restrict__ sums, const float* __restrict__ partials) {
    constexpr int ROWS = SPIO_LN_GRID;
    constexpr int COLS = 32;
    constexpr int SLICES = 256 / COLS;
    // as many rows in flight per thread as a slice has, up to 32: one round trip to memory for up
    // to 256 rows (with 8 in flight the stage took 1.5-2 us longer on the 7x7 and 14x14 shapes)
    constexpr int UNR = (ROWS + SLICES - 1) / SLICES < 32 ? (ROWS + SLICES - 1) / SLICES : 32;
    __shared__ float red[SLICES][COLS];
    const int tid = (int)__builtin_amdgcn_workitem_id_x();
    const int cl = tid % COLS;
    const int slice = tid / COLS;
    const int col = (int)__builtin_amdgcn_workgroup_id_x() * COLS + cl;
    float sum = 0.f;
    if (col < 2 * C) {
        for (int base = slice; base < ROWS; base += SLICES * UNR) {
            float v[UNR];
#pragma unroll
            for (int i = 0; i < UNR; ++i) {
                const int r = base + i * SLICES;
                v[i] = r < ROWS ? partials[(long long)r * 2 * C + col] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < UNR; ++i) sum += v[i];
        }
    }
    red[slice][cl] = sum;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (slice == 0 && col < 2 * C) {
#pragma unroll
        for (int i = 1; i < SLICES; ++i) sum += red[i][cl];
        sums[col] = sum;
    }
}

