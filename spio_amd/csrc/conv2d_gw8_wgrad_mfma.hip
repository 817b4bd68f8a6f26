// Row-streaming MFMA kernel for the conv2d_gw8 weight gradient (gfx950).
//
// Contract (reference kernel: spio/src/conv2d_gw8_wgrad.cu:10-226):
//   dw[k,r,s,c] += sum_{n,p,q} x[n,p+r-py,q+s-px,8g+c] * dy[n,p,q,k]      g = k / 8
// fp16 operands, fp32 accumulation, fp32 result added into `grad_weight`
// ([K][R][S][8] floats) with atomics, so the caller zeroes it first
// (spio/functional/conv2d_gw8_function.py:124-130).
//
// Design
//   * A workgroup owns SPIO_BH rows of dy (output rows) of SPIO_NB images side
//     by side, for SPIO_GB channel groups, and repeats that for SPIO_ITERS
//     image blocks before it publishes its sums.  Per step it stages one row
//     of x and one row of dy in LDS ([group][flattened pixel][8 ch], zero
//     halo materialised once, as in the forward kernel).
//   * One wave owns one group.  The contraction runs over pixels, so both MFMA
//     operands need "8 pixels of one channel" per lane while memory holds
//     "8 channels of one pixel"; the transposing LDS read of gfx950
//     (ds_read_b64_tr_b16) delivers exactly that from the pixel-major rows.
//   * v_mfma_f32_16x16x32_f16 per 32-pixel chunk:
//         A (16 x 32) = dy:  rows m = 8*j + k    (two dy rows j of an aligned row pair, 8 k)
//         B (32 x 16) = x:   cols n = 8*sj + c   (two column taps sj, 8 c)
//     so one MFMA yields dw for 2 filter rows x 2 filter columns.  For the x
//     row of step t and the dy row pair (2i, 2i+1) the filter rows are
//     r = delta - j with delta = t - 2i in [0, R]; there is one accumulator per
//     (delta, column-tap pair).  Entries with r or s out of range are never read.
//   * At the end dw[k,r,s,c] = acc[delta=r] (lanes with j=0) + acc[delta=r+1]
//     (lanes with j=1); the halves are combined through LDS.  fp32 atomics are
//     the scarce resource (the device retires roughly 128 per clock in total,
//     and every workgroup owes R*S*64 of them per group), so there are two
//     ways to publish: SPIO_PARTIALS=0 adds straight into grad_weight with
//     atomics; SPIO_PARTIALS=1 stores each workgroup's sums into its own
//     partial image of a workspace with plain stores, and the small
//     <name>_reduce kernel below folds the partial images into grad_weight.
//     (Reducing inside the kernel by "the last workgroup of a group to finish"
//     was measured and rejected: the device-scope release/acquire fences it
//     needs write back and invalidate the L2 of an XCD and cost more than the
//     atomics they save.)
#include "spio_conv_common.h"

using namespace spio;

#ifndef SPIO_NB
#define SPIO_NB 1
#endif
#ifndef SPIO_ITERS
#define SPIO_ITERS 1
#endif
#ifndef SPIO_PF
#define SPIO_PF 2
#endif
#ifndef SPIO_PARTIALS
#define SPIO_PARTIALS 0
#endif
#ifndef SPIO_TS
#define SPIO_TS 1
#endif

namespace {

constexpr int GB = SPIO_GB;        // groups (waves) per workgroup
constexpr int BH = SPIO_BH;        // dy rows per workgroup
constexpr int NB = SPIO_NB;        // images side by side
constexpr int ITERS = SPIO_ITERS;  // image blocks per workgroup
constexpr int TS = SPIO_TS;        // waves sharing the 32-pixel chunks of one group
constexpr int WAVES = GB * TS;
constexpr int THREADS = 64 * WAVES;
constexpr int PF = SPIO_PF;  // prefetch distance in rows (even)

constexpr int S2 = 2 * ((kS + 1) / 2);
constexpr int NBLK = S2 / 2;   // column-tap pairs
constexpr int ND = kR + 1;     // values of delta
constexpr int WPI = kQ + kS - 1;  // padded width of one image (= W + 2*px)
constexpr int F = NB * WPI;
constexpr int KSPAN = (NB - 1) * WPI + kQ;  // flattened pixels that carry dy
constexpr int KC = (KSPAN + 31) / 32;       // 32-pixel chunks
constexpr int FPX = 32 * KC + S2 - 1;
constexpr int GSX = FPX + ((9 - FPX % 16) + 16) % 16;  // x group stride (pixels), = 9 mod 16
constexpr int FPD = 32 * KC;
constexpr int GSD = FPD + ((9 - FPD % 16) + 16) % 16;  // dy group stride
constexpr int NRX = 2;                                 // x ring rows
constexpr int NRD = 2 * ((kR + 2) / 2);                // dy ring rows: even, >= R+1
constexpr int XROW_UNITS = GB * GSX;
// dy ring rows are 64 bytes apart modulo the 256-byte bank period, so the two rows of a
// pair that one transposing read touches fall into different banks.
constexpr int DROW_UNITS = GB * GSD + ((4 - (GB * GSD) % 16) + 16) % 16;
constexpr int X_CELLS = F * GB;
constexpr int LPTX = (X_CELLS + THREADS - 1) / THREADS;
constexpr int D_CELLS = NB * kQ * GB;
constexpr int LPTD = (D_CELLS + THREADS - 1) / THREADS;
constexpr int GBLKS = (kGroups + GB - 1) / GB;
constexpr int PBLKS = (kP + BH - 1) / BH;
constexpr int NBLKS = (kN + NB * ITERS - 1) / (NB * ITERS);
constexpr int NUM_BLOCKS = GBLKS * PBLKS * NBLKS;
constexpr int STEPS = BH + kR - 1;

static_assert((NRX * XROW_UNITS + NRD * DROW_UNITS) * 16 <= 160 * 1024, "LDS overflow");
static_assert(NRD % 2 == 0 && NRD >= kR + 1, "dy ring too small");
static_assert(PF >= 2 && PF % 2 == 0, "prefetch distance must be even");
constexpr int PART_WAVE_FLOATS = kR * NBLK * 4 * 32;  // floats one wave publishes (partial-block layout)


SPIO_DEVICE spio_half8 read_tr_pair(const unsigned char* lo, const unsigned char* hi) {
    typedef spio_short4 __attribute__((address_space(3))) * lds_ptr;
    union {
        spio_short4 s[2];
        spio_half8 h;
    } v;
    v.s[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)lo);
    v.s[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)hi);
    return v.h;
}

}  // namespace

extern "C" __global__ void SPIO_LAUNCH_BOUNDS(THREADS)
SPIO_KERNEL_NAME(float* __restrict__ grad_weight, const spio_uint4* __restrict__ x,
                 const spio_uint4* __restrict__ dy) {
    // One LDS block: the x ring, then the dy ring; reused as reduction scratch at the end.
    __shared__ spio_uint4 lds[NRX * XROW_UNITS + NRD * DROW_UNITS];
    spio_uint4* const xring = lds;
    spio_uint4* const dring = lds + NRX * XROW_UNITS;

    const int tid = thread_id();
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wg = wave % GB;  // group within the workgroup
    const int ws = wave / GB;  // which share of the 32-pixel chunks this wave multiplies

    int b = block_id();
    if (NUM_BLOCKS % 8 == 0) b = (b & 7) * (NUM_BLOCKS / 8) + (b >> 3);
    const int pb = b % PBLKS;
    const int cb = (b / PBLKS) % GBLKS;
    const int nbk = b / (PBLKS * GBLKS);
    const int p0 = pb * BH;
    const int bh_eff = imin(BH, kP - p0);  // dy rows that exist in this block
    const int gglob = cb * GB + wg;
    const bool wave_active = gglob < kGroups;

    // zero both rings once: halo, gap and slack cells are never written again
    for (int i = tid; i < NRX * XROW_UNITS; i += THREADS) xring[i] = spio_uint4{0u, 0u, 0u, 0u};
    for (int i = tid; i < NRD * DROW_UNITS; i += THREADS) dring[i] = spio_uint4{0u, 0u, 0u, 0u};

    // lane roles inside the transposing reads: block kb = lane/16 covers pixels 8*kb..8*kb+7,
    // source lane sigma = lane%16 = 4*jr + t supplies pixel jr (+4 for the second read) of
    // unit t/2 (dy row j or column tap sj) and channel half t%2.
    const int kb = lane >> 4;
    const int jr = (lane & 15) >> 2;
    const int tt = lane & 3;
    const int sel = tt >> 1;  // j for A, sj for B
    const int xfrag_off = ((wg * GSX + 8 * kb + jr + sel) * 16) + (tt & 1) * 8;   // bytes in an x row
    const int dfrag_off = ((wg * GSD + 8 * kb + jr) * 16) + (tt & 1) * 8;         // bytes in a dy row

    spio_float4 acc[ND][NBLK];
#pragma unroll
    for (int d = 0; d < ND; ++d)
#pragma unroll
        for (int nb = 0; nb < NBLK; ++nb) acc[d][nb] = spio_float4{0.f, 0.f, 0.f, 0.f};

    const long long xrow_units = (long long)kW * kGroups;
    const long long drow_units = (long long)kQ * kGroups;

    for (int it = 0; it < ITERS; ++it) {
        const int n0 = (nbk * ITERS + it) * NB;
        if (n0 >= kN) break;

        // ---- loop-invariant addressing for this image block ----
        int x_off[LPTX], x_lds[LPTX];
#pragma unroll
        for (int l = 0; l < LPTX; ++l) {
            const int cell = tid + THREADS * l;
            x_off[l] = -1;
            x_lds[l] = -1;
            if (cell < X_CELLS) {
                const int g = cell % GB;
                const int f = cell / GB;
                const int img = f / WPI;
                const int col = f % WPI - kPadX;
                x_lds[l] = g * GSX + f;
                if (col >= 0 && col < kW && n0 + img < kN && cb * GB + g < kGroups)
                    x_off[l] = ((n0 + img) * kH * kW + col) * kGroups + cb * GB + g;
            }
        }
        int d_off[LPTD], d_lds[LPTD];
#pragma unroll
        for (int l = 0; l < LPTD; ++l) {
            const int cell = tid + THREADS * l;
            d_off[l] = -1;
            d_lds[l] = -1;
            if (cell < D_CELLS) {
                const int g = cell % GB;
                const int q = (cell / GB) % kQ;
                const int img = cell / (GB * kQ);
                d_lds[l] = g * GSD + img * WPI + q;
                if (n0 + img < kN && cb * GB + g < kGroups)
                    d_off[l] = ((n0 + img) * kP * kQ + q) * kGroups + cb * GB + g;
            }
        }

        // ---- prologue: rows 0..PF-1 into registers, row 0 into LDS ----
        spio_uint4 xpre[PF][LPTX], dpre[PF][LPTD];
#pragma unroll
        for (int t = 0; t < PF; ++t) {
            const int h = p0 + t - kPadY;
            const bool x_ok = t < STEPS && h >= 0 && h < kH;
#pragma unroll
            for (int l = 0; l < LPTX; ++l) {
                xpre[t][l] = spio_uint4{0u, 0u, 0u, 0u};
                if (x_ok && x_off[l] >= 0) xpre[t][l] = load_stream(x + x_off[l] + h * xrow_units);
            }
            const bool d_ok = t < bh_eff;
#pragma unroll
            for (int l = 0; l < LPTD; ++l) {
                dpre[t][l] = spio_uint4{0u, 0u, 0u, 0u};
                if (d_ok && d_off[l] >= 0) dpre[t][l] = load_stream(dy + d_off[l] + (p0 + t) * drow_units);
            }
        }
        block_sync();  // rings zeroed / previous image block finished
#pragma unroll
        for (int l = 0; l < LPTX; ++l)
            if (x_lds[l] >= 0) xring[x_lds[l]] = xpre[0][l];
#pragma unroll
        for (int l = 0; l < LPTD; ++l)
            if (d_lds[l] >= 0) dring[d_lds[l]] = dpre[0][l];
        block_sync();

        for (int tb = 0; tb < STEPS; tb += PF) {
#pragma unroll
            for (int uf = 0; uf < PF; ++uf) {
                const int t = tb + uf;
                if (t >= STEPS) break;
                const int uu = uf & 1;  // parity of t: x ring row and the parity of delta

                // 1. prefetch rows t+PF (their register buffer held row t, now in LDS)
                {
                    const int t2 = t + PF;
                    const int h = p0 + t2 - kPadY;
                    const bool x_ok = t2 < STEPS && h >= 0 && h < kH;
#pragma unroll
                    for (int l = 0; l < LPTX; ++l) {
                        spio_uint4 v = spio_uint4{0u, 0u, 0u, 0u};
                        if (x_ok && x_off[l] >= 0) v = load_stream(x + x_off[l] + h * xrow_units);
                        xpre[uf][l] = v;
                    }
                    const bool d_ok = t2 < bh_eff;
#pragma unroll
                    for (int l = 0; l < LPTD; ++l) {
                        spio_uint4 v = spio_uint4{0u, 0u, 0u, 0u};
                        if (d_ok && d_off[l] >= 0) v = load_stream(dy + d_off[l] + (p0 + t2) * drow_units);
                        dpre[uf][l] = v;
                    }
                }

                // 2. x row t against the dy row pairs it overlaps
                const int hcur = p0 + t - kPadY;
                if (wave_active && hcur >= 0 && hcur < kH) {
                    const unsigned char* xrow =
                        reinterpret_cast<const unsigned char*>(xring + uu * XROW_UNITS) + xfrag_off;
#pragma unroll
                    for (int ci = 0; ci < (KC + TS - 1) / TS; ++ci) {
                        const int ch = ws + TS * ci;
                        if (TS > 1 && ch >= KC) break;
                        spio_half8 bfrag[NBLK];
#pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb) {
                            const unsigned char* pb0 = xrow + (32 * ch + 2 * nb) * 16;
                            bfrag[nb] = read_tr_pair(pb0, pb0 + 4 * 16);
                        }
#pragma unroll
                        for (int d = uu; d < ND; d += 2) {
                            // delta = d has the parity of t: pair index i = (t - d) / 2
                            const int i2 = t - d;  // first row of the pair, relative to p0
                            if (i2 >= 0 && i2 < bh_eff) {
                                const int slot = (i2 + sel) % NRD;
                                const unsigned char* pa0 =
                                    reinterpret_cast<const unsigned char*>(dring + slot * DROW_UNITS) +
                                    dfrag_off + (32 * ch) * 16;
                                const spio_half8 afrag = read_tr_pair(pa0, pa0 + 4 * 16);
#pragma unroll
                                for (int nb = 0; nb < NBLK; ++nb)
                                    acc[d][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                        afrag, bfrag[nb], acc[d][nb], 0, 0, 0);
                            }
                        }
                    }
                }

                // 3. rows t+1 into LDS
                if (t + 1 < STEPS) {
                    const int hn = p0 + t + 1 - kPadY;
                    if (hn >= 0 && hn < kH) {
#pragma unroll
                        for (int l = 0; l < LPTX; ++l)
                            if (x_lds[l] >= 0) xring[((uu + 1) & 1) * XROW_UNITS + x_lds[l]] = xpre[(uf + 1) % PF][l];
                    }
                    const int dslot = (t + 1) % NRD;
#pragma unroll
                    for (int l = 0; l < LPTD; ++l)
                        if (d_lds[l] >= 0) dring[dslot * DROW_UNITS + d_lds[l]] = dpre[(uf + 1) % PF][l];
                }
                block_sync();
            }
        }
    }

    // ---- publish ----
    // dw[k,r,s,c] = acc[delta = r] (lanes 0-31: j = 0) + acc[delta = r+1] (lanes 32-63: j = 1).
    // The j = 1 halves travel through a 512-byte per-wave LDS scratch (LDS operations of one
    // wave execute in order, so no barrier is needed inside the wave).  With TS > 1 the waves of
    // one group then add their sums through LDS so that only one wave per group publishes:
    // fp32 atomics into grad_weight, or plain stores into this workgroup's partial image when a
    // second kernel does the reduction.
    constexpr int SCRATCH_FLOATS = NBLK * 128;  // per wave
    static_assert((WAVES * SCRATCH_FLOATS + GB * (TS - 1) * NBLK * 128) * 4 <= (NRX * XROW_UNITS + NRD * DROW_UNITS) * 16,
                  "reduction scratch does not fit in LDS");
    block_sync();  // every wave is done with the rings; reuse them as scratch
    {
        float* scratch = reinterpret_cast<float*>(lds) + wave * SCRATCH_FLOATS;
        float* red = reinterpret_cast<float*>(lds) + WAVES * SCRATCH_FLOATS;  // [group][ts-1][nb][e][32 lanes]
        const int k4 = 4 * ((lane >> 4) & 1);
        const int sj = (lane & 15) >> 3;
        const int c = lane & 7;
#if SPIO_PARTIALS
        // this wave's slice of the workgroup's partial block: [r][tap pair][e][32 lanes], so that
        // every store instruction writes 128 contiguous bytes
        float* out = grad_weight + (((long long)(nbk * PBLKS + pb) * GBLKS + cb) * GB + wg) * PART_WAVE_FLOATS;
#else
        float* out = grad_weight;
#endif
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            float total[NBLK][4];
#pragma unroll
            for (int nb = 0; nb < NBLK; ++nb) {
                if (lane >= 32) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) scratch[e * 32 + (lane - 32)] = acc[r + 1][nb][e];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    total[nb][e] = 0.f;
                    if (lane < 32) total[nb][e] = acc[r][nb][e] + scratch[e * 32 + lane];
                }
            }
            if (TS > 1) {
                if (ws > 0 && lane < 32) {
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            red[(((wg * (TS - 1) + ws - 1) * NBLK + nb) * 4 + e) * 32 + lane] = total[nb][e];
                }
                block_sync();
                if (ws == 0 && lane < 32) {
#pragma unroll
                    for (int w2 = 0; w2 < TS - 1; ++w2)
#pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb)
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                total[nb][e] += red[(((wg * (TS - 1) + w2) * NBLK + nb) * 4 + e) * 32 + lane];
                }
            }
#if SPIO_PARTIALS
            // through the wave's LDS scratch once more so that all 64 lanes store 16 bytes each
            if (wave_active && ws == 0) {
                float* stage = scratch;  // NBLK * 128 floats: [tap pair][e][32 lanes]
                if (lane < 32) {
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb)
#pragma unroll
                        for (int e = 0; e < 4; ++e) stage[(nb * 4 + e) * 32 + lane] = total[nb][e];
                }
                const spio_float4* stage4 = reinterpret_cast<const spio_float4*>(stage);
                spio_float4* out4 = reinterpret_cast<spio_float4*>(out) + r * NBLK * 32;
#pragma unroll
                for (int i = lane; i < NBLK * 32; i += 64) __builtin_nontemporal_store(stage4[i], out4 + i);
            }
#else
            if (wave_active && ws == 0 && lane < 32) {
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    const int s = 2 * nb + sj;
                    if (s < kS) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            atomic_add_f32(out + (((long long)(8 * gglob + k4 + e) * kR + r) * kS + s) * 8 + c,
                                           total[nb][e]);
                    }
                }
            }
#endif
            if (TS > 1) block_sync();  // the scratch is rewritten for the next filter row
        }
    }

}

#if SPIO_PARTIALS
// Second stage: grad_weight += sum over the partial blocks.  A workgroup owns 8 float4 columns
// of one channel block (128 contiguous bytes of every partial block); its 32 slices each add the
// blocks p = slice, slice + 32, ... with 8 loads in flight, the slices are added through LDS and
// slice 0 adds the total onto grad_weight.  Every element of grad_weight has exactly one owner,
// so no atomics are needed and the sum does not depend on timing.  A column is four consecutive
// lanes of the publishing wave, i.e. four consecutive channels c of one (k, r, s).
#define SPIO_CONCAT2(a, b) a##b
#define SPIO_CONCAT(a, b) SPIO_CONCAT2(a, b)
extern "C" __global__ void SPIO_LAUNCH_BOUNDS(256)
SPIO_CONCAT(SPIO_KERNEL_NAME, _reduce)(float* __restrict__ grad_weight, const spio_float4* __restrict__ partials) {
    constexpr int BLOCK_F4 = GB * PART_WAVE_FLOATS / 4;  // float4 columns of one partial block
    constexpr int NPART = NBLKS * PBLKS;
    constexpr int SLICES = 32;
    constexpr int UN = 8;
    __shared__ spio_float4 red[SLICES][8];
    const int tid = thread_id();
    const int cl = tid & 7;
    const int slice = tid >> 3;
    const int col = (block_id() % (BLOCK_F4 / 8)) * 8 + cl;
    const int cb = block_id() / (BLOCK_F4 / 8);
    spio_float4 sum = spio_float4{0.f, 0.f, 0.f, 0.f};
    for (int base = slice; base < NPART; base += SLICES * UN) {
        spio_float4 v[UN];
#pragma unroll
        for (int i = 0; i < UN; ++i) {
            const int p = base + i * SLICES;
            v[i] = spio_float4{0.f, 0.f, 0.f, 0.f};
            if (p < NPART) v[i] = partials[((long long)p * GBLKS + cb) * BLOCK_F4 + col];
        }
#pragma unroll
        for (int i = 0; i < UN; ++i) sum += v[i];
    }
    red[slice][cl] = sum;
    block_sync();
    if (slice == 0) {
#pragma unroll 4
        for (int i = 1; i < SLICES; ++i) sum += red[i][cl];
        // float index inside the block -> (group, r, tap pair, e, lane)
        const int f = 4 * col;
        const int l32 = f & 31;
        const int e = (f >> 5) & 3;
        const int rn = (f >> 7) % (kR * NBLK);
        const int g = (f >> 7) / (kR * NBLK);
        const int r = rn / NBLK;
        const int s = 2 * (rn % NBLK) + ((l32 & 15) >> 3);
        const int k = 8 * (cb * GB + g) + 4 * (l32 >> 4) + e;
        if (cb * GB + g < kGroups && s < kS) {
            spio_float4* dst =
                reinterpret_cast<spio_float4*>(grad_weight + (((long long)k * kR + r) * kS + s) * 8 + (l32 & 7));
            *dst = *dst + sum;
        }
    }
}
#endif
