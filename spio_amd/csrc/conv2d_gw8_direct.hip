// Direct (one thread per output pixel-group) conv2d_gw8 kernels for gfx950.
//
// These kernels make no assumption about the shape beyond C % 8 == 0.  They are
// the general-purpose configuration of the tile sweep: always legal, never the
// fastest for large tensors.  Contract (reference: spio/src/conv2d_gw8.cu:10-225
// for fprop/dgrad, spio/src/conv2d_gw8_wgrad.cu:10-226 for wgrad):
//
//   fprop : y[n,p,q,k]  = rn16(bias[k] + sum_{c,r,s} x[n,p+r-py,q+s-px,8g+c] * w[k,r,s,c])
//   dgrad : dx[n,h,w,8g+c] = rn16(sum_{j,r,s} dy[n,h-r+py,w-s+px,8g+j] * w[8g+j,r,s,c])
//   wgrad : dw[k,r,s,c] += sum_{n,p,q} x[n,p+r-py,q+s-px,8g+c] * dy[n,p,q,k]   (fp32, atomics)
//
// with g = k / 8, out-of-range reads equal to zero, fp32 accumulation and a
// single round-to-nearest conversion to fp16 at the store.
#include "spio_conv_common.h"

using namespace spio;

#ifndef SPIO_IGRAD
#define SPIO_IGRAD 0
#endif
#ifndef SPIO_HAS_BIAS
#define SPIO_HAS_BIAS 0
#endif
#ifndef SPIO_BLOCK_THREADS
#define SPIO_BLOCK_THREADS 256
#endif

#if !defined(SPIO_WGRAD)

// Source / destination geometry of this direction.
constexpr bool kIgrad = SPIO_IGRAD != 0;
constexpr int kSrcH = kIgrad ? kP : kH;
constexpr int kSrcW = kIgrad ? kQ : kW;
constexpr int kDstH = kIgrad ? kH : kP;
constexpr int kDstW = kIgrad ? kW : kQ;
constexpr int kEffPadY = kIgrad ? kR - 1 - kPadY : kPadY;
constexpr int kEffPadX = kIgrad ? kS - 1 - kPadX : kPadX;

extern "C" __global__ void SPIO_LAUNCH_BOUNDS(SPIO_BLOCK_THREADS)
SPIO_KERNEL_NAME(spio_uint4* __restrict__ dst, const spio_uint4* __restrict__ src,
                 const spio_half* __restrict__ weights, const float* __restrict__ bias) {
    const long long total = (long long)kN * kDstH * kDstW * kGroups;
    const long long idx = (long long)block_id() * SPIO_BLOCK_THREADS + thread_id();
    if (idx >= total) return;
    const int g = (int)(idx % kGroups);
    long long pix = idx / kGroups;
    const int ow = (int)(pix % kDstW);
    pix /= kDstW;
    const int oh = (int)(pix % kDstH);
    const int n = (int)(pix / kDstH);

    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
#if SPIO_HAS_BIAS
        acc[k] = kIgrad ? 0.f : bias[8 * g + k];
#else
        acc[k] = 0.f;
#endif
    }

    for (int r = 0; r < kR; ++r) {
        const int ih = oh + r - kEffPadY;
        if (ih < 0 || ih >= kSrcH) continue;
        for (int s = 0; s < kS; ++s) {
            const int iw = ow + s - kEffPadX;
            if (iw < 0 || iw >= kSrcW) continue;
            Pack16 v;
            v.u = src[(((long long)n * kSrcH + ih) * kSrcW + iw) * kGroups + g];
            if (!kIgrad) {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    Pack16 wv;
                    wv.u = *reinterpret_cast<const spio_uint4*>(
                        weights + ((((long long)(8 * g + k)) * kR + r) * kS + s) * 8);
#pragma unroll
                    for (int c = 0; c < 8; ++c) acc[k] = __builtin_fmaf((float)v.h[c], (float)wv.h[c], acc[k]);
                }
            } else {
                // Transposed, flipped filter: output channel c of the group,
                // input (dy) channel j, tap (R-1-r, S-1-s).
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    Pack16 wv;
                    wv.u = *reinterpret_cast<const spio_uint4*>(
                        weights +
                        ((((long long)(8 * g + j)) * kR + (kR - 1 - r)) * kS + (kS - 1 - s)) * 8);
#pragma unroll
                    for (int c = 0; c < 8; ++c) acc[c] = __builtin_fmaf((float)v.h[j], (float)wv.h[c], acc[c]);
                }
            }
        }
    }
    Pack16 o;
#pragma unroll
    for (int k = 0; k < 8; ++k) o.h[k] = (spio_half)acc[k];
    dst[idx] = o.u;
}

#else  // SPIO_WGRAD

#ifndef SPIO_WGRAD_CHUNKS
#define SPIO_WGRAD_CHUNKS 64
#endif

// One workgroup per (group, pixel chunk); every wave owns a slice of the chunk
// and every lane one (k, c) pair of the 8x8 block, looping over all R*S taps.
// Partial sums go to grad_weight with fp32 atomics, so grad_weight must be
// zero (or hold a value to accumulate onto) before the launch.
extern "C" __global__ void SPIO_LAUNCH_BOUNDS(SPIO_BLOCK_THREADS)
SPIO_KERNEL_NAME(float* __restrict__ grad_weight, const spio_half* __restrict__ x,
                 const spio_half* __restrict__ dy
#if SPIO_HAS_BIAS
                 , float* __restrict__ grad_bias  // [K] fp32, accumulated into; null = not wanted
#endif
) {
    constexpr int kWaves = SPIO_BLOCK_THREADS / 64;
    const int g = block_id() % kGroups;
    const int chunk = block_id() / kGroups;
    const int lane = thread_id() % 64;
    const int wave = thread_id() / 64;
    const int k = lane / 8;
    const int c = lane % 8;

    const long long total_pix = (long long)kN * kP * kQ;
    const long long per_chunk = (total_pix + SPIO_WGRAD_CHUNKS - 1) / SPIO_WGRAD_CHUNKS;
    const long long begin = chunk * per_chunk;
    long long end = begin + per_chunk;
    if (end > total_pix) end = total_pix;

    float acc[kR * kS];
#pragma unroll
    for (int t = 0; t < kR * kS; ++t) acc[t] = 0.f;

    float dsum = 0.f;  // grad_output summed over this wave's pixels (same in the 8 lanes of a k)
    for (long long pix = begin + wave; pix < end; pix += kWaves) {
        const int q = (int)(pix % kQ);
        const long long t0 = pix / kQ;
        const int p = (int)(t0 % kP);
        const int n = (int)(t0 / kP);
        const float d = (float)dy[pix * kC + 8 * g + k];
        dsum += d;
#pragma unroll
        for (int r = 0; r < kR; ++r) {
            const int ih = p + r - kPadY;
#pragma unroll
            for (int s = 0; s < kS; ++s) {
                const int iw = q + s - kPadX;
                float xv = 0.f;
                if (ih >= 0 && ih < kH && iw >= 0 && iw < kW)
                    xv = (float)x[(((long long)n * kH + ih) * kW + iw) * kC + 8 * g + c];
                acc[r * kS + s] = __builtin_fmaf(xv, d, acc[r * kS + s]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kR; ++r)
#pragma unroll
        for (int s = 0; s < kS; ++s)
            atomic_add_f32(grad_weight + ((((long long)(8 * g + k)) * kR + r) * kS + s) * 8 + c,
                      acc[r * kS + s]);
#if SPIO_HAS_BIAS
    if (grad_bias != nullptr && c == 0) atomic_add_f32(grad_bias + 8 * g + k, dsum);
#else
    (void)dsum;
#endif
}

#endif  // SPIO_WGRAD
