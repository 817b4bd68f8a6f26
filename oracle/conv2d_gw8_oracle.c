/*
 * Plain-C restatement of the conv2d_gw8 contract -- TEST INFRASTRUCTURE ONLY.
 *
 * Independent of the torch and numpy statements in conv2d_gw8_oracle.py; the
 * tests cross-check all three.  It works on the physical layouts the kernels
 * use: activations [N][H][W][C] fp16, weights [K][R][S][8] fp16, bias [K] fp32,
 * grad_weight [K][R][S][8] fp32.  Results are fp32 (accumulated in double),
 * i.e. the value before the single round-to-fp16 the kernels apply
 * (spio/src/conv2d_gw8.cu:213-220).  Never linked into the product.
 *
 * Follows: spio/src/conv2d_gw8.cu:10-225 (fprop, dgrad),
 *          spio/src/conv2d_gw8_wgrad.cu:10-226 (wgrad),
 *          spio/functional/conv2d_gw8_function.py:134-136 (grad_bias).
 */
#include <stdint.h>
#include <string.h>

static float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                ++e;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

/* y[n][p][q][k] = bias[k] + sum x[n][p+r-py][q+s-px][8g+c] * w[k][r][s][c] */
void gw8_fprop_f32(const uint16_t* x, const uint16_t* w, const float* bias, float* y, int N, int C,
                   int H, int W, int R, int S, int py, int px) {
    const int P = H + 2 * py - R + 1, Q = W + 2 * px - S + 1;
#pragma omp parallel for collapse(2)
    for (int n = 0; n < N; ++n)
        for (int p = 0; p < P; ++p)
            for (int q = 0; q < Q; ++q)
                for (int k = 0; k < C; ++k) {
                    const int g = k / 8;
                    double acc = bias ? (double)bias[k] : 0.0;
                    for (int r = 0; r < R; ++r) {
                        const int ih = p + r - py;
                        if (ih < 0 || ih >= H) continue;
                        for (int s = 0; s < S; ++s) {
                            const int iw = q + s - px;
                            if (iw < 0 || iw >= W) continue;
                            const uint16_t* xp = x + (((int64_t)n * H + ih) * W + iw) * C + 8 * g;
                            const uint16_t* wp = w + (((int64_t)k * R + r) * S + s) * 8;
                            for (int c = 0; c < 8; ++c)
                                acc += (double)half_to_float(xp[c]) * (double)half_to_float(wp[c]);
                        }
                    }
                    y[(((int64_t)n * P + p) * Q + q) * C + k] = (float)acc;
                }
}

/* dx[n][h][w][8g+c] = sum dy[n][h-r+py][w-s+px][8g+j] * w[8g+j][r][s][c] */
void gw8_dgrad_f32(const uint16_t* dy, const uint16_t* w, float* dx, int N, int C, int H, int W,
                   int R, int S, int py, int px) {
    const int P = H + 2 * py - R + 1, Q = W + 2 * px - S + 1;
#pragma omp parallel for collapse(2)
    for (int n = 0; n < N; ++n)
        for (int h = 0; h < H; ++h)
            for (int ww = 0; ww < W; ++ww)
                for (int ch = 0; ch < C; ++ch) {
                    const int g = ch / 8, c = ch % 8;
                    double acc = 0.0;
                    for (int r = 0; r < R; ++r) {
                        const int p = h - r + py;
                        if (p < 0 || p >= P) continue;
                        for (int s = 0; s < S; ++s) {
                            const int q = ww - s + px;
                            if (q < 0 || q >= Q) continue;
                            const uint16_t* dp = dy + (((int64_t)n * P + p) * Q + q) * C + 8 * g;
                            for (int j = 0; j < 8; ++j)
                                acc += (double)half_to_float(dp[j]) *
                                       (double)half_to_float(
                                           w[(((int64_t)(8 * g + j) * R + r) * S + s) * 8 + c]);
                        }
                    }
                    dx[(((int64_t)n * H + h) * W + ww) * C + ch] = (float)acc;
                }
}

/* dw[k][r][s][c] = sum_{n,p,q} x[n][p+r-py][q+s-px][8g+c] * dy[n][p][q][k] */
void gw8_wgrad_f32(const uint16_t* x, const uint16_t* dy, float* dw, int N, int C, int H, int W,
                   int R, int S, int py, int px) {
    const int P = H + 2 * py - R + 1, Q = W + 2 * px - S + 1;
#pragma omp parallel for
    for (int k = 0; k < C; ++k) {
        const int g = k / 8;
        for (int r = 0; r < R; ++r)
            for (int s = 0; s < S; ++s)
                for (int c = 0; c < 8; ++c) {
                    double acc = 0.0;
                    for (int n = 0; n < N; ++n)
                        for (int p = 0; p < P; ++p) {
                            const int ih = p + r - py;
                            if (ih < 0 || ih >= H) continue;
                            for (int q = 0; q < Q; ++q) {
                                const int iw = q + s - px;
                                if (iw < 0 || iw >= W) continue;
                                acc += (double)half_to_float(
                                           x[(((int64_t)n * H + ih) * W + iw) * C + 8 * g + c]) *
                                       (double)half_to_float(
                                           dy[(((int64_t)n * P + p) * Q + q) * C + k]);
                            }
                        }
                    dw[(((int64_t)k * R + r) * S + s) * 8 + c] = (float)acc;
                }
    }
}

/* db[k] = sum_{n,p,q} dy[n][p][q][k] */
void gw8_dbias_f32(const uint16_t* dy, float* db, int N, int C, int P, int Q) {
    for (int k = 0; k < C; ++k) {
        double acc = 0.0;
        for (int64_t i = 0; i < (int64_t)N * P * Q; ++i) acc += (double)half_to_float(dy[i * C + k]);
        db[k] = (float)acc;
    }
}
