/*
 * Plain-C restatement of the convolution and pooling formulas of the inter-operator scheduler runtime.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/_build/libios_oracle.so and called from tests and from the
 * CPU-baseline leg of the benchmark; the shipped runtime never links or loads it.
 *
 * conv: y[n,o,p,q] = act(b[o] + sum_{c,i,j} x[n, g*ICg + c, p*sh - ph + i, q*sw - pw + j] * w[o,c,i,j]),
 *       g = o / (OC / groups), out-of-range x is zero, OH = 1 + (H - KH + 2 ph) / sh
 *       (geometry and group semantics of reference src/ios/ios_runtime.cu:254-255,275-277).
 * pool: max over in-range window elements, or sum of in-range elements divided by KH*KW
 *       (CUDNN_POOLING_AVERAGE_COUNT_INCLUDE_PADDING, reference src/ios/ios_runtime.cu:542-550).
 * Accumulation is in double so that the result is the correctly rounded reference for fp32 kernels.
 */
#include <math.h>
#include <stddef.h>

static float apply_act(double v, int act) {
    switch (act) {
        case 1: return (float)(v > 0.0 ? v : 0.0);
        case 2: return (float)tanh(v);
        case 3: return (float)(1.0 / (1.0 + exp(-v)));
        default: return (float)v;
    }
}

/* act: 0 identity, 1 relu, 2 tanh, 3 sigmoid */
void oracle_conv2d(const float *x, const float *w, const float *b, float *y, int n, int ic, int h, int wd,
                   int oc, int kh, int kw, int sh, int sw, int ph, int pw, int groups, int act) {
    const int icg = ic / groups, ocg = oc / groups;
    const int oh = 1 + (h - kh + 2 * ph) / sh, ow = 1 + (wd - kw + 2 * pw) / sw;
#pragma omp parallel for collapse(2) schedule(static)
    for (int bi = 0; bi < n; bi++) {
        for (int o = 0; o < oc; o++) {
            const int g = o / ocg;
            for (int p = 0; p < oh; p++) {
                for (int q = 0; q < ow; q++) {
                    double acc = b ? (double)b[o] : 0.0;
                    for (int c = 0; c < icg; c++) {
                        const float *xc = x + ((size_t)bi * ic + (size_t)g * icg + c) * h * wd;
                        const float *wc = w + ((size_t)o * icg + c) * kh * kw;
                        for (int i = 0; i < kh; i++) {
                            const int ih = p * sh - ph + i;
                            if (ih < 0 || ih >= h) continue;
                            for (int j = 0; j < kw; j++) {
                                const int iw = q * sw - pw + j;
                                if (iw < 0 || iw >= wd) continue;
                                acc += (double)xc[(size_t)ih * wd + iw] * (double)wc[i * kw + j];
                            }
                        }
                    }
                    y[(((size_t)bi * oc + o) * oh + p) * ow + q] = apply_act(acc, act);
                }
            }
        }
    }
}

/* is_max: 1 max pool, 0 average pool that counts padded positions */
void oracle_pool2d(const float *x, float *y, int n, int c, int h, int wd, int kh, int kw, int sh, int sw,
                   int ph, int pw, int is_max) {
    const int oh = 1 + (h - kh + 2 * ph) / sh, ow = 1 + (wd - kw + 2 * pw) / sw;
#pragma omp parallel for schedule(static)
    for (int pc = 0; pc < n * c; pc++) {
        const float *xc = x + (size_t)pc * h * wd;
        for (int p = 0; p < oh; p++) {
            for (int q = 0; q < ow; q++) {
                double best = -INFINITY, total = 0.0;
                for (int i = 0; i < kh; i++) {
                    const int ih = p * sh - ph + i;
                    if (ih < 0 || ih >= h) continue;
                    for (int j = 0; j < kw; j++) {
                        const int iw = q * sw - pw + j;
                        if (iw < 0 || iw >= wd) continue;
                        const double v = xc[(size_t)ih * wd + iw];
                        if (v > best) best = v;
                        total += v;
                    }
                }
                y[((size_t)pc * oh + p) * ow + q] = (float)(is_max ? best : total / (double)(kh * kw));
            }
        }
    }
}
