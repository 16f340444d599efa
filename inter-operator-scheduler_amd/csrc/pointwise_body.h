// Device-side bodies of the memory-bound kernels (pooling, depth-wise and direct convolution, n-ary add /
// multiply / activation / strided copy).  Every body processes the elements of logical block `block` out of
// `num_blocks` with a block-stride loop, so the same code serves a stand-alone launch and a slice of the
// fused stage kernel.  Tensors are NCHW views; consecutive lanes cover consecutive output columns.
#pragma once

#include "kernels.h"

namespace ios {

typedef float pw_floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float act_apply(float v, int act) {
    switch (act) {
        case ACT_RELU: return fmaxf(v, 0.0f);
        case ACT_TANH: return tanhf(v);
        case ACT_SIGMOID: return 1.0f / (1.0f + __expf(-v));
        default: return v;
    }
}

struct PoolArgs {
    const float *x;
    float *y;
    long long x_bs, y_bs;
    PoolProblem p;
    int strip_rows;   // 3 x 3 windows: output rows per thread (see pool3x3_body); 0 selects the generic body
    int vec_columns;  // 3 x 3 windows: output columns per thread, 1 or kPoolVecColumns (see pool3x3_vec_body)
    // the pool behind a bias-free convolution (an average pool and a 1 x 1 convolution exchanged): y = act(pool(x) + bias[c]);
    // nullptr for a plain pool
    const float *bias;
    int act;
};

__device__ __forceinline__ float pool_finish(const PoolArgs &a, float v, unsigned c) {
    return a.bias != nullptr ? act_apply(v + a.bias[c], a.act) : v;
}

__device__ __forceinline__ void pool_generic_body(const PoolArgs &a, int block, int num_blocks, unsigned threads) {
    const PoolProblem &p = a.p;
    // 32-bit index arithmetic: the host side rejects tensors with 2^31 or more elements
    const unsigned plane = (unsigned)(p.OH * p.OW);
    const unsigned per_image = (unsigned)p.C * plane;
    const unsigned total = per_image * (unsigned)p.B;
    const float inv = 1.0f / (float)(p.KH * p.KW);
    for (unsigned i = block * threads + threadIdx.x; i < total; i += num_blocks * threads) {
        const unsigned b = i / per_image;
        const unsigned o = i - b * per_image;
        const unsigned c = o / plane;
        const unsigned r = o - c * plane;
        const int oh = (int)(r / (unsigned)p.OW);
        const int ow = (int)r - oh * p.OW;
        const float *xc = a.x + (long long)b * a.x_bs + (long long)c * p.H * p.W;
        const int h0 = oh * p.sh - p.ph, w0 = ow * p.sw - p.pw;
        const int hb = max(h0, 0), he = min(h0 + p.KH, p.H);
        const int wb = max(w0, 0), we = min(w0 + p.KW, p.W);
        float best = -INFINITY, sum = 0.f;
        for (int h = hb; h < he; h++)
            for (int w = wb; w < we; w++) {
                const float v = xc[h * p.W + w];
                best = fmaxf(best, v);
                sum += v;
            }
        a.y[(long long)b * a.y_bs + o] = pool_finish(a, p.is_max ? best : sum * inv, c);
    }
}

// Most rows of outputs a thread of the 3 x 3 pooling body produces: a thread walks down one output column and keeps
// the horizontal partial results of the input rows two consecutive windows share.  Small problems use shorter
// strips (down to one row) so that the launch still fills the device.
constexpr int kPoolStripRows = 8;

// 3 x 3 windows, stride 1 or 2 in h (any stride in w).  Consecutive lanes take consecutive output columns, so the
// three loads of an input row are contiguous (stride 1) or interleaved (stride 2) across a wavefront.  Per output
// this reads 3 * (1 + 2 / 8) (stride 1) or 3 * (2 + 1 / 8) (stride 2) elements instead of 9.
__device__ __forceinline__ void pool3x3_body(const PoolArgs &a, int block, int num_blocks, unsigned threads) {
    const PoolProblem &p = a.p;
    const int R = a.strip_rows;
    const unsigned strips = (unsigned)((p.OH + R - 1) / R);
    const unsigned per_plane = strips * (unsigned)p.OW;
    const unsigned total = per_plane * (unsigned)(p.C * p.B);
    const bool is_max = p.is_max != 0;
    const float neutral = is_max ? -INFINITY : 0.f;
    for (unsigned i = block * threads + threadIdx.x; i < total; i += num_blocks * threads) {
        const unsigned pc = i / per_plane;
        const unsigned rest = i - pc * per_plane;
        const unsigned strip = rest / (unsigned)p.OW;
        const int ow = (int)(rest - strip * (unsigned)p.OW);
        const unsigned b = pc / (unsigned)p.C;
        const unsigned c = pc - b * (unsigned)p.C;
        const float *xc = a.x + (long long)b * a.x_bs + (long long)c * p.H * p.W;
        float *yc = a.y + (long long)b * a.y_bs + (long long)c * p.OH * p.OW + ow;
        const int w0 = ow * p.sw - p.pw;
        const bool c0 = (unsigned)w0 < (unsigned)p.W, c1 = (unsigned)(w0 + 1) < (unsigned)p.W, c2 = (unsigned)(w0 + 2) < (unsigned)p.W;
        // clamped addresses and selects instead of conditional loads: the loads of a window are independent and in
        // flight together
        const int wa = min(max(w0, 0), p.W - 1), wb = min(max(w0 + 1, 0), p.W - 1), wc2 = min(max(w0 + 2, 0), p.W - 1);
        auto row = [&](int h) -> float {
            const bool in_h = (unsigned)h < (unsigned)p.H;
            const float *xr = xc + min(max(h, 0), p.H - 1) * p.W;
            const float l0 = xr[wa], l1 = xr[wb], l2 = xr[wc2];
            const float v0 = (c0 && in_h) ? l0 : neutral;
            const float v1 = (c1 && in_h) ? l1 : neutral;
            const float v2 = (c2 && in_h) ? l2 : neutral;
            return is_max ? fmaxf(fmaxf(v0, v1), v2) : (v0 + v1) + v2;
        };
        auto combine = [&](float r0, float r1, float r2) -> float {
            return pool_finish(a, is_max ? fmaxf(fmaxf(r0, r1), r2) : ((r0 + r1) + r2) * (1.0f / 9.0f), c);
        };
        const int oh_begin = (int)strip * R;
        const int oh_end = min(p.OH, oh_begin + R);
        if (p.sh == 1) {
            float r0 = row(oh_begin - p.ph), r1 = row(oh_begin - p.ph + 1);
            for (int oh = oh_begin; oh < oh_end; oh++) {
                const float r2 = row(oh - p.ph + 2);
                yc[oh * p.OW] = combine(r0, r1, r2);
                r0 = r1;
                r1 = r2;
            }
        } else {
            float r0 = row(oh_begin * 2 - p.ph);
            for (int oh = oh_begin; oh < oh_end; oh++) {
                const float r1 = row(oh * 2 - p.ph + 1);
                const float r2 = row(oh * 2 - p.ph + 2);
                yc[oh * p.OW] = combine(r0, r1, r2);
                r0 = r2;
            }
        }
    }
}

// The same strips, four output columns wide: the form for all but small tensors, where the load instructions per byte decide.  A
// thread reads an input row of its strip with one clamped scalar load and one (stride 1) or two (stride 2) 16-byte loads
// at any 4-byte alignment instead of three loads per output column, and stores four outputs with one 16-byte store.  The
// 16-byte loads may run up to eight elements past the end of a row; what they bring from there (the next row, the next
// plane, or the padding that ends every arena) is replaced by the neutral element.  SW: stride along w (1 or 2), the
// padding along w is at most 1.
typedef float pw_floatx4_u __attribute__((ext_vector_type(4), aligned(4)));
constexpr int kPoolVecColumns = 4;

template <int SW>
__device__ __forceinline__ void pool3x3_vec_body(const PoolArgs &a, int block, int num_blocks, unsigned threads) {
    const PoolProblem &p = a.p;
    const int R = a.strip_rows;
    constexpr int V = kPoolVecColumns;
    constexpr int IN = SW * (V - 1) + 3;   // input columns of a row a thread reads: 6 or 9
    const unsigned strips = (unsigned)((p.OH + R - 1) / R);
    const unsigned quads = (unsigned)((p.OW + V - 1) / V);
    const unsigned per_plane = strips * quads;
    const unsigned total = per_plane * (unsigned)(p.C * p.B);
    const bool is_max = p.is_max != 0;
    const float neutral = is_max ? -INFINITY : 0.f;
    for (unsigned i = block * threads + threadIdx.x; i < total; i += num_blocks * threads) {
        const unsigned pc = i / per_plane;
        const unsigned rest = i - pc * per_plane;
        const unsigned strip = rest / quads;
        const int ow0 = (int)(rest - strip * quads) * V;
        const unsigned b = pc / (unsigned)p.C;
        const unsigned c = pc - b * (unsigned)p.C;
        const float *xc = a.x + (long long)b * a.x_bs + (long long)c * p.H * p.W;
        float *yc = a.y + (long long)b * a.y_bs + (long long)c * p.OH * p.OW + ow0;
        const int w0 = ow0 * SW - p.pw;          // first input column (-1 at the left edge with padding)
        const int w0c = max(w0, 0);
        // horizontal results of one input row for the four windows
        auto row = [&](int h, float (&out)[V]) {
            const bool in_h = (unsigned)h < (unsigned)p.H;
            const float *xr = xc + min(max(h, 0), p.H - 1) * p.W;
            float v[IN];
            v[0] = xr[w0c];
            const pw_floatx4_u q0 = *reinterpret_cast<const pw_floatx4_u *>(xr + w0 + 1);
            v[1] = q0.x; v[2] = q0.y; v[3] = q0.z; v[4] = q0.w;
            if constexpr (SW == 1) {
                v[5] = xr[min(w0 + 5, p.W - 1)];
            } else {
                const pw_floatx4_u q1 = *reinterpret_cast<const pw_floatx4_u *>(xr + w0 + 5);
                v[5] = q1.x; v[6] = q1.y; v[7] = q1.z; v[8] = q1.w;
            }
#pragma unroll
            for (int j = 0; j < IN; j++) v[j] = (in_h && (unsigned)(w0 + j) < (unsigned)p.W) ? v[j] : neutral;
#pragma unroll
            for (int k = 0; k < V; k++)
                out[k] = is_max ? fmaxf(fmaxf(v[SW * k], v[SW * k + 1]), v[SW * k + 2]) : (v[SW * k] + v[SW * k + 1]) + v[SW * k + 2];
        };
        auto store = [&](int oh, const float (&r0)[V], const float (&r1)[V], const float (&r2)[V]) {
            float o[V];
#pragma unroll
            for (int k = 0; k < V; k++)
                o[k] = pool_finish(a, is_max ? fmaxf(fmaxf(r0[k], r1[k]), r2[k]) : ((r0[k] + r1[k]) + r2[k]) * (1.0f / 9.0f), c);
            float *yr = yc + oh * p.OW;
            if (ow0 + V <= p.OW) {
                pw_floatx4_u q;
                q.x = o[0]; q.y = o[1]; q.z = o[2]; q.w = o[3];
                *reinterpret_cast<pw_floatx4_u *>(yr) = q;
            } else {
#pragma unroll
                for (int k = 0; k < V; k++)
                    if (ow0 + k < p.OW) yr[k] = o[k];
            }
        };
        const int oh_begin = (int)strip * R;
        const int oh_end = min(p.OH, oh_begin + R);
        float r0[V], r1[V], r2[V];
        if (p.sh == 1) {
            row(oh_begin - p.ph, r0);
            row(oh_begin - p.ph + 1, r1);
            for (int oh = oh_begin; oh < oh_end; oh++) {
                row(oh - p.ph + 2, r2);
                store(oh, r0, r1, r2);
#pragma unroll
                for (int k = 0; k < V; k++) {
                    r0[k] = r1[k];
                    r1[k] = r2[k];
                }
            }
        } else {
            row(oh_begin * 2 - p.ph, r0);
            for (int oh = oh_begin; oh < oh_end; oh++) {
                row(oh * 2 - p.ph + 1, r1);
                row(oh * 2 - p.ph + 2, r2);
                store(oh, r0, r1, r2);
#pragma unroll
                for (int k = 0; k < V; k++) r0[k] = r2[k];
            }
        }
    }
}

__device__ __forceinline__ void pool_body(const PoolArgs &a, int block, int num_blocks, unsigned threads) {
    if (a.strip_rows > 0 && a.vec_columns > 1) {
        if (a.p.sw == 1) pool3x3_vec_body<1>(a, block, num_blocks, threads);
        else pool3x3_vec_body<2>(a, block, num_blocks, threads);
    } else if (a.strip_rows > 0) {
        pool3x3_body(a, block, num_blocks, threads);
    } else {
        pool_generic_body(a, block, num_blocks, threads);
    }
}

// window == whole map, many planes (strip_rows == 1): one lane reduces one (image, channel) plane with 16-byte loads, four
// independent partial results, no cross-lane step; the 64 planes of a wavefront are 64 consecutive rows of H * W floats, so
// every cache line a load touches is used up by the loads that follow, and the 64 results leave as one coalesced store.
// (One wavefront per plane, below, spends a 64-lane load and a six-step cross-lane reduction on 256 bytes.)
__device__ __forceinline__ void global_pool_rows_body(const PoolArgs &a, int block, int num_blocks, unsigned threads) {
    const PoolProblem &p = a.p;
    const unsigned planes = (unsigned)(p.B * p.C);
    const int HW = p.H * p.W;
    const bool is_max = p.is_max != 0;
    for (unsigned plane = block * threads + threadIdx.x; plane < planes; plane += num_blocks * threads) {
        const unsigned b = plane / (unsigned)p.C, c = plane - b * (unsigned)p.C;
        const float *xc = a.x + (long long)b * a.x_bs + (long long)c * HW;
        float best[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}, sum[4] = {0.f, 0.f, 0.f, 0.f};
        int i = 0;
#pragma unroll 4
        for (; i + 4 <= HW; i += 4) {
            const pw_floatx4_u q = *reinterpret_cast<const pw_floatx4_u *>(xc + i);
            best[0] = fmaxf(best[0], q.x); best[1] = fmaxf(best[1], q.y); best[2] = fmaxf(best[2], q.z); best[3] = fmaxf(best[3], q.w);
            sum[0] += q.x; sum[1] += q.y; sum[2] += q.z; sum[3] += q.w;
        }
        for (; i < HW; i++) {
            best[0] = fmaxf(best[0], xc[i]);
            sum[0] += xc[i];
        }
        const float m = fmaxf(fmaxf(best[0], best[1]), fmaxf(best[2], best[3]));
        const float t = (sum[0] + sum[1]) + (sum[2] + sum[3]);
        a.y[(long long)b * a.y_bs + c] = pool_finish(a, is_max ? m : t / (float)HW, c);
    }
}

// window == whole map: one wavefront reduces one (image, channel) plane
__device__ __forceinline__ void global_pool_body(const PoolArgs &a, int block, int num_blocks, unsigned threads) {
    if (a.strip_rows == 1) {
        global_pool_rows_body(a, block, num_blocks, threads);
        return;
    }
    const PoolProblem &p = a.p;
    const int planes = p.B * p.C;
    const int HW = p.H * p.W;
    const int waves_per_block = threads >> 6;
    const int lane = threadIdx.x & 63;
    for (int plane = block * waves_per_block + (threadIdx.x >> 6); plane < planes; plane += num_blocks * waves_per_block) {
        const int b = plane / p.C, c = plane - b * p.C;
        const float *xc = a.x + b * a.x_bs + (long long)c * HW;
        float best = -INFINITY, sum = 0.f;
        for (int i = lane; i < HW; i += 64) {
            const float v = xc[i];
            best = fmaxf(best, v);
            sum += v;
        }
        for (int off = 32; off > 0; off >>= 1) {
            best = fmaxf(best, __shfl_xor(best, off, 64));
            sum += __shfl_xor(sum, off, 64);
        }
        if (lane == 0) a.y[b * a.y_bs + c] = pool_finish(a, p.is_max ? best : sum / (float)HW, (unsigned)c);
    }
}

struct DirectConvArgs {
    const float *x;
    const float *w;
    const float *bias;
    float *y;
    long long x_bs, y_bs;
    ConvProblem p;
    unsigned x_bytes;   // extent of the input view in bytes when it is below 2^31 (branch-free depth-wise loads), else 0
    int thin;           // direct convolution: 1 selects conv_thin_body (needs kThinConvSmemFloats floats of LDS)
    // depth-wise convolution of a sum: the input is x + more[0] + ... + more[nmore - 1] (added left to right, then the
    // folded ReLU), every view of the shape of x; the reference adds them with a kernel of its own (src/ios/ops.cu:26-48)
    const float *more[kMaxNaryInputs - 1];
    long long more_bs[kMaxNaryInputs - 1];
    unsigned more_bytes[kMaxNaryInputs - 1];
    int nmore;
};

// raw buffer loads as in the matrix-path convolution: an offset with the top bit set is out of range and reads zero
__device__ __forceinline__ float pw_buffer_load(__amdgpu_buffer_rsrc_t r, unsigned byte_offset) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, byte_offset, 0, 0));
}

// SUM: the instantiation that adds further inputs in its loader (kept apart so that the common single-input form stays small)
template <int KH, int KW, bool SUM = false>
__device__ __forceinline__ void dwconv_body(const DirectConvArgs &a, int block, int num_blocks, unsigned threads) {
    const ConvProblem &p = a.p;
    const int kh_n = KH > 0 ? KH : p.KH, kw_n = KW > 0 ? KW : p.KW;
    const unsigned plane = (unsigned)(p.OH * p.OW);
    const unsigned per_image = (unsigned)p.OC * plane;
    const unsigned total = per_image * (unsigned)p.B;
    const int relu_floor = p.pre_relu ? 0 : (int)0x80000000;   // folded ReLU as an integer max
    for (unsigned i = block * threads + threadIdx.x; i < total; i += num_blocks * threads) {
        const unsigned b = i / per_image;
        const unsigned o = i - b * per_image;
        const unsigned c = o / plane;
        const unsigned r = o - c * plane;
        const int oh = (int)(r / (unsigned)p.OW);
        const int ow = (int)r - oh * p.OW;
        const float *wc = a.w + (size_t)c * kh_n * kw_n;
        const int h0 = oh * p.sh - p.ph, w0 = ow * p.sw - p.pw;
        float acc = a.bias[c];
        if (KH > 0 && a.x_bytes != 0) {
            // fixed window: every tap is one independent load, taps outside the image get the out-of-range bit, so
            // the KH * KW loads of an output are in flight together instead of one bounds-checked load after another
            const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.x), 0, a.x_bytes, 0x00020000);
            const unsigned base = (unsigned)(((long long)b * a.x_bs + (long long)c * p.H * p.W + (long long)h0 * p.W + w0) * 4);
            float v[KH > 0 ? KH * KW : 1];
#pragma unroll
            for (int i2 = 0; i2 < KH; i2++) {
                const unsigned row_kill = (unsigned)(h0 + i2) < (unsigned)p.H ? 0u : 0x80000000u;
#pragma unroll
                for (int j = 0; j < KW; j++) {
                    const unsigned kill = (unsigned)(w0 + j) < (unsigned)p.W ? row_kill : 0x80000000u;
                    v[i2 * KW + j] = pw_buffer_load(xr, (base + (unsigned)(i2 * p.W + j) * 4u) | kill);
                }
            }
            // further inputs of the sum (windows up to 5 x 5; the host refuses larger ones): two at a time for 3 x 3 windows,
            // where a missing second one has extent zero and reads zeros, one at a time for 5 x 5
            if constexpr (SUM && KH * KW <= 25) {
                constexpr int PAIR = KH * KW <= 9 ? 2 : 1;
                // unrolled with wavefront-uniform guards: indexing the argument arrays with a loop variable would move them to scratch memory
#pragma unroll
                for (int s = 0; s < kMaxNaryInputs - 1; s += PAIR) {
                    if (s >= a.nmore) break;
                    float u[PAIR][KH > 0 ? KH * KW : 1];
#pragma unroll
                    for (int e = 0; e < PAIR; e++) {
                        constexpr int kLast = kMaxNaryInputs - 2;
                        const int se = s + e < kLast ? s + e : kLast;
                        const __amdgpu_buffer_rsrc_t sr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(a.more[se]), 0,
                                                                                             s + e < a.nmore ? a.more_bytes[se] : 0u, 0x00020000);
                        const unsigned sbase = (unsigned)(((long long)b * a.more_bs[se] + (long long)c * p.H * p.W + (long long)h0 * p.W + w0) * 4);
#pragma unroll
                        for (int i2 = 0; i2 < KH; i2++) {
                            const unsigned row_kill = (unsigned)(h0 + i2) < (unsigned)p.H ? 0u : 0x80000000u;
#pragma unroll
                            for (int j = 0; j < KW; j++) {
                                const unsigned kill = (unsigned)(w0 + j) < (unsigned)p.W ? row_kill : 0x80000000u;
                                u[e][i2 * KW + j] = pw_buffer_load(sr, (sbase + (unsigned)(i2 * p.W + j) * 4u) | kill);
                            }
                        }
                    }
#pragma unroll
                    for (int t = 0; t < KH * KW; t++) {
                        v[t] += u[0][t];
                        if (PAIR > 1 && s + 1 < a.nmore) v[t] += u[PAIR - 1][t];   // wavefront-uniform; skipping keeps -0.0 + 0.0 out of the sum
                    }
                }
            }
#pragma unroll
            for (int t = 0; t < KH * KW; t++) acc = fmaf(__int_as_float(max(__float_as_int(v[t]), relu_floor)), wc[t], acc);
        } else {
            const float *xc = a.x + (long long)b * a.x_bs + (long long)c * p.H * p.W;
            for (int i2 = 0; i2 < kh_n; i2++) {
                const int h = h0 + i2;
                if ((unsigned)h >= (unsigned)p.H) continue;
                for (int j = 0; j < kw_n; j++) {
                    const int ww = w0 + j;
                    if ((unsigned)ww >= (unsigned)p.W) continue;
                    float v = xc[h * p.W + ww];
                    if (p.pre_relu) v = fmaxf(v, 0.f);
                    acc = fmaf(v, wc[i2 * kw_n + j], acc);
                }
            }
        }
        a.y[(long long)b * a.y_bs + o] = act_apply(acc, p.act);
    }
}

__device__ __forceinline__ void dwconv_dispatch(const DirectConvArgs &a, int block, int num_blocks, unsigned threads) {
    const ConvProblem &p = a.p;
    if (a.nmore > 0) {   // the host only builds such launches for 3 x 3 and 5 x 5 windows
        if (p.KH == 3) dwconv_body<3, 3, true>(a, block, num_blocks, threads);
        else dwconv_body<5, 5, true>(a, block, num_blocks, threads);
        return;
    }
    if (p.KH == 3 && p.KW == 3) dwconv_body<3, 3>(a, block, num_blocks, threads);
    else if (p.KH == 5 && p.KW == 5) dwconv_body<5, 5>(a, block, num_blocks, threads);
    else if (p.KH == 7 && p.KW == 7) dwconv_body<7, 7>(a, block, num_blocks, threads);
    else dwconv_body<0, 0>(a, block, num_blocks, threads);
}

// 3 x 3 convolution of a 3-channel image (the first layer of an image network) for large batches: K is 27, so the layer is
// bound by the bytes of its output, not by arithmetic.  A block takes blockDim.x consecutive output pixels and kThinConvChannels
// output channels: their 27 x 32 filter taps wait transposed in LDS and are read as broadcasts, a thread walks the nine filter rows with the three
// input values of the next row in flight (clamped addresses, zeros selected for the padding), keeps 32 accumulators, and
// every store instruction of a wavefront writes 64 consecutive pixels of one output channel.  Sum order: bias, then taps in
// (channel, kh, kw) order, like the direct kernel.  `smem`: kThinConvSmemFloats floats.
constexpr int kThinConvChannels = 32;
constexpr int kThinConvTaps = 27;
constexpr int kThinConvSmemFloats = (kThinConvTaps + 1) * kThinConvChannels;

__device__ __forceinline__ void conv_thin_body(const DirectConvArgs &a, float *smem, int block, int num_blocks) {
    const ConvProblem &p = a.p;
    constexpr int OCB = kThinConvChannels, K = kThinConvTaps;
    const unsigned ohw = (unsigned)(p.OH * p.OW);
    const unsigned npix = ohw * (unsigned)p.B;
    const unsigned pix_blocks = (npix + blockDim.x - 1) / blockDim.x;
    const unsigned chunks = (unsigned)(p.OC + OCB - 1) / OCB;
    const unsigned units = pix_blocks * chunks;
    for (unsigned u = block; u < units; u += num_blocks) {
        const unsigned chunk = u / pix_blocks;   // consecutive blocks share their filters
        const unsigned pb = u - chunk * pix_blocks;
        const int oc0 = (int)chunk * OCB;
        __syncthreads();   // the previous unit's filters are no longer read
        for (int i = threadIdx.x; i < (K + 1) * OCB; i += blockDim.x) {
            const int t = i / OCB, o = i - t * OCB;
            const int oc = min(oc0 + o, p.OC - 1);
            smem[i] = t < K ? a.w[(size_t)oc * K + t] : a.bias[oc];
        }
        __syncthreads();
        const unsigned n = pb * blockDim.x + threadIdx.x;
        const bool valid = n < npix;
        const unsigned nn = min(n, npix - 1);
        const unsigned b = nn / ohw;
        const unsigned r = nn - b * ohw;
        const int oh = (int)(r / (unsigned)p.OW);
        const int ow = (int)r - oh * p.OW;
        const int h0 = oh * p.sh - p.ph, w0 = ow * p.sw - p.pw;
        const float *xb = a.x + (long long)b * a.x_bs;
        auto tap = [&](int c, int i2, int j) -> float {
            const int h = h0 + i2, w = w0 + j;
            const bool inside = (unsigned)h < (unsigned)p.H && (unsigned)w < (unsigned)p.W;
            const float l = xb[(c * p.H + min(max(h, 0), p.H - 1)) * p.W + min(max(w, 0), p.W - 1)];
            const float value = inside ? l : 0.f;
            return p.pre_relu ? fmaxf(value, 0.f) : value;
        };
        float acc[OCB];
#pragma unroll
        for (int o = 0; o < OCB; o++) acc[o] = smem[K * OCB + o];
        // a rolled loop over the taps (unrolled, the compiler fetches all 27 x 32 filter values first and spills them); the
        // input values of one filter row (three taps) are requested while the previous row is being used
        float v0 = tap(0, 0, 0), v1 = tap(0, 0, 1), v2 = tap(0, 0, 2);
#pragma unroll 1
        for (int row = 0; row < 9; row++) {
            const int next = min(row + 1, 8);
            const int nc = next / 3, ni = next - nc * 3;
            const float n0 = tap(nc, ni, 0), n1 = tap(nc, ni, 1), n2 = tap(nc, ni, 2);
            const pw_floatx4 *wt = reinterpret_cast<const pw_floatx4 *>(smem + row * 3 * OCB);
#pragma unroll
            for (int j = 0; j < 3; j++) {
                const float value = j == 0 ? v0 : (j == 1 ? v1 : v2);
#pragma unroll
                for (int q = 0; q < OCB / 4; q++) {
                    const pw_floatx4 w4 = wt[j * (OCB / 4) + q];
                    acc[q * 4 + 0] = fmaf(value, w4.x, acc[q * 4 + 0]);
                    acc[q * 4 + 1] = fmaf(value, w4.y, acc[q * 4 + 1]);
                    acc[q * 4 + 2] = fmaf(value, w4.z, acc[q * 4 + 2]);
                    acc[q * 4 + 3] = fmaf(value, w4.w, acc[q * 4 + 3]);
                }
            }
            v0 = n0;
            v1 = n1;
            v2 = n2;
        }
        if (valid) {
            float *yb = a.y + (long long)b * a.y_bs + r;
#pragma unroll
            for (int o = 0; o < OCB; o++)
                if (oc0 + o < p.OC) yb[(long long)(oc0 + o) * ohw] = act_apply(acc[o], p.act);
        }
    }
}

__device__ __forceinline__ void conv_direct_body(const DirectConvArgs &a, int block, int num_blocks, unsigned threads) {
    const ConvProblem &p = a.p;
    const int icg = p.IC / p.groups, ocg = p.OC / p.groups;
    const long long per_image = (long long)p.OC * p.OH * p.OW;
    const long long total = per_image * p.B;
    for (long long i = block * (long long)threads + threadIdx.x; i < total; i += (long long)num_blocks * threads) {
        const int b = (int)(i / per_image);
        const int o = (int)(i - b * per_image);
        const int oc = o / (p.OH * p.OW);
        const int r = o - oc * p.OH * p.OW;
        const int oh = r / p.OW;
        const int ow = r - oh * p.OW;
        const int g = oc / ocg;
        const float *xg = a.x + b * a.x_bs + (long long)g * icg * p.H * p.W;
        const float *wo = a.w + (size_t)oc * icg * p.KH * p.KW;
        const int h0 = oh * p.sh - p.ph, w0 = ow * p.sw - p.pw;
        float acc = a.bias[oc];
        for (int c = 0; c < icg; c++)
            for (int i2 = 0; i2 < p.KH; i2++) {
                const int h = h0 + i2;
                if ((unsigned)h >= (unsigned)p.H) continue;
                for (int j = 0; j < p.KW; j++) {
                    const int ww = w0 + j;
                    if ((unsigned)ww >= (unsigned)p.W) continue;
                    float v = xg[(long long)c * p.H * p.W + h * p.W + ww];
                    if (p.pre_relu) v = fmaxf(v, 0.f);
                    acc = fmaf(v, wo[(c * p.KH + i2) * p.KW + j], acc);
                }
            }
        a.y[b * a.y_bs + o] = act_apply(acc, p.act);
    }
}

struct NaryKernelArgs {
    NaryArgs in;
    float *y;
    long long y_bs, chw, total;   // total counts VEC-wide packets
    int multiply, accumulate, act, vec;
};

template <int VEC>
__device__ __forceinline__ void nary_body(const NaryKernelArgs &k, int block, int num_blocks, unsigned threads) {
    // indices count VEC-wide packets; chw and every batch stride are multiples of VEC on this path
    const NaryArgs &a = k.in;
    const unsigned chw_v = (unsigned)(k.chw / VEC);
    const unsigned total = (unsigned)k.total;
    for (unsigned i = block * threads + threadIdx.x; i < total; i += num_blocks * threads) {
        const unsigned b = i / chw_v;
        const long long o = (long long)(i - b * chw_v) * VEC;
        float r[VEC];
        float *dst = k.y + (long long)b * k.y_bs + o;
        int first = 0;
        if (k.accumulate) {
#pragma unroll
            for (int e = 0; e < VEC; e++) r[e] = dst[e];
        } else {
            const float *s0 = a.src[0] + (long long)b * a.src_bstride[0] + o;
            if (VEC == 4) {
                const pw_floatx4 v = *reinterpret_cast<const pw_floatx4 *>(s0);
#pragma unroll
                for (int e = 0; e < VEC; e++) r[e] = v[e];
            } else {
                r[0] = s0[0];
            }
            first = 1;
        }
        for (int j = first; j < a.count; j++) {
            const float *s = a.src[j] + (long long)b * a.src_bstride[j] + o;
            float t[VEC];
            if (VEC == 4) {
                const pw_floatx4 v = *reinterpret_cast<const pw_floatx4 *>(s);
#pragma unroll
                for (int e = 0; e < VEC; e++) t[e] = v[e];
            } else {
                t[0] = s[0];
            }
#pragma unroll
            for (int e = 0; e < VEC; e++) r[e] = k.multiply ? r[e] * t[e] : r[e] + t[e];
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) r[e] = act_apply(r[e], k.act);
        if (VEC == 4) {
            pw_floatx4 v = {r[0], r[1], r[2], r[3]};
            *reinterpret_cast<pw_floatx4 *>(dst) = v;
        } else {
            dst[0] = r[0];
        }
    }
}

__device__ __forceinline__ void nary_dispatch(const NaryKernelArgs &k, int block, int num_blocks, unsigned threads) {
    if (k.vec == 4) nary_body<4>(k, block, num_blocks, threads);
    else nary_body<1>(k, block, num_blocks, threads);
}

}  // namespace ios
