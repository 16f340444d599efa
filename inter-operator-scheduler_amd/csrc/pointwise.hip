// Memory-bound kernels: pooling, depth-wise and direct convolution, n-ary add / multiply, activation /
// strided copy, fills.  All of them read and write NCHW views (channel stride H*W, arbitrary batch
// stride), consecutive lanes cover consecutive output columns so that global accesses coalesce.
#include "kernels.h"

#include <algorithm>
#include <stdexcept>

namespace ios {

typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float act_apply(float v, int act) {
    switch (act) {
        case ACT_RELU: return fmaxf(v, 0.0f);
        case ACT_TANH: return tanhf(v);
        case ACT_SIGMOID: return 1.0f / (1.0f + __expf(-v));
        default: return v;
    }
}

static unsigned grid_for(size_t n, int block, unsigned cap = 1u << 20) {
    return (unsigned)std::max<size_t>(1, std::min<size_t>((n + block - 1) / block, cap));
}

// ---- pooling --------------------------------------------------------------------------------------------
__global__ void pool_kernel(const float *x, float *y, long long x_bs, long long y_bs, PoolProblem p) {
    const long long per_image = (long long)p.C * p.OH * p.OW;
    const long long total = per_image * p.B;
    const float inv = 1.0f / (float)(p.KH * p.KW);
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int b = (int)(i / per_image);
        const int o = (int)(i - b * per_image);
        const int c = o / (p.OH * p.OW);
        const int r = o - c * p.OH * p.OW;
        const int oh = r / p.OW;
        const int ow = r - oh * p.OW;
        const float *xc = x + b * x_bs + (long long)c * p.H * p.W;
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
        y[b * y_bs + o] = p.is_max ? best : sum * inv;
    }
}

void launch_pool(const PoolProblem &p, const TensorView &x, const TensorView &y, hipStream_t stream) {
    if (x.C != p.C || x.H != p.H || x.W != p.W || y.C != p.C || y.H != p.OH || y.W != p.OW)
        throw std::runtime_error("pool: tensor views do not match the problem");
    const size_t total = (size_t)p.B * p.C * p.OH * p.OW;
    hipLaunchKernelGGL(pool_kernel, dim3(grid_for(total, 256)), dim3(256), 0, stream, x.ptr, y.ptr, x.bstride, y.bstride, p);
}

__global__ void global_pool_kernel(const float *x, float *y, long long x_bs, long long y_bs, int C, int HW, int planes,
                                   int is_max) {
    const int plane = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (plane >= planes) return;
    const int lane = threadIdx.x & 63;
    const int b = plane / C, c = plane - b * C;
    const float *xc = x + b * x_bs + (long long)c * HW;
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
    if (lane == 0) y[b * y_bs + c] = is_max ? best : sum / (float)HW;
}

void launch_global_pool(const PoolProblem &p, const TensorView &x, const TensorView &y, hipStream_t stream) {
    if (p.KH != p.H || p.KW != p.W || p.OH != 1 || p.OW != 1) throw std::runtime_error("global pool: window must be the whole map");
    const int planes = p.B * p.C;
    hipLaunchKernelGGL(global_pool_kernel, dim3((planes + 3) / 4), dim3(256), 0, stream, x.ptr, y.ptr, x.bstride, y.bstride,
                       p.C, p.H * p.W, planes, p.is_max);
}

// ---- depth-wise convolution -----------------------------------------------------------------------------------
template <int KH, int KW>
__global__ void dwconv_kernel(const float *x, const float *w, const float *bias, float *y, long long x_bs, long long y_bs,
                              ConvProblem p) {
    const int kh_n = KH > 0 ? KH : p.KH, kw_n = KW > 0 ? KW : p.KW;
    const long long per_image = (long long)p.OC * p.OH * p.OW;
    const long long total = per_image * p.B;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int b = (int)(i / per_image);
        const int o = (int)(i - b * per_image);
        const int c = o / (p.OH * p.OW);
        const int r = o - c * p.OH * p.OW;
        const int oh = r / p.OW;
        const int ow = r - oh * p.OW;
        const float *xc = x + b * x_bs + (long long)c * p.H * p.W;
        const float *wc = w + (size_t)c * kh_n * kw_n;
        const int h0 = oh * p.sh - p.ph, w0 = ow * p.sw - p.pw;
        float acc = bias[c];
#pragma unroll
        for (int i2 = 0; i2 < kh_n; i2++) {
            const int h = h0 + i2;
            if ((unsigned)h >= (unsigned)p.H) continue;
#pragma unroll
            for (int j = 0; j < kw_n; j++) {
                const int ww = w0 + j;
                if ((unsigned)ww >= (unsigned)p.W) continue;
                float v = xc[h * p.W + ww];
                if (p.pre_relu) v = fmaxf(v, 0.f);
                acc = fmaf(v, wc[i2 * kw_n + j], acc);
            }
        }
        y[b * y_bs + o] = act_apply(acc, p.act);
    }
}

void launch_dwconv(const ConvProblem &p, const TensorView &x, const float *w, const float *bias, const TensorView &y,
                   hipStream_t stream) {
    if (!p.is_depthwise()) throw std::runtime_error("dwconv: not a depth-wise problem");
    if (x.C != p.IC || x.H != p.H || x.W != p.W || y.C != p.OC || y.H != p.OH || y.W != p.OW)
        throw std::runtime_error("dwconv: tensor views do not match the problem");
    const size_t total = (size_t)p.B * p.OC * p.OH * p.OW;
    const dim3 grid(grid_for(total, 256)), block(256);
    if (p.KH == 3 && p.KW == 3)
        hipLaunchKernelGGL((dwconv_kernel<3, 3>), grid, block, 0, stream, x.ptr, w, bias, y.ptr, x.bstride, y.bstride, p);
    else if (p.KH == 5 && p.KW == 5)
        hipLaunchKernelGGL((dwconv_kernel<5, 5>), grid, block, 0, stream, x.ptr, w, bias, y.ptr, x.bstride, y.bstride, p);
    else if (p.KH == 7 && p.KW == 7)
        hipLaunchKernelGGL((dwconv_kernel<7, 7>), grid, block, 0, stream, x.ptr, w, bias, y.ptr, x.bstride, y.bstride, p);
    else
        hipLaunchKernelGGL((dwconv_kernel<0, 0>), grid, block, 0, stream, x.ptr, w, bias, y.ptr, x.bstride, y.bstride, p);
}

// ---- direct convolution (any groups) ------------------------------------------------------------------------------
__global__ void conv_direct_kernel(const float *x, const float *w, const float *bias, float *y, long long x_bs,
                                   long long y_bs, ConvProblem p) {
    const int icg = p.IC / p.groups, ocg = p.OC / p.groups;
    const long long per_image = (long long)p.OC * p.OH * p.OW;
    const long long total = per_image * p.B;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int b = (int)(i / per_image);
        const int o = (int)(i - b * per_image);
        const int oc = o / (p.OH * p.OW);
        const int r = o - oc * p.OH * p.OW;
        const int oh = r / p.OW;
        const int ow = r - oh * p.OW;
        const int g = oc / ocg;
        const float *xg = x + b * x_bs + (long long)g * icg * p.H * p.W;
        const float *wo = w + (size_t)oc * icg * p.KH * p.KW;
        const int h0 = oh * p.sh - p.ph, w0 = ow * p.sw - p.pw;
        float acc = bias[oc];
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
        y[b * y_bs + o] = act_apply(acc, p.act);
    }
}

void launch_conv_direct(const ConvProblem &p, const TensorView &x, const float *w, const float *bias, const TensorView &y,
                        hipStream_t stream) {
    if (x.C != p.IC || x.H != p.H || x.W != p.W || y.C != p.OC || y.H != p.OH || y.W != p.OW)
        throw std::runtime_error("conv: tensor views do not match the problem");
    const size_t total = (size_t)p.B * p.OC * p.OH * p.OW;
    hipLaunchKernelGGL(conv_direct_kernel, dim3(grid_for(total, 256)), dim3(256), 0, stream, x.ptr, w, bias, y.ptr,
                       x.bstride, y.bstride, p);
}

// ---- n-ary add / multiply, activation, copy ---------------------------------------------------------------------------
template <int VEC>
__global__ void nary_kernel(NaryArgs a, int multiply, int accumulate, int act, long long chw, long long total, float *y,
                            long long y_bs) {
    // indices count VEC-wide packets; chw and every batch stride are multiples of VEC on this path
    const long long chw_v = chw / VEC;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const long long b = i / chw_v;
        const long long o = (i - b * chw_v) * VEC;
        float r[VEC];
        float *dst = y + b * y_bs + o;
        int first = 0;
        if (accumulate) {
#pragma unroll
            for (int e = 0; e < VEC; e++) r[e] = dst[e];
        } else {
            const float *s0 = a.src[0] + b * a.src_bstride[0] + o;
            if (VEC == 4) {
                const floatx4 v = *reinterpret_cast<const floatx4 *>(s0);
#pragma unroll
                for (int e = 0; e < VEC; e++) r[e] = v[e];
            } else {
                r[0] = s0[0];
            }
            first = 1;
        }
        for (int j = first; j < a.count; j++) {
            const float *s = a.src[j] + b * a.src_bstride[j] + o;
            float t[VEC];
            if (VEC == 4) {
                const floatx4 v = *reinterpret_cast<const floatx4 *>(s);
#pragma unroll
                for (int e = 0; e < VEC; e++) t[e] = v[e];
            } else {
                t[0] = s[0];
            }
#pragma unroll
            for (int e = 0; e < VEC; e++) r[e] = multiply ? r[e] * t[e] : r[e] + t[e];
        }
#pragma unroll
        for (int e = 0; e < VEC; e++) r[e] = act_apply(r[e], act);
        if (VEC == 4) {
            floatx4 v = {r[0], r[1], r[2], r[3]};
            *reinterpret_cast<floatx4 *>(dst) = v;
        } else {
            dst[0] = r[0];
        }
    }
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

void launch_nary(const NaryArgs &a, int multiply, int accumulate, int act, int B, long long chw, const TensorView &y,
                 hipStream_t stream) {
    if (a.count < 1 || a.count > kMaxNaryInputs) throw std::runtime_error("nary: bad input count");
    bool vec = (chw % 4 == 0) && (y.bstride % 4 == 0) && aligned16(y.ptr);
    for (int j = 0; j < a.count; j++) vec = vec && (a.src_bstride[j] % 4 == 0) && aligned16(a.src[j]);
    if (vec) {
        const long long total = (long long)B * chw / 4;
        hipLaunchKernelGGL(nary_kernel<4>, dim3(grid_for((size_t)total, 256)), dim3(256), 0, stream, a, multiply, accumulate,
                           act, chw, total, y.ptr, y.bstride);
    } else {
        const long long total = (long long)B * chw;
        hipLaunchKernelGGL(nary_kernel<1>, dim3(grid_for((size_t)total, 256)), dim3(256), 0, stream, a, multiply, accumulate,
                           act, chw, total, y.ptr, y.bstride);
    }
}

void launch_unary(const TensorView &x, const TensorView &y, int act, int B, hipStream_t stream) {
    if (x.C != y.C || x.H != y.H || x.W != y.W) throw std::runtime_error("unary: shape mismatch");
    NaryArgs a;
    a.count = 1;
    a.src[0] = x.ptr;
    a.src_bstride[0] = x.bstride;
    launch_nary(a, 0, 0, act, B, (long long)x.C * x.H * x.W, y, stream);
}

// ---- fills ---------------------------------------------------------------------------------------------------------
__global__ void fill_pattern_kernel(float *dst, size_t n, unsigned seed) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        unsigned h = (unsigned)i * 2654435761u ^ seed;
        h ^= h >> 16;
        h *= 0x85ebca6bu;
        h ^= h >> 13;
        h *= 0xc2b2ae35u;
        h ^= h >> 16;
        dst[i] = (float)(h >> 8) * (1.0f / 8388608.0f) - 1.0f;
    }
}

__global__ void fill_u32_kernel(unsigned *dst, size_t n, unsigned value) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = value;
}

void launch_fill_pattern(float *dst, size_t n, unsigned seed, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(fill_pattern_kernel, dim3(grid_for(n, 256, 65535)), dim3(256), 0, stream, dst, n, seed);
}

void launch_fill_u32(unsigned *dst, size_t n, unsigned value, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(n, 256, 65535)), dim3(256), 0, stream, dst, n, value);
}

}  // namespace ios
