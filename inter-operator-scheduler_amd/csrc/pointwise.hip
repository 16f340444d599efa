// Stand-alone memory-bound kernels and their launchers.  Device code: pointwise_body.h.
#include "pointwise_body.h"

#include <algorithm>
#include <stdexcept>

#include "launch_internal.h"

namespace ios {

__global__ void pool_kernel(PoolArgs a) { pool_body(a, blockIdx.x, gridDim.x, blockDim.x); }
__global__ void global_pool_kernel(PoolArgs a) { global_pool_body(a, blockIdx.x, gridDim.x, blockDim.x); }
__global__ void dwconv_kernel(DirectConvArgs a) { dwconv_dispatch(a, blockIdx.x, gridDim.x, blockDim.x); }
__global__ void conv_direct_kernel(DirectConvArgs a) { conv_direct_body(a, blockIdx.x, gridDim.x, blockDim.x); }
__global__ __launch_bounds__(256) void conv_thin_kernel(DirectConvArgs a) {
    __shared__ float filters[kThinConvSmemFloats];
    conv_thin_body(a, filters, blockIdx.x, gridDim.x);
}
__global__ void nary_kernel(NaryKernelArgs a) { nary_dispatch(a, blockIdx.x, gridDim.x, blockDim.x); }

static int blocks_for(long long n, int per_block, int cap) {
    return (int)std::max<long long>(1, std::min<long long>((n + per_block - 1) / per_block, cap));
}

// ---- argument builders (shared with the fused stage kernel) ---------------------------------------------------------
PoolArgs make_pool_args(const PoolProblem &p, const TensorView &x, const TensorView &y, bool global, int *blocks, const float *bias, int act) {
    if (x.C != p.C || x.H != p.H || x.W != p.W || y.C != p.C || y.H != p.OH || y.W != p.OW)
        throw std::runtime_error("pool: tensor views do not match the problem");
    if (global && (p.KH != p.H || p.KW != p.W || p.OH != 1 || p.OW != 1))
        throw std::runtime_error("global pool: window must be the whole map");
    if ((long long)p.B * p.C * p.OH * p.OW >= (1LL << 31)) throw std::runtime_error("pool: tensor too large for 32-bit indexing");
    PoolArgs a;
    a.x = x.ptr;
    a.y = y.ptr;
    a.x_bs = x.bstride;
    a.y_bs = y.bstride;
    a.p = p;
    a.strip_rows = 0;
    a.vec_columns = 1;
    a.bias = bias;
    a.act = act;
    if (global) {
        // from 2^14 planes on (a lane per plane still gives every compute unit a wavefront) the row form, else a wavefront per plane
        const long long planes = (long long)p.B * p.C;
        if (planes >= (1LL << 14) && p.H * p.W <= 1024) {
            a.strip_rows = 1;
            *blocks = blocks_for(planes, 256, 4096);
        } else {
            *blocks = blocks_for(planes, 4, 4096);
        }
    } else if (p.KH == 3 && p.KW == 3 && (p.sh == 1 || p.sh == 2)) {
        // one thread per strip of output rows; the longest strip that still leaves a million threads
        int rows = kPoolStripRows;
        while (rows > 1 && (long long)p.B * p.C * ((p.OH + rows - 1) / rows) * p.OW < (1LL << 20)) rows >>= 1;
        a.strip_rows = rows;
        long long threads = (long long)p.B * p.C * ((p.OH + rows - 1) / rows) * p.OW;
        // larger tensors: four output columns per thread (16-byte loads and stores) while that leaves 65536 threads
        if ((p.sw == 1 || p.sw == 2) && p.pw <= 1 && p.W >= 8) {
            const long long kVecMinThreads = 1LL << 16;   // measured: 2^16 beats the one-column form from 64x147x147 at batch 1 on, 2^14 loses
            auto quads = [&](int r) { return (long long)p.B * p.C * ((p.OH + r - 1) / r) * ((p.OW + kPoolVecColumns - 1) / kPoolVecColumns); };
            // Tensors that give half a million threads even with the shortest strips (batch 16 and more) are bound by how many
            // loads the device has in flight, not by the rows neighbouring strips read twice: one output row per thread for
            // stride 2, two for stride 1 (batch 64, launched back to back: 64x147x147 stride 2 101.9 -> 89.7 us = 4.9 TB/s,
            // 192x71x71 87.5 -> 77.3, 288x35x35 26.8 -> 22.3, 768x17x17 17.8 -> 15.9; stride 1 on 32x35x35 9.2 -> 7.5,
            // 192x17x17 10.8 -> 9.7 us; longer strips there are 5-15 % slower, one column per thread 30-60 %)
            const long long kShortStripThreads = 1LL << 19;
            int vrows = kPoolStripRows;
            if (quads(1) >= kShortStripThreads) vrows = p.sh == 2 ? 1 : 2;
            while (vrows > 1 && quads(vrows) < kVecMinThreads) vrows >>= 1;
            if (quads(vrows) >= kVecMinThreads) {
                a.vec_columns = kPoolVecColumns;
                a.strip_rows = vrows;
                threads = quads(vrows);
            }
        }
        *blocks = blocks_for(threads, 256, 16384);
    } else {
        *blocks = blocks_for((long long)p.B * p.C * p.OH * p.OW, 256, 8192);
    }
    return a;
}

DirectConvArgs make_direct_conv_args(const ConvProblem &p, const TensorView &x, const float *w, const float *bias,
                                     const TensorView &y, int *blocks, bool thin) {
    if (x.C != p.IC || x.H != p.H || x.W != p.W || y.C != p.OC || y.H != p.OH || y.W != p.OW)
        throw std::runtime_error("conv: tensor views do not match the problem");
    if ((long long)p.B * p.OC * p.OH * p.OW >= (1LL << 31)) throw std::runtime_error("conv: tensor too large for 32-bit indexing");
    DirectConvArgs a;
    a.x = x.ptr;
    a.w = w;
    a.bias = bias;
    a.y = y.ptr;
    a.x_bs = x.bstride;
    a.y_bs = y.bstride;
    a.p = p;
    const unsigned long long x_bytes = ((unsigned long long)(p.B - 1) * x.bstride + (unsigned long long)p.IC * p.H * p.W) * 4ull;
    a.x_bytes = x_bytes < (1ull << 31) ? (unsigned)x_bytes : 0u;
    a.nmore = 0;
    for (int s = 0; s < kMaxNaryInputs - 1; s++) {
        a.more[s] = x.ptr;
        a.more_bs[s] = x.bstride;
        a.more_bytes[s] = 0;
    }
    *blocks = blocks_for((long long)p.B * p.OC * p.OH * p.OW, 256, 8192);
    a.thin = 0;
    if (thin) {
        if (!conv_thin_applies(p)) throw std::runtime_error("conv: the thin-input kernel serves 3 x 3 convolutions of 3-channel inputs");
        a.thin = 1;
        // one block per 256 pixels and 32 output channels (sized for 256-thread blocks like the other bodies)
        const long long units = (((long long)p.B * p.OH * p.OW + 255) / 256) * ((p.OC + kThinConvChannels - 1) / kThinConvChannels);
        *blocks = (int)std::min<long long>(units, 1 << 20);
    }
    return a;
}

bool dwconv_sums_inputs(const ConvProblem &p) { return p.is_depthwise() && p.KH == p.KW && (p.KH == 3 || p.KH == 5); }

void add_dwconv_sources(DirectConvArgs &a, const TensorView *more, int count) {
    if (count < 0 || count > kMaxNaryInputs - 1) throw std::runtime_error("dwconv: too many summed inputs");
    const ConvProblem &p = a.p;
    if (count > 0 && !dwconv_sums_inputs(p)) throw std::runtime_error("dwconv: this window does not add inputs in its loader");
    for (int s = 0; s < count; s++) {
        if (more[s].C != p.IC || more[s].H != p.H || more[s].W != p.W) throw std::runtime_error("dwconv: summed inputs of different shapes");
        const unsigned long long bytes = ((unsigned long long)(p.B - 1) * more[s].bstride + (unsigned long long)p.IC * p.H * p.W) * 4ull;
        if (bytes >= (1ull << 31) || a.x_bytes == 0) throw std::runtime_error("dwconv: summed inputs beyond 31-bit offsets");
        a.more[s] = more[s].ptr;
        a.more_bs[s] = more[s].bstride;
        a.more_bytes[s] = (unsigned)bytes;
    }
    a.nmore = count;
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

NaryKernelArgs make_nary_args(const NaryArgs &in, int multiply, int accumulate, int act, int B, long long chw,
                              const TensorView &y, int *blocks) {
    if (in.count < 1 || in.count > kMaxNaryInputs) throw std::runtime_error("nary: bad input count");
    bool vec = (chw % 4 == 0) && (y.bstride % 4 == 0) && aligned16(y.ptr);
    for (int j = 0; j < in.count; j++) vec = vec && (in.src_bstride[j] % 4 == 0) && aligned16(in.src[j]);
    if ((long long)B * chw >= (1LL << 31)) throw std::runtime_error("nary: tensor too large for 32-bit indexing");
    NaryKernelArgs a;
    a.in = in;
    a.y = y.ptr;
    a.y_bs = y.bstride;
    a.chw = chw;
    a.vec = vec ? 4 : 1;
    a.total = (long long)B * chw / a.vec;
    a.multiply = multiply;
    a.accumulate = accumulate;
    a.act = act;
    *blocks = blocks_for(a.total, 256, 8192);
    return a;
}

// ---- launchers ---------------------------------------------------------------------------------------------------------
void launch_pool(const PoolProblem &p, const TensorView &x, const TensorView &y, hipStream_t stream, const float *bias, int act) {
    int blocks;
    const PoolArgs a = make_pool_args(p, x, y, false, &blocks, bias, act);
    hipLaunchKernelGGL(pool_kernel, dim3(blocks), dim3(256), 0, stream, a);
}

void launch_global_pool(const PoolProblem &p, const TensorView &x, const TensorView &y, hipStream_t stream) {
    int blocks;
    const PoolArgs a = make_pool_args(p, x, y, true, &blocks);
    hipLaunchKernelGGL(global_pool_kernel, dim3(blocks), dim3(256), 0, stream, a);
}

void launch_dwconv(const ConvProblem &p, const TensorView &x, const float *w, const float *bias, const TensorView &y,
                   hipStream_t stream, const TensorView *more, int nmore) {
    if (!p.is_depthwise()) throw std::runtime_error("dwconv: not a depth-wise problem");
    int blocks;
    DirectConvArgs a = make_direct_conv_args(p, x, w, bias, y, &blocks);
    add_dwconv_sources(a, more, nmore);
    hipLaunchKernelGGL(dwconv_kernel, dim3(blocks), dim3(256), 0, stream, a);
}

void launch_conv_direct(const ConvProblem &p, const TensorView &x, const float *w, const float *bias, const TensorView &y,
                        hipStream_t stream, bool thin) {
    int blocks;
    const DirectConvArgs a = make_direct_conv_args(p, x, w, bias, y, &blocks, thin);
    if (thin) hipLaunchKernelGGL(conv_thin_kernel, dim3(blocks), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(conv_direct_kernel, dim3(blocks), dim3(256), 0, stream, a);
}

void launch_nary(const NaryArgs &in, int multiply, int accumulate, int act, int B, long long chw, const TensorView &y,
                 hipStream_t stream) {
    int blocks;
    const NaryKernelArgs a = make_nary_args(in, multiply, accumulate, act, B, chw, y, &blocks);
    hipLaunchKernelGGL(nary_kernel, dim3(blocks), dim3(256), 0, stream, a);
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
    hipLaunchKernelGGL(fill_pattern_kernel, dim3(blocks_for((long long)n, 256, 65535)), dim3(256), 0, stream, dst, n, seed);
}

void launch_fill_u32(unsigned *dst, size_t n, unsigned value, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks_for((long long)n, 256, 65535)), dim3(256), 0, stream, dst, n, value);
}

}  // namespace ios
