// Host-side builders of kernel argument blocks, shared by the stand-alone launchers and the fused stage kernel.
#pragma once

#include "conv_body.h"
#include "pointwise_body.h"

namespace ios {

struct ConvDispatch {
    ConvKernelArgs args;
    int variant;
    int threads, smem_bytes;
    int tiles, groups, slices;       // grid of the main kernel: (tiles, groups, slices), or
    int xcd_blocks;                  // > 0: a one-dimensional grid of this many blocks, numbered for XCD-local split-K
    int grid_blocks() const { return xcd_blocks > 0 ? xcd_blocks : tiles * groups * slices; }
    bool has_reduce;                 // split-K: a reduce pass must follow the main kernel
    ReduceArgs reduce;
    int reduce_blocks;
};

ConvDispatch make_conv_dispatch(const ConvProblem &p, const ConvLaunch &l, const TensorView &x, const float *packed,
                                const float *bias, const TensorView &y, float *workspace, const SplitKReduce &reduce,
                                const TensorView *residual = nullptr, bool post_relu = false);
PoolArgs make_pool_args(const PoolProblem &p, const TensorView &x, const TensorView &y, bool global, int *blocks,
                        const float *bias = nullptr, int act = ACT_NONE);
DirectConvArgs make_direct_conv_args(const ConvProblem &p, const TensorView &x, const float *w, const float *bias,
                                     const TensorView &y, int *blocks, bool thin = false);
// further inputs of a depth-wise convolution of a sum (see DirectConvArgs::more)
void add_dwconv_sources(DirectConvArgs &a, const TensorView *more, int count);
NaryKernelArgs make_nary_args(const NaryArgs &in, int multiply, int accumulate, int act, int B, long long chw,
                              const TensorView &y, int *blocks);

}  // namespace ios
