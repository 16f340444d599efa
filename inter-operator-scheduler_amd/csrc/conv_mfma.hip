// Stand-alone convolution kernels, the configuration table and the launchers.  Device code: conv_body.h.
#include "conv_body.h"
#include "launch_internal.h"

#include <algorithm>
#include <stdexcept>
#include <string>

namespace ios {

// stand-alone kernel around a body: grid = (tiles, groups, K slices), dynamic LDS = Body::SMEM_FLOATS floats
// RES: the residual form of the epilogue (a.res is not null)
template <typename Body, bool RES = false>
__global__ __launch_bounds__(Body::THREADS) void conv_kernel(ConvKernelArgs a) {
    extern __shared__ floatx4 conv_smem[];
    if (a.xcd_local) {   // one-dimensional grid numbered for split-K inside an XCD
        const XcdSlot slot = xcd_enter(a, blockIdx.x, blockIdx.x);
        if (slot.idle) return;
        Body::template run<RES>(a, reinterpret_cast<float *>(conv_smem), slot.tile, 0, slot.slice);
        return;
    }
    Body::template run<RES>(a, reinterpret_cast<float *>(conv_smem), blockIdx.x, blockIdx.y, blockIdx.z);
}

__global__ void splitk_reduce_kernel(ReduceArgs a) { splitk_reduce_body(a, blockIdx.x, gridDim.x, blockDim.x); }

// ---- variant table --------------------------------------------------------------------------------------------
typedef void (*ConvKernelFn)(ConvKernelArgs);

struct VariantEntry {
    ConvVariant v;
    ConvKernelFn kernel, kernel_residual;
    int smem_floats;
};

#define IOS_TILED_ENTRY(IDX, NAME, BM, BN, BK, WM, WN, WK, MT, PD)                                        \
    {{NAME, BM, BN, BK, WM, WN, WK, MT, false, ConvTiled<BM, BN, BK, WM, WN, WK, MT, PD>::CPAD, false, \
      ConvTiled<BM, BN, BK, WM, WN, WK, MT, PD>::FUSABLE, false},    \
     conv_kernel<ConvTiled<BM, BN, BK, WM, WN, WK, MT, PD>>, conv_kernel<ConvTiled<BM, BN, BK, WM, WN, WK, MT, PD>, true>, \
     ConvTiled<BM, BN, BK, WM, WN, WK, MT, PD>::SMEM_FLOATS},
#define IOS_WSPLIT_ENTRY(IDX, NAME, MT, TM, TN, NW, U, QUAD, D, BF16)                                                                  \
    {{NAME, TM * MT, TN * MT, U *(MT == 32 ? 2 : 4), 1, 1, NW, MT, true, ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16>::CPAD, QUAD, \
      ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16>::FUSABLE, BF16},      \
     conv_kernel<ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16>>, conv_kernel<ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16>, true>,    \
     ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16>::SMEM_FLOATS},
#define IOS_WSPLIT_C4_ENTRY(IDX, NAME, MT, TM, TN, NW, U, QUAD, D, BF16)                                                                  \
    {{NAME, TM * MT, TN * MT, U *(MT == 32 ? 2 : 4), 1, 1, NW, MT, true, ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16, 4>::CPAD, QUAD, \
      ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16, 4>::FUSABLE, BF16},                                                                 \
     conv_kernel<ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16, 4>>, conv_kernel<ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16, 4>, true>,    \
     ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16, 4>::SMEM_FLOATS},

#define IOS_SPLIT3_ENTRY(IDX, NAME, TMW, TNW, WM, WN, PD)                                                                              \
    {{NAME, ConvSplit3<TMW, TNW, WM, WN, PD>::BM, ConvSplit3<TMW, TNW, WM, WN, PD>::BN, 16, WM, WN, 1, 32, false,                         \
      ConvSplit3<TMW, TNW, WM, WN, PD>::CPAD, false, false, PREC_FP32, 3},                                                                \
     conv_kernel<ConvSplit3<TMW, TNW, WM, WN, PD>>, conv_kernel<ConvSplit3<TMW, TNW, WM, WN, PD>, true>,                                  \
     ConvSplit3<TMW, TNW, WM, WN, PD>::SMEM_FLOATS},

#define IOS_WSPLIT_X3_ENTRY(IDX, NAME, TM, TN, NW, D)                                                                        \
    {{NAME, TM * 32, TN * 32, 16, 1, 1, NW, 32, true, ConvWsplit<32, TM, TN, NW, 8, true, D, 3>::CPAD, true, false, PREC_FP32, 3, \
      ConvWsplit<32, TM, TN, NW, 8, true, D, 3>::FUSABLE_WIDE},      \
     conv_kernel<ConvWsplit<32, TM, TN, NW, 8, true, D, 3>>, conv_kernel<ConvWsplit<32, TM, TN, NW, 8, true, D, 3>, true>,              \
     ConvWsplit<32, TM, TN, NW, 8, true, D, 3>::SMEM_FLOATS},

#define IOS_SPLIT1_ENTRY(IDX, NAME, TMW, TNW, WM, WN, PD)                                                                              \
    {{NAME, ConvSplit3<TMW, TNW, WM, WN, PD, 1>::BM, ConvSplit3<TMW, TNW, WM, WN, PD, 1>::BN, 16, WM, WN, 1, 32, false,                   \
      ConvSplit3<TMW, TNW, WM, WN, PD, 1>::CPAD, false, false, PREC_BF16, 1},                                                             \
     conv_kernel<ConvSplit3<TMW, TNW, WM, WN, PD, 1>>, conv_kernel<ConvSplit3<TMW, TNW, WM, WN, PD, 1>, true>,                            \
     ConvSplit3<TMW, TNW, WM, WN, PD, 1>::SMEM_FLOATS},

#define IOS_WSPLIT_X1_ENTRY(IDX, NAME, TM, TN, NW, D)                                                                        \
    {{NAME, TM * 32, TN * 32, 16, 1, 1, NW, 32, true, ConvWsplit<32, TM, TN, NW, 8, true, D, 4>::CPAD, true, false, PREC_BF16, 1},      \
     conv_kernel<ConvWsplit<32, TM, TN, NW, 8, true, D, 4>>, conv_kernel<ConvWsplit<32, TM, TN, NW, 8, true, D, 4>, true>,              \
     ConvWsplit<32, TM, TN, NW, 8, true, D, 4>::SMEM_FLOATS},

static const VariantEntry kVariants[] = {IOS_TILED_VARIANTS(IOS_TILED_ENTRY) IOS_WSPLIT_VARIANTS(IOS_WSPLIT_ENTRY)
                                             IOS_WSPLIT_C4_VARIANTS(IOS_WSPLIT_C4_ENTRY)
                                             IOS_WSPLIT_T32_VARIANTS(IOS_WSPLIT_ENTRY) IOS_WSPLIT_F16_VARIANTS(IOS_WSPLIT_ENTRY)
                                             IOS_WSPLIT_LONGK_VARIANTS(IOS_WSPLIT_ENTRY) IOS_SPLIT3_VARIANTS(IOS_SPLIT3_ENTRY) IOS_WSPLIT_X3_VARIANTS(IOS_WSPLIT_X3_ENTRY)
                                             IOS_SPLIT1_VARIANTS(IOS_SPLIT1_ENTRY) IOS_WSPLIT_X1_VARIANTS(IOS_WSPLIT_X1_ENTRY)};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);
static_assert(kNumVariants == kNumConvVariants, "variant lists and count disagree");

int conv_num_variants() { return kNumVariants; }

const ConvVariant &conv_variant(int index) {
    if (index < 0 || index >= kNumVariants) throw std::runtime_error("conv variant index out of range");
    return kVariants[index].v;
}

static int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

static int k_chunk_of(const ConvProblem &p, const ConvLaunch &l) {
    const ConvVariant &v = kVariants[l.variant].v;
    const int kq = p.Kq(v.cpad);
    // for the wave-split kernels BK is the K extent of one register batch, which may not divide kq
    const int tiles_k = ceil_div(kq, v.BK);
    return ceil_div(tiles_k, std::max(1, l.split_k)) * v.BK;
}

// split_k may ask for more slices than there are K tiles; the effective count leaves no slice empty
static int effective_split(const ConvProblem &p, const ConvLaunch &l) {
    return std::max(1, ceil_div(p.Kq(kVariants[l.variant].v.cpad), k_chunk_of(p, l)));
}

int conv_effective_split(const ConvProblem &p, const ConvLaunch &l) { return effective_split(p, l); }

size_t conv_workspace_floats(const ConvProblem &p, const ConvLaunch &l) {
    const int s = effective_split(p, l);
    if (s <= 1) return 0;
    // two-kernel form: [slice][OC][pixels]; one-kernel forms: [group][tile][slice][BM * BN] with the tile count rounded up
    // to a multiple of 8 (the numbering of the XCD-local form, see XcdSlot)
    const ConvVariant &v = kVariants[l.variant].v;
    const size_t tiles = (size_t)xcd_padded_tiles(ceil_div(p.OCg(), v.BM) * ceil_div(p.Npix(), v.BN));
    const size_t padded = (size_t)p.groups * tiles * v.BM * v.BN;
    return (size_t)s * std::max((size_t)p.OC * (size_t)p.Npix(), padded);
}

size_t conv_counter_count(const ConvProblem &p, const ConvLaunch &l) {
    if (effective_split(p, l) <= 1) return 0;
    const ConvVariant &v = kVariants[l.variant].v;
    return (size_t)p.groups * (size_t)xcd_padded_tiles(ceil_div(p.OCg(), v.BM) * ceil_div(p.Npix(), v.BN));
}

static int variant_by_name(const char *name) {
    for (int i = 0; i < kNumVariants; i++)
        if (std::string(kVariants[i].v.name) == name) return i;
    throw std::runtime_error(std::string("conv: no kernel configuration named ") + name);
}

ConvLaunch conv_pick_launch(const ConvProblem &p, int num_cus, bool fusable_only, int precision) {
    // Closed-form model distilled from measured choices on Inception-v3 at batch 1, 16 and 64: problems that fill
    // the device several times over with 64 x 64 tiles take the LDS-tiled kernel (the largest tile that still
    // offers two blocks per compute unit); smaller ones take the wave-split kernel with the largest tile that
    // still offers a block per compute unit; the smallest split K over the grid as well.
    const long long M = p.OCg(), N = p.Npix();
    auto blocks_of = [&](int idx) {
        const ConvVariant &v = kVariants[idx].v;
        return (long long)ceil_div(M, v.BM) * ceil_div(N, v.BN) * p.groups;
    };
    ConvLaunch best;
    if (precision != PREC_FP32) {
        // reduced precision: wave-split configurations only, the largest tile that offers two blocks per compute unit
        static const int bf16_large_to_small[] = {variant_by_name("wb_m64n64_w4"), variant_by_name("wb_m64n32_w8"),
                                                  variant_by_name("wb_m32n32_w8"), variant_by_name("wb_m32n16_w8"),
                                                  variant_by_name("wb_m16n16_w16")};
        static const int fp16_large_to_small[] = {variant_by_name("wh_m64n64_w4"), variant_by_name("wh_m64n32_w8"),
                                                  variant_by_name("wh_m32n32_w8"), variant_by_name("wh_m32n16_w8"),
                                                  variant_by_name("wh_m16n16_w16")};
        const int *large_to_small = precision == PREC_BF16 ? bf16_large_to_small : fp16_large_to_small;
        for (int i = 0; i < 4; i++) {
            const int idx = large_to_small[i];
            if ((!fusable_only || kVariants[idx].v.fusable()) && blocks_of(idx) >= 2LL * num_cus) {
                best.variant = idx;
                return best;
            }
        }
        best.variant = large_to_small[4];
        const ConvVariant &v = kVariants[best.variant].v;
        const long long blocks = blocks_of(best.variant);
        const int batches = ceil_div(p.Kq(v.cpad), v.BK);
        const long long split = std::min<long long>((num_cus + blocks - 1) / blocks, std::max(1, batches / (2 * v.WK)));
        best.split_k = (int)std::max<long long>(1, std::min<long long>(split, 16));
        return best;
    }
    static const int tiled_mid = variant_by_name("m64n64k16_w2x2x1_t32");
    if (!fusable_only && blocks_of(tiled_mid) >= 4LL * num_cus) {
        static const int by_size[] = {variant_by_name("m128n128k16_w2x2x1_t32"), variant_by_name("m128n64k16_w2x2x1_t32"),
                                      variant_by_name("m64n128k16_w2x2x1_t32")};
        best.variant = tiled_mid;
        for (int idx : by_size) {
            if (fusable_only && !kVariants[idx].v.fusable()) continue;
            if (blocks_of(idx) >= 2LL * num_cus) {
                best.variant = idx;
                break;
            }
        }
        return best;
    }
    static const int split_large_to_small[] = {variant_by_name("wq_m64n32_w8_t16"), variant_by_name("wq_m32n32_w8_t16"),
                                               variant_by_name("wq_m32n16_w8_t16")};
    for (int idx : split_large_to_small)
        if ((!fusable_only || kVariants[idx].v.fusable()) && blocks_of(idx) >= num_cus) {
            best.variant = idx;
            return best;
        }
    best.variant = variant_by_name("wq_m16n16_w16_t16");
    const ConvVariant &v = kVariants[best.variant].v;
    const long long blocks = blocks_of(best.variant);
    const int batches = ceil_div(p.Kq(v.cpad), v.BK);          // register batches along K
    const int per_slice = 2 * v.WK;                            // leave every wavefront two batches
    const long long split = std::min<long long>((num_cus + blocks - 1) / blocks, std::max(1, batches / per_slice));
    best.split_k = (int)std::max<long long>(1, std::min<long long>(split, 16));
    return best;
}

bool conv_matrix_path_supported(const ConvProblem &p) {
    // packed filter rows are indexed with 16 bits, input and filter byte offsets with 31 bits
    const unsigned long long x_bytes = (unsigned long long)p.B * p.IC * p.H * p.W * 4ull;
    const unsigned long long w_bytes = (unsigned long long)p.groups * p.Kq(128) * p.OCgP() * 4ull;
    // image sides below 2^15 and output planes below 2^23 elements keep the kernels' signed 24-bit index multiplies exact
    return p.Kq(128) < 65536 && p.Npix() < (1LL << 31) && x_bytes < (1ull << 30) && w_bytes < (1ull << 31) && p.H < 32768 && p.W < 32768 &&
           (long long)p.OH * p.OW < (1LL << 23) && p.B < (1 << 23);
}

ConvDispatch make_conv_dispatch(const ConvProblem &p, const ConvLaunch &l, const TensorView &x, const float *packed,
                                const float *bias, const TensorView &y, float *workspace, const SplitKReduce &reduce,
                                const TensorView *residual, bool post_relu) {
    if (l.variant < 0 || l.variant >= kNumVariants) throw std::runtime_error("conv: bad variant");
    const VariantEntry &e = kVariants[l.variant];
    if (x.C != p.IC || x.H != p.H || x.W != p.W || y.C != p.OC || y.H != p.OH || y.W != p.OW)
        throw std::runtime_error("conv: tensor views do not match the problem");
    if (p.IC % p.groups != 0 || p.OC % p.groups != 0) throw std::runtime_error("conv: channels not divisible by groups");
    if (!conv_matrix_path_supported(p)) throw std::runtime_error("conv: problem too large for the matrix path");
    ConvDispatch d;
    ConvKernelArgs &a = d.args;
    a.x = x.ptr;
    a.wp = packed;
    a.bias = bias;
    a.y = y.ptr;
    a.ws = workspace;
    a.counters = reduce.counters;
    a.H = p.H; a.W = p.W; a.OH = p.OH; a.OW = p.OW;
    a.sh = p.sh; a.sw = p.sw; a.ph = p.ph; a.pw = p.pw;
    a.KW = p.KW;
    a.ICg = p.ICg(); a.ICgP = p.ICgP(e.v.cpad); a.OCg = p.OCg(); a.OCgP = p.OCgP(); a.Kq = p.Kq(e.v.cpad);
    a.magic_icgp = (unsigned)((1ULL << 32) / (unsigned)a.ICgP + 1);   // ICgP >= 8
    a.magic_kw = (unsigned)((1ULL << 32) / (unsigned)a.KW + 1);       // unused when KW == 1
    a.HW = p.H * p.W; a.OHW = p.OH * p.OW; a.groups = p.groups;
    a.x_bs = x.bstride; a.y_bs = y.bstride;
    const unsigned long long x_bytes = ((unsigned long long)(p.B - 1) * x.bstride + (unsigned long long)p.IC * p.H * p.W) * 4ull;
    const unsigned long long w_bytes = (unsigned long long)p.groups * p.Kq(e.v.cpad) * p.OCgP() * (e.v.koct ? 2ull * e.v.koct : e.v.precision != PREC_FP32 ? 2ull : 4ull);
    if (x_bytes >= (1ull << 31) || w_bytes >= (1ull << 31)) throw std::runtime_error("conv: tensor too large for 31-bit buffer offsets");
    a.x_bytes = (unsigned)x_bytes;
    a.w_bytes = (unsigned)w_bytes;
    a.Npix = (int)p.Npix();
    a.act = p.act; a.pre_relu = p.pre_relu;
    a.k_chunk = k_chunk_of(p, l);
    a.split_k = effective_split(p, l);
    {
        // the wave-split kernels' division of a grid slice among the wavefronts of a block (BK = U k-steps, WK wavefronts)
        const int kstep = e.v.MT == 32 ? 2 : 4;
        const int u = std::max(1, e.v.BK / kstep);
        a.steps_total = a.Kq / kstep;
        a.steps_chunk = a.k_chunk / kstep;
        a.steps_per_wave = e.v.kquad ? ceil_div(ceil_div(a.steps_chunk, u), e.v.WK) * u : ceil_div(a.steps_chunk, e.v.WK);
    }
    a.tiles_m = ceil_div(p.OCg(), e.v.BM);
    a.tiles_n = ceil_div(p.Npix(), e.v.BN);
    a.weights_major = (double)p.OC * p.K() > (double)p.B * p.IC * p.H * p.W ? 1 : 0;
    a.tile_div = a.weights_major ? a.tiles_n : a.tiles_m;
    a.xcd_q = (a.tiles_m * a.tiles_n) >> 3;
    a.xcd_r = (a.tiles_m * a.tiles_n) & 7;
    a.div_tile = make_fast_div((unsigned)a.tile_div);
    a.div_ohw = make_fast_div((unsigned)a.OHW);
    a.div_ow = make_fast_div((unsigned)a.OW);
    a.res = nullptr;
    a.res_bs = 0;
    a.post_relu = post_relu ? 1 : 0;
    if (residual != nullptr) {
        if (residual->C != p.OC || residual->H != p.OH || residual->W != p.OW) throw std::runtime_error("conv: residual view does not match the output");
        if ((unsigned long long)(p.B - 1) * residual->bstride + (unsigned long long)p.OC * p.OH * p.OW >= (1ull << 31))
            throw std::runtime_error("conv: residual view too large");
        a.res = residual->ptr;
        a.res_bs = (int)residual->bstride;
    } else if (post_relu) {
        throw std::runtime_error("conv: activation after a residual that is not there");
    }
    if (a.split_k > 1 && workspace == nullptr) throw std::runtime_error("conv: split-K launch without workspace");
    if (p.groups > 65535 || a.split_k > 65535) throw std::runtime_error("conv: grid too large");
    d.variant = l.variant;
    d.threads = e.v.threads();
    d.smem_bytes = e.smem_floats * (int)sizeof(float);
    d.tiles = a.tiles_m * a.tiles_n;
    d.groups = p.groups;
    d.slices = a.split_k;
    if (a.split_k <= 1) a.counters = nullptr;
    // K slices that meet inside an XCD: a one-dimensional grid in the numbering of XcdSlot (plain convolutions without
    // groups; the fields share their place with those of the residual form)
    a.xcd_local = a.counters != nullptr && reduce.xcd_local && reduce.fault != nullptr && p.groups == 1 && residual == nullptr &&
                          a.split_k <= 64 && xcd_grid_blocks(d.tiles, a.split_k) / 8 < (1 << 26)
                      ? 1 : 0;
    d.xcd_blocks = 0;
    if (a.xcd_local) {
        a.fault = reduce.fault;
        a.xcd_map = reduce.xcd_map;
        a.magic_split = (unsigned)((1ULL << 32) / (unsigned)a.split_k + 1);
        d.xcd_blocks = xcd_grid_blocks(d.tiles, a.split_k);
    }
    d.has_reduce = a.split_k > 1 && a.counters == nullptr;
    d.reduce_blocks = 0;
    if (d.has_reduce) {
        ReduceArgs &r = d.reduce;
        r.ws = workspace;
        r.bias = bias;
        r.y = y.ptr;
        r.slices = a.split_k;
        r.OC = p.OC;
        r.Npix = a.Npix;
        r.OHW = a.OHW;
        r.act = p.act;
        r.slice_floats = (long long)p.OC * a.Npix;
        r.y_bs = y.bstride;
        r.res = a.res;
        r.res_bs = a.res_bs;
        r.post_relu = a.post_relu;
        d.reduce_blocks = (int)std::min<long long>((r.slice_floats + 255) / 256, 4096);
    }
    return d;
}

void launch_conv_mfma(const ConvProblem &p, const ConvLaunch &l, const TensorView &x, const float *packed,
                      const float *bias, const TensorView &y, float *workspace, const SplitKReduce &reduce, hipStream_t stream,
                      const TensorView *residual, bool post_relu) {
    const ConvDispatch d = make_conv_dispatch(p, l, x, packed, bias, y, workspace, reduce, residual, post_relu);
    const VariantEntry &e = kVariants[d.variant];
    const dim3 grid = d.xcd_blocks > 0 ? dim3((unsigned)d.xcd_blocks) : dim3((unsigned)d.tiles, (unsigned)d.groups, (unsigned)d.slices);
    const ConvKernelFn kernel = !d.args.xcd_local && d.args.res != nullptr ? e.kernel_residual : e.kernel;
    if (d.smem_bytes > 64 * 1024) {   // beyond the default limit of dynamic LDS: raised once per kernel
        static bool raised[kNumConvVariants][2] = {};
        bool &done = raised[d.variant][kernel == e.kernel_residual ? 1 : 0];
        if (!done) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, d.smem_bytes) != hipSuccess)
                throw std::runtime_error(std::string("conv: cannot reserve LDS for configuration ") + e.v.name);
            done = true;
        }
    }
    hipLaunchKernelGGL(kernel, grid, dim3(d.threads), d.smem_bytes, stream, d.args);
    if (d.has_reduce) hipLaunchKernelGGL(splitk_reduce_kernel, dim3(d.reduce_blocks), dim3(256), 0, stream, d.reduce);
}

// ---- filter packing ------------------------------------------------------------------------
__global__ void pack_filters_kernel(const float *w, float *packed, int OCg, int OCgP, int ICg, int ICgP, int taps, int groups, int kvec,
                                    int precision, int planes) {
    // packed[g][k][m] = w[g * OCg + m][c][tap] with k = tap * ICgP + c;  rows with c >= ICg and columns with m >= OCg are zero.
    // kvec = 4: packed[g][k / 4][m][k % 4] instead (ICgP is a multiple of 4)
    // kvec = 8: planes of bfloat16, packed[g][k / 8][plane][m][k % 8]: three planes with the exact three-term split of every filter
    // value, or one plane with the value rounded to nearest even (the reduced-precision mode)
    const size_t total = (size_t)groups * taps * ICgP * OCgP;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        int m;
        size_t gk;
        if (kvec > 1) {
            const size_t chunk = i / kvec;                       // (g, k / kvec, m)
            m = (int)(chunk % OCgP);
            gk = (chunk / OCgP) * kvec + (i % kvec);             // (g, k)
        } else {
            m = (int)(i % OCgP);
            gk = i / OCgP;
        }
        const int c = (int)(gk % ICgP);
        const size_t gt = gk / ICgP;
        const int tap = (int)(gt % taps);
        const int g = (int)(gt / taps);
        const float value = (m < OCg && c < ICg) ? w[(((size_t)g * OCg + m) * ICg + c) * taps + tap] : 0.f;
        if (kvec == 8) {
            const size_t octet = gk / 8;                         // (g, k / 8)
            const size_t at = (octet * planes * OCgP + m) * 8 + (gk % 8);
            if (planes == 3) {
                unsigned hi, mid, lo;
                split3(value, hi, mid, lo);
                unsigned short *out = reinterpret_cast<unsigned short *>(packed);
                out[at] = (unsigned short)(hi >> 16);
                out[at + (size_t)OCgP * 8] = (unsigned short)(mid >> 16);
                out[at + (size_t)OCgP * 16] = (unsigned short)(lo >> 16);
            } else {
                reinterpret_cast<__bf16 *>(packed)[at] = (__bf16)value;   // round to nearest even
            }
        } else if (precision == PREC_BF16) reinterpret_cast<__bf16 *>(packed)[i] = (__bf16)value;   // round to nearest even
        else if (precision == PREC_FP16) reinterpret_cast<_Float16 *>(packed)[i] = (_Float16)value;   // round to nearest even
        else packed[i] = value;
    }
}

size_t conv_packed_floats(const ConvProblem &p, const ConvLaunch &l) {
    if (l.variant < 0 || l.variant >= kNumVariants) throw std::runtime_error("conv: bad variant");
    const size_t elements = (size_t)p.groups * p.Kq(kVariants[l.variant].v.cpad) * p.OCgP();
    if (kVariants[l.variant].v.koct) return (elements * kVariants[l.variant].v.koct + 1) / 2;   // planes of bfloat16
    return kVariants[l.variant].v.precision != PREC_FP32 ? (elements + 1) / 2 : elements;
}

size_t conv_packed_floats_max(const ConvProblem &p) {
    size_t most = 0;
    for (const VariantEntry &e : kVariants) {
        const size_t elements = (size_t)p.groups * p.Kq(e.v.cpad) * p.OCgP();
        most = std::max(most, e.v.koct ? (elements * e.v.koct + 1) / 2 : elements);
    }
    return most;
}

void launch_pack_filters(const ConvProblem &p, const ConvLaunch &l, const float *w, float *packed, hipStream_t stream) {
    const int cpad = kVariants[l.variant].v.cpad;
    const size_t total = (size_t)p.groups * p.Kq(cpad) * p.OCgP();   // elements
    const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 65535);
    hipLaunchKernelGGL(pack_filters_kernel, dim3(blocks), dim3(256), 0, stream, w, packed, p.OCg(), p.OCgP(), p.ICg(), p.ICgP(cpad),
                       p.KH * p.KW, p.groups, kVariants[l.variant].v.kvec(), kVariants[l.variant].v.precision, kVariants[l.variant].v.koct);
}

}  // namespace ios
