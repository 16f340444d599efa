// Implicit-GEMM convolution on the CDNA4 fp32 matrix cores.
//
// GEMM view per group:  Y[m][n] = sum_k Wp[k][m] * X_im2col[k][n]
//   m = output channel inside the group (OCg), n = flattened (image, oh, ow) pixel, k = (c, kh, kw).
// The filter matrix is pre-packed k-major (launch_pack_filters) so that a block's BK x BM slice is read
// with 16-byte loads along m.  The BK x BN input slice is gathered straight from the NCHW input view:
// consecutive lanes take consecutive pixels, k is decomposed into (c, kh, kw) with multiply-high
// divisions by launch constants, and padding is resolved by predication.  Global loads run PD tiles
// ahead of the math in registers (the loop is latency bound at batch 1, where a block sees only a few
// K tiles), tiles are staged in LDS (double buffered, one barrier per K tile) and consumed by
// v_mfma_f32_32x32x2_f32 / v_mfma_f32_16x16x4_f32: lane l supplies A[k = l / MT][m = l % MT] and
// B[k = l / MT][n = l % MT].
//
// Parallelism for small problems comes from three places: WK wavefronts of a block split each K tile
// and add their accumulators through LDS at the end; split_k grid slices along K write partial tiles
// to a workspace that a second small kernel sums in slice order (fixed order, so results do not depend
// on scheduling; no device-scope fences inside the main kernel); everything else is M x N tiling.
// The epilogue adds the bias, applies the activation and stores through the output view, i.e. directly
// into the consumer's channel window when the output lives inside a concat buffer.
#include "kernels.h"

#include <algorithm>
#include <stdexcept>
#include <string>

namespace ios {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

struct ConvKernelArgs {
    const float *x;
    const float *wp;
    const float *bias;
    float *y;
    float *ws;
    int H, W, OH, OW, sh, sw, ph, pw;
    int KW, KHKW;
    unsigned magic_khkw, magic_kw;   // floor(2^32 / d) + 1; exact quotients for k < 2^16
    int ICg, OCg, OCgP, K, HW, OHW, groups;
    long long x_bs, y_bs;
    int Npix;
    int act, pre_relu;
    int split_k, k_chunk;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ float apply_act(float v, int act) {
    switch (act) {
        case ACT_RELU: return fmaxf(v, 0.0f);
        case ACT_TANH: return tanhf(v);
        case ACT_SIGMOID: return 1.0f / (1.0f + __expf(-v));
        default: return v;
    }
}

template <int MT>
struct Mfma;

template <>
struct Mfma<32> {
    static constexpr int KSTEP = 2;
    static constexpr int ACC = 16;
    typedef floatx16 acc_t;
    __device__ static __forceinline__ acc_t run(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    // row of accumulator element v held by `lane` inside the 32 x 32 tile; the column is lane % 32
    __device__ static __forceinline__ int row(int v, int lane) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }
};

template <>
struct Mfma<16> {
    static constexpr int KSTEP = 4;
    static constexpr int ACC = 4;
    typedef floatx4 acc_t;
    __device__ static __forceinline__ acc_t run(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ int row(int v, int lane) { return 4 * (lane >> 4) + v; }
};

template <int BM, int BN, int BK, int WM, int WN, int WK, int MT, int PD, bool POINTWISE>
__global__ __launch_bounds__(64 * WM * WN * WK) void conv_mfma_kernel(ConvKernelArgs a) {
    using M = Mfma<MT>;
    constexpr int T = 64 * WM * WN * WK;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / MT, TN = WTN / MT;
    constexpr int KSLICE = BK / WK;
    constexpr int PAD = MT == 16 ? 16 : 4;   // MT 16 reads four rows per instruction: rows must not share banks
    constexpr int LDA = BM + PAD, LDB = BN + PAD;
    constexpr int A_VEC_PER_ROW = BM / 4;
    constexpr int A_SLOTS = BK * A_VEC_PER_ROW;
    constexpr int A_ITERS = (A_SLOTS + T - 1) / T;
    constexpr int B_ROWS_PER_PASS = T / BN;
    constexpr int B_ITERS = BK / B_ROWS_PER_PASS;
    static_assert(WTM % MT == 0 && WTN % MT == 0, "wave tile must be a multiple of the MFMA tile");
    static_assert(KSLICE % M::KSTEP == 0, "K slice per wavefront must be a multiple of the MFMA depth");
    static_assert(T % BN == 0 && BK % B_ROWS_PER_PASS == 0, "input loader shape");
    constexpr int TILE_FLOATS = 2 * BK * (LDA + LDB);
    constexpr int RED_FLOATS = (WK - 1) * BM * BN;
    constexpr int SMEM_FLOATS = TILE_FLOATS > RED_FLOATS ? TILE_FLOATS : RED_FLOATS;
    __shared__ __attribute__((aligned(16))) float smem[SMEM_FLOATS];
    float *As = smem;                  // [2][BK][LDA]
    float *Bs = smem + 2 * BK * LDA;   // [2][BK][LDB]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave % WN;
    const int wm = (wave / WN) % WM;
    const int wk = wave / (WN * WM);

    const int tile = blockIdx.x;
    const int tm = tile % a.tiles_m;
    const int tn = tile / a.tiles_m;
    const int g = blockIdx.y;
    const int z = blockIdx.z;
    const int m0 = tm * BM;
    const int n0 = tn * BN;
    const int k_begin = z * a.k_chunk;
    const int k_end = min(a.K, k_begin + a.k_chunk);
    const int nkt = (k_end - k_begin + BK - 1) / BK;

    // ---- per-thread loader state ---------------------------------------------------------------------
    const int bn_l = tid % BN;
    const int bk_l = tid / BN;
    const int n = n0 + bn_l;
    const bool n_ok = n < a.Npix;
    int ih0 = 0, iw0 = 0;
    long long x_off = 0;
    {
        const int nn = n_ok ? n : 0;
        const int b = nn / a.OHW;
        const int r = nn - b * a.OHW;
        const int oh = r / a.OW;
        const int ow = r - oh * a.OW;
        ih0 = oh * a.sh - a.ph;
        iw0 = ow * a.sw - a.pw;
        x_off = (long long)b * a.x_bs + (long long)g * a.ICg * a.HW + (long long)ih0 * a.W + iw0;
    }
    const float *xg = a.x + x_off;
    const float *wg = a.wp + (size_t)g * a.K * a.OCgP;

    floatx4 a_reg[PD][A_ITERS];
    float b_reg[PD][B_ITERS];

    auto load_tile = [&](int kt, floatx4(&ar)[A_ITERS], float(&br)[B_ITERS]) {
        const int k0 = k_begin + kt * BK;
#pragma unroll
        for (int i = 0; i < A_ITERS; i++) {
            const int slot = tid + i * T;
            const int row = slot / A_VEC_PER_ROW;
            const int c4 = slot % A_VEC_PER_ROW;
            const int k = k0 + row;
            const int m = m0 + c4 * 4;
            floatx4 v = {0.f, 0.f, 0.f, 0.f};
            if ((A_SLOTS % T == 0 || slot < A_SLOTS) && k < k_end && m < a.OCgP)
                v = *reinterpret_cast<const floatx4 *>(wg + (size_t)k * a.OCgP + m);
            ar[i] = v;
        }
#pragma unroll
        for (int i = 0; i < B_ITERS; i++) {
            const int k = k0 + bk_l + i * B_ROWS_PER_PASS;
            float v = 0.f;
            if (k < k_end && n_ok) {
                if (POINTWISE) {
                    v = xg[(long long)k * a.HW];
                } else {
                    const int c = a.KHKW == 1 ? k : (int)__umulhi((unsigned)k, a.magic_khkw);
                    const int rem = k - c * a.KHKW;
                    const int kh = a.KW == 1 ? rem : (int)__umulhi((unsigned)rem, a.magic_kw);
                    const int kw = rem - kh * a.KW;
                    if ((unsigned)(ih0 + kh) < (unsigned)a.H && (unsigned)(iw0 + kw) < (unsigned)a.W)
                        v = xg[(long long)c * a.HW + kh * a.W + kw];
                }
            }
            br[i] = v;
        }
    };

    auto store_tile = [&](int buf, const floatx4(&ar)[A_ITERS], const float(&br)[B_ITERS]) {
        float *Ab = As + buf * BK * LDA;
        float *Bb = Bs + buf * BK * LDB;
#pragma unroll
        for (int i = 0; i < A_ITERS; i++) {
            const int slot = tid + i * T;
            if (A_SLOTS % T == 0 || slot < A_SLOTS) {
                const int row = slot / A_VEC_PER_ROW;
                const int c4 = slot % A_VEC_PER_ROW;
                *reinterpret_cast<floatx4 *>(Ab + row * LDA + c4 * 4) = ar[i];
            }
        }
#pragma unroll
        for (int i = 0; i < B_ITERS; i++) {
            float v = br[i];
            if (a.pre_relu) v = fmaxf(v, 0.f);
            Bb[(bk_l + i * B_ROWS_PER_PASS) * LDB + bn_l] = v;
        }
    };

    typename M::acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < M::ACC; v++) acc[i][j][v] = 0.f;

    // ---- main loop: global -> registers (PD tiles ahead) -> LDS (double buffered) -> MFMA -----------------
    // Register stage s holds tile kt with kt % PD == s.  In iteration kt the stage of tile kt is free (the
    // tile already sits in LDS buffer kt & 1), so it is refilled with tile kt + PD; the stage of tile kt + 1,
    // requested PD - 1 iterations ago, is written to the other LDS buffer after the math.
#pragma unroll
    for (int s = 0; s < PD; s++)
        if (s < nkt) load_tile(s, a_reg[s], b_reg[s]);
    if (nkt > 0) store_tile(0, a_reg[0], b_reg[0]);
    __syncthreads();
    const int lk = lane / MT;   // k offset of this lane inside an MFMA step
    const int lc = lane % MT;   // row (A) / column (B) of this lane inside an MFMA tile
    for (int kt0 = 0; kt0 < nkt; kt0 += PD) {
#pragma unroll
        for (int s = 0; s < PD; s++) {
            const int kt = kt0 + s;
            if (kt >= nkt) break;
            const int buf = kt & 1;
            if (kt + PD < nkt) load_tile(kt + PD, a_reg[s], b_reg[s]);
            const float *Ab = As + buf * BK * LDA + (wk * KSLICE + lk) * LDA + wm * WTM + lc;
            const float *Bb = Bs + buf * BK * LDB + (wk * KSLICE + lk) * LDB + wn * WTN + lc;
#pragma unroll
            for (int kk = 0; kk < KSLICE; kk += M::KSTEP) {
                float av[TM], bv[TN];
#pragma unroll
                for (int i = 0; i < TM; i++) av[i] = Ab[kk * LDA + i * MT];
#pragma unroll
                for (int j = 0; j < TN; j++) bv[j] = Bb[kk * LDB + j * MT];
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] = M::run(av[i], bv[j], acc[i][j]);
            }
            if (kt + 1 < nkt) store_tile(buf ^ 1, a_reg[(s + 1) % PD], b_reg[(s + 1) % PD]);
            __syncthreads();
        }
    }

    // ---- fold the WK wavefronts that worked on the same output tile -------------------------------------------
    if (WK > 1) {
        constexpr int PER_WAVE = TM * TN * M::ACC;        // accumulator floats per lane
        constexpr int MN_WAVES = WM * WN;
        float *red = smem;                                // [(WK-1)][PER_WAVE][MN_WAVES * 64]
        const int slot = (wm * WN + wn) * 64 + lane;
        if (wk > 0) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int v = 0; v < M::ACC; v++)
                        red[((size_t)(wk - 1) * PER_WAVE + (i * TN + j) * M::ACC + v) * (MN_WAVES * 64) + slot] =
                            acc[i][j][v];
        }
        __syncthreads();
        if (wk == 0) {
            for (int s = 0; s < WK - 1; s++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int v = 0; v < M::ACC; v++)
                            acc[i][j][v] += red[((size_t)s * PER_WAVE + (i * TN + j) * M::ACC + v) * (MN_WAVES * 64) + slot];
        }
    }

    // ---- epilogue -------------------------------------------------------------------------------------------
    if (a.split_k == 1) {
        if (wk == 0) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int nn = n0 + wn * WTN + j * MT + lc;
                if (nn >= a.Npix) continue;
                const int b = nn / a.OHW;
                const int r = nn - b * a.OHW;
                float *yb = a.y + (long long)b * a.y_bs + (long long)g * a.OCg * a.OHW + r;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int v = 0; v < M::ACC; v++) {
                        const int m = m0 + wm * WTM + i * MT + M::row(v, lane);
                        if (m < a.OCg) yb[(long long)m * a.OHW] = apply_act(acc[i][j][v] + a.bias[g * a.OCg + m], a.act);
                    }
            }
        }
        return;
    }

    // split-K: store this slice's partial tile; splitk_reduce_kernel adds the slices, bias and activation
    float *wsz = a.ws + ((size_t)z * a.groups + g) * a.OCg * (size_t)a.Npix;
    if (wk == 0) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int nn = n0 + wn * WTN + j * MT + lc;
            if (nn >= a.Npix) continue;
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int v = 0; v < M::ACC; v++) {
                    const int m = m0 + wm * WTM + i * MT + M::row(v, lane);
                    if (m < a.OCg) wsz[(size_t)m * a.Npix + nn] = acc[i][j][v];
                }
        }
    }
}

// y[b][oc][r] = act(bias[oc] + sum_s ws[s][oc][n]),  n = b * OHW + r; slices are added in index order
__global__ void splitk_reduce_kernel(const float *ws, const float *bias, float *y, int slices, long long slice_floats, int OC,
                                     int Npix, int OHW, long long y_bs, int act) {
    const long long total = (long long)OC * Npix;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        const int oc = (int)(i / Npix);
        const int n = (int)(i - (long long)oc * Npix);
        float sum = 0.f;
        for (int s = 0; s < slices; s++) sum += ws[s * slice_floats + i];
        const int b = n / OHW;
        const int r = n - b * OHW;
        y[b * y_bs + (long long)oc * OHW + r] = apply_act(sum + bias[oc], act);
    }
}

// ---- variant table --------------------------------------------------------------------------------------------
typedef void (*ConvKernelFn)(ConvKernelArgs);

struct VariantEntry {
    ConvVariant v;
    ConvKernelFn general;
    ConvKernelFn pointwise;
};

#define IOS_CONV_VARIANT(NAME, BM, BN, BK, WM, WN, WK, MT, PD)                                        \
    {                                                                                                 \
        {NAME, BM, BN, BK, WM, WN, WK, MT}, conv_mfma_kernel<BM, BN, BK, WM, WN, WK, MT, PD, false>, \
            conv_mfma_kernel<BM, BN, BK, WM, WN, WK, MT, PD, true>                                   \
    }

static const VariantEntry kVariants[] = {
    IOS_CONV_VARIANT("m64n64k32_w2x2x1_t32", 64, 64, 32, 2, 2, 1, 32, 3),
    IOS_CONV_VARIANT("m128n128k16_w2x2x1_t32", 128, 128, 16, 2, 2, 1, 32, 3),
    IOS_CONV_VARIANT("m32n32k64_w1x1x4_t32", 32, 32, 64, 1, 1, 4, 32, 4),
    IOS_CONV_VARIANT("m64n32k32_w2x1x2_t32", 64, 32, 32, 2, 1, 2, 32, 4),
    IOS_CONV_VARIANT("m32n64k32_w1x2x2_t32", 32, 64, 32, 1, 2, 2, 32, 4),
    IOS_CONV_VARIANT("m128n64k16_w2x2x1_t32", 128, 64, 16, 2, 2, 1, 32, 3),
    IOS_CONV_VARIANT("m64n16k64_w4x1x1_t16", 64, 16, 64, 4, 1, 1, 16, 3),
    IOS_CONV_VARIANT("m32n16k64_w2x1x2_t16", 32, 16, 64, 2, 1, 2, 16, 4),
    IOS_CONV_VARIANT("m16n16k128_w1x1x4_t16", 16, 16, 128, 1, 1, 4, 16, 3),
    IOS_CONV_VARIANT("m32n32k128_w1x1x8_t32", 32, 32, 128, 1, 1, 8, 32, 3),
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

int conv_num_variants() { return kNumVariants; }

const ConvVariant &conv_variant(int index) {
    if (index < 0 || index >= kNumVariants) throw std::runtime_error("conv variant index out of range");
    return kVariants[index].v;
}

static int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

static int k_chunk_of(const ConvProblem &p, const ConvLaunch &l) {
    const int BK = kVariants[l.variant].v.BK;
    const int tiles_k = ceil_div(p.K(), BK);
    return ceil_div(tiles_k, l.split_k) * BK;
}

// split_k may ask for more slices than there are K tiles; the effective count leaves no slice empty
static int effective_split(const ConvProblem &p, const ConvLaunch &l) {
    return std::max(1, ceil_div(p.K(), k_chunk_of(p, l)));
}

size_t conv_workspace_floats(const ConvProblem &p, const ConvLaunch &l) {
    const int s = effective_split(p, l);
    return s > 1 ? (size_t)s * p.OC * (size_t)p.Npix() : 0;
}

ConvLaunch conv_pick_launch(const ConvProblem &p, int num_cus) {
    // Occupancy model: a launch should offer about two blocks per compute unit.  Prefer the largest tile
    // that still does so without splitting K; otherwise take a small tile, sized to the pixel count, and
    // split K, keeping at least two K tiles per slice.
    const long long M = p.OCg(), N = p.Npix();
    const long long want = 2LL * num_cus;
    static const int by_size[] = {1, 5, 0, 3, 4, 2, 7};   // large to small tiles
    ConvLaunch best;
    for (int idx : by_size) {
        const ConvVariant &v = kVariants[idx].v;
        const long long blocks = (long long)ceil_div(M, v.BM) * ceil_div(N, v.BN) * p.groups;
        if (blocks >= want) {
            best.variant = idx;
            best.split_k = 1;
            return best;
        }
    }
    const int pick = 7;   // 32 x 16 tile, four wavefronts
    const ConvVariant &v = kVariants[pick].v;
    const long long blocks = (long long)ceil_div(M, v.BM) * ceil_div(N, v.BN) * p.groups;
    const int tiles_k = ceil_div(p.K(), v.BK);
    int split = (int)std::min<long long>((want + blocks - 1) / blocks, std::max(1, tiles_k / 2));
    best.variant = pick;
    best.split_k = std::max(1, std::min(split, 32));
    return best;
}

bool conv_matrix_path_supported(const ConvProblem &p) {
    return p.K() < 65536 && p.Npix() < (1LL << 31) && (long long)p.IC * p.H * p.W < (1LL << 31);
}

void launch_conv_mfma(const ConvProblem &p, const ConvLaunch &l, const TensorView &x, const float *packed,
                      const float *bias, const TensorView &y, float *workspace, hipStream_t stream) {
    if (l.variant < 0 || l.variant >= kNumVariants) throw std::runtime_error("conv: bad variant");
    const VariantEntry &e = kVariants[l.variant];
    if (x.C != p.IC || x.H != p.H || x.W != p.W || y.C != p.OC || y.H != p.OH || y.W != p.OW)
        throw std::runtime_error("conv: tensor views do not match the problem");
    if (p.IC % p.groups != 0 || p.OC % p.groups != 0) throw std::runtime_error("conv: channels not divisible by groups");
    if (!conv_matrix_path_supported(p)) throw std::runtime_error("conv: problem too large for the matrix path");
    ConvKernelArgs a;
    a.x = x.ptr;
    a.wp = packed;
    a.bias = bias;
    a.y = y.ptr;
    a.ws = workspace;
    a.H = p.H; a.W = p.W; a.OH = p.OH; a.OW = p.OW;
    a.sh = p.sh; a.sw = p.sw; a.ph = p.ph; a.pw = p.pw;
    a.KW = p.KW; a.KHKW = p.KH * p.KW;
    a.magic_khkw = (unsigned)((1ULL << 32) / (unsigned)a.KHKW + 1);   // unused when the divisor is 1
    a.magic_kw = (unsigned)((1ULL << 32) / (unsigned)a.KW + 1);
    a.ICg = p.ICg(); a.OCg = p.OCg(); a.OCgP = p.OCgP(); a.K = p.K();
    a.HW = p.H * p.W; a.OHW = p.OH * p.OW; a.groups = p.groups;
    a.x_bs = x.bstride; a.y_bs = y.bstride;
    a.Npix = (int)p.Npix();
    a.act = p.act; a.pre_relu = p.pre_relu;
    a.k_chunk = k_chunk_of(p, l);
    a.split_k = effective_split(p, l);
    a.tiles_m = ceil_div(p.OCg(), e.v.BM);
    a.tiles_n = ceil_div(p.Npix(), e.v.BN);
    if (a.split_k > 1 && workspace == nullptr) throw std::runtime_error("conv: split-K launch without workspace");
    dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)p.groups, (unsigned)a.split_k);
    if (grid.y > 65535 || grid.z > 65535) throw std::runtime_error("conv: grid too large");
    ConvKernelFn fn = (p.is_pointwise() ? e.pointwise : e.general);
    hipLaunchKernelGGL(fn, grid, dim3(e.v.threads()), 0, stream, a);
    if (a.split_k > 1) {
        const long long total = (long long)p.OC * a.Npix;
        const unsigned blocks = (unsigned)std::min<long long>((total + 255) / 256, 4096);
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, stream, (const float *)workspace, bias, y.ptr,
                           a.split_k, total, p.OC, a.Npix, a.OHW, (long long)y.bstride, p.act);
    }
}

// ---- filter packing ------------------------------------------------------------------------
__global__ void pack_filters_kernel(const float *w, float *packed, int OCg, int OCgP, int K, int groups) {
    // packed[g][k][m] = w[g*OCg + m][k]   (k runs over (c, kh, kw) exactly as in the original layout)
    const size_t total = (size_t)groups * K * OCgP;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int m = (int)(i % OCgP);
        const size_t gk = i / OCgP;
        const int k = (int)(gk % K);
        const int g = (int)(gk / K);
        packed[i] = m < OCg ? w[((size_t)g * OCg + m) * K + k] : 0.f;
    }
}

size_t conv_packed_floats(const ConvProblem &p) { return (size_t)p.groups * p.K() * p.OCgP(); }

void launch_pack_filters(const ConvProblem &p, const float *w, float *packed, hipStream_t stream) {
    const size_t total = conv_packed_floats(p);
    const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 65535);
    hipLaunchKernelGGL(pack_filters_kernel, dim3(blocks), dim3(256), 0, stream, w, packed, p.OCg(), p.OCgP(), p.K(),
                       p.groups);
}

}  // namespace ios
