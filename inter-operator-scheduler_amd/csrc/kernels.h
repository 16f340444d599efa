// Device kernels of the runtime and their host-side launchers (gfx950 / CDNA4 only).
//
// All tensors are fp32 NCHW *views*: a base pointer to (n=0, c=0), the extents C/H/W and a batch stride
// in elements.  The channel stride is always H*W, so a channel slice or a window inside a wider concat
// buffer is again a view; producers write straight into such windows and consumers read slices without
// copies.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace ios {

enum Act : int { ACT_NONE = 0, ACT_RELU = 1, ACT_TANH = 2, ACT_SIGMOID = 3 };
enum Precision : int { PREC_FP32 = 0, PREC_BF16 = 1, PREC_FP16 = 2 };   // operand type of the matrix-path convolutions

constexpr int kMaxNaryInputs = 8;   // views one launch adds (or multiplies)

struct TensorView {
    float *ptr = nullptr;  // element (0, 0, 0, 0)
    int C = 0, H = 0, W = 0;
    long long bstride = 0;  // elements between images
};

// ---- convolution ------------------------------------------------------------------------------------
struct ConvProblem {
    int B, IC, H, W, OC, KH, KW, sh, sw, ph, pw, groups;
    int OH, OW;
    int act;       // Act applied after bias
    int pre_relu;  // apply max(x, 0) to the input while loading it
    int ICg() const { return IC / groups; }
    int OCg() const { return OC / groups; }
    int K() const { return ICg() * KH * KW; }
    // rows of the packed filter matrix when the channels of every tap are padded to a multiple of cpad
    int ICgP(int cpad) const { return (ICg() + cpad - 1) / cpad * cpad; }
    int Kq(int cpad) const { return KH * KW * ICgP(cpad); }
    long long Npix() const { return (long long)B * OH * OW; }
    int OCgP() const { return (OCg() + 3) & ~3; }  // row length of the packed filter matrix
    bool is_depthwise() const { return groups > 1 && IC == groups && OC == groups; }
    double flops() const { return 2.0 * (double)Npix() * OC * K(); }
};

// One implicit-GEMM kernel configuration: block tile BM (output channels) x BN (pixels) x BK, a grid of
// WM x WN x WK wavefronts (WK wavefronts split K) built from MT x MT fp32 MFMA tiles.  `wave_split` selects
// the kernel without LDS staging whose WK wavefronts each own a contiguous range of K (of the block's K slice).
struct ConvVariant {
    const char *name;
    int BM, BN, BK, WM, WN, WK, MT;
    bool wave_split;
    int cpad;   // channel padding of the packed filters this configuration reads
    bool kquad; // packed filters are [k / 4][m][4] (16-byte loads along k) instead of [k][m]
    int threads() const { return 64 * WM * WN * WK; }
    bool fusable_;   // light enough on registers to run inside a fused stage launch
    int precision;   // PREC_FP32, or a reduced-precision mode: bfloat16 / IEEE half filters and inputs, fp32 accumulation
    // packed filters as planes of bfloat16, [k / 8][plane][m][8]: 3 = the exact three-term split of fp32 values (fp32 results from
    // the bfloat16 matrix pipe), 1 = one plane rounded to nearest even (the reduced-precision mode on the same kernels), 0 = neither
    int koct = 0;
    // fits a fused stage launch of the wide-register kernel family only (the three-term wave-split configurations)
    bool fusable_wide_ = false;
    bool fusable() const { return fusable_ || fusable_wide_; }
    bool needs_wide() const { return fusable_wide_ && !fusable_; }
    int kvec() const { return koct ? 8 : kquad ? 4 : 1; }   // consecutive k of one output channel that lie together
};

int conv_num_variants();
const ConvVariant &conv_variant(int index);

struct ConvLaunch {
    int variant = 0;
    int split_k = 1;  // number of grid slices along K; > 1 needs workspace
};

// Grid slices along K a launch configuration really uses (split_k may ask for more than there are K tiles).
int conv_effective_split(const ConvProblem &p, const ConvLaunch &l);
// Floats of workspace a launch configuration needs (split_k partial outputs; large enough for both split-K forms).
size_t conv_workspace_floats(const ConvProblem &p, const ConvLaunch &l);
// Ticket counters the one-kernel split-K form needs: one unsigned per (group, output tile), zero before the
// first launch (the kernel leaves them zero); 0 when the configuration does not split K.
size_t conv_counter_count(const ConvProblem &p, const ConvLaunch &l);
// The matrix path indexes packed filter rows with 16 bits and pixels / input offsets with 31 bits.
bool conv_matrix_path_supported(const ConvProblem &p);

// Default configuration from a closed-form occupancy model (num_cus = compute units of the device);
// fusable_only restricts the choice to configurations that can run inside a fused stage launch.
// precision selects the family of configurations (fp32, bfloat16 or half operands).
ConvLaunch conv_pick_launch(const ConvProblem &p, int num_cus, bool fusable_only = false, int precision = PREC_FP32);

// Filter packing for a kernel configuration: w[OC][ICg][KH][KW] -> packed[g][k = (kh*KW + kw)*ICgP + c][OCgP]
// (or [g][k / 4][OCgP][k % 4] for kquad configurations, three bfloat16 planes [g][k / 8][plane][OCgP][k % 8] for koct ones), ICgP = ICg rounded up to the configuration's channel
// padding (zero rows), OCgP = OCg rounded up to 4.  16-bit configurations pack bfloat16 or half (round to nearest even), two
// per float of the returned size.
size_t conv_packed_floats(const ConvProblem &p, const ConvLaunch &l);
size_t conv_packed_floats_max(const ConvProblem &p);   // over all configurations
void launch_pack_filters(const ConvProblem &p, const ConvLaunch &l, const float *w, float *packed, hipStream_t stream);

// How the K slices of a split-K launch meet.  Without `counters` a second kernel adds them on the same stream.  With
// counters (conv_counter_count of them, zero before the first launch) the block that finishes a tile last adds the slices
// inside the kernel; `xcd_local` additionally numbers the grid so that the slices of a tile share an XCD and meet in its L2
// (only for convolutions without groups; others silently use the device-wide form).  All forms add in slice order.
struct SplitKReduce {
    unsigned *counters = nullptr;
    bool xcd_local = false;
    unsigned xcd_map = 0;        // XCC id of the blocks with index % 8 == c, four bits per c (DeviceContext measures it)
    unsigned *fault = nullptr;   // device-visible word in host memory, set to 1 by a block that runs on an unexpected XCC
};

// y = act(conv(x, w) + bias).  `packed` comes from launch_pack_filters.  `workspace` holds the split_k
// partial outputs (conv_workspace_floats).
void launch_conv_mfma(const ConvProblem &p, const ConvLaunch &l, const TensorView &x, const float *packed,
                      const float *bias, const TensorView &y, float *workspace, const SplitKReduce &reduce, hipStream_t stream,
                      const TensorView *residual = nullptr, bool post_relu = false);

// Depth-wise convolution (groups == IC == OC), filters in their original [C][1][KH][KW] layout.  With `more`, the input is
// x + more[0] + ... + more[nmore - 1] (at most kMaxNaryInputs views in all, added left to right before the folded ReLU).
void launch_dwconv(const ConvProblem &p, const TensorView &x, const float *w, const float *bias,
                   const TensorView &y, hipStream_t stream, const TensorView *more = nullptr, int nmore = 0);
bool dwconv_sums_inputs(const ConvProblem &p);   // the kernel for this window can add further inputs in its loader (3 x 3, 5 x 5)

// Direct convolution for any geometry (one thread per output element); used for grouped convolutions
// whose groups are too thin for the matrix path.  `thin` selects the form for 3 x 3 convolutions of 3-channel images
// (conv_thin_applies), which is bound by the bytes of its output and serves first layers at large batches.
inline bool conv_thin_applies(const ConvProblem &p) { return p.groups == 1 && p.IC == 3 && p.KH == 3 && p.KW == 3; }
void launch_conv_direct(const ConvProblem &p, const TensorView &x, const float *w, const float *bias,
                        const TensorView &y, hipStream_t stream, bool thin = false);

// ---- pooling ----------------------------------------------------------------------------------------
struct PoolProblem {
    int B, C, H, W, KH, KW, sh, sw, ph, pw, OH, OW;
    int is_max;  // 1: max over in-range elements, 0: sum of in-range elements / (KH*KW)
};
// With `bias` (one value per channel): y = act(pool(x) + bias[c]).
void launch_pool(const PoolProblem &p, const TensorView &x, const TensorView &y, hipStream_t stream, const float *bias = nullptr,
                 int act = ACT_NONE);
// Window == whole map: one wavefront reduces one (n, c) plane.
void launch_global_pool(const PoolProblem &p, const TensorView &x, const TensorView &y, hipStream_t stream);

// ---- element-wise -----------------------------------------------------------------------------------
struct NaryArgs {
    const float *src[kMaxNaryInputs];
    long long src_bstride[kMaxNaryInputs];
    int count;
};
// y = act(src0 (+|*) src1 (+|*) ...), left to right; more than kMaxNaryInputs inputs are handled by the
// caller through accumulation (accumulate != 0 also combines the current contents of y first).
void launch_nary(const NaryArgs &a, int multiply, int accumulate, int act, int B, long long chw,
                 const TensorView &y, hipStream_t stream);
// y = act(x) for views; act == ACT_NONE is a strided copy.
void launch_unary(const TensorView &x, const TensorView &y, int act, int B, hipStream_t stream);
// Fill n floats with a deterministic pattern in [-1, 1) (seeded), or with a constant.
void launch_fill_pattern(float *dst, size_t n, unsigned seed, hipStream_t stream);
void launch_fill_u32(unsigned *dst, size_t n, unsigned value, hipStream_t stream);

}  // namespace ios
