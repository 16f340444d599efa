// Device-side bodies of the convolution kernels; included by the translation units that instantiate them
// (the stand-alone kernels and the fused stage kernel).
//
// Implicit-GEMM convolution on the CDNA4 fp32 matrix cores, in two forms: ConvTiled stages operand tiles in LDS
// (large problems), ConvWsplit feeds the matrix cores straight from global memory and divides K among the
// wavefronts of a block (small and medium problems, and the bfloat16 mode).  This comment describes ConvTiled;
// ConvWsplit is described at its definition.
//
// GEMM view per group:  Y[m][n] = sum_k Wp[k][m] * X_im2col[k][n]
//   m = output channel inside the group (OCg), n = flattened (image, oh, ow) pixel,
//   k = (kh, kw, c) tap-major with the channels of every tap zero-padded to a multiple of the K tile.
// The filter matrix is pre-packed k-major (launch_pack_filters) so that a block's BK x BM slice is read
// with 16-byte loads along m.  The BK x BN input slice is gathered straight from the NCHW input view:
// consecutive lanes take consecutive pixels; because a K tile lies inside one filter tap, the tap's
// (kh, kw), its padding test and its base offset are computed once per tile and an element costs one
// address add (with k = (c, kh, kw) the gather spent ~17 VALU instructions per MFMA).  Global loads run PD tiles
// ahead of the math in registers (the loop is latency bound at batch 1, where a block sees only a few
// K tiles), tiles are staged in LDS (double buffered, one barrier per K tile) and consumed by
// v_mfma_f32_32x32x2_f32 / v_mfma_f32_16x16x4_f32: lane l supplies A[k = l / MT][m = l % MT] and
// B[k = l / MT][n = l % MT].
//
// Parallelism for small problems comes from three places: WK wavefronts of a block split each K tile
// and add their accumulators through LDS at the end; split_k grid slices along K write partial tiles
// to a workspace, and the block that finishes a tile last (or a second small kernel) sums them in slice
// order (fixed order, so results do not depend on scheduling; no device-scope fences, which would write
// back and invalidate whole L2s); everything else is M x N tiling.
// The epilogue adds the bias, applies the activation and stores through the output view, i.e. directly
// into the consumer's channel window when the output lives inside a concat buffer.
#pragma once

#include "kernels.h"

#include <type_traits>

namespace ios {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// Division of a 32-bit unsigned by a divisor fixed at launch time (Granlund-Montgomery): exact for every dividend,
// five instructions instead of the ~20 of a hardware-less integer division.
struct FastDiv {
    unsigned m, s1, s2;
};

inline FastDiv make_fast_div(unsigned d) {   // d >= 1
    unsigned l = 0;
    while ((1ull << l) < d) l++;   // ceil(log2(d))
    FastDiv f;
    f.m = (unsigned)((((1ull << l) - d) << 32) / d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 0 ? l - 1 : 0;
    return f;
}

__device__ __forceinline__ unsigned fast_div(unsigned n, const FastDiv &f) {
    const unsigned t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

struct ConvKernelArgs {
    const float *x;
    const float *wp;
    const float *bias;
    float *y;
    float *ws;
    unsigned *counters;               // split-K tickets, one per (group, tile), zero between launches; null: two-kernel split-K
    int H, W, OH, OW, sh, sw, ph, pw;
    int KW;
    int xcd_local;                    // split-K inside one XCD, see below
    unsigned magic_icgp, magic_kw;    // floor(2^32 / d) + 1: exact quotients for dividends < 2^16
    int ICg, ICgP, OCg, OCgP, Kq, HW, OHW, groups;   // Kq = taps * ICgP rows of the packed filter matrix
    long long x_bs, y_bs;
    unsigned x_bytes, w_bytes;        // extents of the input view and of the packed filters, both < 2^31
    int Npix;
    int act, pre_relu;
    int split_k, k_chunk;
    int steps_total, steps_chunk, steps_per_wave;   // wave-split kernels: MFMA k-steps in K, in a grid slice, in a wavefront's share of a full slice
    int tiles_m, tiles_n;
    int weights_major;   // 1: consecutive tiles share filter rows (filters larger than the input), 0: share pixels
    int xcd_q, xcd_r;    // tiles_m * tiles_n = 8 * xcd_q + xcd_r
    int tile_div;        // tiles_n (weights_major) or tiles_m
    FastDiv div_tile;    // by tile_div
    FastDiv div_ohw, div_ow;
    // Either the residual form (stand-alone kernels only): y = res + act(conv + bias), then max(., 0) when post_relu; res is a
    // dense view of the output's shape (batch stride res_bs elements), null for a plain convolution.
    // Or split-K inside one XCD (xcd_local != 0; plain convolutions without groups, counters set): the grid is numbered so
    // that all K slices of an output tile run on the same XCD and meet in that XCD's L2 (see XcdSlot).  xcd_map: the XCC id
    // that blocks with index % 8 == c run on, four bits per c, as measured when the device context was created; fault: a
    // word in host memory that a block finding itself elsewhere sets to 1 (the host then stops using this form);
    // magic_split = floor(2^32 / split_k) + 1: exact quotients by split_k for dividends below 2^26.
    union {
        struct {
            const float *res;
            int res_bs, post_relu;
        };
        struct {
            unsigned *fault;
            unsigned xcd_map, magic_split;
        };
    };
};

// Numbering of the blocks of a launch whose K slices meet inside one XCD.  The dispatcher deals workgroups to the XCDs
// round-robin, so the blocks with index % 8 == c share an XCD.  Class c owns the tiles [c * q + min(c, r), ...) (q + 1 of
// them for c < r, q for the others, where tiles = 8 q + r, the same ranges xcd_tile() uses) and its blocks, in index order,
// are (first tile, slice 0), (first tile, slice 1), ... : a launch has 8 * split * (q + (r > 0)) blocks, of which the last
// ones of the classes c >= r (when r > 0) have no tile and end at once.  `tile` is the value xcd_tile() takes
// (slot-in-class * 8 + c), which also numbers the tile's partial sums and its ticket: those arrays have
// 8 * (q + (r > 0)) entries.
struct XcdSlot {
    int tile, slice;
    bool idle;
};
__host__ __device__ inline int xcd_padded_tiles(int tiles) { return 8 * ((tiles + 7) / 8); }
__host__ __device__ inline int xcd_grid_blocks(int tiles, int split) { return xcd_padded_tiles(tiles) * split; }
__host__ __device__ inline XcdSlot xcd_slot(int local, int tile_in_class, int xcd_q, int xcd_r, int split) {
    // local: index of the block inside the launch (or inside its item of a fused launch); tile_in_class = (local / 8) / split
    const int c = local & 7;
    XcdSlot s;
    s.slice = (local >> 3) - tile_in_class * split;
    s.tile = tile_in_class * 8 + c;
    s.idle = tile_in_class >= xcd_q + (c < xcd_r ? 1 : 0);
    return s;
}

// XCC id of the executing wavefront (bits 3:0 of the hardware register XCC_ID)
__device__ __forceinline__ unsigned xcc_id() { return __builtin_amdgcn_s_getreg(20 | (3 << 11)); }

// One block of an XCD-local split-K launch: its slot, and the check that the dispatcher put it where the numbering assumes.
// `block` is the block's index in the whole launch (the XCD follows from it), `local` its index inside the convolution.
__device__ __forceinline__ XcdSlot xcd_enter(const ConvKernelArgs &a, int block, int local) {
    const XcdSlot s = xcd_slot(local, (int)__umulhi((unsigned)local >> 3, a.magic_split), a.xcd_q, a.xcd_r, a.split_k);
    const unsigned expected = (a.xcd_map >> (4 * (block & 7))) & 15u;
    if (xcc_id() != expected && threadIdx.x == 0) __hip_atomic_store(a.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    return s;
}

// Partial sums and tickets of the one-kernel split-K.  Device-wide form: the slices of a tile run on different XCDs, whose
// L2s are not coherent with each other, so partial sums travel with agent-scope stores and loads (written through to and
// read from memory) and the ticket is an agent-scope atomic.  XCD-local form: all slices share one L2; plain stores are
// written through the L1 to that L2, the ticket is a workgroup-scope atomic (executed in the L2), and the sums are read
// with workgroup-scope loads, which do not use a line the L1 might hold.  In both forms a block waits for its stores to
// be acknowledged before it takes its ticket.
template <bool LOCAL>
__device__ __forceinline__ void partial_store(float *p, float v) {
    if constexpr (LOCAL) *p = v;
    else __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool LOCAL>
__device__ __forceinline__ float partial_load(const float *p) {
    if constexpr (LOCAL) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    else return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// thread 0 of the block: draws the tile's ticket; the block that draws the last one puts the counter back to zero
template <bool LOCAL>
__device__ __forceinline__ int draw_ticket(unsigned *counter, int split_k) {
    unsigned ticket;
    if constexpr (LOCAL) ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    else ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = ticket == (unsigned)split_k - 1u ? 1 : 0;
    if (last) {
        if constexpr (LOCAL) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return last;
}

// v = act(conv + bias) of output element (image b, channel, pixel r): adds the residual operand.  The residual form is a
// compile-time property of a body (RES): the plain form, which every fused stage launch uses, carries no test for it.
template <bool RES>
__device__ __forceinline__ float add_residual(const ConvKernelArgs &a, float v, int b, int channel, int r) {
    if constexpr (RES) {
        v += a.res[(long long)b * a.res_bs + (long long)channel * a.OHW + r];
        if (a.post_relu) v = fmaxf(v, 0.0f);
    }
    return v;
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Tiles are renumbered so that an XCD
// receives a contiguous range of them, and the range runs along the operand that is cheaper to duplicate: the
// more expensive operand (filters at batch 1, activations at large batch) is then fetched into one L2 only.
__device__ __forceinline__ void xcd_tile(const ConvKernelArgs &a, int block, int &tm, int &tn) {
    // XCD x owns tiles [x * q + min(x, r), ...): q + 1 tiles for the first r XCDs, q for the others
    const int xcd = block & 7, slot = block >> 3;
    const int t = slot + xcd * a.xcd_q + min(xcd, a.xcd_r);
    const int q2 = (int)fast_div((unsigned)t, a.div_tile);
    const int rest = t - q2 * a.tile_div;
    tm = a.weights_major ? q2 : rest;
    tn = a.weights_major ? rest : q2;
}

__device__ __forceinline__ float apply_act(float v, int act) {
    switch (act) {
        case ACT_RELU: return fmaxf(v, 0.0f);
        case ACT_TANH: return tanhf(v);
        case ACT_SIGMOID: return 1.0f / (1.0f + __expf(-v));
        default: return v;
    }
}

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

// Raw buffer loads: a 32-bit byte offset against a base + extent descriptor; offsets at or beyond the extent
// read as zero, so an invalid element (padding, channel padding, tile overhang) is a load from kOutOfRange
// and no branch or select on the loaded value is needed.
constexpr unsigned kOutOfRange = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const float *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, bytes, 0x00020000);
}
// `scalar_offset` must be wavefront-uniform; it is added to the address after the range check of `byte_offset`.
__device__ __forceinline__ float buffer_load_f32(__amdgpu_buffer_rsrc_t r, unsigned byte_offset, unsigned scalar_offset = 0) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, byte_offset, scalar_offset, 0));
}
__device__ __forceinline__ floatx4 buffer_load_f32x4(__amdgpu_buffer_rsrc_t r, unsigned byte_offset, unsigned scalar_offset = 0) {
    const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, scalar_offset, 0);
    floatx4 f = {__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w)};
    return f;
}

typedef unsigned int uintx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uintx2 buffer_load_u32x2(__amdgpu_buffer_rsrc_t r, unsigned byte_offset, unsigned scalar_offset = 0) {
    return __builtin_amdgcn_raw_buffer_load_b64(r, byte_offset, scalar_offset, 0);
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

// Tail of the LDS-tiled kernels once a block holds its accumulators (wavefronts with wk == 0; the others only take part in the
// barriers): the split-K exchange in its three forms, then bias, activation and the store through the output view.
template <int MT, int BM, int BN, int TM, int TN, int WM, int WN, bool RES>
__device__ __forceinline__ void tiled_tail(const ConvKernelArgs &a, float *smem, typename Mfma<MT>::acc_t (&acc)[TM][TN], int tile, int g, int z,
                                           int m0, int n0, int wm, int wn, int wk) {
    using M = Mfma<MT>;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int lc = lane % MT;
    // ---- split-K ----------------------------------------------------------------------------------------------
    if (a.split_k > 1) {
        if (a.counters == nullptr) {
            // two-kernel form: store this slice's partial tile; splitk_reduce_kernel adds the slices, bias and activation
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
            return;
        }
        // one-kernel form: every slice stores its partial tile in accumulator layout ([element][thread], so a
        // wavefront writes 256 contiguous bytes), then takes a ticket on the tile's counter; the block that
        // draws the last ticket adds all slices in slice order (its own included, so the sum does not depend
        // on which block came last) and runs the epilogue.  Partials and tickets move with device-scope
        // atomics, which are coherent across the per-XCD L2s without cache-wide write-backs or invalidations;
        // the wait on the outstanding stores before the barrier orders a block's partials before its ticket.
        constexpr int T0 = 64 * WM * WN;
        constexpr int E = TM * TN * M::ACC;
        static_assert(T0 * E == BM * BN, "accumulator layout covers the tile");
        const size_t tiles = (size_t)xcd_padded_tiles(a.tiles_m * a.tiles_n);   // (both forms size their arrays for the padded count)
        float *slices = a.ws + (((size_t)g * tiles + tile) * a.split_k) * (size_t)(BM * BN);
        unsigned *counter = a.counters + (size_t)g * tiles + tile;
        int *last_flag = reinterpret_cast<int *>(smem);
        auto exchange = [&](auto local) -> bool {   // true: this block drew the last ticket and holds the sum of all slices
            constexpr bool LOCAL = decltype(local)::value;
            if (wk == 0) {
                float *mine = slices + (size_t)z * (BM * BN) + tid;
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int v = 0; v < M::ACC; v++) partial_store<LOCAL>(mine + ((i * TN + j) * M::ACC + v) * T0, acc[i][j][v]);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) *last_flag = draw_ticket<LOCAL>(counter, a.split_k);
            __syncthreads();
            if (*last_flag == 0) return false;
            if (wk == 0) {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
#pragma unroll
                        for (int v = 0; v < M::ACC; v++) acc[i][j][v] = 0.f;
                for (int s = 0; s < a.split_k; s++) {
                    const float *theirs = slices + (size_t)s * (BM * BN) + tid;
#pragma unroll
                    for (int i = 0; i < TM; i++)
#pragma unroll
                        for (int j = 0; j < TN; j++)
#pragma unroll
                            for (int v = 0; v < M::ACC; v++) acc[i][j][v] += partial_load<LOCAL>(theirs + ((i * TN + j) * M::ACC + v) * T0);
                }
            }
            return true;
        };
        const bool last = a.xcd_local ? exchange(std::true_type{}) : exchange(std::false_type{});
        if (!last) return;
    }

    // ---- epilogue -------------------------------------------------------------------------------------------
    if (wk == 0) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int nn = n0 + wn * WTN + j * MT + lc;
            if (nn >= a.Npix) continue;
            const int b = (int)fast_div((unsigned)nn, a.div_ohw);
            const int r = nn - b * a.OHW;
            float *yb = a.y + (long long)b * a.y_bs + (long long)g * a.OCg * a.OHW + r;
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int v = 0; v < M::ACC; v++) {
                    const int m = m0 + wm * WTM + i * MT + M::row(v, lane);
                    if (m < a.OCg)
                        yb[(long long)m * a.OHW] = add_residual<RES>(a, apply_act(acc[i][j][v] + a.bias[g * a.OCg + m], a.act), b, g * a.OCg + m, r);
                }
        }
    }
}

template <int BM, int BN, int BK, int WM, int WN, int WK, int MT, int PD>
struct ConvTiled {
    using M = Mfma<MT>;
    static constexpr int T = 64 * WM * WN * WK;
    static constexpr int THREADS = T;
    static constexpr int CPAD = BK;   // channel padding of the packed filters: a K tile never straddles two taps
    static constexpr int PAD = MT == 16 ? 16 : 4;   // MT 16 reads four rows per instruction: rows must not share banks
    static constexpr int LDA = BM + PAD, LDB = BN + PAD;
    static constexpr int TILE_FLOATS = 2 * BK * (LDA + LDB);
    static constexpr int RED_FLOATS = (WK - 1) * BM * BN;
    // The LDS-tiled bodies need 85 registers and more per lane; inside a fused stage launch they would lower the
    // occupancy of every other operator (the wave-split bodies that serve small problems need 32-72), so they
    // only run as stand-alone kernels.
    static constexpr bool FUSABLE = false;
    static constexpr int SMEM_FLOATS = TILE_FLOATS > RED_FLOATS ? TILE_FLOATS : RED_FLOATS;

    // one block: output tile `tile` of group `g`, K slice `z`; smem holds SMEM_FLOATS floats, 16-byte aligned
    template <bool RES = false>
    __device__ static __forceinline__ void run(const ConvKernelArgs &a, float *smem, int tile, int g, int z) {
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / MT, TN = WTN / MT;
    constexpr int KSLICE = BK / WK;
    constexpr int A_VEC_PER_ROW = BM / 4;
    constexpr int A_SLOTS = BK * A_VEC_PER_ROW;
    constexpr int A_ITERS = (A_SLOTS + T - 1) / T;
    constexpr int B_ROWS_PER_PASS = T / BN;
    constexpr int B_ITERS = BK / B_ROWS_PER_PASS;
    static_assert(WTM % MT == 0 && WTN % MT == 0, "wave tile must be a multiple of the MFMA tile");
    static_assert(KSLICE % M::KSTEP == 0, "K slice per wavefront must be a multiple of the MFMA depth");
    static_assert(T % BN == 0 && BK % B_ROWS_PER_PASS == 0, "input loader shape");
    float *As = smem;                  // [2][BK][LDA]
    float *Bs = smem + 2 * BK * LDA;   // [2][BK][LDB]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: keeps per-wavefront K ranges and loop control on the SALU
    const int wn = wave % WN;
    const int wm = (wave / WN) % WM;
    const int wk = wave / (WN * WM);

    int tm, tn;
    xcd_tile(a, tile, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;
    const int k_begin = z * a.k_chunk;
    const int k_end = min(a.Kq, k_begin + a.k_chunk);
    const int nkt = (k_end - k_begin) / BK;   // Kq and k_chunk are multiples of BK

    // ---- per-thread loader state ---------------------------------------------------------------------
    const int bn_l = tid % BN;
    const int bk_l = tid / BN;
    const int n = n0 + bn_l;
    const bool n_ok = n < a.Npix;
    int ih0 = 0, iw0 = 0;
    unsigned x_thread = 0;   // byte offset of (image, group, ih0, iw0); may wrap below zero, the tap offset brings it back
    {
        const int nn = n_ok ? n : 0;
        const int b = (int)fast_div((unsigned)nn, a.div_ohw);
        const int r = nn - b * a.OHW;
        const int oh = (int)fast_div((unsigned)r, a.div_ow);
        const int ow = r - oh * a.OW;
        ih0 = oh * a.sh - a.ph;
        iw0 = ow * a.sw - a.pw;
        x_thread = (unsigned)(((long long)b * a.x_bs + (long long)g * a.ICg * a.HW + (long long)ih0 * a.W + iw0) * 4);
    }
    const __amdgpu_buffer_rsrc_t xr = buffer_of(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = buffer_of(a.wp, a.w_bytes);
    // constant per-thread byte offsets inside a tile: filter element (row, 4 columns) and input row (channel)
    unsigned a_off[A_ITERS];
#pragma unroll
    for (int i = 0; i < A_ITERS; i++) {
        const int slot = tid + i * T;
        const int row = slot / A_VEC_PER_ROW;
        const int c4 = slot % A_VEC_PER_ROW;
        const bool ok = (A_SLOTS % T == 0 || slot < A_SLOTS) && m0 + c4 * 4 < a.OCgP;
        a_off[i] = ok ? (unsigned)(((size_t)g * a.Kq * a.OCgP + (size_t)row * a.OCgP + m0 + c4 * 4) * 4) : kOutOfRange;
    }
    unsigned b_off[B_ITERS];
#pragma unroll
    for (int i = 0; i < B_ITERS; i++) b_off[i] = x_thread + (unsigned)((bk_l + i * B_ROWS_PER_PASS) * a.HW) * 4u;

    floatx4 a_reg[PD][A_ITERS];
    float b_reg[PD][B_ITERS];

    // K is ordered tap-major: row k of the packed filters is (tap = k / ICgP, c = k % ICgP) with ICgP a
    // multiple of BK, so a K tile lies inside one filter tap: (kh, kw) and the tile's base offsets are scalar,
    // the padding test is one compare pair per thread, and an element costs an add and a select of its offset.
    auto load_tile = [&](int kt, floatx4(&ar)[A_ITERS], float(&br)[B_ITERS]) {
        const int k0 = k_begin + kt * BK;
        const int tap = (int)__umulhi((unsigned)k0, a.magic_icgp);
        const int c0 = k0 - tap * a.ICgP;
        const int kh = a.KW == 1 ? tap : (int)__umulhi((unsigned)tap, a.magic_kw);
        const int kw = tap - kh * a.KW;
        const unsigned w_tile = (unsigned)(k0 * a.OCgP) * 4u;
        const unsigned tile_kill = kt < nkt ? 0u : kOutOfRange;   // tiles past the end of the K range load zeros
#pragma unroll
        for (int i = 0; i < A_ITERS; i++) ar[i] = buffer_load_f32x4(wr, (a_off[i] + w_tile) | tile_kill);
        // invalid elements get the top offset bit set, which is beyond every extent; plain bit arithmetic keeps
        // the loads of a tile in one basic block so that they are issued back to back
        const unsigned in_h = (unsigned)(ih0 + kh) < (unsigned)a.H ? 1u : 0u;
        const unsigned in_w = (unsigned)(iw0 + kw) < (unsigned)a.W ? 1u : 0u;
        const unsigned kill = (((in_h & in_w & (n_ok ? 1u : 0u)) ^ 1u) << 31) | tile_kill;
        const unsigned x_tile = (unsigned)(c0 * a.HW + kh * a.W + kw) * 4u;
        const int c_last = a.ICg - c0 - 1 - bk_l;   // this thread's rows beyond c_last are channel padding
#pragma unroll
        for (int i = 0; i < B_ITERS; i++) {
            const unsigned pad = (unsigned)(c_last - i * B_ROWS_PER_PASS) & kOutOfRange;   // sign bit
            br[i] = buffer_load_f32(xr, (b_off[i] + x_tile) | kill | pad);
        }
    };

    const int relu_floor = a.pre_relu ? 0 : (int)0x80000000;
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
            // folded ReLU of the producer as one integer max (negative floats are negative integers)
            Bb[(bk_l + i * B_ROWS_PER_PASS) * LDB + bn_l] = __int_as_float(max(__float_as_int(br[i]), relu_floor));
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
    // The loop runs in rounds of PD tiles with a straight-line body; tiles past the end of the K range are
    // loaded as zeros (see tile_kill) and cost at most PD - 1 idle MFMA tiles per block.
#pragma unroll
    for (int s = 0; s < PD; s++) load_tile(s, a_reg[s], b_reg[s]);
    store_tile(0, a_reg[0], b_reg[0]);
    __syncthreads();
    const int lk = lane / MT;   // k offset of this lane inside an MFMA step
    const int lc = lane % MT;   // row (A) / column (B) of this lane inside an MFMA tile
    for (int kt0 = 0; kt0 < nkt; kt0 += PD) {
#pragma unroll
        for (int s = 0; s < PD; s++) {
            const int kt = kt0 + s;
            const int buf = kt & 1;
            load_tile(kt + PD, a_reg[s], b_reg[s]);
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
            store_tile(buf ^ 1, a_reg[(s + 1) % PD], b_reg[(s + 1) % PD]);
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

    tiled_tail<MT, BM, BN, TM, TN, WM, WN, RES>(a, smem, acc, tile, g, z, m0, n0, wm, wn, wk);
    }   // run
};

// ---- LDS-tiled kernel on the bfloat16 matrix pipe with fp32-exact operands ---------------------------------------------------
// The fp32 matrix instructions run at 1/16 of the rate of the bfloat16 ones (measured: 149-156 against 2340 TFLOP/s).  An fp32
// number is exactly the sum of three bfloat16 numbers (its 24 significant bits in three groups of eight: x = hi + mid + lo,
// each term obtained by truncating the remainder to its leading eight bits, all subtractions exact), so a product of two
// fp32 numbers is the sum of nine products of bfloat16 numbers, each exact in fp32.  This kernel adds the six largest of them
// (hi*hi, hi*mid, mid*hi, hi*lo, mid*mid, lo*hi) on v_mfma_f32_32x32x16_bf16 with fp32 accumulation; the three that are left
// out are below 2^-23 of the product, the size of the rounding error of an fp32 multiplication.  Six instructions of 8 passes
// cover 16 k where the fp32 form needs eight instructions of 16 passes: 2.7 times the matrix throughput at fp32 accuracy.
//
// Filters are split when they are packed: three planes of bfloat16 in octets of eight consecutive k, [k / 8][plane][m][8],
// which is the operand layout of the instruction (lane l: row l % 32, k = 8 * (l / 32) ... + 7): a wavefront reads the filter
// operand of a 32 x 32 tile straight from global memory, one 16-byte load per lane and plane, PD K tiles ahead (the filters
// are small and stay in the caches; the LDS, whose bandwidth bounds this kernel, carries the inputs only).  Inputs are split
// by the thread that stages them: eight channels of one pixel, loaded PD K tiles ahead into registers, three 16-byte LDS
// stores into [plane][octet][pixel][8 k], again the operand layout: an input operand is one conflict-free 16-byte LDS load
// per lane and plane.  K tiles are 16 deep and lie inside one filter tap (channels padded to 16); LDS is double buffered, one
// barrier per K tile.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// the three bfloat16 terms of an fp32 value, each in the upper half of a word (hi + mid + lo == x exactly for normal x)
__device__ __host__ inline void split3(float x, unsigned &hi, unsigned &mid, unsigned &lo) {
    union { float f; unsigned u; } v, r;
    v.f = x;
    hi = v.u & 0xffff0000u;
    r.u = hi;
    v.f = x - r.f;
    mid = v.u & 0xffff0000u;
    r.u = mid;
    v.f = v.f - r.f;
    lo = v.u & 0xffff0000u;
}

// three bfloat16 terms of eight fp32 values, each term as four words of two bfloat16 (lower k in the lower half)
__device__ __forceinline__ void split_bf16x3(const float (&x)[8], uintx4 &hi, uintx4 &mid, uintx4 &lo) {
    unsigned h[8], m[8], l[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        h[i] = __float_as_uint(x[i]) & 0xffff0000u;
        const float r1 = x[i] - __uint_as_float(h[i]);
        m[i] = __float_as_uint(r1) & 0xffff0000u;
        const float r2 = r1 - __uint_as_float(m[i]);
        l[i] = __float_as_uint(r2);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {   // high halves of two words side by side
        hi[i] = __builtin_amdgcn_perm(h[2 * i + 1], h[2 * i], 0x07060302u);
        mid[i] = __builtin_amdgcn_perm(m[2 * i + 1], m[2 * i], 0x07060302u);
        lo[i] = __builtin_amdgcn_perm(l[2 * i + 1], l[2 * i], 0x07060302u);
    }
}

// eight fp32 values rounded to bfloat16 (nearest even), as four words of two (lower k in the lower half)
typedef float floatx8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ uintx4 round_bf16x8(const float (&x)[8]) {
    const floatx8 v = {x[0], x[1], x[2], x[3], x[4], x[5], x[6], x[7]};
    return __builtin_bit_cast(uintx4, __builtin_convertvector(v, bf16x8));
}

// TMW x TNW MFMA tiles of 32 x 32 per wavefront, WM x WN wavefronts per block
// TERMS = 3: fp32 accuracy as described above.  TERMS = 1: the reduced-precision mode with bfloat16 operands (inputs and
// filters rounded to nearest even, fp32 accumulation): one plane, one matrix instruction per tile and K tile, a sixth of the
// matrix work and a third of the LDS traffic.
template <int TMW, int TNW, int WM, int WN, int PD, int TERMS = 3>
struct ConvSplit3 {
    static_assert(TERMS == 3 || TERMS == 1, "three exact terms or one rounded term");
    static constexpr int MT = 32, BK = 16;
    using M = Mfma<32>;
    static constexpr int BM = 32 * TMW * WM, BN = 32 * TNW * WN;
    static constexpr int WAVES = WM * WN;
    static constexpr int T = 64 * WAVES;
    static constexpr int THREADS = T;
    static constexpr int CPAD = BK;
    static constexpr bool FUSABLE = false;
    // LDS in slots of 16 bytes (eight bfloat16): per stage the input planes [TERMS][2][BN]
    static constexpr int STAGE = 2 * TERMS * BN;
    static constexpr int SMEM_FLOATS = 2 * STAGE * 4;
    static constexpr int B_OCT = 2 * BN;
    static constexpr int B_IT = (B_OCT + T - 1) / T;                   // octets a thread stages per K tile
    static_assert(T % BN == 0, "a thread stages the same pixel in every pass");

    template <bool RES = false>
    __device__ static __forceinline__ void run(const ConvKernelArgs &a, float *smem, int tile, int g, int z) {
    constexpr int WTM = 32 * TMW, WTN = 32 * TNW;
    constexpr int TM = TMW, TN = TNW;
    uintx4 *lds = reinterpret_cast<uintx4 *>(smem);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave % WN;
    const int wm = wave / WN;
    const int lk = lane >> 5;   // which eight k of a K tile this lane supplies to the matrix instruction
    const int lc = lane & 31;   // row (A) / column (B) of this lane inside an MFMA tile
    int tm, tn;
    xcd_tile(a, tile, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;
    const int k_begin = z * a.k_chunk;
    const int k_end = min(a.Kq, k_begin + a.k_chunk);
    const int nkt = (k_end - k_begin) / BK;

    // ---- filters: every wavefront reads the operands of its own tiles from global memory, in operand layout -------------
    const __amdgpu_buffer_rsrc_t xr = buffer_of(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = buffer_of(a.wp, a.w_bytes);
    unsigned a_off[TM];      // byte offset of this lane's slot (plane 0) inside a K tile of the packed filters, or out of range
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + wm * WTM + i * MT + lc;
        // packed filters: [g][k / 8][plane][OCgP] slots of 16 bytes
        a_off[i] = m < a.OCgP ? (unsigned)(((((size_t)g * (a.Kq >> 3) + lk) * TERMS) * a.OCgP + m) * 16) : kOutOfRange;
    }
    const unsigned a_plane = (unsigned)a.OCgP * 16u;
    // ---- inputs: this thread's pixel and octets ----------------------------------------------------------------------------
    const int pix = tid % BN;
    const int n = n0 + pix;
    const bool n_ok = n < a.Npix;
    int ih0, iw0;
    unsigned x_thread;
    {
        const int nn = n_ok ? n : 0;
        const int b = (int)fast_div((unsigned)nn, a.div_ohw);
        const int r = nn - b * a.OHW;
        const int oh = (int)fast_div((unsigned)r, a.div_ow);
        const int ow = r - oh * a.OW;
        ih0 = oh * a.sh - a.ph;
        iw0 = ow * a.sw - a.pw;
        x_thread = (unsigned)(((long long)b * a.x_bs + (long long)g * a.ICg * a.HW + (long long)ih0 * a.W + iw0) * 4);
    }
    int b_oct[B_IT];       // which half of the K tile (channels 8 * b_oct ... + 7 of the tile) a pass of this thread stages
#pragma unroll
    for (int i = 0; i < B_IT; i++) b_oct[i] = (tid + i * T) / BN;
    const unsigned b_surplus = B_OCT % T == 0 || tid < B_OCT ? 0u : kOutOfRange;   // (more threads than octets: the surplus stages nothing)

    uintx4 a_reg[PD][TERMS][TM];
    float b_reg[PD][B_IT][8];
    auto load_tile = [&](int kt, uintx4 (&ar)[TERMS][TM], float (&br)[B_IT][8]) {
        const int k0 = k_begin + kt * BK;
        const int tap = (int)__umulhi((unsigned)k0, a.magic_icgp);
        const int c0 = k0 - tap * a.ICgP;
        const int kh = a.KW == 1 ? tap : (int)__umulhi((unsigned)tap, a.magic_kw);
        const int kw = tap - kh * a.KW;
        const unsigned tile_kill = kt < nkt ? 0u : kOutOfRange;   // tiles past the end of the K range load zeros
        const unsigned w_tile = (unsigned)((k0 >> 3) * TERMS * a.OCgP) * 16u;
#pragma unroll
        for (int p = 0; p < TERMS; p++)
#pragma unroll
            for (int i = 0; i < TM; i++) ar[p][i] = __builtin_amdgcn_raw_buffer_load_b128(wr, (a_off[i] + w_tile) | tile_kill, (unsigned)p * a_plane, 0);
        const unsigned in_h = (unsigned)(ih0 + kh) < (unsigned)a.H ? 1u : 0u;
        const unsigned in_w = (unsigned)(iw0 + kw) < (unsigned)a.W ? 1u : 0u;
        const unsigned kill = (((in_h & in_w & (n_ok ? 1u : 0u)) ^ 1u) << 31) | tile_kill | b_surplus;
        const unsigned x_tile = x_thread + (unsigned)(c0 * a.HW + kh * a.W + kw) * 4u;
        const unsigned plane = (unsigned)a.HW * 4u;
#pragma unroll
        for (int i = 0; i < B_IT; i++) {
            const int c_left = a.ICg - 1 - c0 - b_oct[i] * 8;   // channels of this octet beyond c_left are padding
            const unsigned at = (x_tile + (unsigned)(b_oct[i] * 8) * plane) | kill;
            // (no branch around loads inside the loop: where paths that issued loads join, the compiler waits for all of them)
#pragma unroll
            for (int j = 0; j < 8; j++) br[i][j] = buffer_load_f32(xr, at | ((unsigned)(c_left - j) & kOutOfRange), (unsigned)j * plane);
        }
    };
    const int relu_floor = a.pre_relu ? 0 : (int)0x80000000;
    auto store_inputs = [&](int buf, const float (&br)[B_IT][8]) {
        uintx4 *stage = lds + buf * STAGE;
#pragma unroll
        for (int i = 0; i < B_IT; i++) {
            if (B_OCT % T != 0 && tid + i * T >= B_OCT) continue;
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = __int_as_float(max(__float_as_int(br[i][j]), relu_floor));   // folded ReLU of the producer
            if constexpr (TERMS == 3) {
                uintx4 hi, mid, lo;
                split_bf16x3(v, hi, mid, lo);
                stage[(0 + b_oct[i]) * BN + pix] = hi;
                stage[(2 + b_oct[i]) * BN + pix] = mid;
                stage[(4 + b_oct[i]) * BN + pix] = lo;
            } else {
                stage[b_oct[i] * BN + pix] = round_bf16x8(v);
            }
        }
    };

    typename M::acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < M::ACC; v++) acc[i][j][v] = 0.f;

    // ---- main loop ---------------------------------------------------------------------------------------------------------
    // Register stage s holds K tile kt with kt % PD == s (filter operands of this wavefront, inputs of this thread).  Iteration
    // kt: the matrix work of tile kt from registers (filters) and LDS stage kt & 1 (inputs), the stage's registers requested
    // again for tile kt + PD, the inputs of tile kt + 1 split and stored into the other LDS stage, one barrier.
#pragma unroll
    for (int s = 0; s < PD; s++) load_tile(s, a_reg[s], b_reg[s]);
    store_inputs(0, b_reg[0]);
    __syncthreads();
    for (int kt0 = 0; kt0 < nkt; kt0 += PD) {
#pragma unroll
        for (int s = 0; s < PD; s++) {
            const int kt = kt0 + s;
            const int buf = kt & 1;
            const uintx4 *Bb = lds + buf * STAGE + lk * BN + wn * WTN + lc;
            bf16x8 av[TERMS][TM], bv[TERMS][TN];
#pragma unroll
            for (int p = 0; p < TERMS; p++) {
#pragma unroll
                for (int i = 0; i < TM; i++) av[p][i] = __builtin_bit_cast(bf16x8, a_reg[s][p][i]);
#pragma unroll
                for (int j = 0; j < TN; j++) bv[p][j] = __builtin_bit_cast(bf16x8, Bb[p * 2 * BN + j * MT]);
            }
            // all LDS reads of the tile are requested before its first matrix instruction (left to itself the scheduler
            // requests each operand right in front of its first use and the wavefront pays the LDS latency once per plane)
            __builtin_amdgcn_sched_barrier(0);
            // the six terms, smallest first; the tiles of a term are independent instructions
            constexpr int NT = TERMS == 3 ? 6 : 1;
            constexpr int TA[6] = {TERMS == 3 ? 2 : 0, 0, 1, 1, 0, 0}, TB[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[TA[t]][i], bv[TB[t]][j], acc[i][j], 0, 0, 0);
            store_inputs(buf ^ 1, b_reg[(s + 1) % PD]);
            load_tile(kt + PD, a_reg[s], b_reg[s]);
            __syncthreads();
        }
    }
    tiled_tail<MT, BM, BN, TM, TN, WM, WN, RES>(a, smem, acc, tile, g, z, m0, n0, wm, wn, 0);
    }   // run
};

// y[b][oc][r] = act(bias[oc] + sum_s ws[s][oc][n]) (+ residual),  n = b * OHW + r; slices are added in index order
struct ReduceArgs {
    const float *ws;
    const float *bias;
    float *y;
    int slices, OC, Npix, OHW, act;
    long long slice_floats, y_bs;
    const float *res;      // residual operand as in ConvKernelArgs, or null
    int res_bs, post_relu;
};

__device__ __forceinline__ void splitk_reduce_body(const ReduceArgs &a, int block, int num_blocks, unsigned threads) {
    const long long total = (long long)a.OC * a.Npix;
    for (long long i = block * (long long)threads + threadIdx.x; i < total; i += (long long)num_blocks * threads) {
        const int oc = (int)(i / a.Npix);
        const int n = (int)(i - (long long)oc * a.Npix);
        float sum = 0.f;
        for (int s = 0; s < a.slices; s++) sum += a.ws[s * a.slice_floats + i];
        const int b = n / a.OHW;
        const int r = n - b * a.OHW;
        float v = apply_act(sum + a.bias[oc], a.act);
        if (a.res != nullptr) {
            v += a.res[(long long)b * a.res_bs + (long long)oc * a.OHW + r];
            if (a.post_relu) v = fmaxf(v, 0.0f);
        }
        a.y[b * a.y_bs + (long long)oc * a.OHW + r] = v;
    }
}


// ---- wave-split variant: no LDS staging, K divided among the wavefronts of a block ---------------------------------------
// For batch-1 layers (tens to hundreds of pixels, K in the thousands) the LDS-tiled kernel is bound by the chain
// load -> LDS -> barrier per K tile, and slicing K over blocks costs a second kernel.  Here every wavefront of a
// block owns a contiguous K range of the same BM x BN output tile and feeds the MFMA straight from global memory in
// the instruction's operand layout (lane l: A[k = l / MT][m = l % MT], B[k = l / MT][n = l % MT]); there is no barrier
// inside the K loop, two register batches of U k-steps keep dozens of loads in flight per lane, and the NW partial
// tiles meet once in LDS, where the wavefronts share the bias + activation + store work.  The sum order is fixed
// (k ascending inside a wavefront, wavefronts ascending), so results are reproducible.
//
// QUAD: within a batch of U k-steps (U * KSTEP consecutive k) the lane group lk supplies k = U * lk + u in step u
// instead of KSTEP * u + lk.  The MFMA only needs A and B to agree on k, and this assignment gives a lane U
// consecutive filter rows, which the quad-packed filter layout [k / 4][m][4] delivers as 16-byte loads: a quarter
// of the filter load instructions.  Channels are padded to the batch (U * KSTEP), so a batch lies inside one tap.
//
// BF16 (reduced-precision mode): filters are packed as bfloat16 in the quad layout (a lane's four k are one 8-byte
// load), inputs are rounded to bfloat16 (nearest even) after loading, and one v_mfma_f32_16x16x16_bf16 consumes
// the four k of a lane group at once - the same k assignment as QUAD; accumulation stays fp32.
//
// CP: channel padding of the packed filters when it should differ from the default (8, or the batch with QUAD); 4 serves
// layers with a handful of input channels (the first layer of an image network), whose K would otherwise be mostly padding.
template <int MT, int TM, int TN, int NW, int U, bool QUAD = false, int D = 2, int RP = 0, int CP = 0>
struct ConvWsplit {
    using M = Mfma<MT>;
    static constexpr int BM = TM * MT, BN = TN * MT;
    static constexpr int E = TM * TN * M::ACC;
    static constexpr int THREADS = 64 * NW;
    static constexpr int SMEM_FLOATS = NW * E * 64;
    static constexpr int CPAD = CP ? CP : (QUAD ? U * M::KSTEP : 8);   // channel padding of the packed filters this kernel expects
    static_assert(CP == 0 || (!QUAD && CP % M::KSTEP == 0), "a k-step must lie inside one filter tap");
    static constexpr bool KQUAD = QUAD;                    // packed filters are [k / 4][m][4] instead of [k][m]
    // accumulators + staged operands per lane decide whether the body fits the register budget of a fused launch
    // (the channel-padding-4 forms serve first layers, which are stages of their own: kept out of the fused launches)
    static constexpr bool FUSABLE = RP < 3 && CP == 0 && E + D * U * (TM + TN) <= (QUAD ? (MT == 32 ? 48 : 56) : 48);   // per-step addressing of the plain layout needs more registers, and so do the 16-register accumulator tuples of the 32 x 32 tiles
    // the three-term bodies of up to two 32 x 32 tiles per wavefront (100-155 registers) run inside fused launches of the
    // wide-register kernel family (fused_kernel_wide)
    static constexpr bool FUSABLE_WIDE = RP == 3 && NW <= 8 && TM * TN <= 2;
    static constexpr int KREDUCED = RP;                    // 0: fp32 filters; 1: packed filters hold bfloat16; 2: IEEE half; 3: three bfloat16 planes; 4: one
    static constexpr int PLANES = RP == 3 ? 3 : 1;
    // RP == 4: the reduced-precision mode on the same instruction and layout: one plane of filters rounded to bfloat16, inputs
    // rounded after the load, one matrix instruction per tile and batch.
    // RP == 3: fp32 results from the bfloat16 matrix pipe, as in ConvSplit3 (operands split exactly into three bfloat16 terms,
    // six of the nine partial products on v_mfma_f32_32x32x16_bf16): filters are split when packed, [k / 8][plane][m][8], and read
    // as operands straight from global memory; a lane splits the eight input values it loads for a batch itself.
    static_assert(!QUAD || U % 4 == 0, "quad loads need whole groups of four k per lane");
    static_assert(RP >= 0 && RP <= 4 && (RP == 0 || (RP >= 3 ? QUAD && MT == 32 && U == 8 : QUAD && MT == 16 && U == 4)),
                  "the 16-bit paths are the 16 x 16 x 16 form of the quad layout, the three-term path its 32 x 32 x 16 form");

    template <bool RES = false>
    __device__ static __forceinline__ void run(const ConvKernelArgs &a, float *red, int tile, int g, int z) {

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: keeps per-wavefront K ranges and loop control on the SALU
    const int lk = lane / MT;
    const int lc = lane % MT;
    int tm, tn;
    xcd_tile(a, tile, tm, tn);
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    // K slice z of the grid (k_chunk is a multiple of the batch U * KSTEP), divided among the wavefronts; the host did the
    // divisions (every wavefront of a block repeats this prologue on the SIMD's one scalar issue slot, so it is kept short)
    const int s_lo = z * a.steps_chunk;
    const int s_hi = min(a.steps_total, s_lo + a.steps_chunk);
    const int s_begin = s_lo + wave * a.steps_per_wave;
    const int s_end = min(s_hi, s_begin + a.steps_per_wave);

    int ih0[TN], iw0[TN];
    unsigned x_lane[TN];   // byte offset of (image, group channel lk, ih0, iw0); wraps like x_thread above
    bool n_ok[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + j * MT + lc;
        n_ok[j] = n < a.Npix;
        const int nn = n_ok[j] ? n : 0;
        // image sizes are below 2^15 per side and OH * OW below 2^23 (checked on the host): signed 24-bit multiplies, which
        // run at full rate, are exact here; byte offsets are wanted modulo 2^32, so 32-bit arithmetic gives them
        const int b = (int)fast_div((unsigned)nn, a.div_ohw);
        const int r = nn - __mul24(b, a.OHW);
        const int oh = (int)fast_div((unsigned)r, a.div_ow);
        const int ow = r - __mul24(oh, a.OW);
        ih0[j] = __mul24(oh, a.sh) - a.ph;
        iw0[j] = __mul24(ow, a.sw) - a.pw;
        const int lane_channel = QUAD ? U * lk : lk;   // first channel of this lane inside a step / batch
        x_lane[j] = ((unsigned)b * (unsigned)a.x_bs + (unsigned)(g * a.ICg + lane_channel) * (unsigned)a.HW +
                     (unsigned)(__mul24(ih0[j], a.W) + iw0[j])) * 4u;
    }
    const __amdgpu_buffer_rsrc_t xr = buffer_of(a.x, a.x_bytes);
    const __amdgpu_buffer_rsrc_t wr = buffer_of(a.wp, a.w_bytes);
    unsigned w_lane[TM], w_kill[TM], n_kill[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        w_kill[i] = m0 + i * MT + lc < a.OCgP ? 0u : kOutOfRange;
        // byte offsets below 2^31 (checked on the host)
        if (RP >= 3)   // [g][k / 8][plane][m] slots of 16 bytes: this lane's octet of a batch is lk
            w_lane[i] = ((((unsigned)g * ((unsigned)a.Kq >> 3) + (unsigned)lk) * (unsigned)PLANES) * (unsigned)a.OCgP + (unsigned)(m0 + i * MT + lc)) * 16u;
        else if (QUAD)   // [g][k / 4][m][4]: this lane's first quad of a batch is row (U / 4) * lk
            w_lane[i] = (((unsigned)g * ((unsigned)a.Kq >> 2) + (unsigned)((U / 4) * lk)) * (unsigned)a.OCgP + (unsigned)(m0 + i * MT + lc)) * (RP != 0 ? 8u : 16u);
        else
            w_lane[i] = (((unsigned)g * (unsigned)a.Kq + (unsigned)lk) * (unsigned)a.OCgP + (unsigned)(m0 + i * MT + lc)) * 4u;
    }
#pragma unroll
    for (int j = 0; j < TN; j++) n_kill[j] = n_ok[j] ? 0u : kOutOfRange;

    // the bias of the outputs this lane finishes in the epilogue, requested now so that its latency hides behind the K loop
    constexpr int EPW = (E + NW - 1) / NW;
    float bias_pre[EPW];
#pragma unroll
    for (int t = 0; t < EPW; t++) {
        const int e = min(wave + t * NW, E - 1);
        const int m = m0 + (e / (M::ACC * TN)) * MT + M::row(e % M::ACC, lane);
        bias_pre[t] = a.bias[g * a.OCg + min(m, a.OCg - 1)];
    }
    typename M::acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < M::ACC; v++) acc[i][j][v] = 0.f;

    // D register batches in flight: filter operands (fp32: U steps x TM tiles; bf16: four packed k per tile) and inputs
    struct FilterStageF32 {
        float v[U][TM];
    };
    struct FilterStageBf16 {
        uintx2 v[TM];
    };
    struct FilterStageX3 {
        uintx4 v[PLANES][TM];
    };
    using FilterStage = std::conditional_t<(RP >= 3), FilterStageX3, std::conditional_t<(RP != 0), FilterStageBf16, FilterStageF32>>;
    FilterStage av[D];
    float bv[D][U][TN];

    // k-step s covers rows k = s * KSTEP + lk of the tap-major packed filters; ICgP is a multiple of KSTEP, so a
    // step lies inside one filter tap and (tap, kh, kw, first channel) are wavefront-uniform
    // QUAD: scalar state of the next batch to request (batches are requested in K order starting at s_begin)
    int q_cb = 0, q_kh = 0, q_kw = 0;
    unsigned q_w = 0;
    const int c_lane_last = a.ICg - 1 - U * lk;   // QUAD: the lane's first channel of a batch starting at channel cb is real while cb <= c_lane_last
    if constexpr (QUAD) {
        const int kb = s_begin * M::KSTEP;
        const int tap = (int)__umulhi((unsigned)kb, a.magic_icgp);
        q_cb = kb - tap * a.ICgP;
        q_kh = a.KW == 1 ? tap : (int)__umulhi((unsigned)tap, a.magic_kw);
        q_kw = tap - q_kh * a.KW;
        q_w = RP >= 3 ? (unsigned)((kb / 8) * PLANES * a.OCgP) * 16u : (unsigned)((kb / 4) * a.OCgP) * (RP != 0 ? 8u : 16u);
    }
    // `live` (wavefront-uniform) is false for a batch beyond the wavefront's K range: its loads are still issued, against
    // descriptors of extent zero, and return zeros without touching memory.  Loads are never skipped by a branch inside
    // the K loop: where a path with and a path without newly issued loads join, the compiler can only wait for *all*
    // outstanding loads before the next use of an older one, which serialises load latency and matrix work.
    // `ragged` (a std::bool_constant, QUAD only): the group's channel count is not a multiple of U, so the U channels of a lane
    // can straddle the end of the real channels and every k-step needs its own test; otherwise a lane's channels are real or
    // padding together and one test per batch, folded into the lane's offsets, covers them.
    auto load_batch = [&](int s0, FilterStage &A, float(&B)[U][TN], bool live, auto ragged) {
        if constexpr (QUAD) {
            // The whole batch lies inside one tap (channels are padded to the batch).  Batches are requested in K
            // order, so (first channel, kh, kw) and the filter offset advance incrementally on the SALU.  Lane-constant
            // offsets go into the vector operand of the buffer loads, the per-batch / per-step parts into the scalar
            // operand: a filter load costs no VALU instruction, an input load one add + one or per batch and tile.
            (void)s0;
            const __amdgpu_buffer_rsrc_t xr = buffer_of(a.x, live ? a.x_bytes : 0u);
            const __amdgpu_buffer_rsrc_t wr = buffer_of(a.wp, live ? a.w_bytes : 0u);
            if constexpr (RP >= 3) {
#pragma unroll
                for (int p = 0; p < PLANES; p++)
#pragma unroll
                    for (int i = 0; i < TM; i++)   // eight bfloat16 = the lane's eight k of this batch, one plane
                        A.v[p][i] = __builtin_amdgcn_raw_buffer_load_b128(wr, w_lane[i] | w_kill[i], q_w + (unsigned)(p * a.OCgP) * 16u, 0);
            } else if constexpr (RP != 0) {
#pragma unroll
                for (int i = 0; i < TM; i++) {   // four 16-bit values = the lane's four k of this batch
                    A.v[i] = buffer_load_u32x2(wr, w_lane[i] | w_kill[i], q_w);
                }
            } else {
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int q = 0; q < U / 4; q++) {
                        const floatx4 w4 = buffer_load_f32x4(wr, w_lane[i] | w_kill[i], q_w + (unsigned)(q * a.OCgP) * 16u);
                        A.v[q * 4 + 0][i] = w4.x;
                        A.v[q * 4 + 1][i] = w4.y;
                        A.v[q * 4 + 2][i] = w4.z;
                        A.v[q * 4 + 3][i] = w4.w;
                    }
            }
            const unsigned x_tap = (unsigned)(q_kh * a.W + q_kw) * 4u;
            const unsigned x_chan = (unsigned)(q_cb * a.HW) * 4u;
            unsigned voff[TN];
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const unsigned in_h = (unsigned)(ih0[j] + q_kh) < (unsigned)a.H ? 1u : 0u;
                const unsigned in_w = (unsigned)(iw0[j] + q_kw) < (unsigned)a.W ? 1u : 0u;
                voff[j] = (x_lane[j] + x_tap) | (((in_h & in_w) ^ 1u) << 31);
            }
            const int c_left = c_lane_last - q_cb;   // channels of this lane beyond c_left are padding (the tap's last batch)
            if constexpr (decltype(ragged)::value) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const unsigned c_kill = (unsigned)(c_left - u) & kOutOfRange;   // sign bit
#pragma unroll
                    for (int j = 0; j < TN; j++) B[u][j] = buffer_load_f32(xr, voff[j] | c_kill, x_chan + (unsigned)(u * a.HW) * 4u);
                }
            } else {
                const unsigned c_kill = (unsigned)c_left & kOutOfRange;   // all U channels of the lane at once
#pragma unroll
                for (int j = 0; j < TN; j++) voff[j] |= c_kill;
#pragma unroll
                for (int u = 0; u < U; u++)
#pragma unroll
                    for (int j = 0; j < TN; j++) B[u][j] = buffer_load_f32(xr, voff[j], x_chan + (unsigned)(u * a.HW) * 4u);
            }
            // next batch (selects, not branches: the loop body stays one basic block)
            q_w += RP >= 3 ? (unsigned)((U * M::KSTEP / 8) * PLANES * a.OCgP) * 16u : (unsigned)((U * M::KSTEP / 4) * a.OCgP) * (RP != 0 ? 8u : 16u);
            q_cb += U * M::KSTEP;
            const bool next_tap = q_cb >= a.ICgP;
            q_cb = next_tap ? 0 : q_cb;
            q_kw += next_tap ? 1 : 0;
            const bool next_row = q_kw == a.KW;
            q_kw = next_row ? 0 : q_kw;
            q_kh += next_row ? 1 : 0;
            return;
        }
        (void)live;   // steps at or beyond s_end are dead by their index
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool s_ok = (s0 + u) < s_end;
            const int kb = (s0 + u) * M::KSTEP;
            const int tap = (int)__umulhi((unsigned)kb, a.magic_icgp);
            const int cb = kb - tap * a.ICgP;
            const int kh = a.KW == 1 ? tap : (int)__umulhi((unsigned)tap, a.magic_kw);
            const int kw = tap - kh * a.KW;
            const unsigned w_step = (unsigned)(kb * a.OCgP) * 4u;
            const unsigned step_kill = s_ok ? 0u : kOutOfRange;   // wavefront-uniform
#pragma unroll
            for (int i = 0; i < TM; i++) A.v[u][i] = buffer_load_f32(wr, (w_lane[i] + w_step) | w_kill[i] | step_kill);
            const unsigned x_step = (unsigned)(cb * a.HW + kh * a.W + kw) * 4u;
            const unsigned c_kill = (unsigned)(a.ICg - 1 - cb - lk) & kOutOfRange;   // sign bit: channel padding
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const unsigned in_h = (unsigned)(ih0[j] + kh) < (unsigned)a.H ? 1u : 0u;
                const unsigned in_w = (unsigned)(iw0[j] + kw) < (unsigned)a.W ? 1u : 0u;
                const unsigned kill = ((in_h & in_w) ^ 1u) << 31;
                B[u][j] = buffer_load_f32(xr, (x_lane[j] + x_step) | kill | c_kill | n_kill[j] | step_kill);
            }
        }
    };
    // folded ReLU of the producer: as integers, negative floats are below 0 and everything is above INT_MIN
    const int relu_floor = a.pre_relu ? 0 : (int)0x80000000;
    auto compute = [&](const FilterStage &A, const float(&B)[U][TN]) {
        if constexpr (RP == 3) {
            bf16x8 bq[3][TN];
#pragma unroll
            for (int j = 0; j < TN; j++) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = __int_as_float(max(__float_as_int(B[u][j]), relu_floor));
                uintx4 hi, mid, lo;
                split_bf16x3(v, hi, mid, lo);
                bq[0][j] = __builtin_bit_cast(bf16x8, hi);
                bq[1][j] = __builtin_bit_cast(bf16x8, mid);
                bq[2][j] = __builtin_bit_cast(bf16x8, lo);
            }
            // the six terms, smallest first; the tiles of a term are independent instructions
            constexpr int TA[6] = {2, 0, 1, 1, 0, 0}, TB[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
            for (int t = 0; t < 6; t++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, A.v[TA[t]][i]), bq[TB[t]][j], acc[i][j], 0, 0, 0);
            return;
        } else if constexpr (RP == 4) {
            // one rounded term: the reduced-precision mode on the 32 x 32 x 16 instruction
#pragma unroll
            for (int j = 0; j < TN; j++) {
                float v[8];
#pragma unroll
                for (int u = 0; u < 8; u++) v[u] = __int_as_float(max(__float_as_int(B[u][j]), relu_floor));
                const bf16x8 bq = __builtin_bit_cast(bf16x8, round_bf16x8(v));
#pragma unroll
                for (int i = 0; i < TM; i++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, A.v[0][i]), bq, acc[i][j], 0, 0, 0);
            }
            return;
        } else if constexpr (RP != 0) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const floatx4 b32 = {__int_as_float(max(__float_as_int(B[0][j]), relu_floor)), __int_as_float(max(__float_as_int(B[1][j]), relu_floor)),
                                     __int_as_float(max(__float_as_int(B[2][j]), relu_floor)), __int_as_float(max(__float_as_int(B[3][j]), relu_floor))};
                if constexpr (RP == 1) {
                    const bf16x4 b4 = __builtin_convertvector(b32, bf16x4);   // round to nearest even
#pragma unroll
                    for (int i = 0; i < TM; i++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(bf16x4, A.v[i]), b4, acc[i][j], 0, 0, 0);
                } else {
                    const halfx4 b4 = __builtin_convertvector(b32, halfx4);   // round to nearest even, overflow to infinity
#pragma unroll
                    for (int i = 0; i < TM; i++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(halfx4, A.v[i]), b4, acc[i][j], 0, 0, 0);
                }
            }
            return;
        } else {
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        const float bval = __int_as_float(max(__float_as_int(B[u][j]), relu_floor));   // one integer max
                        acc[i][j] = M::run(A.v[u][i], bval, acc[i][j]);
                    }
        }
    };

    const int batches = (s_end - s_begin + U - 1) / U;   // <= 0 for wavefronts beyond the end of K
    auto k_loop = [&](auto ragged) {
        if (batches <= 0) return;
        if constexpr (decltype(ragged)::value) {
            // channel counts that are no multiple of U (a few tiny layers): one batch at a time
            for (int b = 0; b < batches; b++) {
                load_batch(s_begin + b * U, av[0], bv[0], true, ragged);
                compute(av[0], bv[0]);
            }
        } else if constexpr (D == 2) {
            // Two stages, peeled so that every load sits in straight-line code: the steady state requests batch b + 1,
            // consumes batch b, requests b + 2, consumes b + 1 with both requests known to be in range; the last one or two
            // batches are consumed behind the loop.  The waits in front of the matrix instructions then count exactly the
            // loads issued since, and the next batch's latency overlaps this batch's matrix work.  (The scheduling fences
            // keep a stage's requests behind the matrix work that still reads the stage: moved ahead of it they need a
            // second set of registers.)
            load_batch(s_begin, av[0], bv[0], true, ragged);
            int b = 0;
            for (; b + 2 < batches; b += 2) {
                load_batch(s_begin + (b + 1) * U, av[1], bv[1], true, ragged);
                __builtin_amdgcn_sched_barrier(0);
                compute(av[0], bv[0]);
                __builtin_amdgcn_sched_barrier(0);
                load_batch(s_begin + (b + 2) * U, av[0], bv[0], true, ragged);
                __builtin_amdgcn_sched_barrier(0);
                compute(av[1], bv[1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (b + 1 < batches) {
                load_batch(s_begin + (b + 1) * U, av[1], bv[1], true, ragged);
                __builtin_amdgcn_sched_barrier(0);
                compute(av[0], bv[0]);
                compute(av[1], bv[1]);
            } else {
                compute(av[0], bv[0]);
            }
        } else {
            // deeper pipeline: D batches requested before the first one is consumed.  The loop body is straight-line
            // (requests beyond the range are issued dead, see load_batch: at most D - 1 of them in the last round that
            // requests anything); the last D batches are consumed behind the loop, where nothing is requested any more.
#pragma unroll
            for (int st = 0; st < D; st++) load_batch(s_begin + st * U, av[st], bv[st], st < batches, ragged);
            int b = 0;
            for (; b + D < batches; b += D) {
#pragma unroll
                for (int st = 0; st < D; st++) {
                    compute(av[st], bv[st]);
                    __builtin_amdgcn_sched_barrier(0);
                    load_batch(s_begin + (b + st + D) * U, av[st], bv[st], b + st + D < batches, ragged);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int st = 0; st < D; st++)
                if (b + st < batches) compute(av[st], bv[st]);
        }
    };
    if constexpr (QUAD) {
        if ((a.ICg & (U - 1)) == 0) k_loop(std::false_type{});
        else k_loop(std::true_type{});
    } else {
        k_loop(std::false_type{});
    }

    // partial tiles meet in LDS: element e of lane l of wavefront w lives at red[(w * E + e) * 64 + l]
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < M::ACC; v++) red[(wave * E + (i * TN + j) * M::ACC + v) * 64 + lane] = acc[i][j][v];
    __syncthreads();
    if (a.split_k > 1 && a.counters == nullptr) {
        // two-kernel split-K: this slice's partial outputs as [slice][group][m][pixel] for splitk_reduce_kernel
        float *wsz = a.ws + ((size_t)z * a.groups + g) * a.OCg * (size_t)a.Npix;
        for (int e = wave; e < E; e += NW) {
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) sum += red[(w * E + e) * 64 + lane];
            const int m = m0 + (e / (M::ACC * TN)) * MT + M::row(e % M::ACC, lane);
            const int nn = n0 + ((e / M::ACC) % TN) * MT + lc;
            if (m < a.OCg && nn < a.Npix) wsz[(size_t)m * a.Npix + nn] = sum;
        }
        return;
    }
    float *slices = nullptr;
    if (a.split_k > 1) {
        // one-kernel split-K, as in the LDS-tiled kernel: partial tiles in [element][lane] order, a ticket per
        // tile, the block drawing the last ticket adds the slices in slice order
        const size_t tiles = (size_t)xcd_padded_tiles(a.tiles_m * a.tiles_n);
        slices = a.ws + (((size_t)g * tiles + tile) * a.split_k) * (size_t)(BM * BN);
        unsigned *counter = a.counters + (size_t)g * tiles + tile;
        int *last_flag = reinterpret_cast<int *>(red);
        auto hand_in = [&](auto local) {
            constexpr bool LOCAL = decltype(local)::value;
            float *mine = slices + (size_t)z * (BM * BN) + lane;
            for (int e = wave; e < E; e += NW) {
                float sum = 0.f;
#pragma unroll
                for (int w = 0; w < NW; w++) sum += red[(w * E + e) * 64 + lane];
                partial_store<LOCAL>(mine + e * 64, sum);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) *last_flag = draw_ticket<LOCAL>(counter, a.split_k);
        };
        if (a.xcd_local) hand_in(std::true_type{});
        else hand_in(std::false_type{});
        __syncthreads();
        if (*last_flag == 0) return;
    }
    const bool xcd_local = a.xcd_local != 0;
#pragma unroll
    for (int t = 0; t < EPW; t++) {
        const int e = wave + t * NW;
        if (e >= E) break;
        float sum = 0.f;
        if (a.split_k > 1) {
            const float *theirs = slices + e * 64 + lane;
            if (xcd_local)
                for (int s2 = 0; s2 < a.split_k; s2++) sum += partial_load<true>(theirs + (size_t)s2 * (BM * BN));
            else
                for (int s2 = 0; s2 < a.split_k; s2++) sum += partial_load<false>(theirs + (size_t)s2 * (BM * BN));
        } else {
#pragma unroll
            for (int w = 0; w < NW; w++) sum += red[(w * E + e) * 64 + lane];
        }
        const int v = e % M::ACC;
        const int j = (e / M::ACC) % TN;
        const int i = e / (M::ACC * TN);
        const int m = m0 + i * MT + M::row(v, lane);
        const int nn = n0 + j * MT + lc;
        if (m < a.OCg && nn < a.Npix) {
            const int b = (int)fast_div((unsigned)nn, a.div_ohw);
            const int r = nn - b * a.OHW;
            a.y[(long long)b * a.y_bs + ((long long)g * a.OCg + m) * a.OHW + r] =
                add_residual<RES>(a, apply_act(sum + bias_pre[t], a.act), b, g * a.OCg + m, r);
        }
    }
}   // run
};

// ---- kernel configurations ------------------------------------------------------------------------------------------
// X(index, name, BM, BN, BK, WM, WN, WK, MT, PD) for the LDS-tiled kernel
#define IOS_TILED_VARIANTS(X)                                    \
    X(0, "m64n64k32_w2x2x1_t32", 64, 64, 32, 2, 2, 1, 32, 3)     \
    X(1, "m128n128k16_w2x2x1_t32", 128, 128, 16, 2, 2, 1, 32, 3) \
    X(2, "m32n32k64_w1x1x4_t32", 32, 32, 64, 1, 1, 4, 32, 4)     \
    X(3, "m64n32k32_w2x1x2_t32", 64, 32, 32, 2, 1, 2, 32, 4)     \
    X(4, "m32n64k32_w1x2x2_t32", 32, 64, 32, 1, 2, 2, 32, 4)     \
    X(5, "m128n64k16_w2x2x1_t32", 128, 64, 16, 2, 2, 1, 32, 3)   \
    X(6, "m64n16k64_w4x1x1_t16", 64, 16, 64, 4, 1, 1, 16, 3)     \
    X(7, "m32n16k64_w2x1x2_t16", 32, 16, 64, 2, 1, 2, 16, 4)     \
    X(8, "m16n16k128_w1x1x4_t16", 16, 16, 128, 1, 1, 4, 16, 3)   \
    X(9, "m64n128k16_w2x2x1_t32", 64, 128, 16, 2, 2, 1, 32, 3)   \
    X(10, "m64n64k16_w2x2x1_t32", 64, 64, 16, 2, 2, 1, 32, 4)    \
    X(11, "m32n128k16_w1x4x1_t32", 32, 128, 16, 1, 4, 1, 32, 4)  \
    X(12, "m192n64k16_w2x2x1_t32", 192, 64, 16, 2, 2, 1, 32, 3)  \
    X(13, "m96n128k16_w1x4x1_t32", 96, 128, 16, 1, 4, 1, 32, 3)  \
    X(14, "m192n128k16_w2x2x1_t32", 192, 128, 16, 2, 2, 1, 32, 3) \
    X(15, "m160n128k16_w1x4x1_t32", 160, 128, 16, 1, 4, 1, 32, 3)
// X(index, name, MT, TM, TN, NW, U, QUAD, D, BF16) for the wave-split kernel
#define IOS_WSPLIT_VARIANTS(X)                     \
    X(16, "ws_m32n16_w16_t16", 16, 2, 1, 16, 4, false, 2, false)    \
    X(17, "ws_m16n16_w16_t16", 16, 1, 1, 16, 8, false, 2, false)    \
    X(18, "ws_m32n32_w16_t16", 16, 2, 2, 16, 4, false, 2, false)    \
    X(19, "ws_m64n16_w16_t16", 16, 4, 1, 16, 4, false, 2, false)    \
    X(20, "ws_m32n16_w8_t16", 16, 2, 1, 8, 4, false, 2, false)      \
    X(21, "ws_m32n16_w4_t16", 16, 2, 1, 4, 8, false, 2, false)      \
    X(22, "ws_m32n32_w16_t32", 32, 1, 1, 16, 8, false, 2, false)    \
    X(23, "ws_m16n32_w16_t16", 16, 1, 2, 16, 4, false, 2, false)    \
    X(24, "wq_m32n16_w16_t16", 16, 2, 1, 16, 4, true, 2, false)     \
    X(25, "wq_m32n16_w8_t16", 16, 2, 1, 8, 4, true, 2, false)       \
    X(26, "wq_m32n32_w16_t16", 16, 2, 2, 16, 4, true, 2, false)     \
    X(27, "wq_m16n16_w16_t16", 16, 1, 1, 16, 4, true, 2, false)     \
    X(28, "wq_m64n16_w8_t16", 16, 4, 1, 8, 4, true, 2, false)       \
    X(29, "wq_m64n32_w8_t16", 16, 4, 2, 8, 4, true, 2, false)       \
    X(30, "wq_m64n64_w4_t16", 16, 4, 4, 4, 4, true, 2, false)       \
    X(31, "wq_m64n32_w4_t16", 16, 4, 2, 4, 4, true, 2, false)       \
    X(32, "wq_m32n32_w8_t16", 16, 2, 2, 8, 4, true, 2, false)       \
    X(33, "wq_m64n64_w4_t32", 32, 2, 2, 4, 8, true, 2, false)       \
    X(34, "wq_m16n16_w16_t16_d4", 16, 1, 1, 16, 4, true, 4, false) \
    X(35, "wq_m32n16_w8_t16_d4", 16, 2, 1, 8, 4, true, 4, false)   \
    X(36, "wq_m32n16_w16_t16_d4", 16, 2, 1, 16, 4, true, 4, false) \
    X(37, "wq_m16n16_w8_t16_d4", 16, 1, 1, 8, 4, true, 4, false)   \
    X(38, "wq_m32n32_w4_t16", 16, 2, 2, 4, 4, true, 2, false)      \
    X(39, "wq_m32n32_w2_t16_d4", 16, 2, 2, 2, 4, true, 4, false)   \
    X(40, "wq_m64n32_w2_t16", 16, 4, 2, 2, 4, true, 2, false)      \
    X(41, "wq_m32n64_w4_t16", 16, 2, 4, 4, 4, true, 2, false)      \
    X(42, "wq_m64n32_w4_t16_d4", 16, 4, 2, 4, 4, true, 4, false) \
    X(43, "wb_m16n16_w16", 16, 1, 1, 16, 4, true, 2, true)    \
    X(44, "wb_m16n16_w8_d4", 16, 1, 1, 8, 4, true, 4, true)   \
    X(45, "wb_m32n16_w8", 16, 2, 1, 8, 4, true, 2, true)      \
    X(46, "wb_m32n16_w16", 16, 2, 1, 16, 4, true, 2, true)    \
    X(47, "wb_m32n32_w8", 16, 2, 2, 8, 4, true, 2, true)      \
    X(48, "wb_m32n32_w4_d4", 16, 2, 2, 4, 4, true, 4, true)   \
    X(49, "wb_m64n16_w8", 16, 4, 1, 8, 4, true, 2, true)      \
    X(50, "wb_m64n32_w8", 16, 4, 2, 8, 4, true, 2, true)      \
    X(51, "wb_m64n32_w4_d4", 16, 4, 2, 4, 4, true, 4, true)   \
    X(52, "wb_m64n64_w4", 16, 4, 4, 4, 4, true, 2, true)
// X(index, name, MT, TM, TN, NW, U, QUAD, D, BF16): wave-split configurations with channels padded to 4
#define IOS_WSPLIT_C4_VARIANTS(X)                                \
    X(53, "ws_m32n32_w1_t16_c4", 16, 2, 2, 1, 4, false, 2, false) \
    X(54, "ws_m32n64_w1_t16_c4", 16, 2, 4, 1, 4, false, 2, false) \
    X(55, "ws_m32n32_w2_t16_c4", 16, 2, 2, 2, 4, false, 2, false) \
    X(56, "ws_m32n16_w4_t16_c4", 16, 2, 1, 4, 4, false, 2, false)
// X(index, name, MT, TM, TN, NW, U, QUAD, D, BF16): quad-load wave-split configurations on the 32 x 32 x 2 MFMA.  A
// wavefront's input load covers two channels x 32 consecutive pixels (two full 128-byte lines) instead of four
// channels x 16 pixels, and the instruction's ceiling is higher than that of the 16 x 16 x 4 form.
#define IOS_WSPLIT_T32_VARIANTS(X)                                   \
    X(57, "wq_m32n32_w8_t32", 32, 1, 1, 8, 8, true, 2, false)        \
    X(58, "wq_m32n32_w16_t32", 32, 1, 1, 16, 8, true, 2, false)      \
    X(59, "wq_m32n32_w4_t32", 32, 1, 1, 4, 8, true, 2, false)        \
    X(60, "wq_m64n32_w8_t32", 32, 2, 1, 8, 8, true, 2, false)        \
    X(61, "wq_m64n32_w4_t32", 32, 2, 1, 4, 8, true, 2, false)        \
    X(62, "wq_m32n64_w8_t32", 32, 1, 2, 8, 8, true, 2, false)        \
    X(63, "wq_m32n64_w4_t32", 32, 1, 2, 4, 8, true, 2, false)        \
    X(64, "wq_m64n64_w8_t32", 32, 2, 2, 8, 8, true, 2, false)        \
    X(65, "wq_m32n32_w8_t32_u4", 32, 1, 1, 8, 4, true, 2, false)     \
    X(66, "wq_m64n32_w8_t32_u4", 32, 2, 1, 8, 4, true, 2, false)     \
    X(67, "wq_m64n64_w4_t32_u4", 32, 2, 2, 4, 4, true, 2, false)     \
    X(68, "wq_m64n32_w4_t32_u4_d4", 32, 2, 1, 4, 4, true, 4, false)
// X(index, name, MT, TM, TN, NW, U, QUAD, D, RP): the reduced-precision configurations once more with IEEE half operands
// (RP = 2, option precision=fp16), the literal counterpart of the reference's USE_FLOAT16 build
#define IOS_WSPLIT_F16_VARIANTS(X)                          \
    X(69, "wh_m16n16_w16", 16, 1, 1, 16, 4, true, 2, 2)     \
    X(70, "wh_m16n16_w8_d4", 16, 1, 1, 8, 4, true, 4, 2)    \
    X(71, "wh_m32n16_w8", 16, 2, 1, 8, 4, true, 2, 2)       \
    X(72, "wh_m32n16_w16", 16, 2, 1, 16, 4, true, 2, 2)     \
    X(73, "wh_m32n32_w8", 16, 2, 2, 8, 4, true, 2, 2)       \
    X(74, "wh_m32n32_w4_d4", 16, 2, 2, 4, 4, true, 4, 2)    \
    X(75, "wh_m64n16_w8", 16, 4, 1, 8, 4, true, 2, 2)       \
    X(76, "wh_m64n32_w8", 16, 4, 2, 8, 4, true, 2, 2)       \
    X(77, "wh_m64n32_w4_d4", 16, 4, 2, 4, 4, true, 4, 2)    \
    X(78, "wh_m64n64_w4", 16, 4, 4, 4, 4, true, 2, 2)
// X(index, name, MT, TM, TN, NW, U, QUAD, D, RP): quad-load configurations with one or two wavefronts per output tile, for
// layers with many pixels and a short K (the first layers of an image network at batch 1, everything at large batches):
// a wavefront walks (half of) K by itself, its next batch's loads in flight under this batch's matrix instructions
#define IOS_WSPLIT_LONGK_VARIANTS(X)                                  \
    X(79, "wq_m32n32_w1_t32", 32, 1, 1, 1, 8, true, 2, 0)             \
    X(80, "wq_m32n32_w2_t32", 32, 1, 1, 2, 8, true, 2, 0)             \
    X(81, "wq_m64n32_w2_t32", 32, 2, 1, 2, 8, true, 2, 0)             \
    X(82, "wq_m64n32_w1_t32", 32, 2, 1, 1, 8, true, 2, 0)             \
    X(83, "wq_m32n64_w2_t32", 32, 1, 2, 2, 8, true, 2, 0)             \
    X(84, "wq_m32n32_w2_t32_d4", 32, 1, 1, 2, 8, true, 4, 0)          \
    X(85, "wq_m64n32_w2_t32_u4_d4", 32, 2, 1, 2, 4, true, 4, 0)       \
    X(86, "wq_m32n32_w1_t16_d4", 16, 2, 2, 1, 4, true, 4, 0)          \
    X(87, "wq_m64n32_w1_t16", 16, 4, 2, 1, 4, true, 2, 0)             \
    X(88, "wq_m64n64_w2_t32", 32, 2, 2, 2, 8, true, 2, 0)
// X(index, name, TMW, TNW, WM, WN, PD): the LDS-tiled kernel with operands split into three bfloat16 terms (ConvSplit3);
// TMW x TNW tiles of 32 x 32 per wavefront, WM x WN wavefronts
#define IOS_SPLIT3_VARIANTS(X)                     \
    X(89, "x3_m64n128_w2x2", 1, 2, 2, 2, 2)        \
    X(90, "x3_m64n128_w2x2_p3", 1, 2, 2, 2, 3)     \
    X(91, "x3_m64n256_w2x4", 1, 2, 2, 4, 2)        \
    X(92, "x3_m64n64_w2x2", 1, 1, 2, 2, 2)         \
    X(93, "x3_m64n64_w1x1", 2, 2, 1, 1, 2)         \
    X(94, "x3_m64n128_w1x2", 2, 2, 1, 2, 2)        \
    X(95, "x3_m128n64_w4x1", 1, 2, 4, 1, 2)        \
    X(96, "x3_m128n128_w4x2", 1, 2, 4, 2, 2)       \
    X(97, "x3_m192n128_w6x2", 1, 2, 6, 2, 2)
// X(index, name, TM, TN, NW, D): wave-split configurations with operands split into three bfloat16 terms (ConvWsplit, RP = 3),
// 32 x 32 x 16 tiles, 16 k per batch
#define IOS_WSPLIT_X3_VARIANTS(X)            \
    X(98, "x3w_m32n32_w8", 1, 1, 8, 2)       \
    X(99, "x3w_m32n32_w4", 1, 1, 4, 2)       \
    X(100, "x3w_m32n32_w16", 1, 1, 16, 2)    \
    X(101, "x3w_m64n32_w8", 2, 1, 8, 2)      \
    X(102, "x3w_m64n32_w4", 2, 1, 4, 2)      \
    X(103, "x3w_m32n64_w4", 1, 2, 4, 2)      \
    X(104, "x3w_m32n64_w8", 1, 2, 8, 2)      \
    X(105, "x3w_m64n64_w4", 2, 2, 4, 2)      \
    X(106, "x3w_m64n32_w2", 2, 1, 2, 2)
// X(index, name, TMW, TNW, WM, WN, PD): ConvSplit3 with one rounded term (option precision=bf16), up to 64 x 64 per wavefront
#define IOS_SPLIT1_VARIANTS(X)                      \
    X(107, "wb_x1_m64n128_w2x2", 1, 2, 2, 2, 2)     \
    X(108, "wb_x1_m128n128_w2x2", 2, 2, 2, 2, 2)    \
    X(109, "wb_x1_m128n256_w2x4", 2, 2, 2, 4, 2)    \
    X(110, "wb_x1_m64n128_w1x2", 2, 2, 1, 2, 2)     \
    X(111, "wb_x1_m128n64_w4x1", 1, 2, 4, 1, 2)     \
    X(112, "wb_x1_m64n256_w2x4", 1, 2, 2, 4, 2)
// X(index, name, TM, TN, NW, D): the wave-split kernel with one rounded term (ConvWsplit, RP = 4)
#define IOS_WSPLIT_X1_VARIANTS(X)              \
    X(113, "wb_x1w_m32n32_w4", 1, 1, 4, 2)     \
    X(114, "wb_x1w_m64n32_w4", 2, 1, 4, 2)     \
    X(115, "wb_x1w_m32n64_w4", 1, 2, 4, 2)     \
    X(116, "wb_x1w_m64n64_w4", 2, 2, 4, 2)     \
    X(117, "wb_x1w_m32n32_w8", 1, 1, 8, 2)     \
    X(118, "wb_x1w_m64n64_w2", 2, 2, 2, 2)
constexpr int kNumConvVariants = 119;

}  // namespace ios
