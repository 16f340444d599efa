// The fused stage kernel itself (see fused.h), shared by the translation units that instantiate it: the 512-thread form,
// which holds most convolution levels, is compiled on its own with other scheduler settings (fused_512.hip, build.sh).
#pragma once

#include "fused.h"

namespace ios {

// One block of a fused launch: the body of `item`.  MATRIX / DIRECT: the matrix-path convolution bodies / the depth-wise and
// direct convolution bodies are part of the kernel.
// WIDE: the kernel also holds the three-term wave-split bodies (fused_kernel_wide, no cap on registers).
template <int T, bool MATRIX = true, bool DIRECT = true, bool WIDE = false>
__device__ __forceinline__ void fused_item(const WorkItem &item, const int bid, float *smem) {
    // An item spans five 64-byte lines of the scalar cache, and the bodies read its fields in two or three dependent steps
    // (kind, then configuration, then arguments): one word of every line is requested together with the first step, so
    // that the later steps find their lines in the cache instead of paying a miss each.  The comparison below never
    // holds (first_block is not negative) and only keeps the compiler from dropping the loads.
    {
        const int *words = reinterpret_cast<const int *>(&item);
        int touched = 0;
#pragma unroll
        for (int line = 1; line * 16 < (int)(sizeof(WorkItem) / sizeof(int)); line++) touched |= words[line * 16];
        if (item.first_block == -1 && touched == 0x5a5a5a5a) return;
    }
    const int local = bid - item.first_block;
    const int num_blocks = item.num_blocks;
    switch (item.kind) {
        case WORK_CONV: {
            if constexpr (!MATRIX) return;
            if ((int)threadIdx.x >= item.threads) return;   // surplus wavefronts of a narrower body
            const ConvKernelArgs &a = item.conv;   // fields are fetched with scalar loads where they are used
            int tile, z, g;
            if (a.xcd_local) {   // blocks numbered so that the K slices of a tile share an XCD (the XCD follows from bid)
                const XcdSlot slot = xcd_enter(a, bid, local);
                if (slot.idle) return;
                tile = slot.tile;
                z = slot.slice;
                g = 0;
            } else {
                const int rest = (int)fast_div((unsigned)local, item.div_tiles);
                tile = local - rest * item.tiles;
                z = (int)fast_div((unsigned)rest, item.div_groups);
                g = rest - z * item.groups;
            }
            switch (item.variant) {
#define IOS_CASE_TILED(IDX, NAME, BM, BN, BK, WM, WN, WK, MT, PD)                                          \
    case IDX:                                                                                              \
        if constexpr (64 * WM * WN * WK <= T && ConvTiled<BM, BN, BK, WM, WN, WK, MT, PD>::FUSABLE)                   \
            ConvTiled<BM, BN, BK, WM, WN, WK, MT, PD>::run(a, smem, tile, g, z);                                      \
        break;
#define IOS_CASE_WSPLIT(IDX, NAME, MT, TM, TN, NW, U, QUAD, D, BF16)                                        \
    case IDX:                                                                                      \
        if constexpr (64 * NW <= T && ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16>::FUSABLE)              \
            ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16>::run(a, smem, tile, g, z);                       \
        break;
#define IOS_CASE_WSPLIT_C4(IDX, NAME, MT, TM, TN, NW, U, QUAD, D, BF16)                                     \
    case IDX:                                                                                      \
        if constexpr (64 * NW <= T && ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16, 4>::FUSABLE)           \
            ConvWsplit<MT, TM, TN, NW, U, QUAD, D, BF16, 4>::run(a, smem, tile, g, z);                    \
        break;
#define IOS_CASE_X3(IDX, NAME, TM, TN, NW, D)                                                         \
    case IDX:                                                                                      \
        if constexpr (WIDE && 64 * NW <= T && ConvWsplit<32, TM, TN, NW, 8, true, D, 3>::FUSABLE_WIDE)   \
            ConvWsplit<32, TM, TN, NW, 8, true, D, 3>::run(a, smem, tile, g, z);                   \
        break;
                IOS_WSPLIT_X3_VARIANTS(IOS_CASE_X3)
#undef IOS_CASE_X3
                IOS_TILED_VARIANTS(IOS_CASE_TILED)
                IOS_WSPLIT_VARIANTS(IOS_CASE_WSPLIT)
                IOS_WSPLIT_C4_VARIANTS(IOS_CASE_WSPLIT_C4)
                IOS_WSPLIT_T32_VARIANTS(IOS_CASE_WSPLIT)
                IOS_WSPLIT_F16_VARIANTS(IOS_CASE_WSPLIT)
                IOS_WSPLIT_LONGK_VARIANTS(IOS_CASE_WSPLIT)
#undef IOS_CASE_WSPLIT_C4
#undef IOS_CASE_TILED
#undef IOS_CASE_WSPLIT
                default: break;
            }
            break;
        }
        case WORK_REDUCE: {
            const ReduceArgs a = item.reduce;
            splitk_reduce_body(a, local, num_blocks, T);
            break;
        }
        case WORK_POOL: {
            const PoolArgs a = item.pool;
            pool_body(a, local, num_blocks, T);
            break;
        }
        case WORK_GLOBAL_POOL: {
            const PoolArgs a = item.pool;
            global_pool_body(a, local, num_blocks, T);
            break;
        }
        case WORK_DWCONV: {
            if constexpr (DIRECT) dwconv_dispatch(item.direct, local, num_blocks, T);   // (the table of summed inputs is read in place)
            break;
        }
        case WORK_CONV_DIRECT: {
            if constexpr (DIRECT) {
                const DirectConvArgs a = item.direct;
                conv_direct_body(a, local, num_blocks, T);
            }
            break;
        }
        case WORK_NARY: {
            nary_dispatch(item.nary, local, num_blocks, T);   // read in place: the source table is indexed dynamically
            break;
        }
        default: break;
    }
}

template <int T>
__device__ __forceinline__ int fused_item_index(const WorkItem *items, int bid, int num_items, int b1, int b2, int b3, int b4, int b5, int b6, int b7) {
    FusedHeader header;
    header.num_items = num_items;
    header.first_block[0] = 0;
    header.first_block[1] = b1; header.first_block[2] = b2; header.first_block[3] = b3; header.first_block[4] = b4;
    header.first_block[5] = b5; header.first_block[6] = b6; header.first_block[7] = b7;
    int index = 0;   // number of further items that start at or before this block
    if (header.num_items <= kFusedHeaderItems) {
#pragma unroll
        for (int i = 1; i < kFusedHeaderItems; i++) index += bid >= header.first_block[i] ? 1 : 0;   // unused entries are INT_MAX
    } else {
        while (index + 1 < header.num_items && bid >= items[index + 1].first_block) index++;
    }
    return index;
}

// The first blocks of the items travel as scalar kernel arguments (b1 ... b7; item 0 starts at block 0): with
// -amdgpu-kernarg-preload-count the command processor hands them to a wavefront in registers, so a block knows its item
// without a load and its first load is the item itself.
template <int T>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(6))) void fused_kernel(const WorkItem *__restrict__ items, int num_items, int b1, int b2,
                                                                                            int b3, int b4, int b5, int b6, int b7) {
    extern __shared__ floatx4 fused_smem[];
    float *smem = reinterpret_cast<float *>(fused_smem);
    const int bid = blockIdx.x;
    const int index = fused_item_index<T>(items, bid, num_items, b1, b2, b3, b4, b5, b6, b7);
    fused_item<T>(items[index], bid, smem);
}

// The same kernel with the items of the launch inside the kernel-argument segment instead of a table in device memory: a
// block's first load (its item) then hits, where the table costs a miss all the way to memory at the start of every launch
// (the caches do not keep it from one launch to the next): 1.0 % of an Inception-v3 pass, 1.2 % of NASNet-A mobile, 2 % of
// SqueezeNet 1.1 in same-device A/B runs.  With the items there the compiler loads all eight source descriptors of the
// summing depth-wise body ahead of its loop, which does not fit beside the matrix-path bodies in 80 registers, so the form
// comes as two kernels: fused_kernel_inline holds the matrix-path convolution bodies and no depth-wise / direct ones,
// fused_kernel_inline_direct the other way round with four wavefronts per SIMD (another 1.9 % of NASNet-A mobile).
// fused_launch_form() chooses.
constexpr int kInlineItems = 8;
struct alignas(64) InlineItems { WorkItem v[kInlineItems]; };
constexpr unsigned kInlineItemsOffset = 64;   // eight ints, then the items at the next multiple of their alignment
static_assert(8 * sizeof(int) <= kInlineItemsOffset && alignof(InlineItems) == kInlineItemsOffset, "layout of the kernel-argument segment");

template <int T, bool MATRIX>
__device__ __forceinline__ void fused_inline_block(int b1, int b2, int b3, int b4, int b5, int b6, int b7) {
    extern __shared__ floatx4 fused_smem[];
    float *smem = reinterpret_cast<float *>(fused_smem);
    const int bid = blockIdx.x;
    int index = 0;   // unused starts are INT_MAX
    index += bid >= b1 ? 1 : 0; index += bid >= b2 ? 1 : 0; index += bid >= b3 ? 1 : 0; index += bid >= b4 ? 1 : 0;
    index += bid >= b5 ? 1 : 0; index += bid >= b6 ? 1 : 0; index += bid >= b7 ? 1 : 0;
    // The item is read in place, through the segment's address: indexing the by-value parameter would copy all of it to
    // scratch memory first.
    typedef const WorkItem __attribute__((address_space(4))) *ConstantItem;
    unsigned long long address = (unsigned long long)__builtin_amdgcn_kernarg_segment_ptr() + kInlineItemsOffset;
    asm volatile("" : "+s"(address));
    address += (unsigned)__builtin_amdgcn_readfirstlane(index) * (unsigned)sizeof(WorkItem);
    fused_item<T, MATRIX, !MATRIX>(*(const WorkItem *)(ConstantItem)address, bid, smem);
}

template <int T>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(6))) void fused_kernel_inline(int num_items, int b1, int b2, int b3, int b4, int b5, int b6,
                                                                                                   int b7, const InlineItems inl) {
    fused_inline_block<T, true>(b1, b2, b3, b4, b5, b6, b7);
}

template <int T>
__global__ __launch_bounds__(T) __attribute__((amdgpu_waves_per_eu(4))) void fused_kernel_inline_direct(int num_items, int b1, int b2, int b3, int b4, int b5,
                                                                                                          int b6, int b7, const InlineItems inl) {
    fused_inline_block<T, false>(b1, b2, b3, b4, b5, b6, b7);
}

// The family with room for the three-term wave-split bodies: no cap on registers (its heaviest body takes ~155, three
// wavefronts per SIMD), every other body as well, items in the table.  For parallel stages at batch 16 and more, where those
// bodies are the fastest convolution kernels and the launches run long enough for the lower occupancy not to matter.
template <int T>
__global__ __launch_bounds__(T) void fused_kernel_wide(const WorkItem *__restrict__ items, int num_items, int b1, int b2, int b3, int b4, int b5, int b6,
                                                        int b7) {
    extern __shared__ floatx4 fused_smem[];
    float *smem = reinterpret_cast<float *>(fused_smem);
    const int bid = blockIdx.x;
    const int index = fused_item_index<T>(items, bid, num_items, b1, b2, b3, b4, b5, b6, b7);
    fused_item<T, true, true, true>(items[index], bid, smem);
}

// fused_wide.hip (256 and 512 threads)
void launch_fused_wide(int threads, const WorkItem *device_items, int num_items, const int *first_blocks, int total_blocks, int smem_bytes, hipStream_t stream);

// fused_512.hip
void launch_fused_512(const WorkItem *device_items, const WorkItem *host_items, int num_items, const int *first_blocks, int total_blocks, int smem_bytes, hipStream_t stream);

}  // namespace ios
