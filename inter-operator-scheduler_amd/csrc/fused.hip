// The fused stage kernel: see fused.h.
#include "fused_kernel.h"

#include <climits>
#include <cstring>
#include <stdexcept>

namespace ios {

FusedForm fused_launch_form(const WorkItem *host_items, int num_items, int threads, int total_blocks, int num_cus) {
    if (host_items)
        for (int i = 0; i < num_items; i++)
            if (host_items[i].kind == WORK_CONV && conv_variant(host_items[i].variant).needs_wide()) return FusedForm::Wide;
    if (!host_items || num_items > kInlineItems) return FusedForm::Table;
    bool matrix = false, direct = false;
    for (int i = 0; i < num_items; i++) {
        matrix = matrix || host_items[i].kind == WORK_CONV;
        direct = direct || host_items[i].kind == WORK_DWCONV || host_items[i].kind == WORK_CONV_DIRECT;
    }
    if (!direct) return FusedForm::InlineMatrix;
    // the kernel with the direct bodies holds four wavefronts per SIMD: for launches of 256 threads that fit the device at once
    if (!matrix && threads == 256 && total_blocks <= 4 * num_cus) return FusedForm::InlineDirect;
    return FusedForm::Table;
}

const char *fused_kernel_name(FusedForm form) {
    return form == FusedForm::Table ? "fused_kernel" : form == FusedForm::InlineMatrix ? "fused_kernel_inline"
           : form == FusedForm::InlineDirect ? "fused_kernel_inline_direct" : "fused_kernel_wide";
}

void launch_fused(int threads, const WorkItem *device_items, const WorkItem *host_items, const FusedHeader &header, int total_blocks, int smem_bytes, int num_cus, hipStream_t stream) {
    if (header.num_items < 1 || header.num_items > kMaxFusedItems || total_blocks < 1) throw std::runtime_error("fused launch: bad item count");
    const dim3 grid((unsigned)total_blocks);
    static_assert(kFusedHeaderItems == 8, "the kernel takes seven first-block arguments");
    int b[kFusedHeaderItems];
    for (int i = 0; i < kFusedHeaderItems; i++) b[i] = i < header.num_items ? header.first_block[i] : INT_MAX;
    const FusedForm form = fused_launch_form(host_items, header.num_items, threads, total_blocks, num_cus);
    if (form == FusedForm::Wide) {
        launch_fused_wide(threads, device_items, header.num_items, b, total_blocks, smem_bytes, stream);
        return;
    }
    if (form == FusedForm::Table) host_items = nullptr;
    if (host_items && threads != 512) {
        InlineItems inl{};
        memcpy(inl.v, host_items, (size_t)header.num_items * sizeof(WorkItem));
        if (form == FusedForm::InlineDirect)
            hipLaunchKernelGGL(fused_kernel_inline_direct<256>, grid, dim3(256), smem_bytes, stream, header.num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7], inl);
        else if (threads == 256)
            hipLaunchKernelGGL(fused_kernel_inline<256>, grid, dim3(256), smem_bytes, stream, header.num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7], inl);
        else if (threads == 1024)
            hipLaunchKernelGGL(fused_kernel_inline<1024>, grid, dim3(1024), smem_bytes, stream, header.num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7], inl);
        else
            throw std::runtime_error("fused launch: unsupported block size");
        return;
    }
    switch (threads) {
        case 256:
            hipLaunchKernelGGL(fused_kernel<256>, grid, dim3(256), smem_bytes, stream, device_items, header.num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7]);
            break;
        case 512: launch_fused_512(device_items, host_items, header.num_items, b, total_blocks, smem_bytes, stream); break;
        case 1024:
            hipLaunchKernelGGL(fused_kernel<1024>, grid, dim3(1024), smem_bytes, stream, device_items, header.num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7]);
            break;
        default: throw std::runtime_error("fused launch: unsupported block size");
    }
}

}  // namespace ios
