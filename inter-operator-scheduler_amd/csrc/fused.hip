// The fused stage kernel: see fused.h.
#include "fused_kernel.h"

#include <climits>
#include <cstring>
#include <stdexcept>

namespace ios {

bool fused_items_inline(const WorkItem *host_items, int num_items) {
    if (!host_items || num_items > kInlineItems) return false;
    for (int i = 0; i < num_items; i++)
        if (host_items[i].kind == WORK_DWCONV || host_items[i].kind == WORK_CONV_DIRECT) return false;   // bodies the inline form leaves out
    return true;
}

void launch_fused(int threads, const WorkItem *device_items, const WorkItem *host_items, const FusedHeader &header, int total_blocks, int smem_bytes, hipStream_t stream) {
    if (header.num_items < 1 || header.num_items > kMaxFusedItems || total_blocks < 1) throw std::runtime_error("fused launch: bad item count");
    const dim3 grid((unsigned)total_blocks);
    static_assert(kFusedHeaderItems == 8, "the kernel takes seven first-block arguments");
    int b[kFusedHeaderItems];
    for (int i = 0; i < kFusedHeaderItems; i++) b[i] = i < header.num_items ? header.first_block[i] : INT_MAX;
    if (!fused_items_inline(host_items, header.num_items)) host_items = nullptr;
    if (host_items && threads != 512) {
        InlineItems inl{};
        memcpy(inl.v, host_items, (size_t)header.num_items * sizeof(WorkItem));
        if (threads == 256)
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
