// The 512-thread form of the fused stage kernel: see fused_kernel.h.
#include "fused_kernel.h"

#include <cstring>

namespace ios {

void launch_fused_512(const WorkItem *device_items, const WorkItem *host_items, int num_items, const int *first_blocks, int total_blocks, int smem_bytes, hipStream_t stream) {
    const int *b = first_blocks;   // b[1] ... b[7]: first blocks of the items 1 ... 7 (INT_MAX beyond num_items)
    if (host_items) {   // (launch_fused has checked that the items fit the inline form)
        InlineItems inl{};
        memcpy(inl.v, host_items, (size_t)num_items * sizeof(WorkItem));
        hipLaunchKernelGGL(fused_kernel_inline<512>, dim3((unsigned)total_blocks), dim3(512), smem_bytes, stream, num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7], inl);
        return;
    }
    hipLaunchKernelGGL(fused_kernel<512>, dim3((unsigned)total_blocks), dim3(512), smem_bytes, stream, device_items, num_items, b[1], b[2], b[3], b[4],
                       b[5], b[6], b[7]);
}

}  // namespace ios
