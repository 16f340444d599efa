// The wide-register family of the fused stage kernel: see fused_kernel.h.
#include "fused_kernel.h"

#include <stdexcept>

namespace ios {

void launch_fused_wide(int threads, const WorkItem *device_items, int num_items, const int *first_blocks, int total_blocks, int smem_bytes, hipStream_t stream) {
    const int *b = first_blocks;   // b[1] ... b[7]: first blocks of the items 1 ... 7 (INT_MAX beyond num_items)
    const dim3 grid((unsigned)total_blocks);
    if (threads == 256)
        hipLaunchKernelGGL(fused_kernel_wide<256>, grid, dim3(256), smem_bytes, stream, device_items, num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7]);
    else if (threads == 512)
        hipLaunchKernelGGL(fused_kernel_wide<512>, grid, dim3(512), smem_bytes, stream, device_items, num_items, b[1], b[2], b[3], b[4], b[5], b[6], b[7]);
    else
        throw std::runtime_error("fused launch: the wide-register kernels come with 256 and 512 threads");
}

}  // namespace ios
