// Fused stage launch: several independent device operations in one kernel launch.
//
// On MI355X a fork + join across HIP streams costs tens of microseconds while the batch-1 operators it would
// overlap run for 3-15 us each, so concurrent groups of a stage are expressed as *one* grid: a table of work
// items, each owning a contiguous range of blocks; every block looks up its item and runs that operator's
// device body.  Operators of one group that depend on each other go to consecutive launches ("levels") on
// the same stream, which orders them without any cross-queue synchronisation.
#pragma once

#include "launch_internal.h"

namespace ios {

enum WorkKind : int { WORK_CONV = 0, WORK_REDUCE, WORK_POOL, WORK_GLOBAL_POOL, WORK_DWCONV, WORK_CONV_DIRECT, WORK_NARY };

struct WorkItem {
    int kind;
    int variant, threads;          // convolution kernel configuration and the threads its body uses (<= block size)
    int tiles, groups;             // convolution grid decomposition: block = (tile, group, K slice)
    int first_block, num_blocks;   // range of this item inside the fused grid
    int reserved;
    FastDiv div_tiles, div_groups; // convolution: exact quotients by tiles and by groups without an integer division
    union {   // (a work item spans five 64-byte lines: the kernel requests one word of each with its first load)
        ConvKernelArgs conv;
        ReduceArgs reduce;
        PoolArgs pool;
        DirectConvArgs direct;
        NaryKernelArgs nary;
    };
};

// Passed by value with the launch: a block finds its item from the kernel-argument segment alone (one scalar load,
// no walk through the item table), then reads the item's fields from the table.
static_assert(sizeof(WorkItem) <= 320, "a work item spans at most five 64-byte lines");
constexpr int kMaxFusedItems = 16;    // = groups per stage
constexpr int kFusedHeaderItems = 8;  // the schedule search builds stages of up to 8 groups; wider stages walk the table
struct FusedHeader {
    int num_items;
    int first_block[kFusedHeaderItems];   // ascending; entries beyond num_items are INT_MAX (no block reaches them)
};

// Thread-block sizes the fused kernel is instantiated for.  A launch uses the size of its widest convolution body;
// bodies that need fewer wavefronts let the surplus wavefronts of their blocks end at once (barriers only count
// wavefronts that have not ended), the memory-bound bodies adapt to any block size.
constexpr int kFusedThreadClasses[] = {256, 512, 1024};

// Launch `num_items` items as one grid of `total_blocks` blocks of `threads` threads.  `device_items` is the table in device
// memory; `host_items` (the same items on the host, or null) lets launches that qualify carry their items in the
// kernel-argument segment instead (fused_kernel.h); `num_cus`: compute units of the device.
// The form of the fused kernel a launch of these items (host copies) takes: the items in a table in device memory, or in the
// kernel-argument segment, where one kernel holds the matrix-path convolution bodies and another the depth-wise / direct ones.
// Wide: a convolution item needs the kernel family without a register cap (ConvVariant::needs_wide): items in the table.
enum class FusedForm { Table, InlineMatrix, InlineDirect, Wide };
FusedForm fused_launch_form(const WorkItem *host_items, int num_items, int threads, int total_blocks, int num_cus);
const char *fused_kernel_name(FusedForm form);   // without the block size
void launch_fused(int threads, const WorkItem *device_items, const WorkItem *host_items, const FusedHeader &header, int total_blocks, int smem_bytes, int num_cus, hipStream_t stream);

}  // namespace ios
