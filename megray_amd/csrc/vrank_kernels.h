// Entry points of the gfx950 kernels (vrank_kernels.hip, vrank_fold_<type>.hip).
#pragma once

#include <hip/hip_runtime_api.h>

#include "megray/common.h"
#include "vrank_types.h"

namespace MegRay {
namespace vrank {

// The kernel that executes a launch descriptor, as a host-side function address usable with
// hipLaunchKernel and hipGraphAddKernelNode; nullptr for a dtype / op without a kernel.
const void* fold_kernel_for(const FoldLaunch& launch, DType dtype, ReduceOp op);
const void* flat_kernel_for(const FlatLaunch& launch, DType dtype, ReduceOp op);  // rank count 2, 3, 4 or 8
const void* tree_kernel_for(const TreeLaunch& launch, DType dtype, ReduceOp op);
const void* pack_kernel_for(const PackLaunch& launch);

// Enqueue `kernel` over `grid` workgroups of `block` threads (one or four wavefronts) with `*launch` as
// its only argument.  `lds` bytes of LDS are reserved per workgroup on top of what the kernel declares (it never
// touches them: fewer workgroups then share a CU).
hipError_t enqueue(const void* kernel, uint32_t grid, uint32_t block, const void* launch, hipStream_t stream,
                   uint32_t lds = 0);

// LDS bytes to reserve per workgroup of `kernel`, on top of what it declares, so that at most `waves_per_cu`
// of its workgroups share a CU (160 KiB of LDS each; for the one-wavefront kernels that is wavefronts per CU, for the
// group forms workgroups of four); 0 if the kernel's own LDS already sees to that.
uint32_t lds_for_waves_per_cu(const void* kernel, uint32_t waves_per_cu);

}  // namespace vrank
}  // namespace MegRay
