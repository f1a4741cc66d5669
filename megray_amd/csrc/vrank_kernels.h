// Launch entry points of the gfx950 kernels (vrank_kernels.hip).
#pragma once

#include <hip/hip_runtime_api.h>

#include "megray/common.h"
#include "vrank_types.h"

namespace MegRay {
namespace vrank {

// Enqueue one fold launch on `stream`.  hipErrorInvalidValue for a dtype / op without a kernel.
hipError_t launch_fold(const FoldLaunch& launch, DType dtype, ReduceOp op, hipStream_t stream);

// Enqueue one flat fold launch on `stream` (rank count 2, 3, 4 or 8).
hipError_t launch_flat(const FlatLaunch& launch, DType dtype, ReduceOp op, hipStream_t stream);

// Enqueue one element-wise binomial-tree launch on `stream`.
hipError_t launch_tree(const TreeLaunch& launch, DType dtype, ReduceOp op, hipStream_t stream);

// Enqueue one pack launch on `stream`.
hipError_t launch_pack(const PackLaunch& launch, hipStream_t stream);

}  // namespace vrank
}  // namespace MegRay
