// Kernels of one element-traits class: I64Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<I64Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I64Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<I64Traits>(const BatchLaunchArgs&);
}  // namespace mi
