// Kernels of one element-traits class: U64Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<U64Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U64Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<U64Traits>(const BatchLaunchArgs&);
}  // namespace mi
