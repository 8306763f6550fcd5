// Kernels of one element-traits class: U8Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<U8Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U8Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<U8Traits>(const BatchLaunchArgs&);
}  // namespace mi
