// Kernels of one element-traits class: U32Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<U32Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U32Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<U32Traits>(const BatchLaunchArgs&);
}  // namespace mi
