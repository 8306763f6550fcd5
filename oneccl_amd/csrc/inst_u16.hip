// Kernels of one element-traits class: U16Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<U16Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U16Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<U16Traits>(const BatchLaunchArgs&);
}  // namespace mi
