// Kernels of one element-traits class: I32Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<I32Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I32Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<I32Traits>(const BatchLaunchArgs&);
}  // namespace mi
