// Kernels of one element-traits class: I8Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<I8Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I8Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<I8Traits>(const BatchLaunchArgs&);
}  // namespace mi
