// Kernels of one element-traits class: I16Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<I16Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I16Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<I16Traits>(const BatchLaunchArgs&);
}  // namespace mi
