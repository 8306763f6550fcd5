// Kernels of one element-traits class: I32Traits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<I32Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I32Traits>(const FusionLaunchArgs&);
}  // namespace mi
