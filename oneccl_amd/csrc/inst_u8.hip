// Kernels of one element-traits class: U8Traits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<U8Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U8Traits>(const FusionLaunchArgs&);
}  // namespace mi
