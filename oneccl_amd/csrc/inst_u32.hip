// Kernels of one element-traits class: U32Traits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<U32Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U32Traits>(const FusionLaunchArgs&);
}  // namespace mi
