// Kernels of one element-traits class: U64Traits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<U64Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U64Traits>(const FusionLaunchArgs&);
}  // namespace mi
