// Kernels of one element-traits class: I64Traits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<I64Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I64Traits>(const FusionLaunchArgs&);
}  // namespace mi
