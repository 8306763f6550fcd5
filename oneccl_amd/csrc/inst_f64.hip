// Kernels of one element-traits class: F64Traits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<F64Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<F64Traits>(const FusionLaunchArgs&);
}  // namespace mi
