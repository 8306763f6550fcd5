// Kernels of one element-traits class: I16Traits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<I16Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I16Traits>(const FusionLaunchArgs&);
}  // namespace mi
