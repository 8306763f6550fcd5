// Kernels of one element-traits class: F64Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<F64Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<F64Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<F64Traits>(const BatchLaunchArgs&);
}  // namespace mi
