// Kernels of one element-traits class: Bf16KeepTraits<false>
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Bf16KeepTraits<false>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16KeepTraits<false>>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<Bf16KeepTraits<false>>(const BatchLaunchArgs&);
}  // namespace mi
