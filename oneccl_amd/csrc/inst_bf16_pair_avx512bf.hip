// Kernels of one element-traits class: Bf16PairwiseTraits<true, true>
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Bf16PairwiseTraits<true, true>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16PairwiseTraits<true, true>>(const FusionLaunchArgs&);
}  // namespace mi
