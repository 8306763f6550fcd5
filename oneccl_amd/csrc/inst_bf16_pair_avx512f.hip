// Kernels of one element-traits class: Bf16PairwiseTraits<false, true>
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Bf16PairwiseTraits<false, true>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16PairwiseTraits<false, true>>(const FusionLaunchArgs&);
}  // namespace mi
