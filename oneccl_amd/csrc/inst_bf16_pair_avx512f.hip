// Kernels of one element-traits class: Bf16PairwiseTraits<false, true>
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Bf16PairwiseTraits<false, true>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16PairwiseTraits<false, true>>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<Bf16PairwiseTraits<false, true>>(const BatchLaunchArgs&);
}  // namespace mi
