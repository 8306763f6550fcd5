// Kernels of one element-traits class: Bf16PairwiseTraits<false, false>
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Bf16PairwiseTraits<false, false>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16PairwiseTraits<false, false>>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<Bf16PairwiseTraits<false, false>>(const BatchLaunchArgs&);
}  // namespace mi
