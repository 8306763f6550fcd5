// Kernels of one element-traits class: Fp16PairwiseTraits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Fp16PairwiseTraits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Fp16PairwiseTraits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<Fp16PairwiseTraits>(const BatchLaunchArgs&);
}  // namespace mi
