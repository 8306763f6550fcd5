// Kernels of one element-traits class: Fp16NativeTraits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Fp16NativeTraits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Fp16NativeTraits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<Fp16NativeTraits>(const BatchLaunchArgs&);
}  // namespace mi
