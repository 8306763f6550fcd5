// Kernels of one element-traits class: Fp16NativeTraits
#include "fusion_kernels.hpp"

namespace mi {
template hipError_t launch_reduce<Fp16NativeTraits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Fp16NativeTraits>(const FusionLaunchArgs&);
}  // namespace mi
