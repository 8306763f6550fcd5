// Kernels of one element-traits class: F32Traits
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template <>
struct HasUnrollVariants<F32Traits> {
    static constexpr bool value = true;
};
template hipError_t launch_reduce<F32Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<F32Traits>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<F32Traits>(const BatchLaunchArgs&);
}  // namespace mi
