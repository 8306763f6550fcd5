// Kernels of one element-traits class: Bf16KeepTraits<true>
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
template <>
struct HasUnrollVariants<Bf16KeepTraits<true>> {
    static constexpr bool value = true;
};
template hipError_t launch_reduce<Bf16KeepTraits<true>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16KeepTraits<true>>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<Bf16KeepTraits<true>>(const BatchLaunchArgs&);
}  // namespace mi
