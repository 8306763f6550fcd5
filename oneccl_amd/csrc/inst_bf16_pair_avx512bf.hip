// Kernels of one element-traits class: Bf16PairwiseTraits<true, true>
#include "batch_kernels.hpp"
#include "fusion_kernels.hpp"

namespace mi {
// ... and with 7 or 8 inputs the streaming kernel is bound by them, not by loads in flight
template <>
struct StreamUnroll<Bf16PairwiseTraits<true, true>> {
    static constexpr int get(int n) { return n <= 6 ? 4 : 2; }
};
template hipError_t launch_reduce<Bf16PairwiseTraits<true, true>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16PairwiseTraits<true, true>>(const FusionLaunchArgs&);
template hipError_t launch_reduce_batch<Bf16PairwiseTraits<true, true>>(const BatchLaunchArgs&);
}  // namespace mi
