// Kernels of one element-traits class: Bf16PairwiseTraits<false, true>
#include "fusion_kernels.hpp"

namespace mi {
// the truncating narrowing works element by element: with eight inputs one register item fewer fits
template <>
struct FusionPhaseRegs<Bf16PairwiseTraits<false, true>> {
    static constexpr int items(int nt) { return nt <= 7 ? 12 : 11; }
};
template hipError_t launch_reduce<Bf16PairwiseTraits<false, true>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16PairwiseTraits<false, true>>(const FusionLaunchArgs&);
}  // namespace mi
