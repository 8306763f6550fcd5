// Kernels of one element-traits class: Bf16PairwiseTraits<false, false>
#include "fusion_kernels.hpp"

namespace mi {
// the truncating narrowing works element by element: with eight inputs one register item fewer fits
template <>
struct FusionPhaseRegs<Bf16PairwiseTraits<false, false>> {
    static constexpr int items(int nt) { return nt <= 7 ? 12 : 11; }
};
template hipError_t launch_reduce<Bf16PairwiseTraits<false, false>>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<Bf16PairwiseTraits<false, false>>(const FusionLaunchArgs&);
}  // namespace mi
