// Kernels of one element-traits class: U8Traits
#include "fusion_kernels.hpp"

namespace mi {
// sixteen one-byte accumulators per vector and input: fewer register-staged items at 7 and 8 inputs
template <>
struct FusionPhaseRegs<U8Traits> {
    static constexpr int items(int nt) { return nt <= 6 ? 12 : 6; }
};
template <>
struct MultiPhaseRegs<U8Traits> {
    static constexpr int groups = 5;
};
template hipError_t launch_reduce<U8Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<U8Traits>(const FusionLaunchArgs&);
}  // namespace mi
