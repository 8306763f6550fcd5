// Kernels of one element-traits class: I8Traits
#include "fusion_kernels.hpp"

namespace mi {
// sixteen one-byte accumulators per vector and input: fewer register-staged items at 7 and 8 inputs
template <>
struct FusionPhaseRegs<I8Traits> {
    static constexpr int items(int nt) { return nt <= 6 ? 12 : 6; }
};
template <>
struct MultiPhaseRegs<I8Traits> {
    static constexpr int groups = 5;
};
template hipError_t launch_reduce<I8Traits>(const LaunchArgs&);
template hipError_t launch_fusion_reduce<I8Traits>(const FusionLaunchArgs&);
}  // namespace mi
