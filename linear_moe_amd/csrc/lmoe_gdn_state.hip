// Instantiation and launch of the sequential passes of the gated delta rule.
#include "lmoe_launch.hpp"
#include "lmoe_gdn_state.hpp"

namespace lmoe {

template <typename T, int K, int V> struct GdnStateFwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BV = GdnStateCfg<T>::BV;
    const int grid = ((a.N * a.H + 7) / 8) * 8 * (V / BV);
    hipLaunchKernelGGL((k_gdn_state_fwd<T, K, V, BV>), dim3(grid), dim3(3 * NTHR), 0, st, a);
  }
};
template <typename T, int K, int V> struct GdnStateBwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BV = GdnStateCfg<T>::BV;
    const int grid = ((a.N * a.H + 7) / 8) * 8 * (V / BV);
    hipLaunchKernelGGL((k_gdn_state_bwd<T, K, V, BV>), dim3(grid), dim3(3 * NTHR), 0, st, a);
  }
};
void launch_gdn_state_fwd(const lmoe_args& a, hipStream_t st) { dispatch<GdnStateFwd>(a, st); }
void launch_gdn_state_bwd(const lmoe_args& a, hipStream_t st) { dispatch<GdnStateBwd>(a, st); }

}  // namespace lmoe
