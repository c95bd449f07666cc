// Instantiation and launch of the gated-delta-rule WY preparation kernel.
#include "lmoe_launch.hpp"
#include "lmoe_gdn_wy.hpp"

namespace lmoe {

template <typename T, int K, int V> struct GdnWyFwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    const int grid = persistent_grid(a.NT * a.H, sizeof(T) == 2 ? (a.tinv ? 3 : 2) : 1);
    // (2-byte elements at V = 256 exist with Tinv only: the entry points reject a call without it; w and u of 256
    // columns formed here would cost the kernel its second work-group per CU)
    if (a.tinv || (V > 128 && sizeof(T) == 2)) hipLaunchKernelGGL((k_gdn_wy_fwd<T, K, V, true>), dim3(grid), dim3(NTHR), 0, st, a);
    else if constexpr (V <= 128 || sizeof(T) == 4) hipLaunchKernelGGL((k_gdn_wy_fwd<T, K, V, false>), dim3(grid), dim3(NTHR), 0, st, a);
  }
};
void launch_gdn_wy_fwd(const lmoe_args& a, hipStream_t st) { dispatch_gdn<GdnWyFwd>(a, st); }

}  // namespace lmoe
