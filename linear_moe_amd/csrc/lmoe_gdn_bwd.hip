// Instantiation and launch of the gated-delta-rule WY backward kernel.
#include "lmoe_launch.hpp"
#include "lmoe_gdn_wy_bwd.hpp"

namespace lmoe {

template <typename T, int K, int V> struct GdnWyBwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    hipLaunchKernelGGL((k_gdn_wy_bwd<T, K, V>), dim3(a.NT, a.H), dim3(NTHR), 0, st, a);
  }
};
void launch_gdn_wy_bwd(const lmoe_args& a, hipStream_t st) { dispatch<GdnWyBwd>(a, st); }

}  // namespace lmoe
