// Instantiation and launch of the gated-delta-rule WY backward kernel.
#include "lmoe_launch.hpp"
#include "lmoe_gdn_wy_bwd.hpp"

namespace lmoe {

template <typename T>
static void launch_gdn_wy_bwd_t(const lmoe_args& a, hipStream_t st) {
  const dim3 grid(a.NT, a.H), block(NTHR);
  if (a.K == 64 && a.V == 64) hipLaunchKernelGGL((k_gdn_wy_bwd<T, 64, 64>), grid, block, 0, st, a);
  else if (a.K == 64 && a.V == 128) hipLaunchKernelGGL((k_gdn_wy_bwd<T, 64, 128>), grid, block, 0, st, a);
  else if (a.K == 128 && a.V == 64) hipLaunchKernelGGL((k_gdn_wy_bwd<T, 128, 64>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((k_gdn_wy_bwd<T, 128, 128>), grid, block, 0, st, a);
}

void launch_gdn_wy_bwd(const lmoe_args& a, hipStream_t st) {
  if (a.dtype == LMOE_BF16) launch_gdn_wy_bwd_t<bf16>(a, st);
  else launch_gdn_wy_bwd_t<float>(a, st);
}

}  // namespace lmoe
