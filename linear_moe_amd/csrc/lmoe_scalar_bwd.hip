// Instantiation and launch of the scalar-gate backward kernels.
#include "lmoe_launch.hpp"
#include "lmoe_scalar_bwd.hpp"

namespace lmoe {

template <typename T, int K, int V, bool GDN>
static void launch_scalar_bwd_t(const lmoe_args& a, hipStream_t st) {
  constexpr int BVS = 32;                                      // V-slice of the sequential pass
  constexpr int BVD = (sizeof(T) == 4 && V == 128) ? 64 : V;   // V-slice of k_bwd_dv
  constexpr int BVH = sizeof(T) == 4 ? 32 : 64;                // V-slice loop of k_bwd_dqk
  const dim3 block(NTHR);
  if constexpr (GDN) {
    hipLaunchKernelGGL((k_bwd_dv<T, K, V, BVD, true>), dim3(a.NT, a.H, V / BVD), block, 0, st, a);
    hipLaunchKernelGGL((k_state_bwd<T, K, V, BVS, true>), dim3(V / BVS, a.H, a.N), block, 0, st, a);
  } else {
    hipLaunchKernelGGL((k_state_bwd<T, K, V, BVS, false>), dim3(V / BVS, a.H, a.N), block, 0, st, a);
    hipLaunchKernelGGL((k_bwd_dv<T, K, V, BVD, false>), dim3(a.NT, a.H, V / BVD), block, 0, st, a);
  }
  hipLaunchKernelGGL((k_bwd_dqk<T, K, V, BVH, GDN>), dim3(a.NT, a.H), block, 0, st, a);
}

template <typename T, bool GDN>
static void launch_scalar_bwd_kv(const lmoe_args& a, hipStream_t st) {
  if (a.K == 64 && a.V == 64) launch_scalar_bwd_t<T, 64, 64, GDN>(a, st);
  else if (a.K == 64 && a.V == 128) launch_scalar_bwd_t<T, 64, 128, GDN>(a, st);
  else if (a.K == 128 && a.V == 64) launch_scalar_bwd_t<T, 128, 64, GDN>(a, st);
  else launch_scalar_bwd_t<T, 128, 128, GDN>(a, st);
}

void launch_scalar_bwd(const lmoe_args& a, bool gdn, hipStream_t st) {
  if (a.dtype == LMOE_BF16) {
    if (gdn) launch_scalar_bwd_kv<bf16, true>(a, st); else launch_scalar_bwd_kv<bf16, false>(a, st);
  } else {
    if (gdn) launch_scalar_bwd_kv<float, true>(a, st); else launch_scalar_bwd_kv<float, false>(a, st);
  }
}

}  // namespace lmoe
