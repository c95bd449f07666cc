// Instantiation and launch of the sequential passes of the gated delta rule.
#include "lmoe_launch.hpp"
#include "lmoe_gdn_state.hpp"
#include "lmoe_gdn_state_reg.hpp"

namespace lmoe {

// Width of the V-slice a work-group carries: the narrow slice gives more work-groups (a problem
// with few (sequence, head) pairs must still reach every CU); with enough pairs the wide slice
// halves the number of times k, w, q, P are read and stores whole 128-byte lines of o, v_new.
template <typename T, int V> inline bool wide_slices(const lmoe_args& a) {
  constexpr int BW = GdnStateCfg<T>::BV_WIDE;
  return BW <= V && BW != GdnStateCfg<T>::BV && (int64_t)a.N * a.H * (V / BW) >= cu_count();
}
template <typename T, int K, int V, int BV> void launch_fwd(const lmoe_args& a, hipStream_t st) {
  const int grid = ((a.N * a.H + 7) / 8) * 8 * (V / BV);
  // w formed on the chip from Tinv where Tinv is there and LDS has room for a second k tile
  constexpr bool CAN_WT = sizeof(T) == 2;
  const bool wt = CAN_WT && a.tinv != nullptr;
  if constexpr (CAN_WT && BV == 32) {
    if (wt) {       // 2-byte elements with Tinv: the state stays in registers (lmoe_gdn_state_reg.hpp)
      if (a.hs) hipLaunchKernelGGL((k_gdn_state_fwd_reg<K, V, true>), dim3(grid), dim3(3 * NTHR), 0, st, a, (long long*)nullptr, -1);
      else hipLaunchKernelGGL((k_gdn_state_fwd_reg<K, V, false>), dim3(grid), dim3(3 * NTHR), 0, st, a, (long long*)nullptr, -1);
      return;
    }
  }
  // (2-byte elements at V = 256 run with Tinv only, i.e. above: the entry points reject a call without it)
  if constexpr (!(CAN_WT && V > 128)) {
    if (a.hs) {
      if (wt) hipLaunchKernelGGL((k_gdn_state_fwd<T, K, V, BV, true, CAN_WT>), dim3(grid), dim3(3 * NTHR), 0, st, a);
      else hipLaunchKernelGGL((k_gdn_state_fwd<T, K, V, BV, true, false>), dim3(grid), dim3(3 * NTHR), 0, st, a);
    } else {
      if (wt) hipLaunchKernelGGL((k_gdn_state_fwd<T, K, V, BV, false, CAN_WT>), dim3(grid), dim3(3 * NTHR), 0, st, a);
      else hipLaunchKernelGGL((k_gdn_state_fwd<T, K, V, BV, false, false>), dim3(grid), dim3(3 * NTHR), 0, st, a);
    }
  }
}
template <typename T, int K, int V, int BV> void launch_bwd(const lmoe_args& a, hipStream_t st) {
  const int grid = ((a.N * a.H + 7) / 8) * 8 * (V / BV);
  hipLaunchKernelGGL((k_gdn_state_bwd<T, K, V, BV>), dim3(grid), dim3(3 * NTHR), 0, st, a);
}
template <typename T, int K, int V> struct GdnStateFwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BW = GdnStateCfg<T>::BV_WIDE <= V ? GdnStateCfg<T>::BV_WIDE : GdnStateCfg<T>::BV;
    // the register-resident pass is bound by its products, not by latency: twice the columns take twice as long,
    // so it keeps the narrow slice (more work-groups) whatever the problem size
    const bool reg = sizeof(T) == 2 && a.tinv != nullptr;
    if (!reg && wide_slices<T, V>(a)) launch_fwd<T, K, V, BW>(a, st);
    else launch_fwd<T, K, V, GdnStateCfg<T>::BV>(a, st);
  }
};
template <typename T, int K, int V> struct GdnStateBwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BW = GdnStateCfg<T>::BV_WIDE <= V ? GdnStateCfg<T>::BV_WIDE : GdnStateCfg<T>::BV;
    if (wide_slices<T, V>(a)) launch_bwd<T, K, V, BW>(a, st);
    else launch_bwd<T, K, V, GdnStateCfg<T>::BV>(a, st);
  }
};
void launch_gdn_state_fwd(const lmoe_args& a, hipStream_t st) { dispatch_gdn<GdnStateFwd>(a, st); }
// the traced instance of the register-resident forward pass (2-byte elements, K = V = 128, saving call)
bool launch_gdn_state_fwd_trace(const lmoe_args& a, long long* tr, int work_group, hipStream_t st) {
  if (a.dtype != LMOE_BF16 || a.K != 128 || a.V != 128 || !a.tinv || !a.hs) return false;
  const int grid = ((a.N * a.H + 7) / 8) * 8 * (128 / 32);
  if (work_group < 0 || work_group >= grid) return false;
  hipLaunchKernelGGL((k_gdn_state_fwd_reg<128, 128, true, true>), dim3(grid), dim3(3 * NTHR), 0, st, a, tr, work_group);
  return true;
}
void launch_gdn_state_bwd(const lmoe_args& a, hipStream_t st) { dispatch_gdn<GdnStateBwd>(a, st); }

}  // namespace lmoe
