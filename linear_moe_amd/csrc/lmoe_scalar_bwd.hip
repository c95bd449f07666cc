// Instantiation and launch of the backward kernels of chunk_simple_gla.
#include "lmoe_launch.hpp"
#include "lmoe_scalar_bwd.hpp"

namespace lmoe {

template <typename T, int V> struct BwdTiles {
  static constexpr int BVS = sizeof(T) == 4 ? 16 : 32;                // V-slice of the sequential pass
  static constexpr int BVD = V == 128 ? 64 : V;                       // V-slice of k_bwd_dv (LDS for 2-3 work-groups per CU)
  static constexpr int BVH = sizeof(T) == 4 ? 32 : 64;                // V-slice loop of k_bwd_dqk
};

template <bool LOCAL> struct BwdDv {
  template <typename T, int K, int V> struct F {
    static void run(const lmoe_args& a, hipStream_t st) {
      constexpr int BV = BwdTiles<T, V>::BVD;
      hipLaunchKernelGGL((k_bwd_dv<T, K, V, BV, LOCAL>), dim3(a.NT, a.H, V / BV), dim3(NTHR), 0, st, a);
    }
  };
};
template <typename T, int K, int V> struct StateBwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BV = BwdTiles<T, V>::BVS;
    // 64-wide slices where they still fill the chip (2-byte elements): every V slice of a (sequence, head) fetches all
    // of q and k, so two wide slices ask the memory system for less per output column than four narrow ones; a state
    // element is the same sum over the tokens in either split
    constexpr int BW = (sizeof(T) == 2 && V >= 64) ? 64 : BV;
    if (BW != BV && (int64_t)a.N * a.H * (V / BW) >= cu_count()) {
      launch<BW>(a, st);
      return;
    }
    launch<BV>(a, st);
  }
  template <int BVX> static void launch(const lmoe_args& a, hipStream_t st) {
    const dim3 grid(((a.N * a.H + 7) / 8) * 8 * (V / BVX)), block(2 * NTHR);
    if constexpr (sizeof(T) == 2) {        // the pass behind the normalised output exists for 2-byte elements
      if (a.normalize == 1) {
        hipLaunchKernelGGL((k_state_bwd<T, K, V, BVX, 1>), grid, block, 0, st, a);
        return;
      }
      if (a.normalize == 2) {
        hipLaunchKernelGGL((k_state_bwd<T, K, V, BVX, 2>), grid, block, 0, st, a);
        return;
      }
    }
    hipLaunchKernelGGL((k_state_bwd<T, K, V, BVX>), grid, block, 0, st, a);
  }
};
template <typename T, int K, int V> struct BwdDqk {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BVH = BwdTiles<T, V>::BVH;
    const int grid = persistent_grid(a.NT * a.H, 1);
    if constexpr (sizeof(T) == 2) {
      if (a.normalize == 1) hipLaunchKernelGGL((k_bwd_dqkv<T, K, V, BVH, 1>), dim3(grid), dim3(2 * NTHR), 0, st, a);
      else if (a.normalize == 2) hipLaunchKernelGGL((k_bwd_dqkv<T, K, V, BVH, 2>), dim3(grid), dim3(2 * NTHR), 0, st, a);
      else hipLaunchKernelGGL((k_bwd_dqkv<T, K, V, BVH>), dim3(grid), dim3(2 * NTHR), 0, st, a);
    } else {
      hipLaunchKernelGGL((k_bwd_dqk<T, K, V, BVH>), dim3(grid), dim3(2 * NTHR), 0, st, a);
    }
  }
};

void launch_bwd_dv(const lmoe_args& a, bool local, hipStream_t st) {
  if (local) dispatch<BwdDv<true>::F>(a, st); else dispatch<BwdDv<false>::F>(a, st);
}
void launch_state_bwd(const lmoe_args& a, hipStream_t st) { dispatch<StateBwd>(a, st); }
void launch_bwd_dqk(const lmoe_args& a, hipStream_t st) { dispatch<BwdDqk>(a, st); }

}  // namespace lmoe
