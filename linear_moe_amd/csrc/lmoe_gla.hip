// Instantiation and launch of the chunk_gla kernels.
#include "lmoe_launch.hpp"
#include "lmoe_gla.hpp"

namespace lmoe {

template <typename T, int V> struct GlaTiles {
  static constexpr int BVS = 32;                                      // sequential passes
  // ... 64 where that still fills the chip (2-byte elements): the V slices of a (sequence, head) each fetch all of the
  // gated k (q) rows, so two wide slices ask the memory system for a quarter less per output column than four narrow
  // ones.  A state element is the same sum over the tokens in either split: the results do not depend on the choice.
  static constexpr int BVS_WIDE = (sizeof(T) == 2 && V >= 64) ? 64 : BVS;
  static constexpr int BVO = (sizeof(T) == 4 && V == 128) ? 64 : V;   // output / dv kernels
  static constexpr int BVH = sizeof(T) == 4 ? 32 : 64;                // V-slice loop of dq/dk/dg
};

template <typename T, typename GT, int K, int V>
static void launch_gla_t(const lmoe_args& a, int stage, hipStream_t st) {
  typedef GlaTiles<T, V> Tl;
  const dim3 block(NTHR);
  const bool wide = Tl::BVS_WIDE != Tl::BVS && (int64_t)a.N * a.H * (V / Tl::BVS_WIDE) >= cu_count();
  switch (stage) {
    case ST_GLA_INTRA_FWD:
      hipLaunchKernelGGL((k_gla_intra_fwd<T, GT, K>), dim3(persistent_grid(a.NT * a.H, 2)), block, 0, st, a); break;
    case ST_STATE_FWD:
      if constexpr (sizeof(T) == 2) {
        // 2-byte elements: the pass that holds the state also forms the output (k_gla_fwd_fused); hs == NULL: nothing
        // saved
        const int pairs8 = (a.N * a.H + 7) / 8 * 8;
        if constexpr (Tl::BVS_WIDE != Tl::BVS) {
          // (the saving instance of a wide slice at K = 128 has no registers left for the copy of the state beside the
          // loaders' three register sets: saving calls keep the narrow slice there)
          if (wide && (K == 64 || !a.hs)) {
            if constexpr (K == 64) {
              if (a.hs) {
                hipLaunchKernelGGL((k_gla_fwd_fused<T, K, V, Tl::BVS_WIDE, true>), dim3(pairs8 * (V / Tl::BVS_WIDE)), dim3(3 * NTHR), 0, st, a);
                break;
              }
            }
            hipLaunchKernelGGL((k_gla_fwd_fused<T, K, V, Tl::BVS_WIDE, false>), dim3(pairs8 * (V / Tl::BVS_WIDE)), dim3(3 * NTHR), 0, st, a);
            break;
          }
        }
        if (a.hs) hipLaunchKernelGGL((k_gla_fwd_fused<T, K, V, Tl::BVS, true>), dim3(pairs8 * (V / Tl::BVS)), dim3(3 * NTHR), 0, st, a);
        else hipLaunchKernelGGL((k_gla_fwd_fused<T, K, V, Tl::BVS, false>), dim3(pairs8 * (V / Tl::BVS)), dim3(3 * NTHR), 0, st, a);
        break;
      }
      if (wide) hipLaunchKernelGGL((k_gla_state_fwd<T, GT, K, V, Tl::BVS_WIDE>), dim3((a.N * a.H + 7) / 8 * 8 * (V / Tl::BVS_WIDE)), block, 0, st, a);
      else hipLaunchKernelGGL((k_gla_state_fwd<T, GT, K, V, Tl::BVS>), dim3((a.N * a.H + 7) / 8 * 8 * (V / Tl::BVS)), block, 0, st, a);
      break;
    case ST_OUT_FWD:
      hipLaunchKernelGGL((k_gla_out_fwd<T, GT, K, V, Tl::BVO>), dim3(a.NT, a.H, V / Tl::BVO), block, 0, st, a); break;
    case ST_STATE_BWD:
      if (wide) hipLaunchKernelGGL((k_gla_state_bwd<T, GT, K, V, Tl::BVS_WIDE>), dim3((a.N * a.H + 7) / 8 * 8 * (V / Tl::BVS_WIDE)), block, 0, st, a);
      else hipLaunchKernelGGL((k_gla_state_bwd<T, GT, K, V, Tl::BVS>), dim3((a.N * a.H + 7) / 8 * 8 * (V / Tl::BVS)), block, 0, st, a);
      break;
    case ST_DV:
      hipLaunchKernelGGL((k_gla_bwd_dv<T, GT, K, V, Tl::BVO>), dim3(a.NT, a.H, V / Tl::BVO), block, 0, st, a); break;
    case ST_DQK:
      hipLaunchKernelGGL((k_gla_bwd_dqkg<T, GT, K, V, Tl::BVH>), dim3(a.NT, a.H), block, 0, st, a); break;
    default: break;
  }
}

template <typename T, typename GT>
static void launch_gla_kv(const lmoe_args& a, int stage, hipStream_t st) {
  if (a.K == 64 && a.V == 64) launch_gla_t<T, GT, 64, 64>(a, stage, st);
  else if (a.K == 64 && a.V == 128) launch_gla_t<T, GT, 64, 128>(a, stage, st);
  else if (a.K == 128 && a.V == 64) launch_gla_t<T, GT, 128, 64>(a, stage, st);
  else launch_gla_t<T, GT, 128, 128>(a, stage, st);
}

// whether the forward state pass of this problem also forms the output (then ST_OUT_FWD is not part of the forward)
bool gla_fwd_fused(const lmoe_args& a) { return a.dtype == LMOE_BF16; }

// (dtype, g_dtype) must be (bf16, bf16), (bf16, f32) or (f32, f32): checked by the caller
void launch_gla(const lmoe_args& a, int stage, hipStream_t st) {
  if (a.dtype == LMOE_BF16) {
    if (a.g_dtype == LMOE_BF16) launch_gla_kv<bf16, bf16>(a, stage, st);
    else launch_gla_kv<bf16, float>(a, stage, st);
  } else {
    launch_gla_kv<float, float>(a, stage, st);
  }
}

}  // namespace lmoe
