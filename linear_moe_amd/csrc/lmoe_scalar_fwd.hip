// Instantiation and launch of the forward kernel of chunk_simple_gla, plus the toolkit self-test.
#include "lmoe_launch.hpp"
#include "lmoe_scalar_fwd.hpp"

namespace lmoe {

// V-slice of the sequential state pass
template <typename T, int V> struct FwdTiles {
  static constexpr int BVS = sizeof(T) == 4 ? 16 : 32;
};

// the pass for 2-byte elements on V slices of BV columns: saving or forward-only, plain or with the normalised output
template <typename T, int K, int V, int BV> void launch_fwd_b(const lmoe_args& a, hipStream_t st) {
  const dim3 grid(((a.N * a.H + 7) / 8) * 8 * (V / BV)), block(3 * NTHR);
  long long* const no_trace = nullptr;
  if (a.normalize) {
    if (a.hs) hipLaunchKernelGGL((k_state_fwd_b<T, K, V, BV, true, false, true>), grid, block, 0, st, a, no_trace, -1);
    else hipLaunchKernelGGL((k_state_fwd_b<T, K, V, BV, false, false, true>), grid, block, 0, st, a, no_trace, -1);
  } else {
    if (a.hs) hipLaunchKernelGGL((k_state_fwd_b<T, K, V, BV, true>), grid, block, 0, st, a, no_trace, -1);
    else hipLaunchKernelGGL((k_state_fwd_b<T, K, V, BV, false>), grid, block, 0, st, a, no_trace, -1);
  }
}
template <typename T, int K, int V> struct StateFwd {
  static void run(const lmoe_args& a, hipStream_t st) {
    constexpr int BV = FwdTiles<T, V>::BVS;
    if constexpr (sizeof(T) == 2) {
      // 64-wide slices where they still fill the chip: every V slice of a (sequence, head) fetches all of q and k and
      // forms all of P, so two wide slices cost less per output column than four narrow ones; the results do not
      // depend on the width (a state element and an output element are the same sums in either split)
      if constexpr (V >= 64) {
        if ((int64_t)a.N * a.H * (V / 64) >= cu_count()) {
          launch_fwd_b<T, K, V, 64>(a, st);
          return;
        }
      }
      launch_fwd_b<T, K, V, BV>(a, st);
    } else {
      const int grid = ((a.N * a.H + 7) / 8) * 8 * (V / BV);
      if (a.hs) hipLaunchKernelGGL((k_state_fwd<T, K, V, BV, true>), dim3(grid), dim3(3 * NTHR), 0, st, a);
      else hipLaunchKernelGGL((k_state_fwd<T, K, V, BV, false>), dim3(grid), dim3(3 * NTHR), 0, st, a);
    }
  }
};
void launch_state_fwd(const lmoe_args& a, hipStream_t st) { dispatch<StateFwd>(a, st); }
// the traced instance of the pass (2-byte elements, K = V = 128, forward-only call)
bool launch_state_fwd_trace(const lmoe_args& a, long long* tr, int work_group, hipStream_t st) {
  if (a.dtype != LMOE_BF16 || a.K != 128 || a.V != 128 || a.hs) return false;
  constexpr int BV = FwdTiles<bf16, 128>::BVS;
  const int grid = ((a.N * a.H + 7) / 8) * 8 * (128 / BV);
  if (work_group < 0 || work_group >= grid) return false;
  hipLaunchKernelGGL((k_state_fwd_b<bf16, 128, 128, BV, false, true>), dim3(grid), dim3(3 * NTHR), 0, st, a, tr, work_group);
  return true;
}
// C = A B^T (64 x 64, contraction along the tile columns) and G = A^T B (KD x KD, contraction
// along the tile rows, i.e. the transposed-fragment path) over one pair of 64 x KD tiles,
// through the loaders / fragments / accumulator stores of the toolkit
template <typename T, int KD>
__global__ __launch_bounds__(NTHR) void k_selftest(const T* A, const T* B, float* C, float* G) {
  constexpr int LD = KD + LPAD, LDC = CH + LPAD;
  __shared__ __attribute__((aligned(16))) T s_a[CH * LD];
  __shared__ __attribute__((aligned(16))) T s_b[CH * LD];
  __shared__ __attribute__((aligned(16))) float s_c[CH * LDC];
  typedef TileIO<T, CH, KD> IO;
  typename IO::Regs ra, rb;
  IO::load(ra, A, KD, CH);
  IO::load(rb, B, KD, CH);
  IO::store_lds(ra, s_a, LD);
  IO::store_lds(rb, s_b, LD);
  __syncthreads();
  const int wv = wave_id(), l = lane_id();
  f32x4 acc[1][4];
  acc_zero(acc);
  gemm<T, 1, 4, false, false>(acc, s_a, LD, 16 * wv, s_b, LD, 0, 0, KD);
  for (int nj = 0; nj < 4; ++nj) acc_to_lds_t<float>(acc[0][nj], s_c, LDC, 16 * wv, 16 * nj);   // s_c = C^T
  __syncthreads();
  for (int idx = threadIdx.x; idx < CH * CH; idx += NTHR) {
    const int r = idx / CH, c = idx % CH;
    C[idx] = s_c[c * LDC + r];
  }
  // G rows [wv * KD/4, (wv+1) * KD/4)
  constexpr int MB = KD / 64, NB = KD / 16;
  f32x4 g[MB][NB];
  acc_zero(g);
  gemm<T, MB, NB, true, true>(g, s_a, LD, wv * (KD / 4), s_b, LD, 0, 0, CH);
  for (int mi = 0; mi < MB; ++mi)
    for (int ni = 0; ni < NB; ++ni)
      for (int i = 0; i < 4; ++i)
        G[(wv * (KD / 4) + 16 * mi + 4 * (l >> 4) + i) * KD + 16 * ni + (l & 15)] = g[mi][ni][i];
}

void launch_selftest(int dtype, int kd, const void* A, const void* B, float* C, float* G, hipStream_t st) {
  if (dtype == LMOE_BF16) {
    if (kd == 64) hipLaunchKernelGGL((k_selftest<bf16, 64>), dim3(1), dim3(NTHR), 0, st, (const bf16*)A, (const bf16*)B, C, G);
    else hipLaunchKernelGGL((k_selftest<bf16, 128>), dim3(1), dim3(NTHR), 0, st, (const bf16*)A, (const bf16*)B, C, G);
  } else {
    if (kd == 64) hipLaunchKernelGGL((k_selftest<float, 64>), dim3(1), dim3(NTHR), 0, st, (const float*)A, (const float*)B, C, G);
    else hipLaunchKernelGGL((k_selftest<float, 128>), dim3(1), dim3(NTHR), 0, st, (const float*)A, (const float*)B, C, G);
  }
}

}  // namespace lmoe
