// Instantiation and launch of the scalar-gate forward kernels, plus the toolkit self-test.
#include "lmoe_launch.hpp"
#include "lmoe_scalar_fwd.hpp"

namespace lmoe {

// V-slice of the sequential state pass and of the output kernel
template <typename T, int V> struct FwdTiles {
  static constexpr int BVS = 32;
  static constexpr int BVO = (sizeof(T) == 4 && V == 128) ? 64 : V;
};

template <bool GDN> struct StateFwd {
  template <typename T, int K, int V> struct F {
    static void run(const lmoe_args& a, hipStream_t st) {
      constexpr int BV = FwdTiles<T, V>::BVS;
      hipLaunchKernelGGL((k_state_fwd<T, K, V, BV, GDN>), dim3(V / BV, a.H, a.N), dim3(NTHR), 0, st, a);
    }
  };
};
template <bool GDN> struct OutFwd {
  template <typename T, int K, int V> struct F {
    static void run(const lmoe_args& a, hipStream_t st) {
      constexpr int BV = FwdTiles<T, V>::BVO;
      hipLaunchKernelGGL((k_out_fwd<T, K, V, BV, GDN>), dim3(a.NT, a.H, V / BV), dim3(NTHR), 0, st, a);
    }
  };
};

void launch_state_fwd(const lmoe_args& a, bool gdn, hipStream_t st) {
  if (gdn) dispatch<StateFwd<true>::F>(a, st); else dispatch<StateFwd<false>::F>(a, st);
}
void launch_out_fwd(const lmoe_args& a, bool gdn, hipStream_t st) {
  if (gdn) dispatch<OutFwd<true>::F>(a, st); else dispatch<OutFwd<false>::F>(a, st);
}

// C = A B^T over one 64 x KD tile pair, through the loaders / fragments / stores of the toolkit
template <typename T, int KD>
__global__ __launch_bounds__(NTHR) void k_selftest(const T* A, const T* B, float* C, float* Ct) {
  constexpr int LD = KD + LPAD, LDC = CH + LPAD;
  __shared__ __attribute__((aligned(16))) T s_a[CH * LD];
  __shared__ __attribute__((aligned(16))) T s_b[CH * LD];
  __shared__ __attribute__((aligned(16))) T s_bt[KD * LDC];   // B^T, used for Ct = (A B^T)^T check path
  __shared__ __attribute__((aligned(16))) float s_c[CH * LDC];
  __shared__ __attribute__((aligned(16))) float s_ct[CH * LDC];
  typedef TileIO<T, CH, KD> IO;
  typename IO::Regs ra, rb;
  IO::load(ra, A, KD, CH);
  IO::load(rb, B, KD, CH);
  IO::store_lds(ra, s_a, LD);
  IO::store_lds(rb, s_b, LD);
  IO::store_lds_t(rb, s_bt, LDC, nullptr);
  __syncthreads();
  const int wv = wave_id();
  f32x4 acc[1][4];
  acc_zero(acc);
  gemm_nt<T, 1, 4>(acc, s_a, LD, 16 * wv, s_b, LD, 0, 0, KD);
  for (int nj = 0; nj < 4; ++nj) {
    acc_to_lds<float>(acc[0][nj], s_c, LDC, 16 * wv, 16 * nj);
    acc_to_lds_t<float>(acc[0][nj], s_ct, LDC, 16 * wv, 16 * nj);
  }
  __syncthreads();
  // also exercise the transposed-load path: s_bt[k][j] must equal B[j][k]
  float chk = 0.f;
  for (int idx = threadIdx.x; idx < CH * KD; idx += NTHR) {
    const int j = idx / KD, k = idx % KD;
    chk += fabsf(ET<T>::to_f(s_bt[k * LDC + j]) - ET<T>::to_f(B[j * KD + k]));
  }
  for (int idx = threadIdx.x; idx < CH * CH; idx += NTHR) {
    const int r = idx / CH, c = idx % CH;
    C[idx] = s_c[r * LDC + c] + chk;
    Ct[idx] = s_ct[r * LDC + c];
  }
}

void launch_selftest(int dtype, int kd, const void* A, const void* B, float* C, float* Ct, hipStream_t st) {
  if (dtype == LMOE_BF16) {
    if (kd == 64) hipLaunchKernelGGL((k_selftest<bf16, 64>), dim3(1), dim3(NTHR), 0, st, (const bf16*)A, (const bf16*)B, C, Ct);
    else hipLaunchKernelGGL((k_selftest<bf16, 128>), dim3(1), dim3(NTHR), 0, st, (const bf16*)A, (const bf16*)B, C, Ct);
  } else {
    if (kd == 64) hipLaunchKernelGGL((k_selftest<float, 64>), dim3(1), dim3(NTHR), 0, st, (const float*)A, (const float*)B, C, Ct);
    else hipLaunchKernelGGL((k_selftest<float, 128>), dim3(1), dim3(NTHR), 0, st, (const float*)A, (const float*)B, C, Ct);
  }
}

}  // namespace lmoe
