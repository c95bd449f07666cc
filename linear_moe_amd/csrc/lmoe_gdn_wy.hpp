// Gated delta rule, chunk-parallel WY / UT preparation (forward):
//   L = strictlower( diag(beta) (k k^T) . Gamma ),  Gamma_ij = e^{b_i - b_j}
//   Tinv = (I + L)^-1            (unit lower triangular, fp32)
//   w = Tinv (k . beta e^{b}),   u = Tinv (v . beta)
// grid = (NT, H), block = 256.  Writes w, u and Tinv (element type T).
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

// In-LDS inverse of the unit lower triangular matrix I + L (64 x 64, fp32).
//   sL : strictly lower part L (upper part and diagonal must be 0), leading dimension ldl
//   sX : receives (I + L)^-1, leading dimension ldx
//   sY : scratch for one 16 x 16 block per wave... (4 * 256 floats)
// Block forward substitution with 16 x 16 blocks: the four diagonal blocks are inverted by
// the four waves (one column per lane), the off-diagonal blocks follow by block distance:
//   X_IJ = - X_II * sum_{M = J}^{I-1} L_IM X_MJ.
// Must be called by all 256 threads; sL must be complete (barrier before the call).
__device__ __forceinline__ void tri_inverse_64(const float* sL, int ldl, float* sX, int ldx, float* sY) {
  const int wv = wave_id(), l = lane_id(), tid = threadIdx.x;
  // clear X (upper blocks stay zero)
  for (int idx = tid; idx < CH * CH; idx += NTHR) sX[(idx >> 6) * ldx + (idx & 63)] = 0.f;
  __syncthreads();
  if (l < 16) {
    const int o = 16 * wv;
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float s = (i == l) ? 1.f : 0.f;
#pragma unroll
      for (int m = 0; m < i; ++m) s -= sL[(o + i) * ldl + o + m] * x[m];
      x[i] = s;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) sX[(o + i) * ldx + o + l] = x[i];
  }
  __syncthreads();
  const int r = tid >> 4, c = tid & 15;   // one entry of a 16 x 16 block per thread
  for (int d = 1; d < 4; ++d) {
    // Y_IJ = sum_{M=J}^{I-1} L_IM X_MJ for all blocks with I - J = d
    for (int J = 0; J + d < 4; ++J) {
      const int I = J + d;
      float y = 0.f;
      for (int m = 16 * J; m < 16 * I; ++m) y += sL[(16 * I + r) * ldl + m] * sX[m * ldx + 16 * J + c];
      sY[J * 256 + tid] = y;
    }
    __syncthreads();
    for (int J = 0; J + d < 4; ++J) {
      const int I = J + d;
      float x = 0.f;
#pragma unroll
      for (int m = 0; m < 16; ++m) x -= sX[(16 * I + r) * ldx + 16 * I + m] * sY[J * 256 + m * 16 + c];
      sX[(16 * I + r) * ldx + 16 * J + c] = x;
    }
    __syncthreads();
  }
}

template <typename T, int K, int V>
__global__ __launch_bounds__(NTHR) void k_gdn_wy_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD;
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];
  __shared__ __attribute__((aligned(16))) T s_kbgT[K * LDC];
  __shared__ __attribute__((aligned(16))) T s_vbT[V * LDC];
  __shared__ __attribute__((aligned(16))) float s_L[CH * LDC];
  __shared__ __attribute__((aligned(16))) float s_X[CH * LDC];
  // Tinv as an MFMA operand: fp32 reuses s_X in place, bf16 gets its own copy
  __shared__ __attribute__((aligned(16))) T s_Tm_own[sizeof(T) == 4 ? 8 : CH * LDC];
  T* s_Tm = sizeof(T) == 4 ? (T*)s_X : s_Tm_own;
  __shared__ float s_Y[3 * 256];
  __shared__ float s_b[64], s_eb[64], s_beta[64], s_beb[64];

  const int cid = blockIdx.x, h = blockIdx.y;
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  if (threadIdx.x >= 64 && threadIdx.x < 128) {
    const int j = threadIdx.x - 64;
    s_beta[j] = j < ci.len ? load_scalar(a.beta.ptr, a.beta_dtype, row_off(a.beta, ci.b, ci.tok + j, h)) : 0.f;
  }
  chunk_gate_cumsum(a, ci.b, ci.tok, ci.len, h, s_b, s_eb, nullptr);
  if (threadIdx.x < 64) s_beb[threadIdx.x] = s_beta[threadIdx.x] * s_eb[threadIdx.x];
  __syncthreads();

  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, V> IOV;
  {
    typename IOK::Regs rk;
    IOK::load(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
    typename IOV::Regs rv;
    IOV::load(rv, row_ptr<T>(a.v, ci.b, ci.tok, h), a.v.st, ci.len);
    IOK::store_lds(rk, s_k, LDK);
    IOK::store_lds_t(rk, s_kbgT, LDC, s_beb);
    IOV::store_lds_t(rv, s_vbT, LDC, s_beta);
  }
  __syncthreads();
  {
    f32x4 m[1][4];
    acc_zero(m);
    gemm_nt<T, 1, 4>(m, s_k, LDK, 16 * wv, s_k, LDK, 0, 0, K);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r > cc) ? s_beta[r] * m[0][nj][i] * expf(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds<float>(p, s_L, LDC, 16 * wv, 16 * nj);
    }
  }
  __syncthreads();
  tri_inverse_64(s_L, LDC, s_X, LDC, s_Y);
  // Tinv -> element type T (LDS operand + global copy for the backward)
  {
    T* tg = (T*)a.tinv + ((int64_t)cid * a.H + h) * CH * CH;
    for (int idx = threadIdx.x; idx < CH * CH; idx += NTHR) {
      const int r = idx >> 6, c = idx & 63;
      const T x = ET<T>::from_f(s_X[r * LDC + c]);
      if constexpr (sizeof(T) != 4) s_Tm[r * LDC + c] = x;
      tg[idx] = x;
    }
  }
  __syncthreads();
  {
    constexpr int NBK = K / 16;
    f32x4 w[1][NBK];
    acc_zero(w);
    gemm_nt<T, 1, NBK>(w, s_Tm, LDC, 16 * wv, s_kbgT, LDC, 0, 0, CH);
    T* wd = row_ptr<T>(a.w, ci.b, ci.tok, h);
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
        if (r < ci.len) wd[(int64_t)r * a.w.st + cc] = ET<T>::from_f(w[0][ni][i]);
      }
  }
  {
    constexpr int NBV = V / 16;
    f32x4 u[1][NBV];
    acc_zero(u);
    gemm_nt<T, 1, NBV>(u, s_Tm, LDC, 16 * wv, s_vbT, LDC, 0, 0, CH);
    T* ud = row_ptr<T>(a.u, ci.b, ci.tok, h);
#pragma unroll
    for (int ni = 0; ni < NBV; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
        if (r < ci.len) ud[(int64_t)r * a.u.st + cc] = ET<T>::from_f(u[0][ni][i]);
      }
  }
}

}  // namespace lmoe
