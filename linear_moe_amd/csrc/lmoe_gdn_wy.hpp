// Gated delta rule, chunk-parallel WY / UT preparation (forward):
//   L = strictlower( diag(beta) (k k^T) . Gamma ),  Gamma_ij = e^{b_i - b_j}
//   Tinv = (I + L)^-1            (unit lower triangular, fp32)
//   w = Tinv (k . beta e^{b}),   u = Tinv (v . beta)
// and the intra-chunk attention matrix the two sequential passes consume,
//   P = (q k^T) . Gamma  (lower triangle incl. the diagonal).
// grid = (NT, H), block = 256.  Writes w, u, Tinv and P (element type T) and the chunk's
// decay table e^{b}, e^{b_C - b} (fp32).
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
__global__ __launch_bounds__(NTHR, (sizeof(T) == 2 ? 2 : 1)) void k_gdn_wy_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDV = V + LPAD, LDC = CH + LPAD;
  constexpr int NBK = K / 16, NBV = V / 16;
  // k (raw, for k k^T), then overwritten in place by k beta e^{b}; v beta; both stored [64][D]
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];
  __shared__ __attribute__((aligned(16))) T s_vb[CH * LDV];
  __shared__ __attribute__((aligned(16))) float s_L[CH * LDC];   // L, later Tinv in element type T
  __shared__ __attribute__((aligned(16))) float s_X[CH * LDC];
  __shared__ float s_Y[3 * 256];
  __shared__ float s_b[64], s_eb[64], s_beta[64], s_beb[64];
  // Tinv as an MFMA operand: fp32 uses s_X in place, bf16 a copy in the (dead) L tile
  T* s_Tm = sizeof(T) == 4 ? (T*)s_X : (T*)s_L;

  const int cid = blockIdx.x, h = blockIdx.y;
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, V> IOV;
  typedef TileIO<T, CH, CH> IO64;
  typename IOK::Regs rk;
  typename IOV::Regs rv;
  // q enters only as the A operand of q k^T: each wave takes its 16 rows straight into fragments
  RowFrags<T, K> fq;
  fq.load(row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, 16 * wv, ci.len - 1);
  IOK::load(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
  IOV::load(rv, row_ptr<T>(a.v, ci.b, ci.tok, h), a.v.st, ci.len);
  if (threadIdx.x >= 64 && threadIdx.x < 128) {
    const int j = threadIdx.x - 64;
    s_beta[j] = j < ci.len ? load_scalar(a.beta.ptr, a.beta_dtype, row_off(a.beta, ci.b, ci.tok + j, h)) : 0.f;
  }
  chunk_gate_cumsum(a, ci.b, ci.tok, ci.len, h, s_b, s_eb, nullptr);    // barrier inside
  if (threadIdx.x < 64) {
    s_beb[threadIdx.x] = s_beta[threadIdx.x] * s_eb[threadIdx.x];
    // decay table of the chunk for the sequential passes: e^{b_j}, e^{b_C - b_j}
    float* gc = a.gcum + ((int64_t)cid * a.H + h) * 2 * CH;
    gc[threadIdx.x] = s_eb[threadIdx.x];
    gc[CH + threadIdx.x] = expf(s_b[CH - 1] - s_b[threadIdx.x]);
  }
  IOK::store_lds(rk, s_k, LDK);
  IOV::store_lds_scaled(rv, s_vb, LDV, s_beta);
  __syncthreads();
  {
    f32x4 m[1][4];
    acc_zero(m);
    gemm<T, 1, 4, false, false>(m, s_k, LDK, 16 * wv, s_k, LDK, 0, 0, K);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r > cc) ? s_beta[r] * m[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds<float>(p, s_L, LDC, 16 * wv, 16 * nj);
    }
  }
  {
    // P = (q k^T) . Gamma -> global, staged through the (still unused) X tile
    T* s_P = (T*)s_X;
    T* pg = (T*)a.pmat + ((int64_t)cid * a.H + h) * CH * CH;
    f32x4 pm[1][4];
    acc_zero(pm);
    fq.mask(16 * wv, ci.len);
#pragma unroll
    for (int ks = 0; ks < K / 32; ++ks)
#pragma unroll
      for (int nj = 0; nj < 4; ++nj)
        ET<T>::mma(pm[0][nj], fq.f[ks], ET<T>::load_frag(s_k + (16 * nj + (l & 15)) * LDK + 32 * ks + 8 * (l >> 4)));
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        pm[0][nj][i] = (r >= cc) ? pm[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds<T>(pm[0][nj], s_P, LDC, 16 * wv, 16 * nj);
    }
    __syncthreads();
    IO64::lds_to_global(s_P, LDC, pg, CH, CH);
  }
  // k is dead as an operand of k k^T and q k^T: scale it in place to k beta e^{b} (from the registers)
  IOK::store_lds_scaled(rk, s_k, LDK, s_beb);
  __syncthreads();   // L is complete, the P staging has been read: the inverse may overwrite X
  tri_inverse_64(s_L, LDC, s_X, LDC, s_Y);       // barriers inside; s_L is dead afterwards
  {
    T* tg = (T*)a.tinv + ((int64_t)cid * a.H + h) * CH * CH;
    for (int idx = threadIdx.x; idx < CH * CH / 4; idx += NTHR) {
      const int r = idx >> 4, c = (idx & 15) * 4;
      const f32x4 x = *(const f32x4*)(s_X + r * LDC + c);
      if constexpr (sizeof(T) == 2) {
        bf16x4 y; y[0] = (bf16)x[0]; y[1] = (bf16)x[1]; y[2] = (bf16)x[2]; y[3] = (bf16)x[3];
        *(bf16x4*)(s_Tm + r * LDC + c) = y;
        *(bf16x4*)(tg + r * CH + c) = y;
      } else {
        *(f32x4*)(tg + r * CH + c) = x;
      }
    }
  }
  __syncthreads();
  // w = Tinv (k beta e^{b}),  u = Tinv (v beta): contraction over the rows of the [64][D] tiles
  f32x4 w[1][NBK];
  acc_zero(w);
  gemm<T, 1, NBK, false, true>(w, s_Tm, LDC, 16 * wv, s_k, LDK, 0, 0, CH);
  f32x4 u[1][NBV];
  acc_zero(u);
  gemm<T, 1, NBV, false, true>(u, s_Tm, LDC, 16 * wv, s_vb, LDV, 0, 0, CH);
  __syncthreads();   // k, v tiles are dead: wave-private slices of them stage the stores
  store_strip<T, NBK>(w, s_k + wv * 16 * LDK, row_ptr<T>(a.w, ci.b, ci.tok + 16 * wv, h), a.w.st, ci.len - 16 * wv, 1.0f);
  store_strip<T, NBV>(u, s_vb + wv * 16 * LDV, row_ptr<T>(a.u, ci.b, ci.tok + 16 * wv, h), a.u.st, ci.len - 16 * wv, 1.0f);
}

}  // namespace lmoe
