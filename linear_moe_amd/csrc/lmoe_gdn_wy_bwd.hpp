// Gated delta rule, chunk-parallel backward through the WY / UT factors.
// Inputs per chunk: Tinv (saved), du = dv_new, dw, the partial dk and the partial gate gradient
// db left by k_bwd_dqk.  With k_b = beta k, v_b = beta v, k_bg = k_b e^{b}:
//   dT    = du v_b^T + dw k_bg^T  =  (du v^T) . beta_j  +  (dw k^T) . (beta_j e^{b_j})   (column scalings)
//   dv_b  = Tinv^T du,   dk_bg = Tinv^T dw
//   dL    = - strictlower(Tinv^T dT Tinv^T),   dM = dL . Gamma_s        (L = M . Gamma_s, M = k_b k^T)
//   dk_b  = dM k + dk_bg e^{b}
//   dk   += dM^T k_b + dk_b beta;   dv = dv_b beta;   dbeta = <dk_b, k> + <dv_b, v>
//   db   += k_b.(dM k) - k.(dM^T k_b) + dk_bg.k_bg ;   dg = reverse cumsum of db
// grid = (NT, H), block = 256; wave w owns chunk rows 16w .. 16w+15 in every product.
// The partial dk is updated in place with 16-byte read-modify-write vectors.
// All tiles are stored as loaded (du, dw, v, k: [64][D]; Tinv [64][64]); products that contract
// over tile rows use transposed fragments; the small 64 x 64 intermediates are written
// transposed from the accumulators (vector stores) into the space of du / dw once those are dead.
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

template <typename T, int K, int V>
__global__ __launch_bounds__(NTHR, (sizeof(T) == 2 ? 2 : 1)) void k_gdn_wy_bwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDV = V + LPAD, LDC = CH + LPAD;
  constexpr int TILE = CH * LDC;
  constexpr int NBK = K / 16, NBV = V / 16;
  constexpr int O_DU = 0, O_DW = O_DU + CH * LDV, O_V = O_DW + CH * LDK, O_K = O_V + CH * LDV,
                O_TI = O_K + CH * LDK, NELEM = O_TI + TILE;
  // after phase 2 the du / dw region holds the 64 x 64 intermediates:
  //   tile 0: dT^T, later (diag(beta) dM)^T ;  tile 1: X1^T, later dM^T
  constexpr int O_T0 = 0, O_T1 = TILE, O_T2 = O_T0;
  static_assert(2 * TILE <= O_V, "phase 3/4 tiles must fit into the du + dw region");
  __shared__ __attribute__((aligned(16))) T smem[NELEM];
  __shared__ float s_b[64], s_eb[64], s_beta[64], s_db[64], s_dbeta[64];

  const int cid = blockIdx.x, h = blockIdx.y;
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, CH> IO64;
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, V> IOV;
  const T* du_g = row_ptr<T>(a.dvnew, ci.b, ci.tok, h);
  const T* dw_g = row_ptr<T>(a.dw, ci.b, ci.tok, h);
  const T* k_g = row_ptr<T>(a.k, ci.b, ci.tok, h);
  const T* v_g = row_ptr<T>(a.v, ci.b, ci.tok, h);
  T* dk_g = row_ptr<T>(a.dk, ci.b, ci.tok, h);
  const T* tinv_g = (const T*)a.tinv + ((int64_t)cid * a.H + h) * CH * CH;

  {
    typename IOV::Regs ru, rv;
    typename IOK::Regs rw, rk;
    typename IO64::Regs rt;
    IOV::load(ru, du_g, a.dvnew.st, ci.len);
    IOK::load(rw, dw_g, a.dw.st, ci.len);
    IOV::load(rv, v_g, a.v.st, ci.len);
    IOK::load(rk, k_g, a.k.st, ci.len);
    IO64::load(rt, tinv_g, CH, CH);
    if (threadIdx.x >= 64 && threadIdx.x < 128) {
      const int j = threadIdx.x - 64;
      s_beta[j] = j < ci.len ? load_scalar(a.beta.ptr, a.beta_dtype, row_off(a.beta, ci.b, ci.tok + j, h)) : 0.f;
    }
    chunk_gate_cumsum(a, ci.b, ci.tok, ci.len, h, s_b, s_eb, nullptr);   // barrier inside
    IOV::store_lds(ru, smem + O_DU, LDV);
    IOK::store_lds(rw, smem + O_DW, LDK);
    IOV::store_lds(rv, smem + O_V, LDV);
    IOK::store_lds(rk, smem + O_K, LDK);
    IO64::store_lds(rt, smem + O_TI, LDC);
  }
  __syncthreads();
  // ---- phase 1: dT = (du v^T) beta_j + (dw k^T) beta_j e^{b_j} ------------------------
  f32x4 dT[1][4];
  {
    f32x4 t1[1][4], t2[1][4];
    acc_zero(t1); acc_zero(t2);
    gemm<T, 1, 4, false, false>(t1, smem + O_DU, LDV, 16 * wv, smem + O_V, LDV, 0, 0, V);
    gemm<T, 1, 4, false, false>(t2, smem + O_DW, LDK, 16 * wv, smem + O_K, LDK, 0, 0, K);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      const int cc = 16 * nj + (l & 15);
      const float bj = s_beta[cc], bej = bj * s_eb[cc];
#pragma unroll
      for (int i = 0; i < 4; ++i) dT[0][nj][i] = t1[0][nj][i] * bj + t2[0][nj][i] * bej;
    }
  }
  // ---- phase 2: dv_b = Tinv^T du, dk_bg = Tinv^T dw -----------------------------------
  f32x4 dvb[1][NBV], dkbg[1][NBK];
  acc_zero(dvb); acc_zero(dkbg);
  gemm<T, 1, NBV, true, true>(dvb, smem + O_TI, LDC, 16 * wv, smem + O_DU, LDV, 0, 0, CH);
  gemm<T, 1, NBK, true, true>(dkbg, smem + O_TI, LDC, 16 * wv, smem + O_DW, LDK, 0, 0, CH);
  __syncthreads();     // du, dw are dead: their space takes the 64 x 64 intermediates and dk
  // ---- phase 3: dL = -strictlower(Tinv^T dT Tinv^T), dM = dL . Gamma_s ----------------
#pragma unroll
  for (int nj = 0; nj < 4; ++nj) acc_to_lds_t<T>(dT[0][nj], smem + O_T0, LDC, 16 * wv, 16 * nj);   // dT^T [n][i]
  __syncthreads();
  {
    // X1[j][n] = sum_i Tinv[i][j] dT[i][n]
    f32x4 x1[1][4];
    acc_zero(x1);
    gemm<T, 1, 4, true, false>(x1, smem + O_TI, LDC, 16 * wv, smem + O_T0, LDC, 0, 0, CH);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) acc_to_lds_t<T>(x1[0][nj], smem + O_T1, LDC, 16 * wv, 16 * nj);  // X1^T [n][j]
  }
  __syncthreads();
  {
    // dL[j][m] = - sum_n X1[j][n] Tinv[m][n]
    f32x4 dL[1][4];
    acc_zero(dL);
    gemm<T, 1, 4, true, false>(dL, smem + O_T1, LDC, 16 * wv, smem + O_TI, LDC, 0, 0, CH);
    __syncthreads();   // all waves are done with X1^T: dM^T overwrites it
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p, pb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r > cc) ? -dL[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
        pb[i] = p[i] * s_beta[r];
      }
      acc_to_lds_t<T>(p, smem + O_T1, LDC, 16 * wv, 16 * nj);     // dM^T  [j][i]
      acc_to_lds_t<T>(pb, smem + O_T2, LDC, 16 * wv, 16 * nj);    // (diag(beta) dM)^T [j][i]
    }
  }
  __syncthreads();
  // ---- phase 4: dM k, dM^T k_b and the final combination ------------------------------
  f32x4 dMk[1][NBK], dMTkb[1][NBK];
  acc_zero(dMk); acc_zero(dMTkb);
  gemm<T, 1, NBK, true, true>(dMk, smem + O_T1, LDC, 16 * wv, smem + O_K, LDK, 0, 0, CH);
  gemm<T, 1, NBK, false, true>(dMTkb, smem + O_T2, LDC, 16 * wv, smem + O_K, LDK, 0, 0, CH);

  float dbp[4] = {0.f, 0.f, 0.f, 0.f}, dbt[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
      const float kv = ET<T>::to_f(smem[O_K + r * LDK + cc]);
      const float bt = s_beta[r], eb = s_eb[r];
      const float kbv = kv * bt;
      const float dkb = dMk[0][ni][i] + dkbg[0][ni][i] * eb;
      dbt[i] += dkb * kv;
      dbp[i] += kbv * dMk[0][ni][i] - kv * dMTkb[0][ni][i] + dkbg[0][ni][i] * kbv * eb;
      dMk[0][ni][i] = dMTkb[0][ni][i] + dkb * bt;        // what the WY factors add to dk
    }
#pragma unroll
  for (int ni = 0; ni < NBV; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
      dbt[i] += dvb[0][ni][i] * ET<T>::to_f(smem[O_V + r * LDV + cc]);
      dvb[0][ni][i] *= s_beta[r];                                                              // final dv
    }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) {
      dbp[i] += __shfl_xor(dbp[i], d, 64);
      dbt[i] += __shfl_xor(dbt[i], d, 64);
    }
  }
  if ((l & 15) == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s_db[16 * wv + 4 * (l >> 4) + i] = dbp[i];
      s_dbeta[16 * wv + 4 * (l >> 4) + i] = dbt[i];
    }
  }
  __syncthreads();    // k, v tiles are dead: wave-private slices of them stage the stores
  store_strip<T, NBK, true>(dMk, smem + O_K + wv * 16 * LDK, dk_g + (int64_t)16 * wv * a.dk.st, a.dk.st,
                            ci.len - 16 * wv, 1.0f);
  store_strip<T, NBV>(dvb, smem + O_V + wv * 16 * LDV, row_ptr<T>(a.dv, ci.b, ci.tok + 16 * wv, h), a.dv.st,
                      ci.len - 16 * wv, 1.0f);
  if (threadIdx.x < 64) {
    const int j = threadIdx.x;
    float x = 0.f;
    if (j < ci.len) {
      ((float*)a.dbeta.ptr)[row_off(a.dbeta, ci.b, ci.tok + j, h)] = s_dbeta[j];
      x = s_db[j] + ((const float*)a.dg.ptr)[row_off(a.dg, ci.b, ci.tok + j, h)];
    }
    x = wave_rev_scan(x);
    if (j < ci.len) ((float*)a.dg.ptr)[row_off(a.dg, ci.b, ci.tok + j, h)] = x;
  }
}

}  // namespace lmoe
