// Gated delta rule, chunk-parallel backward through the WY / UT factors.
// Inputs per chunk: Tinv (saved), du = dv_new, dw, the partial dk and the partial gate gradient
// db left by k_bwd_dqk.  With k_b = beta k, v_b = beta v, k_bg = k_b e^{b}:
//   dT    = du v_b^T + dw k_bg^T
//   dv_b  = Tinv^T du,   dk_bg = Tinv^T dw
//   dL    = - strictlower(Tinv^T dT Tinv^T),   dM = dL . Gamma_s        (L = M . Gamma_s, M = k_b k^T)
//   dk_b  = dM k + dk_bg e^{b}
//   dk   += dM^T k_b + dk_b beta;   dv = dv_b beta;   dbeta = <dk_b, k> + <dv_b, v>
//   db   += k_b.(dM k) - k.(dM^T k_b) + dk_bg.k_bg ;   dg = reverse cumsum of db
// grid = (NT, H), block = 256; wave w owns chunk rows 16w .. 16w+15 in every product.
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

template <typename T, int K, int V>
__global__ __launch_bounds__(NTHR) void k_gdn_wy_bwd(const lmoe_args a) {
  constexpr int LDC = CH + LPAD;                 // every tile here has 64 (+pad) columns
  constexpr int TILE = CH * LDC;                 // one 64 x 64 tile
  constexpr int NBK = K / 16, NBV = V / 16;
  // LDS map (element offsets):
  //   phase 1: [0] A-slice, [TILE] B-slice
  //   phase 2: [0] Tinv^T, [TILE] du^T (V rows), [TILE + V*LDC] dw^T (K rows)
  //   phase 3: [0] Tinv^T, [TILE] dT^T, [2 TILE] X1, [3 TILE] Tinv ; then [0] dM, [TILE] dM^T
  //   phase 4: [0] dM, [TILE] dM^T, [4 TILE] k^T (K rows), [4 TILE + K*LDC] k_b^T (K rows)
  constexpr int P2_END = TILE + (V + K) * LDC;
  constexpr int P4_END = 4 * TILE + 2 * K * LDC;
  constexpr int NELEM = P2_END > P4_END ? P2_END : P4_END;
  __shared__ __attribute__((aligned(16))) T smem[NELEM];
  __shared__ float s_b[64], s_eb[64], s_beta[64], s_beb[64], s_db[64], s_dbeta[64];

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

  typedef TileIO<T, CH, CH> IO64;     // 64-column slice of a [64 x D] token tile, or a 64x64 matrix
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, V> IOV;
  const T* du_g = row_ptr<T>(a.dvnew, ci.b, ci.tok, h);
  const T* dw_g = row_ptr<T>(a.dw, ci.b, ci.tok, h);
  const T* k_g = row_ptr<T>(a.k, ci.b, ci.tok, h);
  const T* v_g = row_ptr<T>(a.v, ci.b, ci.tok, h);
  const T* tinv_g = (const T*)a.tinv + ((int64_t)cid * a.H + h) * CH * CH;

  // ---- phase 1: dT = du v_b^T + dw k_bg^T ------------------------------------------
  f32x4 dT[1][4];
  acc_zero(dT);
  for (int s = 0; s < (V + K) / 64; ++s) {
    const bool isv = s < V / 64;
    const int off = (isv ? s : s - V / 64) * 64;
    typename IO64::Regs ra, rb;
    if (isv) {
      IO64::load(ra, du_g + off, a.dvnew.st, ci.len);
      IO64::load(rb, v_g + off, a.v.st, ci.len);
    } else {
      IO64::load(ra, dw_g + off, a.dw.st, ci.len);
      IO64::load(rb, k_g + off, a.k.st, ci.len);
    }
    IO64::store_lds(ra, smem, LDC);
    IO64::store_lds_scaled(rb, smem + TILE, LDC, isv ? s_beta : s_beb);
    __syncthreads();
    gemm_nt<T, 1, 4>(dT, smem, LDC, 16 * wv, smem + TILE, LDC, 0, 0, 64);
    __syncthreads();
  }
  // ---- phase 2: dv_b = Tinv^T du, dk_bg = Tinv^T dw ----------------------------------
  {
    typename IO64::Regs rt;
    IO64::load(rt, tinv_g, CH, CH);
    IO64::store_lds_t(rt, smem, LDC, nullptr);
    typename IOV::Regs ru;
    IOV::load(ru, du_g, a.dvnew.st, ci.len);
    IOV::store_lds_t(ru, smem + TILE, LDC, nullptr);
    typename IOK::Regs rw;
    IOK::load(rw, dw_g, a.dw.st, ci.len);
    IOK::store_lds_t(rw, smem + TILE + V * LDC, LDC, nullptr);
  }
  __syncthreads();
  f32x4 dvb[1][NBV], dkbg[1][NBK];
  acc_zero(dvb); acc_zero(dkbg);
  gemm_nt<T, 1, NBV>(dvb, smem, LDC, 16 * wv, smem + TILE, LDC, 0, 0, CH);
  gemm_nt<T, 1, NBK>(dkbg, smem, LDC, 16 * wv, smem + TILE + V * LDC, LDC, 0, 0, CH);
  __syncthreads();
  // ---- phase 3: dL = -strictlower(Tinv^T dT Tinv^T), dM = dL . Gamma_s ---------------
  {
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) acc_to_lds_t<T>(dT[0][nj], smem + TILE, LDC, 16 * wv, 16 * nj);
    typename IO64::Regs rt;
    IO64::load(rt, tinv_g, CH, CH);
    IO64::store_lds(rt, smem + 3 * TILE, LDC);
    // k^T and k_b^T for phase 4 (region not used by phase 3)
    typename IOK::Regs rk;
    IOK::load(rk, k_g, a.k.st, ci.len);
    IOK::store_lds_t(rk, smem + 4 * TILE, LDC, nullptr);
    IOK::store_lds_t(rk, smem + 4 * TILE + K * LDC, LDC, s_beta);
  }
  __syncthreads();
  {
    f32x4 x1[1][4];
    acc_zero(x1);
    gemm_nt<T, 1, 4>(x1, smem, LDC, 16 * wv, smem + TILE, LDC, 0, 0, CH);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) acc_to_lds<T>(x1[0][nj], smem + 2 * TILE, LDC, 16 * wv, 16 * nj);
  }
  __syncthreads();
  {
    f32x4 dL[1][4];
    acc_zero(dL);
    gemm_nt<T, 1, 4>(dL, smem + 2 * TILE, LDC, 16 * wv, smem + 3 * TILE, LDC, 0, 0, CH);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r > cc) ? -dL[0][nj][i] * expf(s_b[r] - s_b[cc]) : 0.f;
      }
      // regions [0] (Tinv^T) and [TILE] (dT^T) are no longer read: every wave passed the
      // barrier after the X1 product
      acc_to_lds<T>(p, smem, LDC, 16 * wv, 16 * nj);
      acc_to_lds_t<T>(p, smem + TILE, LDC, 16 * wv, 16 * nj);
    }
  }
  __syncthreads();
  // ---- phase 4: dM k, dM^T k_b and the final combination -------------------------------
  f32x4 dMk[1][NBK], dMTkb[1][NBK];
  acc_zero(dMk); acc_zero(dMTkb);
  gemm_nt<T, 1, NBK>(dMk, smem, LDC, 16 * wv, smem + 4 * TILE, LDC, 0, 0, CH);
  gemm_nt<T, 1, NBK>(dMTkb, smem + TILE, LDC, 16 * wv, smem + 4 * TILE + K * LDC, LDC, 0, 0, CH);

  float dbp[4] = {0.f, 0.f, 0.f, 0.f}, dbt[4] = {0.f, 0.f, 0.f, 0.f};
  T* dkd = row_ptr<T>(a.dk, ci.b, ci.tok, h);
  const T* kT = smem + 4 * TILE;
#pragma unroll
  for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
      const float kv = ET<T>::to_f(kT[cc * LDC + r]);
      const float bt = s_beta[r], eb = s_eb[r];
      const float kbv = kv * bt;
      const float dkb = dMk[0][ni][i] + dkbg[0][ni][i] * eb;
      dbt[i] += dkb * kv;
      dbp[i] += kbv * dMk[0][ni][i] - kv * dMTkb[0][ni][i] + dkbg[0][ni][i] * kbv * eb;
      if (r < ci.len) {
        T* p = dkd + (int64_t)r * a.dk.st + cc;
        *p = ET<T>::from_f(ET<T>::to_f(*p) + dMTkb[0][ni][i] + dkb * bt);
      }
    }
  T* dvd = row_ptr<T>(a.dv, ci.b, ci.tok, h);
#pragma unroll
  for (int ni = 0; ni < NBV; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
      if (r < ci.len) {
        const float vv = ET<T>::to_f(v_g[(int64_t)r * a.v.st + cc]);
        dbt[i] += dvb[0][ni][i] * vv;
        dvd[(int64_t)r * a.dv.st + cc] = ET<T>::from_f(dvb[0][ni][i] * s_beta[r]);
      }
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
  __syncthreads();
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
