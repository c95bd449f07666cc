// Backward kernels for scalar-gated chunks (chunk_simple_gla and chunk_gated_delta_rule).
// Notation per chunk: b = inclusive cumsum of g, e_b = e^{b}, e_d = e^{b_C - b},
// Gamma_ij = e^{b_i - b_j} [i >= j], P = (q k^T) . Gamma, S = state at chunk start,
// dS' = gradient w.r.t. the state at chunk end, v' = v (simple_gla) or v_new (delta rule).
//
//   k_bwd_dv    : chunk-parallel   dv' = scale P^T do (+ (k . e_d) dS'  unless LOCAL)
//   k_state_bwd : reverse sequential pass over the chunks of one (sequence, head, V-slice):
//                 writes dS' of every chunk (dhs); delta rule: dv_new = dv_loc + (k . e_d) dS';
//                 dS = e^{b_C} dS' + scale (q . e_b)^T do  (- w^T dv_new)
//   k_bwd_dqk   : chunk-parallel   dq, dk (delta rule: the part of dk that does not go through
//                 the WY factors, and dw = -dv_new S^T), gate gradient
//                 db_i = q_i.dq_i - k_i.dk_i (+ on the last row sum_j (dk_d . k_d)_j + e^{b_C} <S, dS'>)
//                 and, for simple_gla, dg = reverse cumsum of db.
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

// ------------------------------------------------------------------------- //
// dv' = scale P^T do + (k . e_d) dS'        grid = (NT, H, V / BV)
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV, bool LOCAL>
__global__ __launch_bounds__(NTHR) void k_bwd_dv(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD;
  constexpr int NB = BV / 16;
  __shared__ __attribute__((aligned(16))) T s_q[CH * LDK];
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];
  __shared__ __attribute__((aligned(16))) T s_doT[BV * LDC];
  __shared__ __attribute__((aligned(16))) T s_dhT[LOCAL ? 8 : BV * LDK];
  __shared__ __attribute__((aligned(16))) T s_PT[CH * LDC];
  __shared__ float s_b[64], s_ed[64];

  const int cid = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * BV;
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  chunk_gate_cumsum(a, ci.b, ci.tok, ci.len, h, s_b, nullptr, s_ed);

  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;
  typedef TileIO<T, K, BV> IOH;
  {
    typename IOK::Regs rq, rk;
    IOK::load(rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
    IOK::load(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
    typename IOV::Regs rd;
    IOV::load(rd, row_ptr<T>(a.d_o, ci.b, ci.tok, h) + v0, a.d_o.st, ci.len);
    IOK::store_lds(rq, s_q, LDK);
    IOK::store_lds(rk, s_k, LDK);
    IOV::store_lds_t(rd, s_doT, LDC, nullptr);
    if constexpr (!LOCAL) {
      typename IOH::Regs rh;
      IOH::load(rh, (const T*)a.dhs + ((int64_t)cid * a.H + h) * K * V + v0, V, K);
      IOH::store_lds_t(rh, s_dhT, LDK, nullptr);
    }
  }
  __syncthreads();
  {
    // P^T stored as s_PT[j][i]; wave w computes rows i = 16w.. of P and writes them transposed
    f32x4 s[1][4];
    acc_zero(s);
    gemm_nt<T, 1, 4>(s, s_q, LDK, 16 * wv, s_k, LDK, 0, 0, K);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r >= cc) ? s[0][nj][i] * expf(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds_t<T>(p, s_PT, LDC, 16 * wv, 16 * nj);
    }
  }
  __syncthreads();
  f32x4 dv[1][NB];
  acc_zero(dv);
  gemm_nt<T, 1, NB>(dv, s_PT, LDC, 16 * wv, s_doT, LDC, 0, 0, CH);
#pragma unroll
  for (int ni = 0; ni < NB; ++ni) dv[0][ni] *= a.scale;
  if constexpr (!LOCAL) {
    f32x4 t[1][NB];
    acc_zero(t);
    gemm_nt<T, 1, NB>(t, s_k, LDK, 16 * wv, s_dhT, LDK, 0, 0, K);
#pragma unroll
    for (int ni = 0; ni < NB; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) dv[0][ni][i] += t[0][ni][i] * s_ed[16 * wv + 4 * (l >> 4) + i];
  }
  const lmoe_tensor& dst = LOCAL ? a.dvnew : a.dv;
  T* dd = row_ptr<T>(dst, ci.b, ci.tok, h) + v0;
#pragma unroll
  for (int ni = 0; ni < NB; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
      if (r < ci.len) dd[(int64_t)r * dst.st + cc] = ET<T>::from_f(dv[0][ni][i]);
    }
}

// ------------------------------------------------------------------------- //
// reverse state pass        grid = (V / BV, H, N)
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV, bool GDN>
__global__ __launch_bounds__(NTHR) void k_state_bwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16;
  __shared__ __attribute__((aligned(16))) T s_qT[K * LDC];             // (scale q e_b)^T  [K][64]
  __shared__ __attribute__((aligned(16))) T s_doT[BV * LDC];           // do^T             [BV][64]
  __shared__ __attribute__((aligned(16))) T s_kd[GDN ? CH * LDK : 8];  // k e_d            [64][K]
  __shared__ __attribute__((aligned(16))) T s_wT[GDN ? K * LDC : 8];   // w^T              [K][64]
  __shared__ __attribute__((aligned(16))) T s_dvl[GDN ? CH * LDU : 8]; // dv_loc           [64][BV]
  __shared__ __attribute__((aligned(16))) T s_dST[GDN ? BV * LDK : 8]; // dS'^T            [BV][K]
  __shared__ __attribute__((aligned(16))) T s_dvT[GDN ? BV * LDC : 8]; // -dv_new^T        [BV][64]
  __shared__ float s_b[64], s_eb[64], s_ed[64], s_qs[64];

  const int v0 = blockIdx.x * BV, h = blockIdx.y, n = blockIdx.z;
  const SeqInfo sq = seq_info(a, n);
  const int wv = wave_id(), l = lane_id();
  const int krow0 = wv * (K / 4);

  f32x4 dS[MB][NB];
  acc_zero(dS);
  if (a.dht) {
    const float* p = a.dht + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          dS[mi][ni][i] = p[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)];
  }
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;

  for (int c = sq.nchunks - 1; c >= 0; --c) {
    const int tok = sq.tok0 + c * CH;
    const int len = min(CH, sq.len - c * CH);
    chunk_gate_cumsum(a, sq.b, tok, len, h, s_b, s_eb, s_ed);
    if (threadIdx.x < 64) s_qs[threadIdx.x] = a.scale * s_eb[threadIdx.x];
    __syncthreads();
    {
      typename IOK::Regs rq;
      IOK::load(rq, row_ptr<T>(a.q, sq.b, tok, h), a.q.st, len);
      IOK::store_lds_t(rq, s_qT, LDC, s_qs);
      typename IOV::Regs rd;
      IOV::load(rd, row_ptr<T>(a.d_o, sq.b, tok, h) + v0, a.d_o.st, len);
      IOV::store_lds_t(rd, s_doT, LDC, nullptr);
      if constexpr (GDN) {
        typename IOK::Regs rk, rw;
        IOK::load(rk, row_ptr<T>(a.k, sq.b, tok, h), a.k.st, len);
        IOK::store_lds_scaled(rk, s_kd, LDK, s_ed);
        IOK::load(rw, row_ptr<T>(a.w, sq.b, tok, h), a.w.st, len);
        IOK::store_lds_t(rw, s_wT, LDC, nullptr);
        typename IOV::Regs rl;
        IOV::load(rl, row_ptr<T>(a.dvnew, sq.b, tok, h) + v0, a.dvnew.st, len);
        IOV::store_lds(rl, s_dvl, LDU);
      }
    }
    {
      T* dhs = (T*)a.dhs + ((int64_t)(sq.chunk0 + c) * a.H + h) * K * V;
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            dhs[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)] = ET<T>::from_f(dS[mi][ni][i]);
          if constexpr (GDN) acc_to_lds_t<T>(dS[mi][ni], s_dST, LDK, krow0 + 16 * mi, 16 * ni);
        }
    }
    __syncthreads();
    if constexpr (GDN) {
      // dv_new = dv_loc + k_d dS'   (rows 16 wv .. of the chunk)
      f32x4 t[1][NB];
      acc_zero(t);
      gemm_nt<T, 1, NB>(t, s_kd, LDK, 16 * wv, s_dST, LDK, 0, 0, K);
      T* vd = row_ptr<T>(a.dvnew, sq.b, tok, h) + v0;
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
          float y = ET<T>::to_f(s_dvl[r * LDU + cc]) + t[0][ni][i];
          y = ET<T>::to_f(ET<T>::from_f(y));
          if (r < len) vd[(int64_t)r * a.dvnew.st + cc] = ET<T>::from_f(y);
          x[i] = -y;
        }
        acc_to_lds_t<T>(x, s_dvT, LDC, 16 * wv, 16 * ni);
      }
      __syncthreads();
    }
    const float dec = expf(s_b[63]);
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) dS[mi][ni] *= dec;
    gemm_nt<T, MB, NB>(dS, s_qT, LDC, krow0, s_doT, LDC, 0, 0, CH);
    if constexpr (GDN) gemm_nt<T, MB, NB>(dS, s_wT, LDC, krow0, s_dvT, LDC, 0, 0, CH);
    __syncthreads();
  }
  if (a.dh0) {
    float* p = a.dh0 + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          p[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)] = dS[mi][ni][i];
  }
}

// ------------------------------------------------------------------------- //
// dq, dk, gate gradient        grid = (NT, H)
//   phase A: loop over V-slices of width BVH accumulating
//              dP = do v'^T, dq_i = do S^T, dk_d = v' dS'^T (, dw = dv_new S^T)
//   phase B: dq = scale e_b dq_i + (scale dP . Gamma) k ; dk = e_d dk_d + (scale dP . Gamma)^T q
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BVH, bool GDN>
__global__ __launch_bounds__(NTHR) void k_bwd_dqk(const lmoe_args a) {
  constexpr int LDV = BVH + LPAD, LDC = CH + LPAD;
  constexpr int NBK = K / 16;
  // phase A tiles
  constexpr int A_DO = 0, A_V = A_DO + CH * LDV, A_H = A_V + CH * LDV, A_DH = A_H + K * LDV,
                A_DVN = A_DH + K * LDV, A_END = A_DVN + (GDN ? CH * LDV : 0);
  // phase B tiles
  constexpr int B_DP = 0, B_DPT = B_DP + CH * LDC, B_KT = B_DPT + CH * LDC, B_QT = B_KT + K * LDC,
                B_END = B_QT + K * LDC;
  constexpr int NELEM = A_END > B_END ? A_END : B_END;
  __shared__ __attribute__((aligned(16))) T smem[NELEM];
  __shared__ float s_b[64], s_eb[64], s_ed[64], s_db[64], s_red[8];

  const int cid = blockIdx.x, h = blockIdx.y;
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  chunk_gate_cumsum(a, ci.b, ci.tok, ci.len, h, s_b, s_eb, s_ed);

  typedef TileIO<T, CH, BVH> IOV;
  typedef TileIO<T, K, BVH> IOH;
  typedef TileIO<T, CH, K> IOK;
  const lmoe_tensor& vs = GDN ? a.vnew : a.v;

  f32x4 dP[1][4], dqi[1][NBK], dkd[1][NBK], dw[1][GDN ? NBK : 1];
  acc_zero(dP); acc_zero(dqi); acc_zero(dkd); acc_zero(dw);
  float hdh = 0.f;   // partial <S, dS'>
  for (int vv = 0; vv < V; vv += BVH) {
    {
      typename IOV::Regs rd, rv;
      IOV::load(rd, row_ptr<T>(a.d_o, ci.b, ci.tok, h) + vv, a.d_o.st, ci.len);
      IOV::load(rv, row_ptr<T>(vs, ci.b, ci.tok, h) + vv, vs.st, ci.len);
      typename IOH::Regs rh, rdh;
      IOH::load(rh, (const T*)a.hs + ((int64_t)cid * a.H + h) * K * V + vv, V, K);
      IOH::load(rdh, (const T*)a.dhs + ((int64_t)cid * a.H + h) * K * V + vv, V, K);
#pragma unroll
      for (int p = 0; p < IOH::PASSES; ++p)
#pragma unroll
        for (int i = 0; i < IOH::VEC; ++i) hdh += ET<T>::to_f(rh.v[p][i]) * ET<T>::to_f(rdh.v[p][i]);
      IOV::store_lds(rd, smem + A_DO, LDV);
      IOV::store_lds(rv, smem + A_V, LDV);
      IOH::store_lds(rh, smem + A_H, LDV);
      IOH::store_lds(rdh, smem + A_DH, LDV);
      if constexpr (GDN) {
        typename IOV::Regs rn;
        IOV::load(rn, row_ptr<T>(a.dvnew, ci.b, ci.tok, h) + vv, a.dvnew.st, ci.len);
        IOV::store_lds(rn, smem + A_DVN, LDV);
      }
    }
    __syncthreads();
    gemm_nt<T, 1, 4>(dP, smem + A_DO, LDV, 16 * wv, smem + A_V, LDV, 0, 0, BVH);
    gemm_nt<T, 1, NBK>(dqi, smem + A_DO, LDV, 16 * wv, smem + A_H, LDV, 0, 0, BVH);
    gemm_nt<T, 1, NBK>(dkd, smem + A_V, LDV, 16 * wv, smem + A_DH, LDV, 0, 0, BVH);
    if constexpr (GDN) gemm_nt<T, 1, NBK>(dw, smem + A_DVN, LDV, 16 * wv, smem + A_H, LDV, 0, 0, BVH);
    __syncthreads();
  }
  // block reduction of <S, dS'>
  hdh = wave_sum(hdh);
  if (l == 0) s_red[wv] = hdh;
  // phase B operands
  {
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r >= cc) ? a.scale * dP[0][nj][i] * expf(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds<T>(p, smem + B_DP, LDC, 16 * wv, 16 * nj);
      acc_to_lds_t<T>(p, smem + B_DPT, LDC, 16 * wv, 16 * nj);
    }
    typename IOK::Regs rq, rk;
    IOK::load(rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
    IOK::load(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
    IOK::store_lds_t(rq, smem + B_QT, LDC, nullptr);
    IOK::store_lds_t(rk, smem + B_KT, LDC, nullptr);
  }
  __syncthreads();
  f32x4 dq[1][NBK], dk[1][NBK];
  acc_zero(dq); acc_zero(dk);
  gemm_nt<T, 1, NBK>(dq, smem + B_DP, LDC, 16 * wv, smem + B_KT, LDC, 0, 0, CH);
  gemm_nt<T, 1, NBK>(dk, smem + B_DPT, LDC, 16 * wv, smem + B_QT, LDC, 0, 0, CH);
  // combine, store, and form db_i = q_i.dq_i - k_i.dk_i ; kk = sum_j (dk_d . k_d)_j
  float dbp[4] = {0.f, 0.f, 0.f, 0.f};
  float kk = 0.f;
  T* dqd = row_ptr<T>(a.dq, ci.b, ci.tok, h);
  T* dkd_ = row_ptr<T>(a.dk, ci.b, ci.tok, h);
  T* dwd = GDN ? row_ptr<T>(a.dw, ci.b, ci.tok, h) : nullptr;
#pragma unroll
  for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
      const float qv = ET<T>::to_f(smem[B_QT + cc * LDC + r]);
      const float kv = ET<T>::to_f(smem[B_KT + cc * LDC + r]);
      const float dqv = a.scale * s_eb[r] * dqi[0][ni][i] + dq[0][ni][i];
      const float dkdv = s_ed[r] * dkd[0][ni][i];
      const float dkv = dkdv + dk[0][ni][i];
      dbp[i] += qv * dqv - kv * dkv;
      kk += kv * dkdv;
      if (r < ci.len) {
        dqd[(int64_t)r * a.dq.st + cc] = ET<T>::from_f(dqv);
        dkd_[(int64_t)r * a.dk.st + cc] = ET<T>::from_f(dkv);
        if constexpr (GDN) dwd[(int64_t)r * a.dw.st + cc] = ET<T>::from_f(-dw[0][ni][i]);
      }
    }
  // reduce db over the 16 lanes that share a row group, kk over the whole block
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int d = 1; d < 16; d <<= 1) dbp[i] += __shfl_xor(dbp[i], d, 64);
  }
  if ((l & 15) == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) s_db[16 * wv + 4 * (l >> 4) + i] = dbp[i];
  }
  kk = wave_sum(kk);
  if (l == 0) s_red[4 + wv] = kk;
  __syncthreads();
  if (threadIdx.x < 64) {
    const int j = threadIdx.x;
    float x = s_db[j];
    // last-row term; rows past the end of a partial chunk carry zero q, k, so the term may sit
    // on the last valid row without changing the reverse cumulative sum
    const float hsum = s_red[0] + s_red[1] + s_red[2] + s_red[3];
    const float ksum = s_red[4] + s_red[5] + s_red[6] + s_red[7];
    if (j == ci.len - 1) x += ksum + expf(s_b[63]) * hsum;
    if constexpr (!GDN) x = wave_rev_scan(x);   // dg; the delta rule finishes db in its WY backward
    if (a.dg.ptr && j < ci.len) ((float*)a.dg.ptr)[row_off(a.dg, ci.b, ci.tok + j, h)] = x;
  }
}

}  // namespace lmoe
