// chunk_gla kernels: per-channel log-decays g_t in R^K.
// Per chunk: b = inclusive cumsum of g over tokens (fp32, [64 x K]);
//   A_ij  = sum_k q_ik k_jk e^{b_ik - b_jk}   (i >= j)     exponent formed per pair: always <= 0
//   o     = scale [ (q . e^{b}) S + A v ]
//   S'    = diag(e^{b_C}) S + (k . e^{b_C - b})^T v
// Backward (dS' = gradient w.r.t. the state at chunk end, dA = scale do v^T masked i >= j):
//   dv    = scale A^T do + (k . e^{b_C - b}) dS'
//   dS    = diag(e^{b_C}) dS' + scale (q . e^{b})^T do
//   dq_ik = scale e^{b_ik} (do S^T)_ik + sum_{j<=i} dA_ij k_jk e^{b_ik - b_jk}
//   dk_jk = e^{b_Ck - b_jk} (v dS'^T)_jk + sum_{i>=j} dA_ij q_ik e^{b_ik - b_jk}
//   db_ik = q_ik dq_ik - k_ik dk_ik (+ on the last row: sum_j (dk_d . k_d)_jk + e^{b_Ck} sum_v S_kv dS'_kv)
//   dg    = reverse cumsum of db over the chunk's tokens
// The gated operands q e^{b} and k e^{b_C - b} and the chunk decay e^{b_C} are formed once, by the
// chunk-parallel kernel that computes A (it holds q, k and b in LDS anyway), and stored per chunk
// ([NT,H,64,K], rows past the end of a partial chunk zero): the two sequential state passes and the
// output / dv kernels then need neither the gate nor a scan nor an exponential.
// Pairwise exponents are formed only inside 16-token sub-chunks (vector ALU, fp32); between
// sub-chunks the decay factors through the cumulative gate at the sub-chunk boundary, which turns
// those parts into products of scaled tiles on MFMA, like every other product here.
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

constexpr int cmax(int a, int b) { return a > b ? a : b; }
// largest decay exponent over one 16-token sub-chunk up to which chunk_gla factors its diagonal blocks through a
// reference gate (e^60 ~ 1e26 leaves fp32 / bf16 range to spare for the operand it multiplies)
constexpr float GLA_SAFE_EXP = 60.0f;
// first row of the k~ copy of block row I inside the stacked tile: 0, 16, 48, 96
constexpr int KT_ROW0(int I) { return 8 * I * (I + 1); }

// N consecutive fp32 values of an LDS tile whose rows start on 16-byte boundaries, as 16-byte reads (left to the
// compiler, a column group of the gate tile arrives as N scalar reads)
template <int N> __device__ __forceinline__ void load_f32_group(const float* p, float (&b)[N]) {
  static_assert(N % 4 == 0, "whole 16-byte pieces");
#pragma unroll
  for (int e4 = 0; e4 < N; e4 += 4) {
    const f32x4 t = *(const f32x4*)(p + e4);
#pragma unroll
    for (int e = 0; e < 4; ++e) b[e4 + e] = t[e];
  }
}

// g tile of the chunk -> fp32 LDS tile s_b[64][LDB] holding the inclusive cumsum over tokens.
// The scan: a thread takes one channel over a segment of 64 K / 256 tokens (its values in registers, so the
// LDS reads are independent of each other), the segment totals go through a small LDS array, and every thread
// adds the totals of the segments before its own.  All 256 threads; ends with a barrier (the barriers order
// LDS traffic only: loads a caller keeps in flight stay in flight).
template <typename GT, int K>
struct GlaGate {
  typedef TileIO<GT, CH, K> IOG;
  typedef typename IOG::Regs Regs;
  static __device__ __forceinline__ void issue(Regs& rg, const lmoe_args& a, int b, int tok, int len, int h) {
    IOG::load_nomask(rg, row_ptr<GT>(a.g, b, tok, h), a.g.st, len);
  }
  // tot: NTHR floats of LDS for the segment totals
  template <int LDB>
  // mult: factor applied to the stored cumsum (1, or TEXP_PRESCALE<T> for kernels that only form exponentials of it)
  static __device__ __forceinline__ void finish(Regs& rg, int len, float* s_b, float* s_tot, float mult = 1.0f) {
    constexpr int NSEG = NTHR / K, SEG = CH / NSEG;
    static_assert(NTHR % K == 0 && CH % NSEG == 0, "one channel and one token segment per thread");
    IOG::mask(rg, len);
    IOG::store_lds_f32(rg, s_b, LDB);
    lds_barrier();
    const int c = threadIdx.x % K, sg = threadIdx.x / K;
    float v[SEG];
#pragma unroll
    for (int r = 0; r < SEG; ++r) v[r] = s_b[(sg * SEG + r) * LDB + c];
#pragma unroll
    for (int r = 1; r < SEG; ++r) v[r] += v[r - 1];
    s_tot[sg * K + c] = v[SEG - 1];
    lds_barrier();
    float off = 0.f;
#pragma unroll
    for (int q = 0; q < NSEG - 1; ++q) off += q < sg ? s_tot[q * K + c] : 0.f;
#pragma unroll
    for (int r = 0; r < SEG; ++r) s_b[(sg * SEG + r) * LDB + c] = (v[r] + off) * mult;
    lds_barrier();
  }
  template <int LDB>
  static __device__ __forceinline__ void finish(Regs& rg, int len, float* s_b) {
    __shared__ float s_tot[NTHR];
    finish<LDB>(rg, len, s_b, s_tot);
  }
};
template <typename GT, int K, int LDB = K + 1>
__device__ __forceinline__ void gla_gate_tile(const lmoe_args& a, int b, int tok, int len, int h, float* s_b) {
  typename GlaGate<GT, K>::Regs rg;
  GlaGate<GT, K>::issue(rg, a, b, tok, len, h);
  GlaGate<GT, K>::template finish<LDB>(rg, len, s_b);
}

// ------------------------------------------------------------------------- //
// A (intra-chunk attention matrix), persistent grid over the (chunk, head) items
//   The chunk is cut into four sub-chunks of 16 tokens.  For a block (I, J) with J < I the decay
//   factors through the cumulative gate at the last token before sub-chunk I, b* = b_{16 I - 1}:
//     A_ij = sum_k (q_ik e^{b_ik - b*_k}) (k_jk e^{b*_k - b_jk}),   both exponents <= 0,
//   which is a matrix product of two scaled tiles (MFMA).  Only the four diagonal blocks need the
//   exponent per pair; they run on the vector ALU in fp32, one block per wave, four pairs per lane.
// ------------------------------------------------------------------------- //
template <typename T, typename GT, int K>
__global__ __launch_bounds__(NTHR) void k_gla_intra_fwd(const lmoe_args a) {
  constexpr int LDB = K + 4, LDK = K + LPAD, LDC = CH + LPAD;
  __shared__ __attribute__((aligned(16))) float s_b[CH * LDB];
  __shared__ __attribute__((aligned(16))) T s_q[CH * LDK];        // q, k as loaded
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];
  // all block rows at once where LDS has room for the stacked k~ tile (everything but fp32 with K = 128), else
  // one block row at a time with the diagonal blocks always on the vector ALU
  constexpr bool ONE_PASS = (CH * LDB * 4 + (3 * CH * LDK + 160 * LDK + CH * LDC) * (int)sizeof(T)) <= 150 * 1024;
  __shared__ __attribute__((aligned(16))) T s_qt[(ONE_PASS ? CH : 16) * LDK];   // q~: rows scaled to the reference of their block row
  __shared__ __attribute__((aligned(16))) T s_kt[(ONE_PASS ? 160 : 48) * LDK];  // k~ of block rows 0..3: 16 + 32 + 48 + 64 rows
  __shared__ __attribute__((aligned(16))) T s_A[CH * LDC];
  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, CH> IOA;
  typedef GlaGate<GT, K> GG;
  // persistent: item = (chunk, head); the next item's q, k, g are requested at the top of an item and stay in
  // flight behind its LDS-only barriers (item index clamped: every load is issued)
  const int nitems = num_chunks(a) * a.H;
  if (nitems <= 0) return;                   // (a chunk count read on the device may be zero)
  struct Pre { typename IOK::Regs rq, rk; typename GG::Regs rg; };
  Pre pre;
  auto issue = [&](int it) {
    it = min(it, nitems - 1);
    const int cid = it / a.H, h = it % a.H;
    const ChunkInfo ci = chunk_info(a, cid);
    IOK::load_nomask(pre.rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
    IOK::load_nomask(pre.rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
    GG::issue(pre.rg, a, ci.b, ci.tok, ci.len, h);
  };
  issue(blockIdx.x);
  for (int it = blockIdx.x; it < nitems; it += gridDim.x) {
  const int cid = it / a.H, h = it % a.H;
  const ChunkInfo ci = chunk_info(a, cid);
  {
    typename IOK::Regs rq = pre.rq, rk = pre.rk;
    IOK::mask(rq, ci.len);
    IOK::mask(rk, ci.len);
    IOK::store_lds(rq, s_q, LDK);
    IOK::store_lds(rk, s_k, LDK);
  }
  typename GG::Regs rg = pre.rg;
  issue(it + gridDim.x);
  {                                                                                        // blocks above the diagonal
    constexpr int VEC = ET<T>::VEC;
    static_assert((CH * LDC) % VEC == 0, "whole 16-byte pieces");
    for (int idx = threadIdx.x; idx < CH * LDC / VEC; idx += NTHR) *(typename ET<T>::vec*)(s_A + idx * VEC) = ET<T>::zero();
  }
  GG::template finish<LDB>(rg, ci.len, s_b, (float*)s_qt, TEXP_PRESCALE<T>);    // barriers inside; b in exp2 units
  // ---- gated operands for the other kernels: q e^{b}, k e^{b_C - b}, e^{b_C} ----
  {
    constexpr int VEC = ET<T>::VEC;
    typedef typename ET<T>::vec vec;
    T* qe = (T*)a.qe + ((int64_t)cid * a.H + h) * CH * K;
    T* ke = (T*)a.ke + ((int64_t)cid * a.H + h) * CH * K;
    static_assert(CH * K / VEC % NTHR == 0, "whole passes");
#pragma unroll
    for (int ps = 0; ps < CH * K / VEC / NTHR; ++ps) {
      const int e = ps * NTHR + threadIdx.x;
      const int r = e / (K / VEC), c0 = (e % (K / VEC)) * VEC;
      const vec qv = *(const vec*)(s_q + r * LDK + c0), kv = *(const vec*)(s_k + r * LDK + c0);
      vec qo, ko;
      float b[VEC], bC[VEC];
      load_f32_group(s_b + r * LDB + c0, b);
      load_f32_group(s_b + 63 * LDB + c0, bC);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        qo[j] = ET<T>::from_f(ET<T>::to_f(qv[j]) * texp_scaled<T>(b[j]));
        ko[j] = ET<T>::from_f(ET<T>::to_f(kv[j]) * texp_scaled<T>(bC[j] - b[j]));
      }
      *(vec*)(qe + r * K + c0) = qo;
      *(vec*)(ke + r * K + c0) = ko;
    }
    if (threadIdx.x < K) a.gcum[((int64_t)cid * a.H + h) * K + threadIdx.x] = texp_scaled<T>(s_b[63 * LDB + threadIdx.x]);
  }
  // ---- is the decay inside every 16-token sub-chunk small enough to factor the diagonal blocks too? ----
  // Block row I (tokens 16 I ..) takes the cumulative gate just before it as its reference, b* = b_{16 I - 1}
  // (0 for I = 0):  A_ij = sum_k (q_ik e^{b_ik - b*_k}) (k_jk e^{b*_k - b_jk}).  For j before the block row both
  // exponents are <= 0.  For j inside it the second one is the decay over at most 16 tokens, >= 0: taken only
  // if it stays below GLA_SAFE_EXP for every channel, otherwise that diagonal block forms its exponent per pair
  // on the vector ALU (always safe; what fla's diagonal sub-blocks do).
  int unsafe = 0;
  if (threadIdx.x < K) {
#pragma unroll
    for (int I = 0; I < 4; ++I) {
      const float ref = I == 0 ? 0.f : s_b[(16 * I - 1) * LDB + threadIdx.x];
      if (!(ref - s_b[(16 * I + 15) * LDB + threadIdx.x] <= GLA_SAFE_EXP * TEXP_PRESCALE<T>)) unsafe |= 1 << I;
    }
  }
  if constexpr (ONE_PASS) {
    // bitwise OR over the work-group (the barrier-with-predicate intrinsics only tell zero from non-zero)
    __shared__ int s_unsafe;
    if (threadIdx.x == 0) s_unsafe = 0;
    lds_barrier();
    if (unsafe) atomicOr(&s_unsafe, unsafe);
    lds_barrier();
    unsafe = s_unsafe;
  } else {
    unsafe = 15;
  }
  // ---- diagonal blocks that cannot be factored: wave w owns block (w, w); lane -> row i, columns j0 .. j0 + 3 ----
  if ((unsafe >> wv) & 1) {
    const int i = 16 * wv + (l & 15), j0 = 16 * wv + 4 * (l >> 4);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k4 = 0; k4 < K; k4 += 4) {
      const f32x4 bi = *(const f32x4*)(s_b + i * LDB + k4);
      float qi[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) qi[e] = ET<T>::to_f(s_q[i * LDK + k4 + e]);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int j = j0 + jj;
        const f32x4 bj = *(const f32x4*)(s_b + j * LDB + k4);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc[jj] += qi[e] * ET<T>::to_f(s_k[j * LDK + k4 + e]) * texp_scaled<T>(fminf(bi[e] - bj[e], 0.f));
      }
    }
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) s_A[i * LDC + j0 + jj] = ET<T>::from_f(i >= j0 + jj ? acc[jj] : 0.f);
  }
  if constexpr (ONE_PASS) {
  // ---- scaled operands of all block rows at once: q~ (64 rows), k~ of block row I = rows 0 .. 16 I + 15 ----
  {
    constexpr int VEC = ET<T>::VEC;
    typedef typename ET<T>::vec vec;
    // stacked rows 0 .. 63: q~; 64 .. 223: k~ of block rows 0 .. 3 (16-byte pieces).  Unrolled: a pass is a chain of
    // LDS reads, exponentials and a write, and seven (fourteen) of them one after the other cost a third of an item
    constexpr int NPASS = (CH + 160) * (K / VEC) / NTHR;
    static_assert((CH + 160) * (K / VEC) % NTHR == 0, "whole passes");
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int idx = ps * NTHR + threadIdx.x;
      const int sr = idx / (K / VEC), c0 = (idx % (K / VEC)) * VEC;
      const bool isq = sr < CH;
      const int kr = sr - CH;                                           // row of the stacked k~ tile
      const int I = isq ? (sr >> 4) : (kr < 16 ? 0 : kr < 48 ? 1 : kr < 96 ? 2 : 3);
      const int tok = isq ? sr : kr - KT_ROW0(I);
      const vec x = *(const vec*)((isq ? s_q : s_k) + tok * LDK + c0);
      vec o;
      float ref[VEC], bt[VEC];
      load_f32_group(s_b + tok * LDB + c0, bt);
      load_f32_group(s_b + (I == 0 ? 0 : 16 * I - 1) * LDB + c0, ref);      // (row 0 for I = 0: read, not used)
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = I == 0 ? bt[e] : bt[e] - ref[e];
        o[e] = ET<T>::from_f(ET<T>::to_f(x[e]) * texp_scaled<T>(isq ? d : -d));
      }
      *(vec*)((isq ? s_qt + sr * LDK : s_kt + kr * LDK) + c0) = o;
    }
  }
  lds_barrier();
  // wave w: the blocks (I, w), I = w .. 3; the diagonal one masked to i >= j
#pragma unroll
  for (int I = 0; I < 4; ++I) {
    if (wv > I || (wv == I && ((unsafe >> I) & 1))) continue;
    f32x4 t[1][1];
    acc_zero(t);
    gemm<T, 1, 1, false, false, true>(t, s_qt, LDK, 16 * I, s_kt + KT_ROW0(I) * LDK, LDK, 16 * wv, 0, K);
    if (wv == I) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (4 * (l >> 4) + e < (l & 15)) t[0][0][e] = 0.f;
    }
    acc_to_lds<T>(t[0][0], s_A, LDC, 16 * I, 16 * wv);
  }
  lds_barrier();
  } else {
    // ---- blocks below the diagonal, one block row at a time ----
    for (int I = 1; I < 4; ++I) {
      const float* bs = s_b + (16 * I - 1) * LDB;                   // b* of this block row
      for (int idx = threadIdx.x; idx < 16 * K; idx += NTHR) {
        const int r = idx / K, c = idx % K, i = 16 * I + r;
        s_qt[r * LDK + c] = ET<T>::from_f(ET<T>::to_f(s_q[i * LDK + c]) * texp_scaled<T>(s_b[i * LDB + c] - bs[c]));
      }
      for (int idx = threadIdx.x; idx < 16 * I * K; idx += NTHR) {
        const int j = idx / K, c = idx % K;
        s_kt[j * LDK + c] = ET<T>::from_f(ET<T>::to_f(s_k[j * LDK + c]) * texp_scaled<T>(bs[c] - s_b[j * LDB + c]));
      }
      lds_barrier();
      if (wv < I) {
        f32x4 t[1][1];
        acc_zero(t);
        gemm<T, 1, 1, false, false, true>(t, s_qt, LDK, 0, s_kt, LDK, 16 * wv, 0, K);
        acc_to_lds<T>(t[0][0], s_A, LDC, 16 * I, 16 * wv);
      }
      lds_barrier();
    }
  }
  IOA::lds_to_global(s_A, LDC, (T*)a.amat + ((int64_t)cid * a.H + h) * CH * CH, CH, CH);
  lds_barrier();      // the tiles are rewritten by the next item
  }
}

// ------------------------------------------------------------------------- //
// forward state pass, 1-D grid (XCD-aware, see the kernel)
// ------------------------------------------------------------------------- //
template <typename T, typename GT, int K, int V, int BV>
__global__ __launch_bounds__(NTHR) void k_gla_state_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16;
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];     // k e^{b_C - b}     [64][K]
  __shared__ __attribute__((aligned(16))) T s_v[CH * LDU];     // v                 [64][BV]
  __shared__ __attribute__((aligned(16))) T s_h[K * LDU];      // S on its way out  [K][BV]
  // 1-D grid of ceil(N H / 8) * 8 * (V / BV) work-groups; the V-slices of one (sequence, head) get ids that are
  // congruent mod 8, i.e. run on the same XCD and share its gated k (q) rows through that XCD's L2
  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = (jj % NVS) * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
  const SeqInfo sq = seq_info(a, n);
  const int wv = wave_id();
  const int krow0 = wv * (K / 4);
  f32x4 S[MB][NB];
  acc_zero(S);
  if (a.h0) {
    const float* h0 = a.h0 + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i) S[mi][ni][i] = h0[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)];
  }
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;
  typedef TileIO<T, K, BV> IOH;
  // The operands of the next PF chunks are kept in flight in PF register sets (chunk index clamped: every load
  // is issued; the surplus ones at the end are never used): one chunk of this pass is shorter than a trip to HBM.
  constexpr int PF = 3;
  struct Pre { typename IOK::Regs rk; typename IOV::Regs rv; float dec[MB][4]; };
  Pre pre[PF];
  auto issue = [&](Pre& P, int c) {
    c = min(c, sq.nchunks - 1);
    const int64_t item = (int64_t)(sq.chunk0 + c) * a.H + h;
    IOK::load_nomask(P.rk, (const T*)a.ke + item * CH * K, K, CH);
    IOV::load_nomask(P.rv, row_ptr<T>(a.v, sq.b, sq.tok0 + c * CH, h) + v0, a.v.st, min(CH, sq.len - c * CH));
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int i = 0; i < 4; ++i) P.dec[mi][i] = a.gcum[item * K + krow0 + acc_row(mi, i)];
  };
  if (sq.nchunks > 0) {
#pragma unroll
    for (int j = 0; j < PF; ++j) issue(pre[j], j);
  }
  for (int c0 = 0; c0 < sq.nchunks; c0 += PF) {
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int c = c0 + j;
      if (c >= sq.nchunks) break;
      const int len = min(CH, sq.len - c * CH);
      Pre& P = pre[j];
      IOK::store_lds(P.rk, s_k, LDK);
      IOV::mask(P.rv, len);
      IOV::store_lds(P.rv, s_v, LDU);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          acc_to_lds<T>(S[mi][ni], s_h, LDU, krow0 + 16 * mi, 16 * ni);
#pragma unroll
          for (int i = 0; i < 4; ++i) S[mi][ni][i] *= P.dec[mi][i];
        }
      issue(P, c + PF);
      lds_barrier();      // LDS-only: the loads stay in flight
      IOH::lds_to_global(s_h, LDU, (T*)a.hs + ((int64_t)(sq.chunk0 + c) * a.H + h) * K * V + v0, V, K);
      // S += (k e^{b_C - b})^T v
#pragma unroll
      for (int kk = 0; kk < CH; kk += 32) {
        typename ET<T>::frag af[MB], bf[NB];
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) af[mi] = ET<T>::load_frag_t(s_k, LDK, kk, krow0 + 16 * mi);
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) bf[ni] = ET<T>::load_frag_t(s_v, LDU, kk, 16 * ni);
#pragma unroll
        for (int mi = 0; mi < MB; ++mi)
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(S[mi][ni], af[mi], bf[ni]);
      }
      lds_barrier();
    }
  }
  if (a.ht) {
    float* ht = a.ht + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i) ht[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)] = S[mi][ni][i];
  }
}

// ------------------------------------------------------------------------- //
// forward state pass AND output in one kernel (2-byte elements), 1-D grid as k_gla_state_fwd, 768 threads.
// The three-team, one-barrier-per-chunk design of the scalar-gate forward pass (k_state_fwd_b, lmoe_scalar_fwd.hpp)
// on the operands k_gla_intra_fwd stored: q e^{b}, k e^{b_C - b}, the intra-chunk matrix A and the chunk decay
// e^{b_C}, so that the pass needs no gate, no exponential and forms no P.  The output leaves the kernel that holds the
// state: S is not read back from memory by a kernel of its own (k_gla_out_fwd fetched hs, q e^{b}, A and v again).
//   consumers (waves 0-3):  S = diag(e^{b_C}) S + (k e^{b_C - b})^T v in fp32 accumulators (wave w: K rows K/4 w ..),
//                           S^T of the next chunk -> s_hT, then the fragments of the next update
//   loaders   (waves 4-7):  three register sets of (k~, q~, v, decay), chunk c + 2 staged into the buffer of
//                           chunk c as window c opens; with SAVE hs[chunk] <- S (layout [K][V]) through transposing
//                           reads of s_hT: a lane holds eight consecutive V columns of one K row, 16-byte stores
//   output    (waves 8-11): rows 16 w .. of o^T = S^T q~^T + v^T A^T in one accumulator (the products, their order
//                           and the rounding of k_gla_out_fwd: the same bits), stored from registers; its rows of A
//                           come straight from memory into the lanes that use them, two chunks ahead
// Two buffers of every tile: what a window reads of a chunk's own operands was read into registers at the end of the
// window before (see k_state_fwd_b).
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV, bool SAVE>
__global__ __launch_bounds__(3 * NTHR) void k_gla_fwd_fused(const lmoe_args a) {
  static_assert(sizeof(T) == 2, "2-byte elements");
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16, KS = K / 32, CS = CH / 32;
  __shared__ __attribute__((aligned(16))) T s_k[2][CH * LDK];                 // k e^{b_C - b}  [64][K]
  __shared__ __attribute__((aligned(16))) T s_q[2][CH * LDK];                 // q e^{b}        [64][K]
  __shared__ __attribute__((aligned(16))) T s_u[2][CH * LDU];                 // v              [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[2][BV * LDK];                // S^T            [BV][K]
  __shared__ __attribute__((aligned(16))) float s_dec[2][K];                  // e^{b_C}        [K]

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = (jj % NVS) * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
  const SeqInfo sq = seq_info(a, n);
  const int l = lane_id();
  // (wave-uniform by construction; said to the compiler, so that the branches on it are scalar branches: a matrix
  // instruction runs whatever the lane mask, and a short masked region is not jumped over)
  const int wave = __builtin_amdgcn_readfirstlane(wave_id());
  const int team = wave >> 2;
  if (sq.nchunks == 0) {
    // empty sequence: the final state is the initial state
    if (a.ht && team == 0) {
      for (int idx = threadIdx.x; idx < K * BV; idx += NTHR) {
        const int r = idx / BV, c = v0 + idx % BV;
        const int64_t o = ((int64_t)n * a.H + h) * K * V + (int64_t)r * V + c;
        a.ht[o] = a.h0 ? a.h0[o] : 0.f;
      }
    }
    return;
  }
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;

  if (team == 1) {
    // --------------------------------- loaders -------------------------------------------
    const int tid = threadIdx.x & (NTHR - 1);
    struct Pre { typename IOK::Regs rk, rq; typename IOV::Regs ru; float dec; int len; };
    Pre pre[3];                                              // register set = chunk % 3
    // Always issued (chunk index clamped to the last chunk; the surplus loads at the end of a sequence are never
    // consumed): a prefetch that is skipped on some path would make the compiler drain all outstanding loads at
    // every consumer of a register set.
    auto issue = [&](Pre& P, int c) {
      c = min(c, sq.nchunks - 1);
      const int64_t item = (int64_t)(sq.chunk0 + c) * a.H + h;
      const int len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rk, (const T*)a.ke + item * CH * K, K, CH);
      IOK::load_nomask(P.rq, (const T*)a.qe + item * CH * K, K, CH);
      IOV::load_nomask(P.ru, row_ptr<T>(a.v, sq.b, sq.tok0 + c * CH, h) + v0, a.v.st, len);
      P.dec = a.gcum[item * K + min(tid, K - 1)];
      P.len = len;
    };
    // registers -> LDS buffer `buf`
    auto stage = [&](Pre& P, int buf) {
      IOV::mask(P.ru, P.len);
      IOK::store_lds(P.rk, s_k[buf], LDK);
      IOK::store_lds(P.rq, s_q[buf], LDK);
      IOV::store_lds(P.ru, s_u[buf], LDU);
      if (tid < K) s_dec[buf][tid] = P.dec;
    };
    // hs[chunk][h][K][v0 .. v0+BV] <- S (only the backward reads it: SAVE = false for forward-only calls): S^T read
    // through the transposing LDS read, lane (c, g): K row 16 kb + c, V columns 32 vb + 8 g .. + 7
    auto save_state = [&](int c) {
      if constexpr (SAVE) {
        T* hs = (T*)a.hs + ((int64_t)(sq.chunk0 + c) * a.H + h) * K * V + v0;
#pragma unroll
        for (int kb = 0; kb < K / 64; ++kb)
#pragma unroll
          for (int vb = 0; vb < BV / 32; ++vb) {
            const int k0 = 16 * (4 * kb + (wave - 4));
            const typename ET<T>::frag x = ET<T>::load_frag_t(s_hT[c & 1], LDK, 32 * vb, k0, l);
            *(typename ET<T>::vec*)(hs + (int64_t)(k0 + (l & 15)) * V + 32 * vb + 8 * (l >> 4)) = x;
          }
      }
    };
#pragma unroll
    for (int j = 0; j < 3; ++j) issue(pre[j], j);
    stage(pre[0], 0);
    issue(pre[0], 3);
    stage(pre[1], 1);
    lds_barrier();                                                                       // chunks 0, 1 staged
    for (int c0 = 0; c0 < sq.nchunks; c0 += 3) {
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int c = c0 + j;
        if (c >= sq.nchunks) break;
        lds_barrier();
        // (both always: past the end it is the last chunk again, never consumed)
        issue(pre[(j + 1) % 3], c + 4);
        stage(pre[(j + 2) % 3], c & 1);          // chunk c + 2 takes the buffers of chunk c
        save_state(c);
      }
    }
    return;
  }

  if (team == 2) {
    // --------------------------------- output --------------------------------------------
    const int ow = wave - 8;
    const int fr = l & 15, fg = 8 * (l >> 4), g4 = 4 * (l >> 4);
    lds_barrier();                                                                       // chunks 0, 1 staged
    typename ET<T>::frag fq[KS], fv[CS][NB];
    // The rows of A of this wave enter only as its own matrix operand: they come straight from memory into the
    // registers of the lane that uses them (row 16 ow + fr, 8 tokens per 32), two chunks ahead, in two register
    // sets (chunk parity) - no LDS tile, nothing for the loaders to stage.  Always requested (chunk index clamped),
    // blocks above the diagonal included (zeros as stored): no load sits behind a branch.
    typename ET<T>::frag fp[2][CS];
    auto issue_A = [&](typename ET<T>::frag (&f)[CS], int c) {
      c = min(c, sq.nchunks - 1);
      const T* A = (const T*)a.amat + ((int64_t)(sq.chunk0 + c) * a.H + h) * CH * CH + (16 * ow + fr) * CH + fg;
#pragma unroll
      for (int kq = 0; kq < CS; ++kq) f[kq] = *(const typename ET<T>::vec*)(A + 32 * kq);
    };
    issue_A(fp[0], 0);
    issue_A(fp[1], 1);
    auto preread = [&](int c) {
      const int cb = c & 1;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) fq[ks] = ET<T>::load_frag(s_q[cb] + (16 * ow + fr) * LDK + 32 * ks + fg);
#pragma unroll
      for (int kq = 0; kq < CS; ++kq) {
        if (2 * kq <= ow) {          // tokens j >= 32 only reach the rows of waves 2, 3 (A is lower triangular)
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) fv[kq][ni] = ET<T>::load_frag_t(s_u[cb], LDU, 32 * kq, 16 * ni, l);
        }
      }
    };
    preread(0);
    for (int c0 = 0; c0 < sq.nchunks; c0 += 2) {
#pragma unroll
     for (int j = 0; j < 2; ++j) {
      const int c = c0 + j;
      if (c >= sq.nchunks) break;
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      lds_barrier();
      typename ET<T>::frag fh[KS][NB];
      const T* hT = s_hT[c & 1];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) fh[ks][ni] = ET<T>::load_frag(hT + (16 * ni + fr) * LDK + 32 * ks + fg);
      __builtin_amdgcn_sched_barrier(0);
      f32x4 o[NB];
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) o[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(o[ni], fh[ks][ni], fq[ks]);            // (q~ S)^T: column x token
#pragma unroll
      for (int kq = 0; kq < CS; ++kq) {
        if (2 * kq <= ow) {
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(o[ni], fv[kq][ni], fp[j][kq]);        // + (A v)^T
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      issue_A(fp[j], c + 2);
      // lane: token 16 ow + fr, columns 16 ni + g4 .. + 3
      if (16 * ow + fr < len) {
        T* orow = row_ptr<T>(a.o, sq.b, tok + 16 * ow + fr, h) + v0 + g4;
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          typename ET<T>::vec4 y;
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] = ET<T>::from_f(o[ni][e] * a.scale);
          *(typename ET<T>::vec4*)(orow + 16 * ni) = y;
        }
      }
      if (c + 1 < sq.nchunks) preread(c + 1);
     }
    }
    return;
  }

  // --------------------------------- consumers -------------------------------------------
  const int wv = wave;
  const int krow0 = wv * (K / 4);
  f32x4 S[MB][NB];
  acc_zero(S);
  if (a.h0) {
    const float* h0 = a.h0 + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i) S[mi][ni][i] = h0[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)];
  }
  auto copy_state = [&](int buf) {          // S -> LDS as S^T
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(S[mi][ni], s_hT[buf], LDK, krow0 + 16 * mi, 16 * ni);
  };
  copy_state(0);
  lds_barrier();                                                                         // chunks 0, 1 staged
  typename ET<T>::frag af[CS][MB], bf[CS][NB];
  f32x4 dec[MB];
  auto preread = [&](int c) {
    const int cb = c & 1;
#pragma unroll
    for (int kq = 0; kq < CS; ++kq) {
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) af[kq][mi] = ET<T>::load_frag_t(s_k[cb], LDK, 32 * kq, krow0 + 16 * mi);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) bf[kq][ni] = ET<T>::load_frag_t(s_u[cb], LDU, 32 * kq, 16 * ni);
    }
#pragma unroll
    for (int mi = 0; mi < MB; ++mi) dec[mi] = *(const f32x4*)&s_dec[cb][krow0 + 16 * mi + 4 * (l >> 4)];
  };
  preread(0);
  for (int c = 0; c < sq.nchunks; ++c) {
    lds_barrier();
    // S = diag(e^{b_C}) S + (k e^{b_C - b})^T v
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) S[mi][ni] *= dec[mi];
#pragma unroll
    for (int kq = 0; kq < CS; ++kq)
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(S[mi][ni], af[kq][mi], bf[kq][ni]);
    __builtin_amdgcn_sched_barrier(0);
    if (c + 1 < sq.nchunks) {
      copy_state((c + 1) & 1);
      preread(c + 1);
    }
  }
  if (a.ht) {
    float* ht = a.ht + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i) ht[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)] = S[mi][ni][i];
  }
}

// ------------------------------------------------------------------------- //
// output, grid = (NT, H, V / BV)
// ------------------------------------------------------------------------- //
template <typename T, typename GT, int K, int V, int BV>
__global__ __launch_bounds__(NTHR) void k_gla_out_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDV = BV + LPAD;
  constexpr int NB = BV / 16;
  // Two LDS regions, each used twice (small LDS -> more work-groups per CU, which is what hides the load
  // latency of these one-shot work-groups):  R0: S, then v;  R1: q e^{b} (as stored by k_gla_intra_fwd),
  // then A.  Every load is requested up front and waits in registers for its region.  S and v are staged as
  // they lie in memory (16-byte writes) and enter the products, which contract over their rows, through
  // transposing reads (staged transposed, element by element, these two kernels spent 70 % of their cycles
  // in LDS bank conflicts).
  constexpr int R0_ELEMS = cmax(K * LDV, CH * LDV);
  constexpr int R1_ELEMS = cmax(CH * LDK, CH * LDC);
  __shared__ __attribute__((aligned(16))) T r0[R0_ELEMS];
  __shared__ __attribute__((aligned(16))) T r1[R1_ELEMS];
  T* s_h = r0; T* s_v = r0;
  T* s_q = r1; T* s_P = r1;
  const int cid = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * BV;
  if (cid >= num_chunks(a)) return;          // launch sized by an upper bound of the chunk count
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;
  typedef TileIO<T, K, BV> IOH;
  typedef TileIO<T, CH, CH> IOA;
  typename IOK::Regs rq;
  typename IOV::Regs rv;
  typename IOH::Regs rh;
  typename IOA::Regs ra;
  IOK::load_nomask(rq, (const T*)a.qe + ((int64_t)cid * a.H + h) * CH * K, K, CH);
  IOH::load_nomask(rh, (const T*)a.hs + ((int64_t)cid * a.H + h) * K * V + v0, V, K);
  IOA::load_nomask(ra, (const T*)a.amat + ((int64_t)cid * a.H + h) * CH * CH, CH, CH);
  IOV::load_nomask(rv, row_ptr<T>(a.v, ci.b, ci.tok, h) + v0, a.v.st, ci.len);
  IOK::store_lds(rq, s_q, LDK);
  IOH::store_lds(rh, s_h, LDV);
  lds_barrier();
  // the products are formed transposed (o^T = S^T (q e^b)^T, then += v^T A^T): a lane then holds four consecutive V
  // columns of one token and stores them as one 8-byte piece
  f32x4 o[NB][1];
  acc_zero(o);
  gemm<T, NB, 1, true, false>(o, s_h, LDV, 0, s_q, LDK, 16 * wv, 0, K);
  lds_barrier();                                                                       // q e^{b}, S are dead
  IOA::store_lds(ra, s_P, LDC);
  IOV::mask(rv, ci.len);
  IOV::store_lds(rv, s_v, LDV);
  lds_barrier();
  gemm<T, NB, 1, true, false>(o, s_v, LDV, 0, s_P, LDC, 16 * wv, 0, CH);
  const int r = 16 * wv + (l & 15);
  if (r < ci.len) {
    T* od = row_ptr<T>(a.o, ci.b, ci.tok + r, h) + v0 + 4 * (l >> 4);
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) {
      typename ET<T>::vec4 x;
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = ET<T>::from_f(o[ni][0][i] * a.scale);
      *(typename ET<T>::vec4*)(od + 16 * ni) = x;
    }
  }
}

// ------------------------------------------------------------------------- //
// reverse state pass, 1-D grid (XCD-aware, see k_gla_state_fwd)
// ------------------------------------------------------------------------- //
template <typename T, typename GT, int K, int V, int BV>
__global__ __launch_bounds__(NTHR) void k_gla_state_bwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16;
  __shared__ __attribute__((aligned(16))) T s_q[CH * LDK];     // q e^{b}             [64][K]
  __shared__ __attribute__((aligned(16))) T s_do[CH * LDU];    // do                  [64][BV]
  __shared__ __attribute__((aligned(16))) T s_h[K * LDU];      // dS' on its way out  [K][BV]
  // 1-D grid of ceil(N H / 8) * 8 * (V / BV) work-groups; the V-slices of one (sequence, head) get ids that are
  // congruent mod 8, i.e. run on the same XCD and share its gated k (q) rows through that XCD's L2
  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = (jj % NVS) * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
  const SeqInfo sq = seq_info(a, n);
  const int wv = wave_id();
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
        for (int i = 0; i < 4; ++i) dS[mi][ni][i] = p[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)];
  }
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;
  typedef TileIO<T, K, BV> IOH;
  const float scale = a.scale;
  // the operands of the next PF chunks are kept in flight in PF register sets (see k_gla_state_fwd)
  constexpr int PF = 3;
  struct Pre { typename IOK::Regs rq; typename IOV::Regs rd; float dec[MB][4]; };
  Pre pre[PF];
  auto issue = [&](Pre& P, int c) {
    c = max(c, 0);
    const int64_t item = (int64_t)(sq.chunk0 + c) * a.H + h;
    IOK::load_nomask(P.rq, (const T*)a.qe + item * CH * K, K, CH);
    IOV::load_nomask(P.rd, row_ptr<T>(a.d_o, sq.b, sq.tok0 + c * CH, h) + v0, a.d_o.st, min(CH, sq.len - c * CH));
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int i = 0; i < 4; ++i) P.dec[mi][i] = a.gcum[item * K + krow0 + acc_row(mi, i)];
  };
  if (sq.nchunks > 0) {
#pragma unroll
    for (int j = 0; j < PF; ++j) issue(pre[j], sq.nchunks - 1 - j);
  }
  for (int c0 = sq.nchunks - 1; c0 >= 0; c0 -= PF) {
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int c = c0 - j;
      if (c < 0) break;
      const int len = min(CH, sq.len - c * CH);
      Pre& P = pre[j];
      IOK::store_lds(P.rq, s_q, LDK);
      IOV::mask(P.rd, len);
      IOV::store_lds(P.rd, s_do, LDU);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          acc_to_lds<T>(dS[mi][ni], s_h, LDU, krow0 + 16 * mi, 16 * ni);
#pragma unroll
          for (int i = 0; i < 4; ++i) dS[mi][ni][i] *= P.dec[mi][i];
        }
      issue(P, c - PF);
      lds_barrier();      // LDS-only: the loads stay in flight
      IOH::lds_to_global(s_h, LDU, (T*)a.dhs + ((int64_t)(sq.chunk0 + c) * a.H + h) * K * V + v0, V, K);
      // dS += scale (q e^{b})^T do
      f32x4 t[MB][NB];
      acc_zero(t);
#pragma unroll
      for (int kk = 0; kk < CH; kk += 32) {
        typename ET<T>::frag af[MB], bf[NB];
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) af[mi] = ET<T>::load_frag_t(s_q, LDK, kk, krow0 + 16 * mi);
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) bf[ni] = ET<T>::load_frag_t(s_do, LDU, kk, 16 * ni);
#pragma unroll
        for (int mi = 0; mi < MB; ++mi)
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(t[mi][ni], af[mi], bf[ni]);
      }
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) dS[mi][ni] += scale * t[mi][ni];
      lds_barrier();
    }
  }
  if (a.dh0) {
    float* p = a.dh0 + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i) p[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)] = dS[mi][ni][i];
  }
}

// ------------------------------------------------------------------------- //
// dv = scale A^T do + (k . e^{b_C - b}) dS',  grid = (NT, H, V / BV)
// ------------------------------------------------------------------------- //
template <typename T, typename GT, int K, int V, int BV>
__global__ __launch_bounds__(NTHR) void k_gla_bwd_dv(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDV = BV + LPAD;
  constexpr int NB = BV / 16;
  // two LDS regions, each used twice (see k_gla_out_fwd):  R0: dS', then do;  R1: k e^{b_C - b} (as stored
  // by k_gla_intra_fwd), then A; all staged as they lie in memory, transposing reads where a product contracts
  // over the rows of a tile
  constexpr int R0_ELEMS = cmax(K * LDV, CH * LDV);
  constexpr int R1_ELEMS = cmax(CH * LDK, CH * LDC);
  __shared__ __attribute__((aligned(16))) T r0[R0_ELEMS];
  __shared__ __attribute__((aligned(16))) T r1[R1_ELEMS];
  T* s_dh = r0; T* s_do = r0;
  T* s_kd = r1; T* s_P = r1;
  const int cid = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * BV;
  if (cid >= num_chunks(a)) return;          // launch sized by an upper bound of the chunk count
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;
  typedef TileIO<T, K, BV> IOH;
  typedef TileIO<T, CH, CH> IOA;
  typename IOK::Regs rk;
  typename IOV::Regs rd;
  typename IOH::Regs rh;
  typename IOA::Regs ra;
  IOK::load_nomask(rk, (const T*)a.ke + ((int64_t)cid * a.H + h) * CH * K, K, CH);
  IOH::load_nomask(rh, (const T*)a.dhs + ((int64_t)cid * a.H + h) * K * V + v0, V, K);
  IOA::load_nomask(ra, (const T*)a.amat + ((int64_t)cid * a.H + h) * CH * CH, CH, CH);
  IOV::load_nomask(rd, row_ptr<T>(a.d_o, ci.b, ci.tok, h) + v0, a.d_o.st, ci.len);
  IOK::store_lds(rk, s_kd, LDK);
  IOH::store_lds(rh, s_dh, LDV);
  lds_barrier();
  // products formed transposed (see k_gla_out_fwd): 8-byte stores of four consecutive V columns per token
  f32x4 dv[NB][1], dv2[NB][1];
  acc_zero(dv); acc_zero(dv2);
  gemm<T, NB, 1, true, false>(dv2, s_dh, LDV, 0, s_kd, LDK, 16 * wv, 0, K);
  lds_barrier();                                                                       // k e^{..}, dS' are dead
  IOA::store_lds(ra, s_P, LDC);
  IOV::mask(rd, ci.len);
  IOV::store_lds(rd, s_do, LDV);
  lds_barrier();
  gemm<T, NB, 1, true, true>(dv, s_do, LDV, 0, s_P, LDC, 16 * wv, 0, CH);
  const int r = 16 * wv + (l & 15);
  if (r < ci.len) {
    T* dd = row_ptr<T>(a.dv, ci.b, ci.tok + r, h) + v0 + 4 * (l >> 4);
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) {
      typename ET<T>::vec4 x;
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = ET<T>::from_f(__builtin_fmaf(a.scale, dv[ni][0][i], dv2[ni][0][i]));
      *(typename ET<T>::vec4*)(dd + 16 * ni) = x;
    }
  }
}

// ------------------------------------------------------------------------- //
// dq, dk, dg (2-byte elements: dv as well), grid = (NT, H)
// ------------------------------------------------------------------------- //
template <typename T, typename GT, int K, int V, int BVH>
__global__ __launch_bounds__(NTHR) __attribute__((amdgpu_waves_per_eu((K <= 64 && sizeof(T) == 2) ? 2 : 1))) void k_gla_bwd_dqkg(const lmoe_args a) {
  // (LDB: rows of the fp32 gate tile start on 16-byte boundaries, and the rows 4 apart that the lanes of an accumulator
  // column read fall into different banks)
  constexpr int LDV = BVH + LPAD, LDB = K + 4, LDP = CH + 1;
  constexpr int NBK = K / 16;
  // phase A (element type T): do, v, S, dS' slices.  phase B (fp32): dA, q, k, b tiles
  constexpr int A_DO = 0, A_V = A_DO + CH * LDV, A_H = A_V + CH * LDV, A_DH = A_H + K * LDV, A_END0 = A_DH + K * LDV;
  // 2-byte elements: dv is formed here as well, from the do and dS' slices that phase A stages anyway and two more
  // tiles, k e^{b_C - b} and A as k_gla_intra_fwd stored them (the chunk-parallel dv kernel, which fetched do and
  // dS' a second time, is not run)
  constexpr bool DV = sizeof(T) == 2;
  constexpr int A_KE = A_END0, A_AM = A_KE + (DV ? CH * (K + LPAD) : 0), A_END = A_AM + (DV ? CH * (CH + LPAD) : 0);
  constexpr int B_DP = 0, B_Q = B_DP + CH * LDP, B_K = B_Q + CH * LDB, B_B = B_K + CH * LDB, B_END = B_B + CH * LDB;
  // Sub-chunk form of the intra-chunk sums (see k_gla_intra_fwd): between 16-token sub-chunks the
  // decay factors through the cumulative gate b* at the sub-chunk boundary,
  //   dq_i += e^{b_i - b*} [ dA (k e^{b* - b}) ]_i      (j in earlier sub-chunks)
  //   dk_j += e^{b* - b_j} [ dA^T (q e^{b - b*}) ]_j    (i in later sub-chunks)
  // two MFMA products per boundary over element-type tiles dA, k~, q~ behind the fp32 tiles; the
  // pairwise loops below then cover the diagonal blocks only.  Used where the extra tiles fit LDS.
  constexpr int LDC = CH + LPAD, LDK = K + LPAD;
  // layout of that form: b (fp32) | q, k as loaded | dA | k~ | q~  (element type T)
  constexpr int S_B = 0, S_TBASE = CH * LDB * 4;
  constexpr int T_Q = 0, T_K = T_Q + CH * LDK, T_DA = T_K + CH * LDK, T_KT = T_DA + CH * LDC, T_END = T_KT + 192 * LDK;
  constexpr int S_BYTES = S_TBASE + T_END * (int)sizeof(T);
  constexpr bool SUB = S_BYTES + 4096 <= 160 * 1024;
  static_assert(!SUB || 192 * LDK * (int)sizeof(T) >= CH * LDB * 4, "the db tile fits over the stacked k~, q~ tile");
  constexpr int B_BYTES = SUB ? S_BYTES : B_END * 4;
  constexpr int NBYTES = (A_END * (int)sizeof(T) > B_BYTES) ? A_END * (int)sizeof(T) : B_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem_raw[NBYTES];
  __shared__ float s_hdh[K], s_kk[4 * K];
  T* smT = (T*)smem_raw;
  float* smF = (float*)smem_raw;

  const int cid = blockIdx.x, h = blockIdx.y;
  if (cid >= num_chunks(a)) return;          // launch sized by an upper bound of the chunk count
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, BVH> IOV;
  typedef TileIO<T, K, BVH> IOH;
  typedef TileIO<T, CH, K> IOK;

  f32x4 dP[1][4], dqi[1][NBK], dkd[1][NBK];
  acc_zero(dP); acc_zero(dqi); acc_zero(dkd);
  float hdh[IOH::PASSES];
#pragma unroll
  for (int p = 0; p < IOH::PASSES; ++p) hdh[p] = 0.f;
  // Loads run one stage ahead of their use: slice s + 1 is requested before slice s is staged, and q, k, g
  // before the last slice is.
  constexpr int NSL = V / BVH;
  struct Slice { typename IOV::Regs rd, rv; typename IOH::Regs rh, rdh; };
  Slice sl[2];
  typename IOK::Regs rq, rk;
  typename GlaGate<GT, K>::Regs rg;
  auto issue_slice = [&](Slice& x, int vv) {
    IOV::load_nomask(x.rd, row_ptr<T>(a.d_o, ci.b, ci.tok, h) + vv, a.d_o.st, ci.len);
    IOV::load_nomask(x.rv, row_ptr<T>(a.v, ci.b, ci.tok, h) + vv, a.v.st, ci.len);
    IOH::load_nomask(x.rh, (const T*)a.hs + ((int64_t)cid * a.H + h) * K * V + vv, V, K);
    IOH::load_nomask(x.rdh, (const T*)a.dhs + ((int64_t)cid * a.H + h) * K * V + vv, V, K);
  };
  issue_slice(sl[0], 0);
  typedef TileIO<T, CH, CH> IOA;
  typename IOK::Regs rke;
  typename IOA::Regs ram;
  if constexpr (DV) {
    IOK::load_nomask(rke, (const T*)a.ke + ((int64_t)cid * a.H + h) * CH * K, K, CH);
    IOA::load_nomask(ram, (const T*)a.amat + ((int64_t)cid * a.H + h) * CH * CH, CH, CH);
  }
  auto issue_qkg = [&]() {
    IOK::load_nomask(rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
    IOK::load_nomask(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
    GlaGate<GT, K>::issue(rg, a, ci.b, ci.tok, ci.len, h);
  };
  // with two slices everything is requested at the start (a load of this kernel takes 5 to 9 thousand cycles to
  // arrive, the work on a slice 1500); with more, q, k, g go out with the last slice
  constexpr bool QKG_EARLY = NSL <= 2;
#pragma unroll
  for (int si = 0; si < NSL; ++si) {
    Slice& x = sl[si & 1];
    if (si + 1 < NSL) issue_slice(sl[(si + 1) & 1], (si + 1) * BVH);
    if (QKG_EARLY ? si == 0 : si + 1 == NSL) issue_qkg();
    IOV::mask(x.rd, ci.len);
    IOV::mask(x.rv, ci.len);
#pragma unroll
    for (int p = 0; p < IOH::PASSES; ++p)
#pragma unroll
      for (int i = 0; i < IOH::VEC; ++i) hdh[p] += ET<T>::to_f(x.rh.v[p][i]) * ET<T>::to_f(x.rdh.v[p][i]);
    IOV::store_lds(x.rd, smT + A_DO, LDV);
    IOV::store_lds(x.rv, smT + A_V, LDV);
    IOH::store_lds(x.rh, smT + A_H, LDV);
    IOH::store_lds(x.rdh, smT + A_DH, LDV);
    if constexpr (DV) {
      if (si == 0) {
        IOK::store_lds(rke, smT + A_KE, LDK);
        IOA::store_lds(ram, smT + A_AM, LDC);
      }
    }
    lds_barrier();      // LDS-only barriers: the loads requested above stay in flight
    gemm_nt<T, 1, 4, true>(dP, smT + A_DO, LDV, 16 * wv, smT + A_V, LDV, 0, 0, BVH);
    gemm_nt<T, 1, NBK, true>(dqi, smT + A_DO, LDV, 16 * wv, smT + A_H, LDV, 0, 0, BVH);
    gemm_nt<T, 1, NBK, true>(dkd, smT + A_V, LDV, 16 * wv, smT + A_DH, LDV, 0, 0, BVH);
    if constexpr (DV) {
      // dv^T of the slice = scale do^T A + dS'^T (k e^{b_C - b})^T, the products and the rounding of k_gla_bwd_dv
      // (same operands, same order): a lane holds four consecutive V columns of one token, 8-byte stores
      constexpr int NBV = BVH / 16;
      f32x4 dv[NBV][1], dv2[NBV][1];
      acc_zero(dv); acc_zero(dv2);
      gemm<T, NBV, 1, true, false>(dv2, smT + A_DH, LDV, 0, smT + A_KE, LDK, 16 * wv, 0, K);
      gemm<T, NBV, 1, true, true>(dv, smT + A_DO, LDV, 0, smT + A_AM, LDC, 16 * wv, 0, CH);
      const int r = 16 * wv + (l & 15);
      if (r < ci.len) {
        T* dd = row_ptr<T>(a.dv, ci.b, ci.tok + r, h) + si * BVH + 4 * (l >> 4);
#pragma unroll
        for (int ni = 0; ni < NBV; ++ni) {
          typename ET<T>::vec4 y;
#pragma unroll
          for (int i = 0; i < 4; ++i) y[i] = ET<T>::from_f(__builtin_fmaf(a.scale, dv[ni][0][i], dv2[ni][0][i]));
          *(typename ET<T>::vec4*)(dd + 16 * ni) = y;
        }
      }
    }
    lds_barrier();
  }
  // per state row k: sum_v S_kv dS'_kv  (the IOH::VPR adjacent threads of a pass share a row)
#pragma unroll
  for (int p = 0; p < IOH::PASSES; ++p) {
    const float x = group_sum<IOH::VPR>(hdh[p]);
    int row, col; IOH::coords(p, row, col);
    if (col == 0 && row < K) s_hdh[row] = x;
  }
  // phase B tiles
  T* tQ = (T*)(smem_raw + S_TBASE) + T_Q;
  T* tK = (T*)(smem_raw + S_TBASE) + T_K;
  T* tDA = (T*)(smem_raw + S_TBASE) + T_DA;
  T* tKT = (T*)(smem_raw + S_TBASE) + T_KT;
  float* sBw = SUB ? smF + S_B / 4 : smF + B_B;
  {
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r >= cc) ? a.scale * dP[0][nj][i] : 0.f;
        if constexpr (!SUB) smF[B_DP + r * LDP + cc] = p[i];
      }
      if constexpr (SUB) acc_to_lds<T>(p, tDA, LDC, 16 * wv, 16 * nj);
    }
    IOK::mask(rq, ci.len);
    IOK::mask(rk, ci.len);
    if constexpr (SUB) {
      IOK::store_lds(rq, tQ, LDK);
      IOK::store_lds(rk, tK, LDK);
    } else {
      IOK::store_lds_f32(rq, smF + B_Q, LDB);
      IOK::store_lds_f32(rk, smF + B_K, LDB);
    }
  }
  GlaGate<GT, K>::template finish<LDB>(rg, ci.len, sBw);   // barriers inside
  const float* sB = sBw;
  // dA, q, k of the pairwise loops and the epilogue, from whichever tiles this layout keeps
  auto Pm = [&](int r, int j) { if constexpr (SUB) return ET<T>::to_f(tDA[r * LDC + j]); else return smF[B_DP + r * LDP + j]; };
  auto Qm = [&](int r, int c) { if constexpr (SUB) return ET<T>::to_f(tQ[r * LDK + c]); else return smF[B_Q + r * LDB + c]; };
  auto Km = [&](int r, int c) { if constexpr (SUB) return ET<T>::to_f(tK[r * LDK + c]); else return smF[B_K + r * LDB + c]; };
  // Intra-chunk sums through reference gates (see k_gla_intra_fwd).  Wave w owns sub-chunk w:
  //   dq rows:  e^{b_i - ref_w}  [ dA(rows of w, j < 16 w + 16) (k_j e^{ref_w - b_j}) ],   ref_w  = b_{16 w - 1} (0 for w = 0)
  //   dk rows:  e^{ref'_w - b_j} [ dA^T(rows of w, i >= 16 w)   (q_i e^{b_i - ref'_w}) ],  ref'_w = b_{16 w + 15}
  // Tokens outside the wave's own sub-chunk have exponents <= 0; inside it the exponent is a decay over at
  // most 16 tokens, taken only if it stays below GLA_SAFE_EXP for every channel of the sub-chunk: otherwise
  // those rows of the scaled operand are zero and the diagonal block takes the per-pair loops below.
  // Two rounds over one stacked LDS tile: sub-chunks {0, 3}, then {1, 2} (contraction ranges in multiples of 32
  // tokens: k~ of sub-chunk 0 / 1 / 2 / 3 holds 32 / 32 / 64 / 64 rows, q~ 64 / 64 / 32 / 32).
  int unsafe = 0;
  f32x4 dqo[1][NBK], dko[1][NBK];
  acc_zero(dqo); acc_zero(dko);
  if constexpr (SUB) {
    __shared__ int s_unsafe;
    if (threadIdx.x == 0) s_unsafe = 0;
    if (threadIdx.x < K) {
#pragma unroll
      for (int I = 0; I < 4; ++I) {
        const float ref = I == 0 ? 0.f : sB[(16 * I - 1) * LDB + threadIdx.x];
        if (!(ref - sB[(16 * I + 15) * LDB + threadIdx.x] <= GLA_SAFE_EXP)) unsafe |= 1 << I;
      }
    }
    __syncthreads();
    if (unsafe) atomicOr(&s_unsafe, unsafe);
    __syncthreads();
    unsafe = s_unsafe;
#pragma unroll
    for (int rd = 0; rd < 2; ++rd) {
      // segment s of the stacked tile: s = 0, 1: k~ of sub-chunks wa, wb; s = 2, 3: q~ of sub-chunks wa, wb
      const int wa = rd == 0 ? 0 : 1, wb = rd == 0 ? 3 : 2;
      constexpr int SEGROW[4] = {0, 32, 96, 160};                       // k~(wa) 32 | k~(wb) 64 | q~(wa) 64 | q~(wb) 32
      constexpr int VEC = ET<T>::VEC;
      typedef typename ET<T>::vec vec;
      // A thread keeps its 16-byte column group c0 and takes one stacked row out of every RPI: the segment of a row
      // is then known at compile time, the gate row that a whole segment shares (its reference) is read once, and
      // every gate value arrives in 16-byte reads
      constexpr int PPR = K / VEC, RPI = NTHR / PPR, NIT = 192 / RPI;
      static_assert(32 % RPI == 0 && NTHR % PPR == 0, "segment boundaries fall between the passes");
      const int c0 = (threadIdx.x % PPR) * VEC, rin = threadIdx.x / PPR;
      auto gate_row = [&](int row, float (&b)[VEC]) { load_f32_group(sB + row * LDB + c0, b); };
      float ref[4][VEC];                                                // k~: b_{16 w - 1} (0 for w = 0); q~: b_{16 w + 15}
#pragma unroll
      for (int sg = 0; sg < 4; ++sg) {
        const int w = (sg & 1) ? wb : wa;
        if (sg < 2 && w == 0) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) ref[sg][e] = 0.f;
        } else {
          gate_row(sg < 2 ? 16 * w - 1 : 16 * w + 15, ref[sg]);
        }
      }
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int sr0 = it * RPI, sg = sr0 < 32 ? 0 : sr0 < 96 ? 1 : sr0 < 160 ? 2 : 3;   // known after unrolling
        const int sr = sr0 + rin;
        const int w = (sg & 1) ? wb : wa;
        const bool own_ok = !((unsafe >> w) & 1);
        // token of this row and whether the row is in use
        int tok;
        bool use;
        if (sg < 2) {
          tok = sr - SEGROW[sg];
          use = tok < 16 * w + 16 && (tok < 16 * w || own_ok);          // k_j e^{ref_w - b_j}
        } else {
          tok = (w < 2 ? 0 : 32) + sr - SEGROW[sg];
          use = tok >= 16 * w && (tok >= 16 * w + 16 || own_ok);        // q_i e^{b_i - ref'_w}
        }
        vec o = ET<T>::zero();
        if (use) {
          const vec x = *(const vec*)((sg < 2 ? tK : tQ) + tok * LDK + c0);
          float bt[VEC];
          gate_row(tok, bt);
#pragma unroll
          for (int e = 0; e < VEC; ++e)
            o[e] = ET<T>::from_f(ET<T>::to_f(x[e]) * texp<T>(sg < 2 ? ref[sg][e] - bt[e] : bt[e] - ref[sg][e]));
        }
        *(vec*)(tKT + sr * LDK + c0) = o;
      }
      __syncthreads();
      if (wv == wa || wv == wb) {
        const int sg = wv == wa ? 0 : 1;
        const int nk = wv < 2 ? 32 : 64;                                // tokens j < nk
        gemm<T, 1, NBK, false, true>(dqo, tDA, LDC, 16 * wv, tKT + SEGROW[sg] * LDK, LDK, 0, 0, nk);
        const int i0 = wv < 2 ? 0 : 32;                                 // tokens i >= i0
        gemm<T, 1, NBK, true, true>(dko, tDA, LDC, 16 * wv, tKT + (SEGROW[2 + sg] - i0) * LDK, LDK, 0, i0, CH);
      }
      __syncthreads();
    }
  }
  const int jlo = SUB ? 16 * wv : 0, ihi = SUB ? 16 * wv + 16 : CH;   // range of the pairwise loops
  T* dqd = row_ptr<T>(a.dq, ci.b, ci.tok, h);
  T* dkd_g = row_ptr<T>(a.dk, ci.b, ci.tok, h);
  float kkp[NBK];                      // per column: sum over this lane's rows of (dk_d . k_d)
  float dbv[NBK][4];
  static_assert(NBK % 4 == 0, "column tiles are taken four at a time");
#pragma unroll
  for (int nh = 0; nh < NBK; nh += 4) {
    // Diagonal block of this wave's sub-chunk, for four column tiles at a time.  One pass over the 16 tokens
    // j of the sub-chunk serves both sums: dA is lower triangular (zero above the diagonal), so
    //   sq[r] += dA(r, j) k_j e,   sk[r] += dA(j, r) q_j e,   e = e^{-|b_r - b_j|}
    // (b decreases along the chunk: the exponent wanted is b_r - b_j for j <= r and b_j - b_r for j >= r;
    // where it is not, the dA factor is zero).  k_j, q_j, b_j are read once per token and column and serve
    // the lane's four rows; the dA values are read once per token and serve the four column tiles.
    float sqv[4][4], skv[4][4], brv[4][4];
#pragma unroll
    for (int n4 = 0; n4 < 4; ++n4)
#pragma unroll
      for (int i = 0; i < 4; ++i) sqv[n4][i] = skv[n4][i] = 0.f;
    if (SUB && ((unsafe >> wv) & 1)) {
#pragma unroll
      for (int n4 = 0; n4 < 4; ++n4)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sqv[n4][i] = skv[n4][i] = 0.f;
          brv[n4][i] = sB[(16 * wv + 4 * (l >> 4) + i) * LDB + 16 * (nh + n4) + (l & 15)] * TEXP_PRESCALE<T>;
        }
      for (int jj = 0; jj < 16; ++jj) {
        const int j = 16 * wv + jj;
        float pq[4], pk[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * wv + 4 * (l >> 4) + i;
          pq[i] = Pm(r, j);
          pk[i] = Pm(j, r);
        }
#pragma unroll
        for (int n4 = 0; n4 < 4; ++n4) {
          const int cc = 16 * (nh + n4) + (l & 15);
          const float kj = Km(j, cc), qj = Qm(j, cc), bj = sB[j * LDB + cc] * TEXP_PRESCALE<T>;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float e = texp_scaled<T>(-fabsf(brv[n4][i] - bj));
            sqv[n4][i] += pq[i] * kj * e;
            skv[n4][i] += pk[i] * qj * e;
          }
        }
      }
    }
#pragma unroll
    for (int n4 = 0; n4 < 4; ++n4) {
      const int ni = nh + n4;
      const int cc = 16 * ni + (l & 15);
      const float bC = sB[63 * LDB + cc];
      // Two exponentials per element, e^{b_r - ref_w} and e^{ref'_w - b_r} (both exponents <= 0); the other two
      // factors of a row follow from them through one factor per column: e^{b_r} = e^{ref_w} e^{b_r - ref_w},
      // e^{b_C - b_r} = e^{b_C - ref'_w} e^{ref'_w - b_r}
      const float refq = wv == 0 ? 0.f : sB[(16 * wv - 1) * LDB + cc], refk = sB[(16 * wv + 15) * LDB + cc];
      const float eref = texp<T>(refq), eC = texp<T>(bC - refk);
      kkp[ni] = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i;
        const float br = sB[r * LDB + cc];
        const float e1 = texp<T>(br - refq), e2 = texp<T>(refk - br);
        float sq_ = 0.f, sk_ = 0.f;
        if constexpr (SUB) {
          sq_ = sqv[n4][i];
          sk_ = skv[n4][i];
          sq_ += dqo[0][ni][i] * e1;
          sk_ += dko[0][ni][i] * e2;
        } else {
          for (int j = jlo; j <= r; ++j) sq_ += Pm(r, j) * Km(j, cc) * texp<T>(br - sB[j * LDB + cc]);
          for (int ii = r; ii < ihi; ++ii) sk_ += Pm(ii, r) * Qm(ii, cc) * texp<T>(sB[ii * LDB + cc] - br);
        }
        const float qv = Qm(r, cc), kv = Km(r, cc);
        const float ed = eC * e2;
        const float dqv = a.scale * (eref * e1) * dqi[0][ni][i] + sq_;
        const float dkdv = dkd[0][ni][i] * ed;
        const float dkv = dkdv + sk_;
        kkp[ni] += kv * dkdv;
        dbv[ni][i] = qv * dqv - kv * dkv;
        if constexpr (SUB) {
          // on their way out through the q, k tiles: this element of them is read by this lane only from here on
          // (the per-pair loops above read other rows' elements of the columns of this group before this point)
          tQ[r * LDK + cc] = ET<T>::from_f(dqv);
          tK[r * LDK + cc] = ET<T>::from_f(dkv);
        } else if (r < ci.len) {
          dqd[(int64_t)r * a.dq.st + cc] = ET<T>::from_f(dqv);
          dkd_g[(int64_t)r * a.dk.st + cc] = ET<T>::from_f(dkv);
        }
      }
      // sum over the 4 row groups of the wave
      kkp[ni] += __shfl_xor(kkp[ni], 16, 64);
      kkp[ni] += __shfl_xor(kkp[ni], 32, 64);
      if (l < 16) s_kk[wv * K + cc] = kkp[ni];
    }
  }
  __syncthreads();   // all reads of the q tile are done: reuse it for db
  if constexpr (SUB) {
    IOK::lds_to_global(tQ, LDK, dqd, a.dq.st, ci.len);
    IOK::lds_to_global(tK, LDK, dkd_g, a.dk.st, ci.len);
  }
  float* sDB = SUB ? (float*)tKT : smF + B_Q;
#pragma unroll
  for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
      sDB[r * LDB + cc] = dbv[ni][i];
    }
  __syncthreads();
  // dg = reverse cumsum of db over the tokens (+ the last-row term): a thread takes one channel over a segment
  // of tokens, the segment totals go through LDS (rows past the end of a partial chunk have zero db)
  {
    constexpr int NSEG = NTHR / K, SEG = CH / NSEG;
    __shared__ float s_seg[NTHR];
    const int cc = threadIdx.x % K, sg = threadIdx.x / K;
    float v[SEG];
#pragma unroll
    for (int r = 0; r < SEG; ++r) v[r] = sDB[(sg * SEG + r) * LDB + cc];
#pragma unroll
    for (int r = SEG - 2; r >= 0; --r) v[r] += v[r + 1];
    s_seg[sg * K + cc] = v[0];
    __syncthreads();
    float off = s_kk[cc] + s_kk[K + cc] + s_kk[2 * K + cc] + s_kk[3 * K + cc] + texp<T>(sB[63 * LDB + cc]) * s_hdh[cc];
#pragma unroll
    for (int q = 1; q < NSEG; ++q) off += q > sg ? s_seg[q * K + cc] : 0.f;
    GT* dg = (GT*)a.dg.ptr + row_off(a.dg, ci.b, ci.tok, h);      // dg in the element type of g
#pragma unroll
    for (int r = 0; r < SEG; ++r) {
      const int row = sg * SEG + r;
      if (row < ci.len) dg[(int64_t)row * a.dg.st + cc] = ET<GT>::from_f(v[r] + off);
    }
  }
}

}  // namespace lmoe
