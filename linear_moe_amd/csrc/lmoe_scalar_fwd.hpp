// Forward kernels for scalar-gated chunks (chunk_simple_gla and chunk_gated_delta_rule):
//   k_state_fwd : sequential pass over the chunks of one (sequence, head, V-slice); keeps the
//                 state S[K x BV] in fp32 MFMA accumulators, writes the state at the start of
//                 every chunk (hs) and, for the delta rule, v_new = u - w S.
//   k_out_fwd   : chunk-parallel output  o = scale [ e^{b_i} q_i S + ((q k^T) . Gamma) v' ].
// Math: S' = e^{b_C} S + (k . e^{b_C - b})^T v',  Gamma_ij = e^{b_i - b_j} [i >= j].
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

// ------------------------------------------------------------------------- //
// state pass (forward): producer / consumer work-group of 512 threads
//   grid = ceil(N*H / 8) * 8 * (V / BV) work-groups (1-D).  Work-group -> (sequence, head,
//   V-slice): the V-slices of one (sequence, head) get ids that are congruent mod 8, i.e. run on
//   the same XCD and share k, w through its L2.
//   Waves 0-3 (consumers) carry the dependency chain of the state and nothing else:
//        S -> LDS (element type T) | B1 | v_new = u - w S -> LDS | B2 | S = e^{b_C} S + (k e_d)^T v_new
//   wave w owns state rows [w*K/4, (w+1)*K/4) x BV columns in fp32 MFMA accumulators.
//   Waves 4-7 (producers) keep the operands of the next PF chunks in flight in registers, form
//   the gate cumsum (lane j = token j), scale k by e^{b_C - b}, fill the other LDS buffer and
//   write hs (layout [V][K]) from the LDS copy of S.  Both teams meet at the two barriers of a
//   step; with two waves per SIMD the producers' memory and LDS latencies hide behind the chain.
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV, bool GDN>
__global__ __launch_bounds__(2 * NTHR) void k_state_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16;
  // bf16: two operand buffers; fp32 (the parity path) has LDS for one and pays a third barrier
  constexpr int NBUF = sizeof(T) == 2 ? 2 : 1;
  __shared__ __attribute__((aligned(16))) T s_kd[NBUF][CH * LDK];             // k e^{b_C-b}   [64][K]
  __shared__ __attribute__((aligned(16))) T s_w[NBUF][GDN ? CH * LDK : 8];    // w             [64][K]
  __shared__ __attribute__((aligned(16))) T s_u[NBUF][CH * LDU];              // u or v        [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[BV * LDK];                // S^T           [BV][K]
  __shared__ __attribute__((aligned(16))) T s_vT[GDN ? BV * LDC : 8];      // v_new^T       [BV][64]
  __shared__ __attribute__((aligned(16))) T s_stg[GDN ? 4 * 16 * LDU : 8]; // v_new store staging
  __shared__ float s_dec[NBUF];                                               // e^{b_C} per buffer

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = pair / a.H;
  const SeqInfo sq = seq_info(a, n);
  const int l = lane_id();
  const bool producer = threadIdx.x >= NTHR;
  if (sq.nchunks == 0) {
    // empty sequence: the final state is the initial state
    if (a.ht && !producer) {
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
  typedef TileIO<T, BV, K> IOHT;

  if (producer) {
    // ------------------------------- producers -------------------------------------------
    constexpr int PF = 3;
    struct Pre { typename IOK::Regs rk, rw; typename IOV::Regs ru; uint32_t graw; int len; };
    Pre pre[PF];
    const lmoe_tensor& us = GDN ? a.u : a.v;
    const bool gated = a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr;
    const void* gptr = gated ? a.g.ptr : a.k.ptr;
    // Always issued (chunk index clamped to the last chunk; the surplus loads at the end of a
    // sequence are never consumed): a prefetch that is skipped on some path would make the
    // compiler drain all outstanding loads at every consumer of a register set.
    auto issue = [&](Pre& P, int c) {
      c = min(c, sq.nchunks - 1);
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rk, row_ptr<T>(a.k, sq.b, tok, h), a.k.st, len);
      if constexpr (GDN) IOK::load_nomask(P.rw, row_ptr<T>(a.w, sq.b, tok, h), a.w.st, len);
      IOV::load_nomask(P.ru, row_ptr<T>(us, sq.b, tok, h) + v0, us.st, len);
      P.len = len;
      P.graw = load_scalar_raw(gptr, a.g_dtype, gated ? row_off(a.g, sq.b, tok + min(l, len - 1), h) : 0);
    };
    // registers -> LDS buffer `buf`
    auto stage = [&](Pre& P, int buf) {
      IOK::mask(P.rk, P.len);
      if constexpr (GDN) IOK::mask(P.rw, P.len);
      IOV::mask(P.ru, P.len);
      const float x = wave_incl_scan((gated && l < P.len) ? scalar_from_raw(P.graw, a.g_dtype) : 0.f);
      const float xl = __shfl(x, 63, 64);
      const float ed = expf(xl - x);                        // lane j: e^{b_C - b_j}
#pragma unroll
      for (int p = 0; p < IOK::PASSES; ++p) {
        int row, col; IOK::coords(p, row, col);
        const float sc = __shfl(ed, row, 64);
        typename IOK::vec o;
#pragma unroll
        for (int i = 0; i < IOK::VEC; ++i) o[i] = ET<T>::from_f(ET<T>::to_f(P.rk.v[p][i]) * sc);
        *(typename IOK::vec*)(&s_kd[buf][row * LDK + col]) = o;
      }
      if constexpr (GDN) IOK::store_lds(P.rw, s_w[buf], LDK);
      IOV::store_lds(P.ru, s_u[buf], LDU);
      if (threadIdx.x == NTHR) s_dec[buf] = expf(xl);
    };
#pragma unroll
    for (int j = 0; j < PF; ++j) issue(pre[j], j);
    stage(pre[0], 0);
    issue(pre[0], PF);
    for (int c0 = 0; c0 < sq.nchunks; c0 += PF) {
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int c = c0 + j;
        if (c >= sq.nchunks) break;
        lds_barrier();                                                                   // B1
        // hs[chunk][h][v0 .. v0+BV][K] <- S^T
        IOHT::lds_to_global(s_hT, LDK, (T*)a.hs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
        if constexpr (NBUF == 2) {
          if (c + 1 < sq.nchunks) stage(pre[(j + 1) % PF], (c + 1) & 1);
        }
        lds_barrier();                                                                   // B2
        if constexpr (NBUF == 1) {
          lds_barrier();                                                                 // B3: buffer read
          if (c + 1 < sq.nchunks) stage(pre[(j + 1) % PF], 0);
        }
        issue(pre[(j + 1) % PF], c + 1 + PF);
      }
    }
    return;
  }

  // --------------------------------- consumers -------------------------------------------
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
        for (int i = 0; i < 4; ++i)
          S[mi][ni][i] = h0[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)];
  }
  for (int c = 0; c < sq.nchunks; ++c) {
    const int cur = NBUF == 2 ? (c & 1) : 0;
    const int tok = sq.tok0 + c * CH;
    const int len = min(CH, sq.len - c * CH);
    // S (state at chunk start) -> LDS as S^T
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(S[mi][ni], s_hT, LDK, krow0 + 16 * mi, 16 * ni);
    lds_barrier();                                                                       // B1
    const float dec = s_dec[cur];
    if constexpr (GDN) {
      // v_new = u - w S  (rows 16*wv .. +15 of the chunk)
      f32x4 vn[1][NB];
      acc_zero(vn);
      gemm<T, 1, NB, false, false>(vn, s_w[cur], LDK, 16 * wv, s_hT, LDK, 0, 0, K);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
          // round once to the storage type so that the state update and the output kernel see
          // the same v_new
          vn[0][ni][i] = ET<T>::to_f(ET<T>::from_f(ET<T>::to_f(s_u[cur][r * LDU + cc]) - vn[0][ni][i]));
        }
        acc_to_lds_t<T>(vn[0][ni], s_vT, LDC, 16 * wv, 16 * ni);
      }
      lds_barrier();                                                                     // B2
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) S[mi][ni] *= dec;
      gemm<T, MB, NB, true, false>(S, s_kd[cur], LDK, krow0, s_vT, LDC, 0, 0, CH);
      store_strip<T, NB>(vn, s_stg + wv * 16 * LDU, row_ptr<T>(a.vnew, sq.b, tok + 16 * wv, h) + v0, a.vnew.st,
                         len - 16 * wv, 1.0f);
    } else {
      lds_barrier();                                                                     // B2
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) S[mi][ni] *= dec;
      gemm<T, MB, NB, true, true>(S, s_kd[cur], LDK, krow0, s_u[cur], LDU, 0, 0, CH);
    }
    if constexpr (NBUF == 1) lds_barrier();                                              // B3
  }
  if (a.ht) {
    float* ht = a.ht + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          ht[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)] = S[mi][ni][i];
  }
}

// ------------------------------------------------------------------------- //
// output (forward), chunk-parallel, persistent
//   grid = min(NT*H, 2 per CU), block = 256; one work item = one (chunk, head), full V;
//   wave w owns chunk rows 16w .. 16w+15.
//   The tiles of the next item are fetched into registers while the current one is computed
//   (barriers order LDS traffic only, so the loads stay in flight).
//   LDS: q, k, S^T stored as loaded (hs holds S^T, [V][K]); P^T overlays k once q k^T is done, v' overlays S once q S is
//   done; products that contract over tile rows use transposed fragments.
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, bool GDN>
__global__ __launch_bounds__(NTHR, (sizeof(T) == 2 ? 2 : 1)) void k_out_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDV = V + LPAD;
  constexpr int NB = V / 16;
  constexpr int H_EL = V * LDK > CH * LDV ? V * LDK : CH * LDV;
  constexpr int Q_EL = CH * LDK > 4 * 16 * LDV ? CH * LDK : 4 * 16 * LDV;   // also the store staging area
  __shared__ __attribute__((aligned(16))) T s_q[Q_EL];
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];      // later: P^T [64][LDC]
  __shared__ __attribute__((aligned(16))) T s_h[H_EL];          // later: v' [64][LDV]
  __shared__ float s_b[64], s_eb[64];
  static_assert(CH * LDC <= CH * LDK, "P^T must fit into the k tile");
  T* s_PT = s_k;
  T* s_v = s_h;

  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, V> IOV;
  typedef TileIO<T, V, K> IOH;        // hs holds S^T: [V][K]
  const lmoe_tensor& vs = GDN ? a.vnew : a.v;
  const int nitems = a.NT * a.H;
  typename IOK::Regs rq, rk;
  typename IOV::Regs rv;
  typename IOH::Regs rh;
  uint32_t graw = 0;
  auto issue = [&](int it) {
    const int cid = it / a.H, h = it % a.H;
    const ChunkInfo ci = chunk_info(a, cid);
    IOK::load_nomask(rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
    IOK::load_nomask(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
    IOH::load_nomask(rh, (const T*)a.hs + ((int64_t)cid * a.H + h) * K * V, K, V);
    graw = gate_prefetch(a, ci.b, ci.tok, ci.len, h);
  };
  auto issue_v = [&](int it) {
    const int cid = it / a.H, h = it % a.H;
    const ChunkInfo ci = chunk_info(a, cid);
    IOV::load_nomask(rv, row_ptr<T>(vs, ci.b, ci.tok, h), vs.st, ci.len);
  };
  // prefetches are always issued (item index clamped): see k_state_fwd
  int it = blockIdx.x;
  if (it < nitems) { issue(it); issue_v(it); }
  for (; it < nitems; it += gridDim.x) {
    const int cid = it / a.H, h = it % a.H;
    const ChunkInfo ci = chunk_info(a, cid);
    const int nxt = min(it + (int)gridDim.x, nitems - 1);
    gate_finish(a, graw, ci.len, s_b, s_eb, nullptr);
    IOK::mask(rq, ci.len);
    IOK::mask(rk, ci.len);
    IOK::store_lds(rq, s_q, LDK);
    IOK::store_lds(rk, s_k, LDK);
    IOH::store_lds(rh, s_h, LDK);
    lds_barrier();
    issue(nxt);
    f32x4 s[1][4];
    acc_zero(s);
    gemm<T, 1, 4, false, false>(s, s_q, LDK, 16 * wv, s_k, LDK, 0, 0, K);
    f32x4 o[1][NB];
    acc_zero(o);
    gemm<T, 1, NB, false, false>(o, s_q, LDK, 16 * wv, s_h, LDK, 0, 0, K);
    lds_barrier();            // every wave is done reading k and S: P^T and v' may overlay them
    IOV::mask(rv, ci.len);
    IOV::store_lds(rv, s_v, LDV);
    issue_v(nxt);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r >= cc) ? s[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds_t<T>(p, s_PT, LDC, 16 * wv, 16 * nj);     // s_PT[j][i]
    }
#pragma unroll
    for (int ni = 0; ni < NB; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[0][ni][i] *= s_eb[16 * wv + 4 * (l >> 4) + i];
    lds_barrier();
    // o += P v' : A = P^T stored [j][i] (contraction j along rows), B = v' stored [j][v]
    gemm<T, 1, NB, true, true>(o, s_PT, LDC, 16 * wv, s_v, LDV, 0, 0, CH);
    // stage through a wave-private slice of the q tile: q was last read before the second
    // barrier of this iteration (as the A operand of the first two products)
    store_strip<T, NB>(o, s_q + wv * 16 * LDV, row_ptr<T>(a.o, ci.b, ci.tok + 16 * wv, h), a.o.st,
                       ci.len - 16 * wv, a.scale);
    lds_barrier();
  }
}

}  // namespace lmoe
