// Gated delta rule: the two sequential passes over the chunks of one (sequence, head, V-slice).
//
//   forward :  v_new = u - w S,   o = scale [ e^{b_i} q_i S + P v_new ],   S' = e^{b_C} S + k^T (e_d v_new)
//   backward:  dv_new = scale P^T do + e_d (k dS'),
//              dS = e^{b_C} dS' + q^T (scale e_b do) - w^T dv_new
//   with P = (q k^T) . Gamma (written by k_gdn_wy_fwd as P and P^T), e_b = e^{b}, e_d = e^{b_C - b}.
//
// Both kernels keep the per-chunk work of the dependency chain as small as it can be made:
//   * work-group = 2 teams of 4 waves.  Team 0 (consumers) owns the state slice [K x BV] in fp32
//     MFMA accumulators (wave w: rows [w K/4, (w+1) K/4)) and, for the products whose rows are
//     tokens, rows 16 w .. 16 w + 15 of the chunk.  Team 1 (loaders) stages the tiles that are
//     contracted along their rows (they need the transposing LDS read) and the gate vectors two
//     chunks ahead, and writes the state checkpoints (hs / dhs, layout [V][K]).
//   * operands that are contracted along their columns and used by one wave only (w, q, P rows in
//     the forward; k, P^T rows in the backward) never touch LDS: every consumer wave loads its own
//     16-row strip as MFMA A-fragments straight from global memory, a few chunks ahead
//     (RowFrags), so the LDS pipe carries only what several waves share.
//   * grid = ceil(N*H / 8) * 8 * (V / BV) work-groups (1-D): the V-slices of one (sequence, head)
//     get ids congruent mod 8, i.e. run on the same XCD and share k, w, q, P through its L2.
#pragma once
#include <type_traits>
#include "lmoe_seq.hpp"

namespace lmoe {

// V-slice / prefetch shape of the sequential passes per element type
template <typename T> struct GdnStateCfg {
  static constexpr int BV = sizeof(T) == 2 ? 32 : 16;    // V columns per work-group
  static constexpr int PF = sizeof(T) == 2 ? 3 : 1;      // consumer-side prefetch depth (chunks)
  static constexpr int LPF = 3;                          // loader-side prefetch depth (chunks)
};

// ------------------------------------------------------------------------- //
// forward
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV>
__global__ __launch_bounds__(2 * NTHR) void k_gdn_state_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16, KS = K / 32;
  constexpr int PF = GdnStateCfg<T>::PF, LPF = GdnStateCfg<T>::LPF;
  static_assert(LPF == 3 && PF <= 3, "the chunk loops are written out for rings of three");
  __shared__ __attribute__((aligned(16))) T s_k[2][CH * LDK];       // k             [64][K]
  __shared__ __attribute__((aligned(16))) T s_u[2][CH * LDU];       // u             [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[BV * LDK];         // S^T           [BV][K]
  __shared__ __attribute__((aligned(16))) T s_vT[BV * LDC];         // v_new^T       [BV][64]
  __shared__ __attribute__((aligned(16))) T s_stg[4 * 16 * LDU];    // v_new store strips
  __shared__ __attribute__((aligned(16))) T s_ost[4 * 16 * LDU];    // o store strips
  __shared__ __attribute__((aligned(16))) float s_eb[2][64], s_ed[2][64];
  __shared__ float s_dec[2];                                        // e^{b_C} per buffer

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = pair / a.H;
  const SeqInfo sq = seq_info(a, n);
  const int l = lane_id();
  const int team = threadIdx.x / NTHR;
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
  typedef TileIO<T, BV, K> IOHT;

  if (team == 1) {
    // --------------------------------- loaders -------------------------------------------
    struct Pre { typename IOK::Regs rk; typename IOV::Regs ru; uint32_t graw; int len; };
    Pre pre[LPF];
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
      IOV::load_nomask(P.ru, row_ptr<T>(a.u, sq.b, tok, h) + v0, a.u.st, len);
      P.len = len;
      P.graw = load_scalar_raw(gptr, a.g_dtype, gated ? row_off(a.g, sq.b, tok + min(l, len - 1), h) : 0);
    };
    auto stage = [&](Pre& P, int buf) {
      IOK::mask(P.rk, P.len);
      IOV::mask(P.ru, P.len);
      IOK::store_lds(P.rk, s_k[buf], LDK);
      IOV::store_lds(P.ru, s_u[buf], LDU);
      if (wave_id() == 4) {
        const float x = wave_incl_scan((gated && l < P.len) ? scalar_from_raw(P.graw, a.g_dtype) : 0.f);
        const float xl = __shfl(x, 63, 64);
        s_eb[buf][l] = expf(x);
        s_ed[buf][l] = expf(xl - x);
        if (l == 0) s_dec[buf] = expf(xl);
      }
    };
#pragma unroll
    for (int j = 0; j < LPF; ++j) issue(pre[j], j);
    stage(pre[0], 0);
    issue(pre[0], LPF);
    wait_all_loads();
    auto step = [&](auto slot, const int c) {
      constexpr int j = decltype(slot)::value;
      lds_barrier();                                                                     // B1
      // hs[chunk][h][v0 .. v0+BV][K] <- S^T
      IOHT::lds_to_global(s_hT, LDK, (T*)a.hs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
      if (c + 1 < sq.nchunks) stage(pre[(j + 1) % LPF], (c + 1) & 1);
      lds_barrier();                                                                     // B2
      issue(pre[(j + 1) % LPF], c + 1 + LPF);
    };
    // whole groups of LPF chunks without an exit in between (see the consumers)
    int c0 = 0;
    for (; c0 + LPF <= sq.nchunks; c0 += LPF) {
      step(std::integral_constant<int, 0>(), c0);
      step(std::integral_constant<int, 1>(), c0 + 1);
      step(std::integral_constant<int, 2>(), c0 + 2);
    }
    if (c0 < sq.nchunks) step(std::integral_constant<int, 0>(), c0);
    if (c0 + 1 < sq.nchunks) step(std::integral_constant<int, 1>(), c0 + 1);
    return;
  }

  // --------------------------------- consumers -------------------------------------------
  const int wv = wave_id();
  const int krow0 = wv * (K / 4);
  const int fr = l & 15, fg = 8 * (l >> 4);          // fragment row / contraction offset of this lane
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
  // this wave's strips of w, q (rows of the chunk) and P, kept PF chunks ahead in registers
  RowFrags<T, K> fw[PF], fq[PF];
  RowFrags<T, CH> fp[PF];
  auto issue = [&](RowFrags<T, K>& W, RowFrags<T, K>& Q, RowFrags<T, CH>& P, int c) {
    c = min(c, sq.nchunks - 1);
    const int tok = sq.tok0 + c * CH;
    const int last = min(CH, sq.len - c * CH) - 1;
    W.load(row_ptr<T>(a.w, sq.b, tok, h), a.w.st, 16 * wv, last);
    Q.load(row_ptr<T>(a.q, sq.b, tok, h), a.q.st, 16 * wv, last);
    P.load((const T*)a.pmat + ((int64_t)(sq.chunk0 + c) * a.H + h) * 2 * CH * CH, CH, 16 * wv, CH - 1);
  };
#pragma unroll
  for (int j = 0; j < PF; ++j) issue(fw[j], fq[j], fp[j], j);
  // The compiler may order these first loads freely; were they still pending at the loop header,
  // its wait-count analysis would merge that order into every iteration (a full drain per trip).
  wait_all_loads();

  // one chunk; `slot` (compile-time) names the register set that holds its strips
  auto step = [&](auto slot, const int c) {
    {
      constexpr int j = decltype(slot)::value;
      const int cur = c & 1;
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      // S (state at chunk start) -> LDS as S^T
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(S[mi][ni], s_hT, LDK, krow0 + 16 * mi, 16 * ni);
      lds_barrier();                                                                     // B1
      // w S and q S over the same S^T fragments (rows 16 wv .. of the chunk)
      f32x4 vn[1][NB], o[1][NB];
      acc_zero(vn);
      acc_zero(o);
      fw[j].mask(16 * wv, len);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        typename ET<T>::frag bS[NB];
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) bS[ni] = ET<T>::load_frag(s_hT + (16 * ni + fr) * LDK + 32 * ks + fg);
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          ET<T>::mma(vn[0][ni], fw[j].f[ks], bS[ni]);
          ET<T>::mma(o[0][ni], fq[j].f[ks], bS[ni]);
        }
      }
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
          // v_new = u - w S, rounded once to the storage type so that the state update, the
          // output and the backward see the same values
          vn[0][ni][i] = ET<T>::to_f(ET<T>::from_f(ET<T>::to_f(s_u[cur][r * LDU + cc]) - vn[0][ni][i]));
          o[0][ni][i] *= s_eb[cur][r];
        }
        acc_to_lds_t<T>(vn[0][ni], s_vT, LDC, 16 * wv, 16 * ni);
      }
      const float dec = s_dec[cur];
      lds_barrier();                                                                     // B2
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) S[mi][ni] *= dec;
      // o += P v_new ;  S += k^T (e_d v_new)   over the same v_new^T fragments
#pragma unroll
      for (int ks = 0; ks < CH / 32; ++ks) {
        typename ET<T>::frag af[MB], bv[NB];
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) af[mi] = ET<T>::load_frag_t(s_k[cur], LDK, 32 * ks, krow0 + 16 * mi);
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          bv[ni] = ET<T>::load_frag(s_vT + (16 * ni + fr) * LDC + 32 * ks + fg);
          ET<T>::mma(o[0][ni], fp[j].f[ks], bv[ni]);
          scale_frag8<T>(bv[ni], &s_ed[cur][32 * ks + fg]);
        }
#pragma unroll
        for (int mi = 0; mi < MB; ++mi)
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(S[mi][ni], af[mi], bv[ni]);
      }
      issue(fw[j], fq[j], fp[j], c + PF);
      store_strip<T, NB>(vn, s_stg + wv * 16 * LDU, row_ptr<T>(a.vnew, sq.b, tok + 16 * wv, h) + v0, a.vnew.st,
                         len - 16 * wv, 1.0f);
      store_strip<T, NB>(o, s_ost + wv * 16 * LDU, row_ptr<T>(a.o, sq.b, tok + 16 * wv, h) + v0, a.o.st,
                         len - 16 * wv, a.scale);
    }
  };
  // Whole groups of PF chunks run without an exit between the chunks: an early exit inside the
  // group would be one more path to the loop header, on which the compiler could count only the
  // loads of the first chunk as issued and would drain the prefetch ring on every trip.
  int c0 = 0;
  for (; c0 + PF <= sq.nchunks; c0 += PF) {
    step(std::integral_constant<int, 0>(), c0);
    if constexpr (PF > 1) step(std::integral_constant<int, 1 % PF>(), c0 + 1);
    if constexpr (PF > 2) step(std::integral_constant<int, 2 % PF>(), c0 + 2);
  }
  if constexpr (PF > 1) {
    if (c0 < sq.nchunks) step(std::integral_constant<int, 0>(), c0);
    if constexpr (PF > 2) {
      if (c0 + 1 < sq.nchunks) step(std::integral_constant<int, 1 % PF>(), c0 + 1);
    }
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
// backward (reverse order over the chunks)
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV>
__global__ __launch_bounds__(2 * NTHR) void k_gdn_state_bwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16, KS = K / 32;
  constexpr int PF = GdnStateCfg<T>::PF, LPF = GdnStateCfg<T>::LPF;
  static_assert(LPF == 3 && PF <= 3, "the chunk loops are written out for rings of three");
  // two operand buffers; fp32 tiles with K = 128 (the parity path) leave LDS for one and pay a
  // third barrier per chunk
  constexpr int NBUF = (sizeof(T) == 4 && K == 128) ? 1 : 2;
  __shared__ __attribute__((aligned(16))) T s_q[NBUF][CH * LDK];    // q        [64][K]
  __shared__ __attribute__((aligned(16))) T s_w[NBUF][CH * LDK];    // w        [64][K]
  __shared__ __attribute__((aligned(16))) T s_do[NBUF][CH * LDU];   // do       [64][BV]
  __shared__ __attribute__((aligned(16))) T s_dST[BV * LDK];        // dS'^T    [BV][K]
  __shared__ __attribute__((aligned(16))) T s_dvT[BV * LDC];        // -dv_new^T [BV][64]
  __shared__ __attribute__((aligned(16))) T s_stg[4 * 16 * LDU];    // dv_new store strips
  __shared__ __attribute__((aligned(16))) float s_qs[NBUF][64], s_ed[NBUF][64];
  __shared__ float s_dec[NBUF];

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = pair / a.H;
  const SeqInfo sq = seq_info(a, n);
  const int l = lane_id();
  const int team = threadIdx.x / NTHR;
  if (sq.nchunks == 0) {
    if (a.dh0 && team == 0) {
      for (int idx = threadIdx.x; idx < K * BV; idx += NTHR) {
        const int r = idx / BV, c = v0 + idx % BV;
        const int64_t o = ((int64_t)n * a.H + h) * K * V + (int64_t)r * V + c;
        a.dh0[o] = a.dht ? a.dht[o] : 0.f;
      }
    }
    return;
  }
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;
  typedef TileIO<T, BV, K> IOHT;

  if (team == 1) {
    // --------------------------------- loaders -------------------------------------------
    struct Pre { typename IOK::Regs rq, rw; typename IOV::Regs rd; uint32_t graw; int len; };
    Pre pre[LPF];
    const bool gated = a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr;
    const void* gptr = gated ? a.g.ptr : a.k.ptr;
    const float scale = a.scale;
    // always issued, chunk index clamped (see k_gdn_state_fwd)
    auto issue = [&](Pre& P, int c) {
      c = max(c, 0);
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rq, row_ptr<T>(a.q, sq.b, tok, h), a.q.st, len);
      IOK::load_nomask(P.rw, row_ptr<T>(a.w, sq.b, tok, h), a.w.st, len);
      IOV::load_nomask(P.rd, row_ptr<T>(a.d_o, sq.b, tok, h) + v0, a.d_o.st, len);
      P.len = len;
      P.graw = load_scalar_raw(gptr, a.g_dtype, gated ? row_off(a.g, sq.b, tok + min(l, len - 1), h) : 0);
    };
    auto stage = [&](Pre& P, int buf) {
      IOK::mask(P.rq, P.len);
      IOK::mask(P.rw, P.len);
      IOV::mask(P.rd, P.len);
      IOK::store_lds(P.rq, s_q[buf], LDK);
      IOK::store_lds(P.rw, s_w[buf], LDK);
      IOV::store_lds(P.rd, s_do[buf], LDU);
      if (wave_id() == 4) {
        const float x = wave_incl_scan((gated && l < P.len) ? scalar_from_raw(P.graw, a.g_dtype) : 0.f);
        const float xl = __shfl(x, 63, 64);
        s_qs[buf][l] = scale * expf(x);
        s_ed[buf][l] = expf(xl - x);
        if (l == 0) s_dec[buf] = expf(xl);
      }
    };
#pragma unroll
    for (int j = 0; j < LPF; ++j) issue(pre[j], sq.nchunks - 1 - j);
    stage(pre[0], 0);
    issue(pre[0], sq.nchunks - 1 - LPF);
    wait_all_loads();
    auto step = [&](auto slot, const int it) {
      constexpr int j = decltype(slot)::value;
      const int c = sq.nchunks - 1 - it;
      lds_barrier();                                                                     // B1
      IOHT::lds_to_global(s_dST, LDK, (T*)a.dhs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
      if constexpr (NBUF == 2) {
        if (c > 0) stage(pre[(j + 1) % LPF], (it + 1) & 1);
      }
      lds_barrier();                                                                     // B2
      if constexpr (NBUF == 1) {
        lds_barrier();                                                                   // B3: buffer read
        if (c > 0) stage(pre[(j + 1) % LPF], 0);
      }
      issue(pre[(j + 1) % LPF], c - 1 - LPF);
    };
    // whole groups of LPF chunks without an exit in between (see k_gdn_state_fwd)
    int it0 = 0;
    for (; it0 + LPF <= sq.nchunks; it0 += LPF) {
      step(std::integral_constant<int, 0>(), it0);
      step(std::integral_constant<int, 1>(), it0 + 1);
      step(std::integral_constant<int, 2>(), it0 + 2);
    }
    if (it0 < sq.nchunks) step(std::integral_constant<int, 0>(), it0);
    if (it0 + 1 < sq.nchunks) step(std::integral_constant<int, 1>(), it0 + 1);
    return;
  }

  // --------------------------------- consumers -------------------------------------------
  const int wv = wave_id();
  const int krow0 = wv * (K / 4);
  const int fr = l & 15, fg = 8 * (l >> 4);
  const float scale = a.scale;
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
  // this wave's strips of k (rows of the chunk) and P^T, kept PF chunks ahead in registers
  RowFrags<T, K> fk[PF];
  RowFrags<T, CH> fpt[PF];
  auto issue = [&](RowFrags<T, K>& Kf, RowFrags<T, CH>& Pt, int c) {
    c = max(c, 0);
    const int tok = sq.tok0 + c * CH;
    const int last = min(CH, sq.len - c * CH) - 1;
    Kf.load(row_ptr<T>(a.k, sq.b, tok, h), a.k.st, 16 * wv, last);
    Pt.load((const T*)a.pmat + (((int64_t)(sq.chunk0 + c) * a.H + h) * 2 + 1) * CH * CH, CH, 16 * wv, CH - 1);
  };
#pragma unroll
  for (int j = 0; j < PF; ++j) issue(fk[j], fpt[j], sq.nchunks - 1 - j);
  wait_all_loads();   // see k_gdn_state_fwd

  // one chunk (the it-th from the end); `slot` (compile-time) names its register set
  auto step = [&](auto slot, const int it) {
    {
      constexpr int j = decltype(slot)::value;
      const int c = sq.nchunks - 1 - it;
      const int cur = NBUF == 2 ? (it & 1) : 0;
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(dS[mi][ni], s_dST, LDK, krow0 + 16 * mi, 16 * ni);
      lds_barrier();                                                                     // B1
      // t = k dS'  and  dv_loc = P^T do   (rows 16 wv .. of the chunk)
      f32x4 t[1][NB], dvl[1][NB];
      acc_zero(t);
      acc_zero(dvl);
      fk[j].mask(16 * wv, len);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          const typename ET<T>::frag bD = ET<T>::load_frag(s_dST + (16 * ni + fr) * LDK + 32 * ks + fg);
          ET<T>::mma(t[0][ni], fk[j].f[ks], bD);
        }
      }
      typename ET<T>::frag bdo[CH / 32][NB];
#pragma unroll
      for (int ks = 0; ks < CH / 32; ++ks)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          bdo[ks][ni] = ET<T>::load_frag_t(s_do[cur], LDU, 32 * ks, 16 * ni);
          ET<T>::mma(dvl[0][ni], fpt[j].f[ks], bdo[ks][ni]);
        }
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        f32x4 x;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = 16 * wv + 4 * (l >> 4) + i;
          // dv_new, rounded once to the storage type (the WY backward reads the stored values)
          t[0][ni][i] = ET<T>::to_f(ET<T>::from_f(scale * dvl[0][ni][i] + s_ed[cur][r] * t[0][ni][i]));
          x[i] = -t[0][ni][i];
        }
        acc_to_lds_t<T>(x, s_dvT, LDC, 16 * wv, 16 * ni);
      }
      const float dec = s_dec[cur];
      lds_barrier();                                                                     // B2
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) dS[mi][ni] *= dec;
      // dS += q^T (scale e_b do) - w^T dv_new
#pragma unroll
      for (int ks = 0; ks < CH / 32; ++ks) {
        typename ET<T>::frag aq[MB], aw[MB], bn[NB];
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) {
          aq[mi] = ET<T>::load_frag_t(s_q[cur], LDK, 32 * ks, krow0 + 16 * mi);
          aw[mi] = ET<T>::load_frag_t(s_w[cur], LDK, 32 * ks, krow0 + 16 * mi);
        }
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          scale_frag8<T>(bdo[ks][ni], &s_qs[cur][32 * ks + fg]);
          bn[ni] = ET<T>::load_frag(s_dvT + (16 * ni + fr) * LDC + 32 * ks + fg);
        }
#pragma unroll
        for (int mi = 0; mi < MB; ++mi)
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) {
            ET<T>::mma(dS[mi][ni], aq[mi], bdo[ks][ni]);
            ET<T>::mma(dS[mi][ni], aw[mi], bn[ni]);
          }
      }
      if constexpr (NBUF == 1) lds_barrier();                                            // B3
      issue(fk[j], fpt[j], c - PF);
      store_strip<T, NB>(t, s_stg + wv * 16 * LDU, row_ptr<T>(a.dvnew, sq.b, tok + 16 * wv, h) + v0, a.dvnew.st,
                         len - 16 * wv, 1.0f);
    }
  };
  // whole groups of PF chunks without an exit in between (see k_gdn_state_fwd)
  int it0 = 0;
  for (; it0 + PF <= sq.nchunks; it0 += PF) {
    step(std::integral_constant<int, 0>(), it0);
    if constexpr (PF > 1) step(std::integral_constant<int, 1 % PF>(), it0 + 1);
    if constexpr (PF > 2) step(std::integral_constant<int, 2 % PF>(), it0 + 2);
  }
  if constexpr (PF > 1) {
    if (it0 < sq.nchunks) step(std::integral_constant<int, 0>(), it0);
    if constexpr (PF > 2) {
      if (it0 + 1 < sq.nchunks) step(std::integral_constant<int, 1 % PF>(), it0 + 1);
    }
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

}  // namespace lmoe
