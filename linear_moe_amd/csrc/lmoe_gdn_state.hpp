// Gated delta rule: the two sequential passes over the chunks of one (sequence, head, V-slice).
//
//   forward :  v_new = u - w S,   o = scale [ e^{b_i} q_i S + P v_new ],   S' = e^{b_C} S + k^T (e_d v_new)
//   backward:  dv_new = scale P^T do + e_d (k dS'),
//              dS = e^{b_C} dS' + q^T (scale e_b do) - w^T dv_new
//   with P = (q k^T) . Gamma (written by k_gdn_wy_fwd), e_b = e^{b}, e_d = e^{b_C - b}.
//
// Both kernels keep the per-chunk work of the dependency chain as small as it can be made:
//   * work-group = 3 teams of 4 waves that meet at two barriers per chunk (B1, B2).
//     Team 0 (consumers) owns the state slice [K x BV] in fp32 MFMA accumulators (wave w: rows
//     [w K/4, (w+1) K/4)) and, for the products whose rows are tokens, rows 16 w .. 16 w + 15 of
//     the chunk.  It touches LDS and the matrix cores only: a wave that issues global loads or
//     stores stalls at the issue whenever the vector memory pipe of the CU is busy, and on this
//     wave every such stall lengthens the chain.
//     Teams 1 and 2 (loaders) own all global traffic: they keep the operand tiles of the next
//     chunks in flight in registers (whole 128-byte lines per row) and stage them into single
//     LDS buffers in the half-step before they are needed.  Team 1 has the tiles phase 2 reads
//     and writes the state checkpoints (hs / dhs, layout [V][K]) and the chunk's results, which
//     it lifts out of LDS during phase 1 and stores during phase 2; team 2 has the tiles phase 1
//     reads: it stages during phase 2 and issues its loads during phase 1, so that in both
//     half-steps one team fills LDS while the other waits on the memory pipe.
//   * the intra-chunk matrix P is not formed here: the chunk-parallel WY preparation writes it
//     once per (chunk, head) instead of once per V-slice.
//   * grid = ceil(N*H / 8) * 8 * (V / BV) work-groups (1-D): the V-slices of one (sequence, head)
//     get ids congruent mod 8, i.e. run on the same XCD and share k, w, q, P through its L2.
#pragma once
#include <type_traits>
#include "lmoe_seq.hpp"

namespace lmoe {

// V-slice / prefetch shape of the sequential passes per element type
template <typename T> struct GdnStateCfg {
  static constexpr int BV = sizeof(T) == 2 ? 32 : 16;    // V columns per work-group
  static constexpr int BV_WIDE = sizeof(T) == 2 ? 64 : 16;   // ... when there are enough work-groups anyway
  static constexpr int LPF = sizeof(T) == 2 ? 2 : 1;     // chunks a loader keeps in flight per ring
};

// Runs step(slot, i) for i = 0 .. n-1 with slot = i % L as a compile-time constant.
// Whole groups of L steps run without an exit in between: an early exit inside a group would be
// one more path to the loop header, on which the compiler could count only the loads of the
// first step as issued and would drain the prefetch ring on every trip.
template <int L, int J = 0, typename F> __device__ __forceinline__ void ring_group(int i, F& step) {
  if constexpr (J < L) {
    step(std::integral_constant<int, J>(), i + J);
    ring_group<L, J + 1>(i, step);
  }
}
template <int L, int J = 0, typename F> __device__ __forceinline__ void ring_tail(int i, int n, F& step) {
  if constexpr (J < L - 1) {
    if (i + J < n) {
      step(std::integral_constant<int, J>(), i + J);
      ring_tail<L, J + 1>(i, n, step);
    }
  }
}
template <int L, typename F> __device__ __forceinline__ void ring_loop(int n, F&& step) {
  int i = 0;
  for (; i + L <= n; i += L) ring_group<L>(i, step);
  ring_tail<L>(i, n, step);
}

// ------------------------------------------------------------------------- //
// forward
//   team 1, chunk c:   B1 | stage k(c), P(c); lift S^T(c), o(c-1) out of LDS |
//                      B2 | lift v_new(c); store hs(c), o(c-1), v_new(c); prefetch k, P
//   team 2, chunk c:   B1 | prefetch w, q, u, decay table | B2 | stage those of chunk c+1
//   consumers, chunk c: S -> LDS | B1 | w S, q S, v_new -> LDS | B2 | S update, P v_new, o -> LDS
//   (team 1 lifts v_new(c) right after B2 and stores it in the same half-step)
// ------------------------------------------------------------------------- //
// SAVE = false (forward-only call): hs and v_new, which only the backward reads, are not written
template <typename T, int K, int V, int BV, bool SAVE, bool WT>
__global__ __launch_bounds__(3 * NTHR) void k_gdn_state_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16, KS = K / 32;
  constexpr int LPF = GdnStateCfg<T>::LPF;
  // WT: w = Tinv (k beta e^{b}) and u = Tinv (v beta) are not read from memory (w: 16 KB per chunk and work-group
  // through a request queue that bounds this kernel; neither is then written by the WY preparation) but formed on
  // the chip: during phase 2 of chunk c consumer wave w forms
  // rows 16 w .. of w(c+1) from Tinv(c+1) (8 KB, columns scaled by beta e^{b}) and k(c+1), which the loaders
  // then stage one chunk early into the second of two k tiles.  WT = false (fp32: LDS has no room for that;
  // or no Tinv given): w is read as written by the WY preparation.
  static_assert(!WT || sizeof(T) == 2, "the second k tile fits for 2-byte elements only");
  __shared__ __attribute__((aligned(16))) T s_k[(WT ? 2 : 1) * CH * LDK];   // k          [64][K] (WT: of chunks c, c + 1)
  __shared__ __attribute__((aligned(16))) T s_w[CH * LDK];          // w             [64][K]
  __shared__ __attribute__((aligned(16))) T s_ti[WT ? CH * LDC : 8];   // Tinv       [64][64]
  __shared__ __attribute__((aligned(16))) T s_v[WT ? CH * LDU : 8];    // v          [64][BV] of the chunk whose u is formed
  __shared__ __attribute__((aligned(16))) float s_f[64], s_be[64];  // beta e^{b}, beta of the chunk whose w, u are formed
  __shared__ __attribute__((aligned(16))) T s_q[CH * LDK];          // q             [64][K]
  __shared__ __attribute__((aligned(16))) T s_p[CH * LDC];          // P             [64][64]
  __shared__ __attribute__((aligned(16))) T s_u[CH * LDU];          // u             [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[BV * LDK];         // S^T           [BV][K]
  __shared__ __attribute__((aligned(16))) T s_vn[CH * LDU];         // v_new         [64][BV] (MFMA operand through transposing reads, and stored)
  __shared__ __attribute__((aligned(16))) T s_o[CH * LDU];          // o             [64][BV] (to be stored)
  __shared__ __attribute__((aligned(16))) float s_eb[2][64], s_ed[2][64];
  __shared__ float s_dec[2];                                        // e^{b_C}; gate arrays: buffer c & 1

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
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
  typedef TileIO<T, CH, CH> IOP;
  typedef TileIO<T, BV, K> IOHT;

  if (team == 1) {
    // ------------------------- loaders, ring A (k, P) and all stores ----------------------
    struct PreA { typename IOK::Regs rk; typename IOP::Regs rp, rt; typename IOV::Regs rv; float be, f; int len; };
    PreA pa[LPF];
    // Always issued (chunk index clamped to the last chunk; the surplus loads at the end of a
    // sequence are never consumed): a prefetch that is skipped on some path would make the
    // compiler drain all outstanding loads at every consumer of a register set.
    auto issue_a = [&](PreA& P, int c) {
      c = min(c, sq.nchunks - 1);
      const int tok = sq.tok0 + c * CH;
      P.len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rk, row_ptr<T>(a.k, sq.b, tok, h), a.k.st, P.len);
      IOP::load_nomask(P.rp, (const T*)a.pmat + ((int64_t)(sq.chunk0 + c) * a.H + h) * CH * CH, CH, CH);
      if constexpr (WT) {
        IOP::load_nomask(P.rt, (const T*)a.tinv + ((int64_t)(sq.chunk0 + c) * a.H + h) * CH * CH, CH, CH);
        IOV::load_nomask(P.rv, row_ptr<T>(a.v, sq.b, tok, h) + v0, a.v.st, P.len);
        const float* gc = a.gcum + ((int64_t)(sq.chunk0 + c) * a.H + h) * GATE_ROWS * CH;
        P.be = gc[2 * CH + l];
        P.f = gc[3 * CH + l];
      }
    };
    auto stage_a = [&](PreA& P) {
      IOK::mask(P.rk, P.len);
      IOK::store_lds(P.rk, s_k, LDK);
      IOP::store_lds(P.rp, s_p, LDC);       // rows and columns past the end are zero as written
    };
    // WT: P of chunk c for its phase 2; k, Tinv, v, beta, beta e^{b} of chunk c + 1 for the w, u the consumers form then
    auto stage_p = [&](PreA& P) { IOP::store_lds(P.rp, s_p, LDC); };
    auto stage_k = [&](PreA& P, int c) {
      IOK::mask(P.rk, P.len);
      IOK::store_lds(P.rk, s_k + (c & 1) * CH * LDK, LDK);
      IOP::store_lds(P.rt, s_ti, LDC);
      IOV::mask(P.rv, P.len);
      IOV::store_lds(P.rv, s_v, LDU);
      if (wave_id() == 4) {
        s_be[l] = P.be;
        s_f[l] = P.f;
      }
    };
    // a result tile of chunk c: registers -> global
    auto store_result = [&](const typename IOV::Regs& r, const lmoe_tensor& dst, int c) {
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      IOV::template store_global<true>(r, row_ptr<T>(dst, sq.b, tok, h) + v0, dst.st, len);
    };
#pragma unroll
    for (int j = 0; j < LPF; ++j) issue_a(pa[j], j);
    // the first loads may be ordered freely by the compiler; were they still pending at the loop
    // header, its wait-count analysis would carry that order into every iteration
    wait_all_loads();
    if constexpr (WT) {
      stage_k(pa[0], 0);
      lds_barrier();                                                                     // B0: the consumers form w(0)
    }
    typename IOHT::Regs rh;
    typename IOV::Regs ro;
    // v_new leaves in blocks of at most 32 columns (the layout of vnew: see slice_ptr)
    constexpr int SBW = BV < SLICE_COLS ? BV : SLICE_COLS, NSB = BV / SBW;
    typedef TileIO<T, CH, SBW> IOS;
    typename IOS::Regs rvn[NSB];
    ring_loop<LPF>(sq.nchunks, [&](auto slot, const int c) {
      constexpr int j = decltype(slot)::value, jn = (j + 1) % LPF;
      lds_barrier();                                                                     // B1
      if constexpr (WT) {
        stage_p(pa[j]);
        stage_k(pa[jn], c + 1);             // (past the last chunk: a clamped copy of it, never used)
      } else {
        stage_a(pa[j]);
      }
      // S^T and the previous chunk's o leave LDS now (the consumers rewrite them after B2)
      if constexpr (SAVE) IOHT::load_lds(rh, s_hT, LDK);
      IOV::load_lds(ro, s_o, LDU);
      lds_barrier();                                                                     // B2
      // v_new of this chunk is complete (the consumers rewrite it after the next B1)
      if constexpr (SAVE) {
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) IOS::load_lds(rvn[sb], s_vn + SBW * sb, LDU);
        // hs[chunk][h][v0 .. v0+BV][K] <- S^T
        IOHT::template store_global<true>(rh, (T*)a.hs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
      }
      if (c > 0) store_result(ro, a.o, c - 1);
      if constexpr (SAVE) {
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb)
          IOS::template store_global<true>(rvn[sb], slice_ptr<T>(a.vnew, sq.chunk0 + c, h, a.H, V, v0 + SBW * sb), SLICE_COLS, min(CH, sq.len - c * CH));
      }
      issue_a(pa[j], c + LPF);
    });
    lds_barrier();                                                                       // o of the last chunk
    IOV::load_lds(ro, s_o, LDU);
    store_result(ro, a.o, sq.nchunks - 1);
    return;
  }
  if (team == 2) {
    // ------------------------- loaders, ring B (w, q, u, decay table) ---------------------
    // staged during phase 2 of the step before the one that reads them in phase 1
    struct PreB { typename IOK::Regs rw, rq; typename IOV::Regs ru; float eb, ed; int len; };   // rw unused with WT
    PreB pb[LPF];
    auto issue_b = [&](PreB& P, int c) {
      c = min(c, sq.nchunks - 1);
      const int tok = sq.tok0 + c * CH;
      P.len = min(CH, sq.len - c * CH);
      if constexpr (!WT) IOK::load_nomask(P.rw, row_ptr<T>(a.w, sq.b, tok, h), a.w.st, P.len);
      IOK::load_nomask(P.rq, row_ptr<T>(a.q, sq.b, tok, h), a.q.st, P.len);
      if constexpr (!WT) IOV::load_nomask(P.ru, row_ptr<T>(a.u, sq.b, tok, h) + v0, a.u.st, P.len);
      const float* gc = a.gcum + ((int64_t)(sq.chunk0 + c) * a.H + h) * GATE_ROWS * CH;
      P.eb = gc[l];
      P.ed = gc[CH + l];
    };
    auto stage_b = [&](PreB& P, int buf) {
      if constexpr (!WT) {
        IOK::mask(P.rw, P.len);
        IOK::store_lds(P.rw, s_w, LDK);
      }
      IOK::store_lds(P.rq, s_q, LDK);       // rows past the end only reach output rows that are not stored
      if constexpr (!WT) {
        IOV::mask(P.ru, P.len);
        IOV::store_lds(P.ru, s_u, LDU);
      }
      if (wave_id() == 8) {
        s_eb[buf][l] = P.eb;
        s_ed[buf][l] = P.ed;
        if (l == 63) s_dec[buf] = P.eb;
      }
    };
#pragma unroll
    for (int j = 0; j < LPF; ++j) issue_b(pb[j], j);
    stage_b(pb[0], 0);
    wait_all_loads();   // see ring A
    if constexpr (WT) lds_barrier();                                                     // B0
    ring_loop<LPF>(sq.nchunks, [&](auto slot, const int c) {
      constexpr int j = decltype(slot)::value, jn = (j + 1) % LPF;
      lds_barrier();                                                                     // B1
      issue_b(pb[j], c + LPF);              // chunk c was staged before this barrier: refill its set
      lds_barrier();                                                                     // B2
      if (c + 1 < sq.nchunks) stage_b(pb[jn], (c + 1) & 1);
    });
    lds_barrier();
    return;
  }

  // --------------------------------- consumers -------------------------------------------
  // the waves that carry the recurrence win every issue slot they ask for over the loader waves of
  // their SIMD
  __builtin_amdgcn_s_setprio(3);
  const int wv = wave_id();
  const int krow0 = wv * (K / 4);
  const int fr = l & 15, fg = 8 * (l >> 4);          // fragment row / contraction offset of this lane
  const float scale = a.scale;
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
  // rows 16 wv .. of w(c) and u(c) into the w and u tiles (read back by this wave only, after the next barrier)
  auto form_w = [&](int c) {
    const T* kt = s_k + (c & 1) * CH * LDK;
    f32x4 wacc[K / 16], uacc[NB];
#pragma unroll
    for (int ni = 0; ni < K / 16; ++ni) wacc[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) uacc[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < CH / 32; ++ks) {
      if (ks == 0 || wv >= 2) {            // Tinv is lower triangular
        typename ET<T>::frag bt = ET<T>::load_frag(s_ti + (16 * wv + fr) * LDC + 32 * ks + fg);
        typename ET<T>::frag bu = bt;
        scale_frag8<T>(bt, &s_f[32 * ks + fg]);
        scale_frag8<T>(bu, &s_be[32 * ks + fg]);
#pragma unroll
        for (int ni = 0; ni < K / 16; ++ni) ET<T>::mma(wacc[ni], ET<T>::load_frag_t(kt, LDK, 32 * ks, 16 * ni), bt);
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(uacc[ni], ET<T>::load_frag_t(s_v, LDU, 32 * ks, 16 * ni), bu);
      }
    }
#pragma unroll
    for (int ni = 0; ni < K / 16; ++ni) acc_to_lds_t<T>(wacc[ni], s_w, LDK, 16 * ni, 16 * wv);
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(uacc[ni], s_u, LDU, 16 * ni, 16 * wv);     // u = Tinv (v beta)
  };
  if constexpr (WT) {
    lds_barrier();                                                                       // B0: k, Tinv of chunk 0 staged
    form_w(0);
  }
  for (int c = 0; c < sq.nchunks; ++c) {
    const int cur = c & 1;
    const T* s_kc = s_k + (WT ? cur * CH * LDK : 0);
    // S (state at chunk start) -> LDS as S^T
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(S[mi][ni], s_hT, LDK, krow0 + 16 * mi, 16 * ni);
    lds_barrier();                                                                       // B1
    // (w S)^T and (q S)^T over the same S^T fragments, for the tokens 16 wv .. of the chunk.  The
    // products are formed transposed (S^T as the A operand): a lane then holds four consecutive V
    // columns of one token, so u is read and v_new, o are written with 8-byte LDS accesses in token-major
    // layout (2-byte LDS accesses cost as many cycles as 8-byte ones).
    f32x4 vn[1][NB], o[1][NB];
    acc_zero(vn);
    acc_zero(o);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const typename ET<T>::frag aw = ET<T>::load_frag(s_w + (16 * wv + fr) * LDK + 32 * ks + fg);
      const typename ET<T>::frag aq = ET<T>::load_frag(s_q + (16 * wv + fr) * LDK + 32 * ks + fg);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        const typename ET<T>::frag bS = ET<T>::load_frag(s_hT + (16 * ni + fr) * LDK + 32 * ks + fg);
        ET<T>::mma(vn[0][ni], bS, aw);
        ET<T>::mma(o[0][ni], bS, aq);
      }
    }
    const int tk = 16 * wv + (l & 15);       // token of this lane in the transposed accumulators
    const float ebt = s_eb[cur][tk];
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) {
      const typename ET<T>::vec4 u4 = *(const typename ET<T>::vec4*)(s_u + tk * LDU + 16 * ni + 4 * (l >> 4));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // v_new = u - w S, rounded once to the storage type so that the state update, the
        // output and the backward see the same values
        vn[0][ni][i] = ET<T>::to_f(ET<T>::from_f(ET<T>::to_f(u4[i]) - vn[0][ni][i]));
        o[0][ni][i] *= ebt;
      }
      acc_to_lds_t<T>(vn[0][ni], s_vn, LDU, 16 * ni, 16 * wv);      // s_vn[token][v]
    }
    const float dec = s_dec[cur];
    lds_barrier();                                                                       // B2
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) S[mi][ni] *= dec;
    // o += P v_new ;  S += k^T (e_d v_new)   over the same v_new^T fragments
#pragma unroll
    for (int ks = 0; ks < CH / 32; ++ks) {
      typename ET<T>::frag af[MB], bv[NB];
      const typename ET<T>::frag ap = ET<T>::load_frag(s_p + (16 * wv + fr) * LDC + 32 * ks + fg);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) af[mi] = ET<T>::load_frag_t(s_kc, LDK, 32 * ks, krow0 + 16 * mi);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        bv[ni] = ET<T>::load_frag_t(s_vn, LDU, 32 * ks, 16 * ni);       // rows: V columns, contraction: tokens
        ET<T>::mma(o[0][ni], bv[ni], ap);
        scale_frag8<T>(bv[ni], &s_ed[cur][32 * ks + fg]);
      }
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(S[mi][ni], af[mi], bv[ni]);
    }
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) {
      // o for the loaders (they lift the previous chunk's during phase 1, hence not earlier)
      o[0][ni] *= scale;
      acc_to_lds_t<T>(o[0][ni], s_o, LDU, 16 * ni, 16 * wv);         // s_o[token][v]
    }
    if constexpr (WT) form_w(c + 1);         // off the chain: the loaders' requests bound this window
  }
  lds_barrier();                                                                         // results of the last chunk
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
// backward (reverse order over the chunks; it = 0 is the last chunk)
//     dv_new = scale P^T do + e_d (k dS'),   dZ = Tinv^T dv_new,
//     dS = e^{b_C} dS' + q^T (scale e_b do) - (k beta e^{b})^T dZ
//   dZ is the gradient with respect to Z = beta (v - e^{b} k S)  (v_new = Tinv Z, i.e. (I + L) v_new = Z).  It is
//   what leaves for the chunk-parallel backward instead of dv_new: with it every gradient of the WY form is one
//   product with dZ -- dv = beta dZ, d(k beta e^{b}) = -dZ S^T, dL = -strictlower(dZ v_new^T) -- and that kernel
//   needs neither Tinv nor a product of three 64 x 64 matrices.  It also carries the recurrence: w^T dv_new with
//   w = Tinv (k beta e^{b}) is (k beta e^{b})^T dZ, so w (a 64 x 64 x K product per chunk on the waves of the
//   chain) is never formed; the 64 x 64 x BV product for dZ runs on the team that stores it while the consumers
//   add q^T (scale e_b do), at the price of a third barrier per chunk.
//   team 1, chunk c:   B1 | stage q(c); lift dS'^T(c) out of LDS; read its rows of Tinv^T |
//                      B2 | dZ(c) for its 16 tokens per wave -> LDS | B3 | store dhs(c), dZ(c); prefetch q
//   team 2, chunk c:   B1 | prefetch k, P, Tinv, do, decay table | B2 | stage those of chunk c-1 | B3 |
//                      (4-byte elements: one k tile, staged behind B3, when the consumers hold its fragments)
//   consumers, chunk c: dS' -> LDS | B1 | k dS', P^T do, dv_new -> LDS | B2 | dS = e^{b_C} dS + q^T (..);
//                      fragments of (k beta e^{b})^T | B3 | dS -= (k beta e^{b})^T dZ
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV>
__global__ __launch_bounds__(3 * NTHR) void k_gdn_state_bwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16, KS = K / 32;
  constexpr int LPF = GdnStateCfg<T>::LPF;
  // 2-byte elements: two k tiles (chunk c is read until B3, chunk c - 1 is staged behind B2); 4-byte elements have
  // the room for one, which team 2 refills behind B3
  constexpr bool LATE = sizeof(T) == 4;
  constexpr int NKB = LATE ? 1 : 2;
  __shared__ __attribute__((aligned(16))) T s_q[CH * LDK];          // q         [64][K]
  __shared__ __attribute__((aligned(16))) T s_ti[CH * LDC];         // Tinv      [64][64]
  __shared__ __attribute__((aligned(16))) T s_k[NKB * CH * LDK];    // k         [64][K]
  __shared__ __attribute__((aligned(16))) T s_p[CH * LDC];          // P         [64][64]
  __shared__ __attribute__((aligned(16))) T s_do[CH * LDU];         // do        [64][BV]
  __shared__ __attribute__((aligned(16))) T s_dST[BV * LDK];        // dS'^T     [BV][K]
  __shared__ __attribute__((aligned(16))) T s_dvn[CH * LDU];        // dv_new    [64][BV] (MFMA operand through transposing reads)
  __shared__ __attribute__((aligned(16))) T s_dz[CH * LDU];         // dZ        [64][BV] (likewise, and stored)
  __shared__ __attribute__((aligned(16))) float s_qs[2][64], s_ed[2][64], s_f[NKB][64];   // s_f = beta e^{b}: goes with the k tile
  __shared__ float s_dec[2];                                        // gate arrays: buffer it & 1

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
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
  typedef TileIO<T, CH, CH> IOP;
  typedef TileIO<T, BV, K> IOHT;

  if (team == 1) {
    // ------------------------- loaders, ring A (q), dZ and all stores ---------------------
    struct PreA { typename IOK::Regs rq; int len; };
    PreA pa[LPF];
    // always issued, chunk index clamped (see k_gdn_state_fwd); `it` counts chunks from the end
    auto issue_a = [&](PreA& P, int it) {
      const int c = max(sq.nchunks - 1 - it, 0);
      const int tok = sq.tok0 + c * CH;
      P.len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rq, row_ptr<T>(a.q, sq.b, tok, h), a.q.st, P.len);
    };
    auto stage_a = [&](PreA& P) {
      IOK::mask(P.rq, P.len);
      IOK::store_lds(P.rq, s_q, LDK);
    };
    // dZ = Tinv^T dv_new: wave wt of this team forms the 16 tokens 16 wt .. (transposed, so that a lane holds four
    // consecutive columns of one token) into its rows of s_dz, which the consumers read behind B3 and which it
    // stores itself.  dZ lies in memory like v_new (blocks of 32 columns, see slice_ptr).
    const int wt = wave_id() - 4;
    constexpr int VEC = ET<T>::VEC, VPRW = BV / VEC, NDZ = (16 * VPRW + 63) / 64;
    typedef typename ET<T>::vec vec;
#pragma unroll
    for (int j = 0; j < LPF; ++j) issue_a(pa[j], j);
    wait_all_loads();   // see k_gdn_state_fwd
    typename IOHT::Regs rh;
    ring_loop<LPF>(sq.nchunks, [&](auto slot, const int it) {
      constexpr int j = decltype(slot)::value;
      const int c = sq.nchunks - 1 - it;
      lds_barrier();                                                                     // B1
      stage_a(pa[j]);
      // dS'^T leaves LDS now (the consumers rewrite it at the end of the chunk)
      IOHT::load_lds(rh, s_dST, LDK);
      // rows 16 wt .. of Tinv^T (team 2 restages the tile behind B2); Tinv is lower triangular
      typename ET<T>::frag tf[CH / 32];
#pragma unroll
      for (int ks = 0; ks < CH / 32; ++ks) tf[ks] = ET<T>::load_frag_t(s_ti, LDC, 32 * ks, 16 * wt, l);
      lds_barrier();                                                                     // B2: dv_new of this chunk is complete
      f32x4 dz[NB];
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) dz[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < CH / 32; ++ks) {
        if (ks == CH / 32 - 1 || wt < 2) {
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(dz[ni], ET<T>::load_frag_t(s_dvn, LDU, 32 * ks, 16 * ni, l), tf[ks]);
        }
      }
      // rounded once to the storage type: the recurrence and the chunk-parallel backward see the same values
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(dz[ni], s_dz, LDU, 16 * ni, 16 * wt, l);
      lds_barrier();                                                                     // B3
      const int len = min(CH, sq.len - c * CH);
      vec zv[NDZ];
#pragma unroll
      for (int x = 0; x < NDZ; ++x) {
        const int idx = min(l + 64 * x, 16 * VPRW - 1);
        zv[x] = *(const vec*)(s_dz + (16 * wt + idx / VPRW) * LDU + (idx % VPRW) * VEC);
      }
      IOHT::template store_global<true>(rh, (T*)a.dhs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
#pragma unroll
      for (int x = 0; x < NDZ; ++x) {
        const int idx = l + 64 * x, tokr = 16 * wt + idx / VPRW, col = (idx % VPRW) * VEC;
        if (idx < 16 * VPRW && tokr < len)
          __builtin_nontemporal_store(zv[x], (vec*)(slice_ptr<T>(a.dvnew, sq.chunk0 + c, h, a.H, V, v0 + col) + tokr * SLICE_COLS));
      }
      issue_a(pa[j], it + LPF);
    });
    lds_barrier();
    return;
  }
  if (team == 2) {
    // ------------------------- loaders, ring B (k, P, Tinv, do, decay table, beta) ------
    // staged during phase 2 of the step before the one that reads them in phase 1
    struct PreB { typename IOK::Regs rk; typename IOP::Regs rp, rt; typename IOV::Regs rd; float eb, ed, f; int len; };
    PreB pb[LPF];
    const float scale = a.scale;
    auto issue_b = [&](PreB& P, int it) {
      const int c = max(sq.nchunks - 1 - it, 0);
      const int tok = sq.tok0 + c * CH;
      P.len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rk, row_ptr<T>(a.k, sq.b, tok, h), a.k.st, P.len);
      IOP::load_nomask(P.rp, (const T*)a.pmat + ((int64_t)(sq.chunk0 + c) * a.H + h) * CH * CH, CH, CH);
      IOP::load_nomask(P.rt, (const T*)a.tinv + ((int64_t)(sq.chunk0 + c) * a.H + h) * CH * CH, CH, CH);
      IOV::load_nomask(P.rd, row_ptr<T>(a.d_o, sq.b, tok, h) + v0, a.d_o.st, P.len);
      const float* gc = a.gcum + ((int64_t)(sq.chunk0 + c) * a.H + h) * GATE_ROWS * CH;
      P.eb = gc[l];
      P.ed = gc[CH + l];
      P.f = gc[3 * CH + l];
    };
    auto stage_b = [&](PreB& P, int buf) {
      const int kb = LATE ? 0 : buf;
      IOK::mask(P.rk, P.len);
      IOV::mask(P.rd, P.len);
      IOK::store_lds(P.rk, s_k + kb * CH * LDK, LDK);
      IOP::store_lds(P.rp, s_p, LDC);       // rows and columns past the end are zero as written
      IOP::store_lds(P.rt, s_ti, LDC);
      IOV::store_lds(P.rd, s_do, LDU);
      if (wave_id() == 8) {
        s_f[kb][l] = P.f;
        s_qs[buf][l] = scale * P.eb;
        s_ed[buf][l] = P.ed;
        if (l == 63) s_dec[buf] = P.eb;
      }
    };
#pragma unroll
    for (int j = 0; j < LPF; ++j) issue_b(pb[j], j);
    stage_b(pb[0], 0);
    wait_all_loads();
    ring_loop<LPF>(sq.nchunks, [&](auto slot, const int it) {
      constexpr int j = decltype(slot)::value, jn = (j + 1) % LPF;
      lds_barrier();                                                                     // B1
      issue_b(pb[j], it + LPF);             // this chunk was staged before the barrier: refill its set
      lds_barrier();                                                                     // B2
      if constexpr (!LATE) {
        if (it + 1 < sq.nchunks) stage_b(pb[jn], (it + 1) & 1);
      }
      lds_barrier();                                                                     // B3
      if constexpr (LATE) {
        if (it + 1 < sq.nchunks) stage_b(pb[jn], (it + 1) & 1);
      }
    });
    lds_barrier();
    return;
  }

  // --------------------------------- consumers -------------------------------------------
  // the waves that carry the recurrence win every issue slot they ask for over the loader waves of
  // their SIMD
  __builtin_amdgcn_s_setprio(3);
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
  for (int it = 0; it < sq.nchunks; ++it) {
    const int cur = it & 1;
    const T* s_kc = s_k + (LATE ? 0 : cur) * CH * LDK;
    const float* s_fc = s_f[LATE ? 0 : cur];
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(dS[mi][ni], s_dST, LDK, krow0 + 16 * mi, 16 * ni);
    lds_barrier();                                                                       // B1
    // t = (k dS')^T  and  dv_loc = (P^T do)^T for the tokens 16 wv .. of the chunk: formed transposed,
    // so that a lane holds four consecutive V columns of one token (see k_gdn_state_fwd)
    f32x4 t[1][NB], dvl[1][NB];
    acc_zero(t);
    acc_zero(dvl);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const typename ET<T>::frag ak = ET<T>::load_frag(s_kc + (16 * wv + fr) * LDK + 32 * ks + fg);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni)
        ET<T>::mma(t[0][ni], ET<T>::load_frag(s_dST + (16 * ni + fr) * LDK + 32 * ks + fg), ak);
    }
    typename ET<T>::frag bdo[CH / 32][NB];
#pragma unroll
    for (int ks = 0; ks < CH / 32; ++ks) {
      // rows 16 wv .. of P^T: P is stored as written, the contraction runs along its rows
      const typename ET<T>::frag ap = ET<T>::load_frag_t(s_p, LDC, 32 * ks, 16 * wv);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        bdo[ks][ni] = ET<T>::load_frag_t(s_do, LDU, 32 * ks, 16 * ni);
        ET<T>::mma(dvl[0][ni], bdo[ks][ni], ap);
      }
    }
#pragma unroll
    for (int ks = 0; ks < CH / 32; ++ks)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) scale_frag8<T>(bdo[ks][ni], &s_qs[cur][32 * ks + fg]);
    const float edt = s_ed[cur][16 * wv + (l & 15)];       // the token of this lane
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        // dv_new, rounded once to the storage type.
        // The fused multiply-add is spelled out: left to the compiler, a sum of two products is contracted
        // one way or the other per instantiation, and the wide and narrow slices then differ in the last bit.
        t[0][ni][i] = ET<T>::to_f(ET<T>::from_f(__builtin_fmaf(scale, dvl[0][ni][i], edt * t[0][ni][i])));
      acc_to_lds_t<T>(t[0][ni], s_dvn, LDU, 16 * ni, 16 * wv);      // s_dvn[token][v]
    }
    const float dec = s_dec[cur];
    lds_barrier();                                                                       // B2
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) dS[mi][ni] *= dec;
    // dS += q^T (scale e_b do), while team 1 forms dZ; the fragments of (k beta e^{b})^T for what follows B3 are
    // requested here too
    typename ET<T>::frag aw[CH / 32][MB];
#pragma unroll
    for (int ks = 0; ks < CH / 32; ++ks) {
      typename ET<T>::frag aq[MB];
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) {
        aq[mi] = ET<T>::load_frag_t(s_q, LDK, 32 * ks, krow0 + 16 * mi);
        aw[ks][mi] = ET<T>::load_frag_t(s_kc, LDK, 32 * ks, krow0 + 16 * mi);
      }
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(dS[mi][ni], aq[mi], bdo[ks][ni]);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) {
        scale_frag8<T>(aw[ks][mi], &s_fc[32 * ks + fg]);
        frag_negate(aw[ks][mi]);
      }
    }
    lds_barrier();                                                                       // B3: dZ of this chunk is complete
    // dS -= (k beta e^{b})^T dZ
#pragma unroll
    for (int ks = 0; ks < CH / 32; ++ks) {
      typename ET<T>::frag bn[NB];
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) bn[ni] = ET<T>::load_frag_t(s_dz, LDU, 32 * ks, 16 * ni);    // rows: V columns, contraction: tokens
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(dS[mi][ni], aw[ks][mi], bn[ni]);
    }
  }
  lds_barrier();
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
