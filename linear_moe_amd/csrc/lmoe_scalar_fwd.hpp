// Forward kernel of chunk_simple_gla (one scalar log-decay per token and head): one sequential
// pass over the chunks of one (sequence, head, V-slice) that carries the state and forms the output
//   o = scale [ e^{b_i} q_i S + ((q k^T) . Gamma) v ],   S' = e^{b_C} S + (k . e^{b_C - b})^T v,
//   Gamma_ij = e^{b_i - b_j} [i >= j].
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

template <typename T> __device__ __forceinline__ void scale_frag(typename ET<T>::frag& f, const float* s8) {
  const f32x4 s0 = *(const f32x4*)s8, s1 = *(const f32x4*)(s8 + 4);
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { f[i] = (bf16)((float)f[i] * s0[i]); f[i + 4] = (bf16)((float)f[i + 4] * s1[i]); }
  } else {
    f.lo *= s0; f.hi *= s1;
  }
}

// ------------------------------------------------------------------------- //
// state pass + output (forward): work-group of three teams of four waves (768 threads)
//   grid = ceil(N*H / 8) * 8 * (V / BV) work-groups (1-D).  Work-group -> (sequence, head,
//   V-slice): the V-slices of one (sequence, head) get ids that are congruent mod 8, i.e. run on
//   the same XCD and share q, k through its L2.
//   Team 0 (waves 0-3, consumers) carries the dependency chain of the state and nothing else:
//        S -> LDS (element type T) | B1 | S = e^{b_C} S + k^T (e_d v) | B2
//     wave w owns state rows [w*K/4, (w+1)*K/4) x BV columns in fp32 MFMA accumulators; the row
//     scaling e_d is applied to the v fragments in registers, so k is staged unscaled.
//   Team 1 (waves 4-7, loaders) keeps the operands of the next PF chunks in flight in registers,
//     forms the gate cumsum, fills the other LDS buffer and writes hs (layout [V][K]) from the
//     LDS copy of S (SAVE; a forward-only call passes hs = NULL and nothing is written).
//   Team 2 (waves 8-11, output) forms the chunk's output rows 16w.. between B1 and B2: e^{b_i} q S, its rows of
//     P = (q k^T) . Gamma (kept in registers as an MFMA operand) and P v; the rows are stored after B2.
//   All teams meet at the same barriers; three waves per SIMD hide each other's latencies.
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV, bool SAVE>
__global__ __launch_bounds__(3 * NTHR) void k_state_fwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16;
  // bf16: two operand buffers; fp32 (the parity path) has LDS for one and pays a third barrier
  constexpr int NBUF = sizeof(T) == 2 ? 2 : 1;
  __shared__ __attribute__((aligned(16))) T s_k[NBUF][CH * LDK];              // k             [64][K]
  __shared__ __attribute__((aligned(16))) T s_q[NBUF][CH * LDK];              // q             [64][K]
  __shared__ __attribute__((aligned(16))) T s_u[NBUF][CH * LDU];              // u or v        [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[BV * LDK];                   // S^T           [BV][K]
  __shared__ __attribute__((aligned(16))) T s_pst[4 * 16 * LDC];              // team 2: P strips
  __shared__ __attribute__((aligned(16))) T s_ost[4 * 16 * LDU];              // team 2: o store
  __shared__ __attribute__((aligned(16))) float s_b[NBUF][64], s_eb[NBUF][64], s_ed[NBUF][64];
  __shared__ float s_dec[NBUF];                                               // e^{b_C} per buffer

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
    constexpr int PF = 2;
    struct Pre { typename IOK::Regs rk, rq; typename IOV::Regs ru; uint32_t graw; int len; };
    Pre pre[PF];
    const lmoe_tensor& us = a.v;
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
      IOK::load_nomask(P.rq, row_ptr<T>(a.q, sq.b, tok, h), a.q.st, len);
      IOV::load_nomask(P.ru, row_ptr<T>(us, sq.b, tok, h) + v0, us.st, len);
      P.len = len;
      P.graw = load_scalar_raw(gptr, a.g_dtype, gated ? row_off(a.g, sq.b, tok + min(l, len - 1), h) : 0);
    };
    // registers -> LDS buffer `buf`
    auto stage = [&](Pre& P, int buf) {
      IOK::mask(P.rk, P.len);
      IOK::mask(P.rq, P.len);
      IOV::mask(P.ru, P.len);
      IOK::store_lds(P.rk, s_k[buf], LDK);
      IOK::store_lds(P.rq, s_q[buf], LDK);
      IOV::store_lds(P.ru, s_u[buf], LDU);
      if (wave_id() == 4) {
        const float x = wave_incl_scan((gated && l < P.len) ? scalar_from_raw(P.graw, a.g_dtype) : 0.f);
        const float xl = __shfl(x, 63, 64);
        s_b[buf][l] = x;
        s_eb[buf][l] = expf(x);
        s_ed[buf][l] = expf(xl - x);
        if (l == 0) s_dec[buf] = expf(xl);
      }
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
        // the next chunk's operands first (always: past the end it is the last chunk again, never consumed),
        // so that the wait for their loads does not sit behind the store below
        if constexpr (NBUF == 2) stage(pre[(j + 1) % PF], (c + 1) & 1);
        // hs[chunk][h][v0 .. v0+BV][K] <- S^T (only the backward reads it: SAVE = false for forward-only calls)
        if constexpr (SAVE)
          IOHT::lds_to_global(s_hT, LDK, (T*)a.hs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
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

  if (team == 2) {
    // --------------------------------- output --------------------------------------------
    const int ow = wave_id() - 8;
    T* pst = s_pst + ow * 16 * LDC;
    for (int c = 0; c < sq.nchunks; ++c) {
      const int cur = NBUF == 2 ? (c & 1) : 0;
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      lds_barrier();                                                                     // B1
      // Everything of output rows 16 ow .. happens in this window, where the consumers only update the state:
      // e^{b} q S, the rows of P = (q k^T) . Gamma (blocks above the diagonal are zero and skipped), and P v.
      const int fr = l & 15, fg = 8 * (l >> 4);
      if constexpr (sizeof(T) == 4) {
        // fp32 (the parity path): looped products, P through this wave's own LDS strip
        f32x4 o[1][NB], pp[1][4];
        acc_zero(o);
        acc_zero(pp);
        const f32x4 bi = *(const f32x4*)&s_b[cur][16 * ow + 4 * (l >> 4)];
        float bj[4];
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) bj[nj] = s_b[cur][16 * nj + fr];
        gemm<T, 1, NB, false, false>(o, s_q[cur], LDK, 16 * ow, s_hT, LDK, 0, 0, K);
        gemm<T, 1, 4, false, false>(pp, s_q[cur], LDK, 16 * ow, s_k[cur], LDK, 0, 0, K);
#pragma unroll
        for (int ni = 0; ni < NB; ++ni)
#pragma unroll
          for (int e = 0; e < 4; ++e) o[0][ni][e] *= s_eb[cur][16 * ow + 4 * (l >> 4) + e];
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) {
          f32x4 x;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int i = 16 * ow + 4 * (l >> 4) + e, j = 16 * nj + fr;
            x[e] = (i >= j) ? pp[0][nj][e] * texp<T>(bi[e] - bj[nj]) : 0.f;
          }
          acc_to_lds<T>(x, pst, LDC, 0, 16 * nj);
        }
        // the strip is this wave's own: ordering inside the wave is enough
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        gemm<T, 1, NB, false, true>(o, pst, LDC, 0, s_u[cur], LDU, 0, 0, CH);
        lds_barrier();                                                                   // B2
        store_strip<T, NB>(o, s_ost + ow * 16 * LDU, row_ptr<T>(a.o, sq.b, tok + 16 * ow, h) + v0, a.o.st,
                           len - 16 * ow, a.scale);
      } else {
        // 2-byte elements.  All three products are formed transposed (the MFMA operands swapped), so that a lane
        // holds four consecutive columns of ONE token: P^T = k q^T then lies in the lanes as the operand of
        // (P v)^T = v^T P^T needs it (frag_of_blocks; v^T read in the matching numbering, load_frag_t_blocks) and
        // never goes through LDS, the gate factors of a lane are one b_i and four consecutive b_j, and the result
        // leaves as 8-byte writes.  Every fragment and gate value is requested before the first product (left to the
        // compiler, each read is waited for where it is used and the window is a chain of LDS round trips).
        constexpr int KS = K / 32, CS = CH / 32;
        const int g4 = 4 * (l >> 4);
        typename ET<T>::frag fq[KS], fh[KS][NB], fk[KS][4], fv[CS][NB];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          fq[ks] = ET<T>::load_frag(s_q[cur] + (16 * ow + fr) * LDK + 32 * ks + fg);
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) fh[ks][ni] = ET<T>::load_frag(s_hT + (16 * ni + fr) * LDK + 32 * ks + fg);
#pragma unroll
          for (int nj = 0; nj < 4; ++nj)
            if (nj <= ow) fk[ks][nj] = ET<T>::load_frag(s_k[cur] + (16 * nj + fr) * LDK + 32 * ks + fg);
        }
        __builtin_amdgcn_sched_barrier(0);
        f32x4 ot[NB], pt[4];
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ot[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) pt[nj] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(ot[ni], fh[ks][ni], fq[ks]);      // (q S)^T: column x token
#pragma unroll
          for (int nj = 0; nj < 4; ++nj)
            if (nj <= ow) ET<T>::mma(pt[nj], fk[ks][nj], fq[ks]);                       // P^T: token j x token i
        }
        // second batch (the fragments above are dead by now: all of them at once do not fit the registers)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kq = 0; kq < CS; ++kq)
#pragma unroll
          for (int ni = 0; ni < NB; ++ni)
            if (2 * kq <= ow) fv[kq][ni] = load_frag_t_blocks(s_u[cur], LDU, 32 * kq, 16 * ni, l);
        const float bi = s_b[cur][16 * ow + fr], ebi = s_eb[cur][16 * ow + fr];
        f32x4 bj[4];
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) bj[nj] = *(const f32x4*)&s_b[cur][16 * nj + g4];
        __builtin_amdgcn_sched_barrier(0);
        const int i = 16 * ow + fr;
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ot[ni] *= ebi;
#pragma unroll
        for (int nj = 0; nj < 4; ++nj)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            pt[nj][e] = (i >= 16 * nj + g4 + e) ? pt[nj][e] * texp<T>(bi - bj[nj][e]) : 0.f;
#pragma unroll
        for (int kq = 0; kq < CS; ++kq) {
          if (2 * kq <= ow) {        // tokens j >= 32 only reach the rows of waves 2, 3
            const typename ET<T>::frag fp = frag_of_blocks(pt[2 * kq], pt[2 * kq + 1]);
#pragma unroll
            for (int ni = 0; ni < NB; ++ni) ET<T>::mma(ot[ni], fv[kq][ni], fp);         // (P v)^T
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier();                                                                   // B2
        store_strip_t<T, NB>(ot, s_ost + ow * 16 * LDU, row_ptr<T>(a.o, sq.b, tok + 16 * ow, h) + v0, a.o.st,
                             len - 16 * ow, a.scale);
      }
      if constexpr (NBUF == 1) lds_barrier();                                            // B3
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
    // S (state at chunk start) -> LDS as S^T
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(S[mi][ni], s_hT, LDK, krow0 + 16 * mi, 16 * ni);
    lds_barrier();                                                                       // B1
    const float dec = s_dec[cur];
    // S = e^{b_C} S + k^T (e_d v'): the row scaling e_d is applied to the v' fragments in registers.  In this
    // window, not behind B2: the copy of S for the output team was written before B1, nothing here waits for
    // the P rows below, and behind B2 the consumers then go straight to the next chunk's copy
    {
      typename ET<T>::frag af[CH / 32][MB], bf[CH / 32][NB];
#pragma unroll
      for (int kq = 0; kq < CH / 32; ++kq) {
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) af[kq][mi] = ET<T>::load_frag_t(s_k[cur], LDK, 32 * kq, krow0 + 16 * mi);
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) bf[kq][ni] = ET<T>::load_frag_t(s_u[cur], LDU, 32 * kq, 16 * ni);
      }
#pragma unroll
      for (int kq = 0; kq < CH / 32; ++kq)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) scale_frag<T>(bf[kq][ni], &s_ed[cur][32 * kq + 8 * (l >> 4)]);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) S[mi][ni] *= dec;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kq = 0; kq < CH / 32; ++kq)
#pragma unroll
        for (int mi = 0; mi < MB; ++mi)
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(S[mi][ni], af[kq][mi], bf[kq][ni]);
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_barrier();                                                                       // B2
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

}  // namespace lmoe
