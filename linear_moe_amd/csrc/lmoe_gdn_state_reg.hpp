// Gated delta rule, forward sequential pass for 2-byte elements with the state held in registers as an MFMA operand.
//
//   per chunk:  X = k S;   Z = beta (v - e^{b} X);   v_new = Tinv Z        ( = u - w S with u = Tinv (v beta), w = Tinv (k beta e^{b}) )
//               o = scale [ e^{b} (q S) + P v_new ];   S' = e^{b_C} S + k^T (e_d v_new)
//
// What bounds a sequential pass on this GPU is the rate at which ONE wave gets LDS reads served (about one wave-wide
// read instruction per 23 cycles, whatever its width; measured), not the matrix cores and not the number of barriers:
// the work of a chunk is therefore laid out so that every operand read from LDS is a single 16-byte read per MFMA, no
// operand is read that can stay in registers, and the reads are spread over four waves.
//   * Consumer wave j (waves 0, 1) owns ALL K rows of the 16 columns 16 j .. of the slice.  An accumulator block holds
//     four rows of one column per lane; two blocks give the 8 contraction elements an MFMA B operand wants, so the
//     state enters  k S  -- and v_new enters  k^T (e_d v_new)  -- straight from the registers the previous product left
//     it in.  For that to fit plain 16-byte row reads of the other operand, accumulator rows are NUMBERED accordingly:
//     block pair (2 s, 2 s + 1), lane group g, element i  <->  index 32 s + 8 g + 4 e + i  (e = block parity).  The row an A
//     operand lane reads (k, Tinv rows) and the columns a transposing read addresses (k^T) follow that numbering;
//     nothing is ever permuted in memory.
//   * w and u are never formed: v_new = Tinv Z costs 6 products (Tinv is lower triangular) on top of X = k S.
//   * Helper wave j (waves 2, 3) forms the output of the same 16 columns from what the consumers leave in LDS anyway
//     (S^T at chunk start, which is the checkpoint the loaders store, and v_new): q S in phase 1, P v_new in phase 2,
//     transposed so that a lane holds four consecutive columns of one token (8-byte writes of o).  
//   * Loader teams as in k_gdn_state_fwd: team 1 stages k(c+1) in phase 1 and carries all stores; team 2
//     stages q, Tinv, v, gates of chunk c+1 in phase 2.
//   * The intra-chunk matrix P = (q k^T) . Gamma is formed here, by the four waves of team 1 in phase 1 (behind their
//     staging of k, where they would otherwise wait for the consumers): the ten 16 x 16 blocks of the lower
//     triangle, three or two per wave, from the q and k tiles and the gate table's b row into the P tile that the
//     helpers read in phase 2.  The WY preparation then reads no q and writes no P, this pass reads none (8 KB per
//     chunk and work-group less through the CU's memory pipe, which bounds it), and a forward-only call never has P
//     in memory.  A call that saves for the backward writes P once: every V-slice work-group stores its share of
//     the rows.  (Formed on the helper waves instead, as registers that feed (P v_new)^T directly, the pass was 45 us
//     slower at T = 8192: 48 more products per chunk on a wave that shares a phase with the consumers.)
#pragma once
#include <type_traits>
#include "lmoe_gdn_state.hpp"

namespace lmoe {

// Time stamps of the traced instance (TRACE = true): every team's leading wave notes the shader clock when it
// arrives at and leaves the two barriers of a chunk and at a few points in between, into LDS (a global store would
// stall the traced wave at the issue); the traced work-group copies them out when it ends.  Slots: 0 consumer wave,
// 1 helper wave, 2 loader team 1, 3 loader team 2; marks per (slot, chunk): see lmoe_trace_gdn_state_fwd in
// include/lmoe.h.  Chunks beyond TRACE_CHUNKS are not recorded.
constexpr int TRACE_CHUNKS = 128, TRACE_MARKS = 8, TRACE_SLOTS = 4;

// A fragment of k^T for the state block mi (see the numbering above): contraction = tokens k0 + 8 g .. + 7 (rows of
// the tile), lane fr <-> state row  32 (mi / 2) + 8 (fr / 4) + 4 (mi % 2) + fr % 4  (columns of the tile)
__device__ __forceinline__ bf16x8 load_frag_t_state(const bf16* tile, int ld, int k0, int mi, int l) {
  const int s = l & 15;
  const bf16* p = tile + (k0 + 8 * (l >> 4) + (s >> 2)) * ld + 32 * (mi >> 1) + 8 * (s & 3) + 4 * (mi & 1);
  typedef __attribute__((address_space(3))) bf16x4 lds_b4;
  const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_b4*)p);
  const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_b4*)(p + 4 * ld));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
// (frag_of_blocks, lmoe_common.hpp: two accumulator blocks -> the 8 contraction elements of an operand)

template <int K, int V, bool SAVE, bool TRACE = false>
__global__ __launch_bounds__(3 * NTHR) void k_gdn_state_fwd_reg(const lmoe_args a, long long* tr, int traced_wg) {
  typedef bf16 T;
  constexpr int BV = 32;
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int KT = K / 16, KS = K / 32;
  // register sets per prefetch ring (deeper rings were measured: 3 and 4 sets for either team change nothing, the pass
  // is bound by what the memory system delivers for its traffic, not by the lead of its requests)
  constexpr int LPA = GdnStateCfg<T>::LPF, LPB = GdnStateCfg<T>::LPF;
  __shared__ __attribute__((aligned(16))) T s_k[2 * CH * LDK];      // k [64][K] of chunks c, c + 1
  __shared__ __attribute__((aligned(16))) T s_q[CH * LDK];          // q [64][K]
  __shared__ __attribute__((aligned(16))) T s_ti[CH * LDC];         // Tinv [64][64]
  __shared__ __attribute__((aligned(16))) T s_p[CH * LDC];          // P [64][64]
  __shared__ __attribute__((aligned(16))) T s_v[CH * LDU];          // v [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[BV * LDK];         // S^T [BV][K] at chunk start
  __shared__ __attribute__((aligned(16))) T s_vn[CH * LDU];         // v_new [64][BV]
  __shared__ __attribute__((aligned(16))) T s_o[CH * LDU];          // o [64][BV]
  __shared__ __attribute__((aligned(16))) float s_f[64], s_be[64];  // beta e^{b}, beta
  __shared__ __attribute__((aligned(16))) float s_b[64];            // cumulative log-decay b
  __shared__ __attribute__((aligned(16))) float s_eb[2][64], s_ed[2][64];
  __shared__ float s_dec[2];                                        // e^{b_C}; buffer c & 1
  __shared__ long long s_tr[TRACE ? TRACE_SLOTS * TRACE_CHUNKS * TRACE_MARKS : 1];
  auto TR = [&](int slot, int c, int mark) {
    if constexpr (TRACE) {
      if ((int)blockIdx.x == traced_wg && (threadIdx.x & 63) == 0 && c < TRACE_CHUNKS)
        s_tr[(slot * TRACE_CHUNKS + c) * TRACE_MARKS + mark] = __builtin_readcyclecounter();
    }
  };
  if constexpr (TRACE) {
    for (int i = threadIdx.x; i < TRACE_SLOTS * TRACE_CHUNKS * TRACE_MARKS; i += 3 * NTHR) s_tr[i] = 0;
    __syncthreads();
  }

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
  const SeqInfo sq = seq_info(a, n);
  const int l = lane_id();
  const int team = threadIdx.x / NTHR;
  if (sq.nchunks == 0) {
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
    struct PreA { typename IOK::Regs rk; int len; };
    PreA pa[LPA];
    auto issue_a = [&](PreA& P, int c) {      // always issued, chunk index clamped (see k_gdn_state_fwd)
      c = min(c, sq.nchunks - 1);
      const int tok = sq.tok0 + c * CH;
      P.len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rk, row_ptr<T>(a.k, sq.b, tok, h), a.k.st, P.len);
    };
    auto stage_k = [&](PreA& P, int c) {
      IOK::mask(P.rk, P.len);
      IOK::store_lds(P.rk, s_k + (c & 1) * CH * LDK, LDK);
    };
    // this work-group's share of the rows of P (formed below, the whole matrix in s_p): 64 / NVS rows, every
    // thread stores (threads beyond the share repeat a row with the same bytes: no store sits behind a branch)
    constexpr int PROWS = CH / NVS;
    const int pidx = (threadIdx.x & (NTHR - 1)) % (PROWS * 8);
    const int prow = vsl * PROWS + pidx / 8, pcol = (pidx % 8) * 8;
    auto store_result = [&](const typename IOV::Regs& r, const lmoe_tensor& dst, int c) {
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      IOV::template store_global<true>(r, row_ptr<T>(dst, sq.b, tok, h) + v0, dst.st, len);
    };
    // P = (q k^T) . Gamma of the chunk in the tiles, Gamma_ij = e^{b_i - b_j} for i >= j (rows past the end of a
    // partial chunk: 0; its columns are zero through k): block number x = wave, wave + 4, wave + 8 of the ten blocks
    // (ti, tj <= ti) of the lower triangle, formed transposed (k rows as the A operand) so that a lane holds four
    // consecutive columns of one row (8-byte writes).  The six blocks above the diagonal are cleared once.
    const int wt = wave_id() - 4;
    auto form_p = [&](int c) {
      const int fr = l & 15, g = l >> 4;
      const T* s_kc = s_k + (c & 1) * CH * LDK;
      const int len = min(CH, sq.len - c * CH);
      int ti[3], tj[3];
#pragma unroll
      for (int x = 0; x < 3; ++x) {
        const int idx = min(wt + 4 * x, 9);
        ti[x] = idx >= 6 ? 3 : idx >= 3 ? 2 : idx >= 1 ? 1 : 0;
        tj[x] = idx - ti[x] * (ti[x] + 1) / 2;
      }
      const int nx = wt < 2 ? 3 : 2;        // wave-uniform
      f32x4 pc[3];
#pragma unroll
      for (int x = 0; x < 3; ++x) pc[x] = f32x4{0.f, 0.f, 0.f, 0.f};
      typename ET<T>::frag fq[2][3], fk[2][3];
      auto fetch = [&](int ks, int buf) {
#pragma unroll
        for (int x = 0; x < 3; ++x) {
          fq[buf][x] = ET<T>::load_frag(s_q + (16 * ti[x] + fr) * LDK + 32 * ks + 8 * g);
          fk[buf][x] = ET<T>::load_frag(s_kc + (16 * tj[x] + fr) * LDK + 32 * ks + 8 * g);
        }
      };
      fetch(0, 0);
      // the decay factors (masked) while the first fragments are on their way: behind the products only a multiply,
      // a conversion and the write are left
      f32x4 gm[3];
#pragma unroll
      for (int x = 0; x < 3; ++x) {
        const int i = 16 * ti[x] + fr, j0 = 16 * tj[x] + 4 * g;
        const float bi = s_b[i];
        const f32x4 bj = *(const f32x4*)&s_b[j0];
#pragma unroll
        for (int e = 0; e < 4; ++e) gm[x][e] = (i >= j0 + e && i < len) ? texp<T>(bi - bj[e]) : 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + 1 < KS) fetch(ks + 1, (ks + 1) & 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int x = 0; x < 3; ++x)
          if (x < nx) ET<T>::mma(pc[x], fk[ks & 1][x], fq[ks & 1][x]);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int x = 0; x < 3; ++x) {
        if (x < nx) {
          const int i = 16 * ti[x] + fr, j0 = 16 * tj[x] + 4 * g;
          bf16x4 y;
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] = (bf16)(pc[x][e] * gm[x][e]);
          *(bf16x4*)(s_p + i * LDC + j0) = y;
        }
      }
    };
    {
      const int t = threadIdx.x & (NTHR - 1), r = t >> 4, cc = t & 15;
#pragma unroll
      for (int I = 0; I < 3; ++I)
#pragma unroll
        for (int J = I + 1; J < 4; ++J) s_p[(16 * I + r) * LDC + 16 * J + cc] = (T)0.f;
    }
#pragma unroll
    for (int j = 0; j < LPA; ++j) issue_a(pa[j], j);
    wait_all_loads();
    stage_k(pa[0], 0);
    lds_barrier();                                                                       // B0
    typename IOHT::Regs rh;
    typename IOV::Regs rvn, ro;
    ring_loop<LPA>(sq.nchunks, [&](auto slot, const int c) {
      constexpr int j = decltype(slot)::value, jn = (j + 1) % LPA;
      if (wave_id() == 4) TR(2, c, 0);
      lds_barrier();                                                                     // B1
      if (wave_id() == 4) TR(2, c, 1);
      stage_k(pa[jn], c + 1);               // (past the last chunk: a clamped copy of it, never used)
      if constexpr (SAVE) IOHT::load_lds(rh, s_hT, LDK);
      IOV::load_lds(ro, s_o, LDU);
      if (wave_id() == 4) TR(2, c, 6);
      // behind the staging: the first thousand cycles after the barrier every wave of the work-group reads LDS and
      // a read of this team's takes that long to come back (measured: formed first, P was ready 250 cycles later
      // and k staged 600 cycles later than in this order)
      form_p(c);
      if (wave_id() == 4) TR(2, c, 2);
      lds_barrier();                                                                     // B2
      if (wave_id() == 4) TR(2, c, 3);
      if constexpr (SAVE) {
        IOV::load_lds(rvn, s_vn, LDU);
        const typename ET<T>::vec pv = *(const typename ET<T>::vec*)(s_p + prow * LDC + pcol);
        IOHT::template store_global<true>(rh, (T*)a.hs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
        __builtin_nontemporal_store(pv, (typename ET<T>::vec*)((T*)a.pmat + (((int64_t)(sq.chunk0 + c) * a.H + h) * CH + prow) * CH + pcol));
      }
      if (c > 0) store_result(ro, a.o, c - 1);
      if constexpr (SAVE) IOV::template store_global<true>(rvn, slice_ptr<T>(a.vnew, sq.chunk0 + c, h, a.H, V, v0), SLICE_COLS, min(CH, sq.len - c * CH));
      if (wave_id() == 4) TR(2, c, 4);
      issue_a(pa[j], c + LPA);
      if (wave_id() == 4) TR(2, c, 5);
    });
    lds_barrier();                                                                       // o of the last chunk
    IOV::load_lds(ro, s_o, LDU);
    store_result(ro, a.o, sq.nchunks - 1);
    if constexpr (TRACE) {
      if ((int)blockIdx.x == traced_wg)
        for (int i = threadIdx.x & (NTHR - 1); i < TRACE_SLOTS * TRACE_CHUNKS * TRACE_MARKS; i += NTHR) tr[i] = s_tr[i];
    }
    return;
  }
  if (team == 2) {
    // ------------------------- loaders, ring B (q, Tinv, v, gates) ------------------------
    struct PreB { typename IOK::Regs rq; typename IOP::Regs rt; typename IOV::Regs rv; float eb, ed, be, f, bb; int len; };
    PreB pb[LPB];
    auto issue_b = [&](PreB& P, int c) {
      c = min(c, sq.nchunks - 1);
      const int tok = sq.tok0 + c * CH;
      P.len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rq, row_ptr<T>(a.q, sq.b, tok, h), a.q.st, P.len);
      IOP::load_nomask(P.rt, (const T*)a.tinv + ((int64_t)(sq.chunk0 + c) * a.H + h) * CH * CH, CH, CH);
      IOV::load_nomask(P.rv, row_ptr<T>(a.v, sq.b, tok, h) + v0, a.v.st, P.len);
      const float* gc = a.gcum + ((int64_t)(sq.chunk0 + c) * a.H + h) * GATE_ROWS * CH;
      P.eb = gc[l];
      P.ed = gc[CH + l];
      P.be = gc[2 * CH + l];
      P.f = gc[3 * CH + l];
      P.bb = gc[4 * CH + l];
    };
    auto stage_b = [&](PreB& P, int buf) {
      IOK::store_lds(P.rq, s_q, LDK);       // rows past the end only reach output rows that are not stored
      IOP::store_lds(P.rt, s_ti, LDC);
      if (a.v_act) {                         // v = silu(v as given): the activation in front of the op, applied here
#pragma unroll
        for (int p = 0; p < IOV::PASSES; ++p)
#pragma unroll
          for (int i = 0; i < IOV::VEC; ++i) P.rv.v[p][i] = ET<T>::from_f(silu_of(ET<T>::to_f(P.rv.v[p][i])));
      }
      IOV::mask(P.rv, P.len);
      IOV::store_lds(P.rv, s_v, LDU);
      if (wave_id() == 8) {
        s_be[l] = P.be;
        s_f[l] = P.f;
        s_b[l] = P.bb;
        s_eb[buf][l] = P.eb;
        s_ed[buf][l] = P.ed;
        if (l == 63) s_dec[buf] = P.eb;
      }
    };
#pragma unroll
    for (int j = 0; j < LPB; ++j) issue_b(pb[j], j);
    wait_all_loads();
    stage_b(pb[0], 0);
    lds_barrier();                                                                       // B0
    ring_loop<LPB>(sq.nchunks, [&](auto slot, const int c) {
      constexpr int j = decltype(slot)::value, jn = (j + 1) % LPB;
      if (wave_id() == 8) TR(3, c, 0);
      lds_barrier();                                                                     // B1
      if (wave_id() == 8) TR(3, c, 1);
      issue_b(pb[j], c + LPB);              // chunk c was staged before this barrier: refill its set
      if (wave_id() == 8) TR(3, c, 2);
      lds_barrier();                                                                     // B2
      if (wave_id() == 8) TR(3, c, 3);
      if (c + 1 < sq.nchunks) stage_b(pb[jn], (c + 1) & 1);
      if (wave_id() == 8) TR(3, c, 4);
    });
    lds_barrier();
    return;
  }

  const int wv = wave_id();
  const int fr = l & 15, g = l >> 4;
  const float scale = a.scale;
  if (wv >= 2) {
    // ------------------------------ helpers: the output ----------------------------------
    const int j = wv - 2;
    lds_barrier();                                                                       // B0
    for (int c = 0; c < sq.nchunks; ++c) {
      const int cur = c & 1;
      if (wv == 2) TR(1, c, 0);
      lds_barrier();                                                                     // B1
      if (wv == 2) TR(1, c, 1);
      // (q S)^T: rows = columns of the slice (S^T as the A operand, read from the checkpoint tile), columns = tokens
      f32x4 oa[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) oa[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      {
        typename ET<T>::frag fs[KS], fq[2][4];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fs[ks] = ET<T>::load_frag(s_hT + (16 * j + fr) * LDK + 32 * ks + 8 * g);
#pragma unroll
        for (int t = 0; t < 4; ++t) fq[0][t] = ET<T>::load_frag(s_q + (16 * t + fr) * LDK + 8 * g);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          if (ks + 1 < KS) {
#pragma unroll
            for (int t = 0; t < 4; ++t) fq[(ks + 1) & 1][t] = ET<T>::load_frag(s_q + (16 * t + fr) * LDK + 32 * (ks + 1) + 8 * g);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int t = 0; t < 4; ++t) ET<T>::mma(oa[t], fs[ks], fq[ks & 1][t]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) oa[t] *= s_eb[cur][16 * t + fr];
      if (wv == 2) TR(1, c, 2);
      lds_barrier();                                                                     // B2
      if (wv == 2) TR(1, c, 3);
      {
        // + (P v_new)^T: v_new^T through transposing reads of the tile the consumers wrote; P is lower triangular
        typename ET<T>::frag fv[2], fp[6];
#pragma unroll
        for (int s = 0; s < 2; ++s) fv[s] = ET<T>::load_frag_t(s_vn, LDU, 32 * s, 16 * j, l);
        fp[0] = ET<T>::load_frag(s_p + (0 + fr) * LDC + 8 * g);
        fp[1] = ET<T>::load_frag(s_p + (16 + fr) * LDC + 8 * g);
        fp[2] = ET<T>::load_frag(s_p + (32 + fr) * LDC + 8 * g);
        fp[3] = ET<T>::load_frag(s_p + (48 + fr) * LDC + 8 * g);
        fp[4] = ET<T>::load_frag(s_p + (32 + fr) * LDC + 32 + 8 * g);
        fp[5] = ET<T>::load_frag(s_p + (48 + fr) * LDC + 32 + 8 * g);
        __builtin_amdgcn_sched_barrier(0);
        ET<T>::mma(oa[0], fv[0], fp[0]);
        ET<T>::mma(oa[1], fv[0], fp[1]);
        ET<T>::mma(oa[2], fv[0], fp[2]);
        ET<T>::mma(oa[3], fv[0], fp[3]);
        ET<T>::mma(oa[2], fv[1], fp[4]);
        ET<T>::mma(oa[3], fv[1], fp[5]);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        oa[t] *= scale;
        acc_to_lds_t<T>(oa[t], s_o, LDU, 16 * j, 16 * t, l);                             // o [token][column]: 8-byte writes
      }
      if (wv == 2) TR(1, c, 4);
    }
    lds_barrier();
    return;
  }

  // --------------------------------- consumers: the chain ---------------------------------
  __builtin_amdgcn_s_setprio(3);
  const int j = wv;
  const int vc = v0 + 16 * j + fr;                   // the column of this lane
  // row of the state / token of a token-row block that accumulator element i of block m holds in this lane
  auto idx_of = [&](int m, int i) { return 32 * (m >> 1) + 8 * g + 4 * (m & 1) + i; };
  // row an A-operand lane reads for block m of a token-row product
  auto arow_of = [&](int m) { return 32 * (m >> 1) + 4 * (m & 1) + 8 * (fr >> 2) + (fr & 3); };
  f32x4 S[KT];
#pragma unroll
  for (int mi = 0; mi < KT; ++mi) S[mi] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (a.h0) {
    const float* h0 = a.h0 + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < KT; ++mi)
#pragma unroll
      for (int i = 0; i < 4; ++i) S[mi][i] = h0[(int64_t)idx_of(mi, i) * V + vc];
  }
  auto put_state = [&]() {                           // S^T [column][K]: four consecutive rows per lane and block
#pragma unroll
    for (int mi = 0; mi < KT; ++mi) {
      bf16x4 x;
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = (bf16)S[mi][i];
      *(bf16x4*)(s_hT + (16 * j + fr) * LDK + idx_of(mi, 0)) = x;
    }
  };
  put_state();
  lds_barrier();                                                                         // B0
  for (int c = 0; c < sq.nchunks; ++c) {
    const int cur = c & 1;
    const T* s_kc = s_k + cur * CH * LDK;
    typename ET<T>::frag bS[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) bS[ks] = frag_of_blocks(S[2 * ks], S[2 * ks + 1]);
    if (wv == 0) TR(0, c, 0);
    lds_barrier();                                                                       // B1
    if (wv == 0) TR(0, c, 1);
    // X = k S
    f32x4 X[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) X[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    typename ET<T>::frag fv[2], fti[6];
    f32x4 be[2][2], ff[2][2];
    {
      typename ET<T>::frag fk[2][4];
#pragma unroll
      for (int t = 0; t < 4; ++t) fk[0][t] = ET<T>::load_frag(s_kc + arow_of(t) * LDK + 8 * g);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + 1 < KS) {
#pragma unroll
          for (int t = 0; t < 4; ++t) fk[(ks + 1) & 1][t] = ET<T>::load_frag(s_kc + arow_of(t) * LDK + 32 * (ks + 1) + 8 * g);
        } else {
          // what follows the product, requested while it runs: v^T, beta, beta e^{b}, and the six Tinv fragments
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            fv[s] = ET<T>::load_frag_t(s_v, LDU, 32 * s, 16 * j, l);
            be[s][0] = *(const f32x4*)&s_be[32 * s + 8 * g]; be[s][1] = *(const f32x4*)&s_be[32 * s + 8 * g + 4];
            ff[s][0] = *(const f32x4*)&s_f[32 * s + 8 * g]; ff[s][1] = *(const f32x4*)&s_f[32 * s + 8 * g + 4];
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) fti[t] = ET<T>::load_frag(s_ti + arow_of(t) * LDC + 8 * g);
          fti[4] = ET<T>::load_frag(s_ti + arow_of(2) * LDC + 32 + 8 * g);
          fti[5] = ET<T>::load_frag(s_ti + arow_of(3) * LDC + 32 + 8 * g);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t) ET<T>::mma(X[t], fk[ks & 1][t], bS[ks]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (wv == 0) TR(0, c, 5);
    // Z = beta v - (beta e^{b}) X  (8 tokens of this lane's column per 32-token step), then v_new = Tinv Z
    typename ET<T>::frag Z[2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          Z[s][4 * e + i] = (bf16)(be[s][e][i] * (float)fv[s][4 * e + i] - ff[s][e][i] * X[2 * s + e][i]);
    f32x4 vn[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) vn[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    ET<T>::mma(vn[0], fti[0], Z[0]);
    ET<T>::mma(vn[1], fti[1], Z[0]);
    ET<T>::mma(vn[2], fti[2], Z[0]);
    ET<T>::mma(vn[3], fti[3], Z[0]);
    ET<T>::mma(vn[2], fti[4], Z[1]);
    ET<T>::mma(vn[3], fti[5], Z[1]);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      uint32_t xb[4], nb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // v_new rounded once to the storage type: the state update, the output and the backward see the same values
        const bf16 x = (bf16)vn[t][i];
        vn[t][i] = (float)x;
        xb[i] = (uint32_t)__builtin_bit_cast(uint16_t, x);
      }
      // v_new [token][column] for the helpers and the loaders: neighbouring lanes hold neighbouring columns of the same
      // four tokens; they swap (quad permutation 1 0 3 2), the even lane writes tokens 0, 1 and the odd lane tokens
      // 2, 3 of the pair of columns as whole 32-bit words
#pragma unroll
      for (int i = 0; i < 4; ++i) nb[i] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)xb[i], 0xB1, 0xf, 0xf, false);
      const bool odd = fr & 1;
      const uint32_t w0 = odd ? (nb[2] | (xb[2] << 16)) : (xb[0] | (nb[0] << 16));
      const uint32_t w1 = odd ? (nb[3] | (xb[3] << 16)) : (xb[1] | (nb[1] << 16));
      uint32_t* dst = (uint32_t*)(s_vn + idx_of(t, odd ? 2 : 0) * LDU + 16 * j + (fr & ~1));
      dst[0] = w0;
      dst[LDU / 2] = w1;
    }
    const float dec = s_dec[cur];
    // the k^T fragments of the first half of the update do not depend on this chunk's results
    typename ET<T>::frag fkt[KT];
#pragma unroll
    for (int mi = 0; mi < KT; ++mi) fkt[mi] = load_frag_t_state(s_kc, LDK, 0, mi, l);
    f32x4 ed[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s) { ed[s][0] = *(const f32x4*)&s_ed[cur][32 * s + 8 * g]; ed[s][1] = *(const f32x4*)&s_ed[cur][32 * s + 8 * g + 4]; }
    if (wv == 0) TR(0, c, 2);
    lds_barrier();                                                                       // B2
    if (wv == 0) TR(0, c, 3);
#pragma unroll
    for (int mi = 0; mi < KT; ++mi) S[mi] *= dec;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      typename ET<T>::frag bvd;
#pragma unroll
      for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int i = 0; i < 4; ++i) bvd[4 * e + i] = (bf16)(vn[2 * s + e][i] * ed[s][e][i]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mi = 0; mi < KT; ++mi) ET<T>::mma(S[mi], fkt[mi], bvd);
      __builtin_amdgcn_sched_barrier(0);
      if (s == 0) {
#pragma unroll
        for (int mi = 0; mi < KT; ++mi) fkt[mi] = load_frag_t_state(s_kc, LDK, 32, mi, l);
      }
    }
    if (wv == 0) TR(0, c, 6);
    put_state();                                      // the state at the start of the next chunk
    if (wv == 0) TR(0, c, 4);
  }
  lds_barrier();                                                                         // results of the last chunk
  if (a.ht) {
    float* ht = a.ht + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int mi = 0; mi < KT; ++mi)
#pragma unroll
      for (int i = 0; i < 4; ++i) ht[(int64_t)idx_of(mi, i) * V + vc] = S[mi][i];
  }
}

}  // namespace lmoe
