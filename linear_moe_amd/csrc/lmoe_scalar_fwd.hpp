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
// state pass + output (forward), fp32 elements (the parity path): work-group of three teams of four waves
// (768 threads); the LDS holds one operand buffer, so a chunk costs three barriers.  k_state_fwd_b below is the pass
// for 2-byte elements.
//   grid = ceil(N*H / 8) * 8 * (V / BV) work-groups (1-D).  Work-group -> (sequence, head,
//   V-slice): the V-slices of one (sequence, head) get ids that are congruent mod 8, i.e. run on
//   the same XCD and share q, k through its L2.
//   Team 0 (waves 0-3, consumers) carries the dependency chain of the state and nothing else:
//        S -> LDS (element type T) | B1 | S = e^{b_C} S + k^T (e_d v) | B2
//     wave w owns state rows [w*K/4, (w+1)*K/4) x BV columns in fp32 MFMA accumulators; the row
//     scaling e_d is applied to the v fragments in registers, so k is staged unscaled.
//   Team 1 (waves 4-7, loaders) keeps the operands of the next PF chunks in flight in registers,
//     forms the gate cumsum, fills the LDS buffer and writes hs (layout [V][K]) from the
//     LDS copy of S (SAVE; a forward-only call passes hs = NULL and nothing is written).
//   Team 2 (waves 8-11, output) forms the chunk's output rows 16w.. between B1 and B2: e^{b_i} q S, its rows of
//     P = (q k^T) . Gamma (through a wave-private LDS strip) and P v; the rows are stored after B2.
//   All teams meet at the same barriers; three waves per SIMD hide each other's latencies.
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV, bool SAVE>
__global__ __launch_bounds__(3 * NTHR) void k_state_fwd(const lmoe_args a) {
  static_assert(sizeof(T) == 4, "fp32 elements; 2-byte elements: k_state_fwd_b");
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16;
  __shared__ __attribute__((aligned(16))) T s_k[1][CH * LDK];              // k             [64][K]
  __shared__ __attribute__((aligned(16))) T s_q[1][CH * LDK];              // q             [64][K]
  __shared__ __attribute__((aligned(16))) T s_u[1][CH * LDU];              // u or v        [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[BV * LDK];                   // S^T           [BV][K]
  __shared__ __attribute__((aligned(16))) T s_pst[4 * 16 * LDC];              // team 2: P strips
  __shared__ __attribute__((aligned(16))) T s_ost[4 * 16 * LDU];              // team 2: o store
  __shared__ __attribute__((aligned(16))) float s_b[1][64], s_eb[1][64], s_ed[1][64];
  __shared__ float s_dec[1];                                               // e^{b_C} per buffer

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
        // hs[chunk][h][v0 .. v0+BV][K] <- S^T (only the backward reads it: SAVE = false for forward-only calls)
        if constexpr (SAVE)
          IOHT::lds_to_global(s_hT, LDK, (T*)a.hs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
        lds_barrier();                                                                   // B2
        lds_barrier();                                                                   // B3: buffer read
        if (c + 1 < sq.nchunks) stage(pre[(j + 1) % PF], 0);
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
      constexpr int cur = 0;
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      lds_barrier();                                                                     // B1
      // Everything of output rows 16 ow .. happens in this window, where the consumers only update the state:
      // e^{b} q S, the rows of P = (q k^T) . Gamma (blocks above the diagonal are zero and skipped), and P v.
      const int fr = l & 15;
      // looped products, P through this wave's own LDS strip
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
      lds_barrier();                                                                     // B2
      store_strip<T, NB>(o, s_ost + ow * 16 * LDU, row_ptr<T>(a.o, sq.b, tok + 16 * ow, h) + v0, a.o.st,
                         len - 16 * ow, a.scale);
      lds_barrier();                                                                     // B3
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
    constexpr int cur = 0;
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
    lds_barrier();                                                                       // B3
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
// The same pass for 2-byte elements, one barrier per chunk: whatever a window reads was completed in the window
// before.  Two operand buffers (chunk c + 1 is complete, chunk c + 2 is being staged over chunk c, whose operands the
// waves already hold in registers), two copies of S^T and two of P = (q k^T) . Gamma.  Window c, between barrier c and
// barrier c + 1:
//   consumers: S = e^{b_C} S + k^T (e_d v) on fragments of chunk c read before the barrier, S -> s_hT[(c + 1) & 1],
//              then the blocks of P of chunk c + 1 below the diagonal -> s_P[(c + 1) & 1] (the output team, which
//              formed its rows of P itself in an earlier version, was the longest chain of the window), then the
//              fragments of chunk c + 1 for the next update
//   loaders:   loads of chunk c + 4 issued into the register set that the last window's staging freed, chunk c + 2
//              staged into buffer c & 1, hs <- s_hT[c & 1] (SAVE)
//   output:    rows 16 w .. of o = e^b q S (s_hT[c & 1]) + P (s_P[c & 1]) v on q rows and v fragments read before
//              the barrier, stored from registers, then the q rows and v fragments of chunk c + 1 and, from those q
//              rows, the diagonal blocks of P of chunk c + 1
// A chunk's own operands are staged two windows before its window: what is read of them is read at the end of the
// window before, when the LDS is quiet, and their buffer is free for the chunk after the next one as the window
// opens.  Behind the barrier, where all twelve waves ask for data at once and a read takes about a thousand cycles
// to return, only S^T and P (written in the window before) are left to read.
// Time stamps of the traced instance (TRACE = true): one wave of each team notes the shader clock where it arrives
// at and leaves the barrier of a chunk and at a few points in between; the stamps sit in LDS (a global store
// per stamp would perturb the wave that is measured) and each of those waves copies its own out at the end:
// tr[slot][chunk][mark], slots 0 consumers, 1 loaders, 2 output team; marks: include/lmoe.h.
// ------------------------------------------------------------------------- //
constexpr int SFWD_TRACE_CHUNKS = 24, SFWD_TRACE_MARKS = 8, SFWD_TRACE_SLOTS = 3;

// NORM (ungated calls): the output leaves divided by den + eps (lmoe_args.normalize = 1; 2: undivided, with den handed
// out beside it for a caller that adds the den of several key blocks first), den_i = scale q_i . (sum of the keys up to i) - the
// op with one more value column of ones, carried beside the state as one more accumulator column (z = the sum of the
// keys of the chunks before, fp32 in LDS and, for the backward, in zs) and formed by every V slice for itself:
// consumers z += k^T 1, output team q z and the row sums of P as two more products against a fragment of ones.
template <typename T, int K, int V, int BV, bool SAVE, bool TRACE = false, bool NORM = false>
__global__ __launch_bounds__(3 * NTHR) void k_state_fwd_b(const lmoe_args a, long long* tr, int traced_wg) {
  static_assert(sizeof(T) == 2, "2-byte elements");
  static_assert(!(NORM && TRACE), "the traced instance is the plain pass");
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16, KS = K / 32, CS = CH / 32;
  __shared__ __attribute__((aligned(16))) T s_k[2][CH * LDK];                 // k             [64][K]
  __shared__ __attribute__((aligned(16))) T s_q[2][CH * LDK];                 // q             [64][K]
  __shared__ __attribute__((aligned(16))) T s_u[2][CH * LDU];                 // v             [64][BV]
  __shared__ __attribute__((aligned(16))) T s_hT[2][BV * LDK];                // S^T           [BV][K]
  __shared__ __attribute__((aligned(16))) T s_P[2][CH * LDC];                 // P             [64][64]
  __shared__ __attribute__((aligned(16))) float s_b[2][64], s_eb[2][64], s_ed[2][64];
  __shared__ float s_dec[2];                                                  // e^{b_C} per buffer
  __shared__ __attribute__((aligned(16))) float s_z[NORM ? 2 : 1][NORM ? K : 4];   // NORM: the sum of the keys before a chunk
  // (the low 32 bits of the clock: whoever reads the stamps takes their differences modulo 2^32)
  __shared__ uint32_t s_tr[TRACE ? SFWD_TRACE_SLOTS * SFWD_TRACE_CHUNKS * SFWD_TRACE_MARKS : 1];
  auto TR = [&](int slot, int c, int mark) {
    if constexpr (TRACE) {
      if ((int)blockIdx.x == traced_wg && (threadIdx.x & 63) == 0 && c < SFWD_TRACE_CHUNKS)
        s_tr[(slot * SFWD_TRACE_CHUNKS + c) * SFWD_TRACE_MARKS + mark] = (uint32_t)__builtin_readcyclecounter();
    }
  };
  auto trace_out = [&](int slot) {       // by the wave that wrote the slot: ordering inside the wave is enough
    if constexpr (TRACE) {
      if ((int)blockIdx.x == traced_wg) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        constexpr int N = SFWD_TRACE_CHUNKS * SFWD_TRACE_MARKS;
        for (int i = threadIdx.x & 63; i < N; i += 64) tr[slot * N + i] = s_tr[slot * N + i];
      }
    }
  };
  if constexpr (TRACE) {
    for (int i = threadIdx.x; i < SFWD_TRACE_SLOTS * SFWD_TRACE_CHUNKS * SFWD_TRACE_MARKS; i += 3 * NTHR) s_tr[i] = 0;
    __syncthreads();
  }

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
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

  // Blocks (ti, tj[0 .. n)) of P of chunk c (16 x 16 each, one q strip against n <= 2 k strips), formed transposed so
  // that a lane holds four consecutive columns of one row (8-byte writes).  The ten blocks on and below the diagonal
  // are dealt to eight waves: the output team takes the diagonal (wave w: block (w, w), p_diag) once its rows are
  // stored, the consumers the six blocks below it (waves 0, 1: rows 3, 2 against k strips 0, 1; wave 2: (3, 2); wave 3: (1, 0)).
  // Every fragment is requested before the first product: the LDS is busiest right behind the barrier, a read comes
  // back after several hundred cycles, and a product loop that requests one step ahead pays that once per step.
  auto p_blocks = [&](int c, int ti, int tja, int tjb, int n) {
    const int cb = c & 1, fr = l & 15, g = l >> 4;
    const T *qc = s_q[cb], *kc = s_k[cb];
    T* Pn = s_P[c & 1];
    typename ET<T>::frag fq[KS], fka[KS], fkb[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      fq[ks] = ET<T>::load_frag(qc + (16 * ti + fr) * LDK + 32 * ks + 8 * g);
      fka[ks] = ET<T>::load_frag(kc + (16 * tja + fr) * LDK + 32 * ks + 8 * g);
      if (n == 2) fkb[ks] = ET<T>::load_frag(kc + (16 * tjb + fr) * LDK + 32 * ks + 8 * g);
    }
    // the decay factors (masked: only the diagonal block has entries above the diagonal) while the fragments are on
    // their way
    const int i = 16 * ti + fr;
    const float bi = s_b[cb][i];
    const f32x4 bja = *(const f32x4*)&s_b[cb][16 * tja + 4 * g], bjb = *(const f32x4*)&s_b[cb][16 * tjb + 4 * g];
    f32x4 ga, gb;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ga[e] = (i >= 16 * tja + 4 * g + e) ? texp<T>(bi - bja[e]) : 0.f;
      gb[e] = texp<T>(bi - bjb[e]);
    }
    f32x4 pa = {0.f, 0.f, 0.f, 0.f}, pb = {0.f, 0.f, 0.f, 0.f};
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      ET<T>::mma(pa, fka[ks], fq[ks]);
      if (n == 2) ET<T>::mma(pb, fkb[ks], fq[ks]);
    }
    __builtin_amdgcn_sched_barrier(0);
    bf16x4 y;
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = (bf16)(pa[e] * ga[e]);
    *(bf16x4*)(Pn + i * LDC + 16 * tja + 4 * g) = y;
    if (n == 2) {
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = (bf16)(pb[e] * gb[e]);
      *(bf16x4*)(Pn + i * LDC + 16 * tjb + 4 * g) = y;
    }
  };

  if (team == 1) {
    // --------------------------------- loaders -------------------------------------------
    struct Pre { typename IOK::Regs rk, rq; typename IOV::Regs ru; uint32_t graw; int len; };
    Pre pre[3];                                              // register set = chunk % 3
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
      IOV::load_nomask(P.ru, row_ptr<T>(a.v, sq.b, tok, h) + v0, a.v.st, len);
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
      if (wave == 4) {
        const float x = wave_incl_scan((gated && l < P.len) ? scalar_from_raw(P.graw, a.g_dtype) : 0.f);
        const float xl = __shfl(x, 63, 64);
        s_b[buf][l] = x;
        s_eb[buf][l] = expf(x);
        s_ed[buf][l] = expf(xl - x);
        if (l == 0) s_dec[buf] = expf(xl);
      }
    };
    // hs[chunk][h][v0 .. v0+BV][K] <- S^T (only the backward reads it: SAVE = false for forward-only calls)
    auto save_state = [&](int c) {
      if constexpr (SAVE) {
        T* hs = (T*)a.hs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K;
        // a wide slice of a 128-wide key has few registers left beside three register sets in flight: a quarter of
        // the rows at a time there
        constexpr int RS = (BV >= 64 && K >= 128) ? BV / 4 : BV;
#pragma unroll
        for (int r0 = 0; r0 < BV; r0 += RS) {
          if constexpr (RS < BV) __builtin_amdgcn_sched_barrier(0);
          TileIO<T, RS, K>::lds_to_global(s_hT[c & 1] + r0 * LDK, LDK, hs + r0 * K, K, RS);
        }
      }
    };
#pragma unroll
    for (int j = 0; j < 3; ++j) issue(pre[j], j);
    stage(pre[0], 0);
    issue(pre[0], 3);
    stage(pre[1], 1);
    {
      // blocks of P above the diagonal: zero, and never written again
      const int t = threadIdx.x & (NTHR - 1), r = t >> 4, cc = t & 15;
#pragma unroll
      for (int I = 0; I < 3; ++I)
#pragma unroll
        for (int J = I + 1; J < 4; ++J) {
          s_P[0][(16 * I + r) * LDC + 16 * J + cc] = (T)0.f;
          s_P[1][(16 * I + r) * LDC + 16 * J + cc] = (T)0.f;
        }
    }
    lds_barrier();                                                                       // chunks 0, 1 staged
    for (int c0 = 0; c0 < sq.nchunks; c0 += 3) {
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int c = c0 + j;
        if (c >= sq.nchunks) break;
        if (wave == 4) TR(1, c, 0);
        lds_barrier();
        if (wave == 4) TR(1, c, 1);
        // (both always: past the end it is the last chunk again, never consumed)
        issue(pre[(j + 1) % 3], c + 4);
        if (wave == 4) TR(1, c, 5);
        stage(pre[(j + 2) % 3], c & 1);          // chunk c + 2 takes the buffer of chunk c
        if (wave == 4) TR(1, c, 2);
        save_state(c);
        if (wave == 4) TR(1, c, 4);
      }
    }
    if (wave == 4) trace_out(1);
    return;
  }

  if (team == 2) {
    // --------------------------------- output --------------------------------------------
    const int ow = wave - 8;
    const int fr = l & 15, fg = 8 * (l >> 4), g4 = 4 * (l >> 4);
    lds_barrier();                                                                       // chunks 0, 1 staged
    // What the window of a chunk reads of its own operand buffer - the q rows, the v^T fragments, the gate factor -
    // was staged two windows earlier: it is read at the end of the window before, when the LDS is quiet, and not in
    // the rush behind the barrier, where only S^T and P (written in the window before) are left to read.
    typename ET<T>::frag fq[KS], fv[CS][NB];
    float ebi;
    auto preread = [&](int c) {
      const int cb = c & 1;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) fq[ks] = ET<T>::load_frag(s_q[cb] + (16 * ow + fr) * LDK + 32 * ks + fg);
#pragma unroll
      for (int kq = 0; kq < CS; ++kq) {
        if (2 * kq <= ow) {          // tokens j >= 32 only reach the rows of waves 2, 3
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) fv[kq][ni] = ET<T>::load_frag_t(s_u[cb], LDU, 32 * kq, 16 * ni, l);
        }
      }
      ebi = s_eb[cb][16 * ow + fr];
    };
    // the diagonal block (ow, ow) of P of chunk c from the q rows that preread(c) has just fetched
    auto p_diag = [&](int c) {
      const int cb = c & 1, g = l >> 4;
      typename ET<T>::frag fk[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) fk[ks] = ET<T>::load_frag(s_k[cb] + (16 * ow + fr) * LDK + 32 * ks + fg);
      const int i = 16 * ow + fr;
      const float bi = s_b[cb][i];
      const f32x4 bj = *(const f32x4*)&s_b[cb][16 * ow + 4 * g];
      f32x4 gm, pa = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int e = 0; e < 4; ++e) gm[e] = (fr >= 4 * g + e) ? texp<T>(bi - bj[e]) : 0.f;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) ET<T>::mma(pa, fk[ks], fq[ks]);
      __builtin_amdgcn_sched_barrier(0);
      bf16x4 y;
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = (bf16)(pa[e] * gm[e]);
      *(bf16x4*)(s_P[c & 1] + i * LDC + 16 * ow + 4 * g) = y;
    };
    preread(0);
    p_diag(0);
    for (int c = 0; c < sq.nchunks; ++c) {
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      if (ow == 0) TR(2, c, 0);
      lds_barrier();
      if (ow == 0) TR(2, c, 1);
      // Both products are formed transposed (the MFMA operands swapped), so that a lane holds four consecutive
      // columns of ONE token and the result leaves as 8-byte stores.  Every fragment is requested before the first
      // product (left to the compiler, each read is waited for where it is used and the window is a chain of LDS
      // round trips).
      typename ET<T>::frag fh[KS][NB], fp[CS];
      const T *Pc = s_P[c & 1], *hT = s_hT[c & 1];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) fh[ks][ni] = ET<T>::load_frag(hT + (16 * ni + fr) * LDK + 32 * ks + fg);
#pragma unroll
      for (int kq = 0; kq < CS; ++kq)
        if (2 * kq <= ow) fp[kq] = ET<T>::load_frag(Pc + (16 * ow + fr) * LDC + 32 * kq + fg);
      f32x4 oz = {0.f, 0.f, 0.f, 0.f};
      if constexpr (NORM) {
        // q z, with z as a matrix operand of sixteen equal rows (every lane group reads the same eight columns):
        // every row of the accumulator holds the same sum
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const f32x4 z0 = *(const f32x4*)&s_z[c & 1][32 * ks + fg], z1 = *(const f32x4*)&s_z[c & 1][32 * ks + fg + 4];
          typename ET<T>::frag fz;
#pragma unroll
          for (int e = 0; e < 4; ++e) { fz[e] = (bf16)z0[e]; fz[e + 4] = (bf16)z1[e]; }
          ET<T>::mma(oz, fz, fq[ks]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      f32x4 ot[NB], pv[NB];
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) ot[ni] = pv[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(ot[ni], fh[ks][ni], fq[ks]);          // (q S)^T: column x token
      if (ow == 0) TR(2, c, 5);
#pragma unroll
      for (int kq = 0; kq < CS; ++kq) {
        if (2 * kq <= ow) {
#pragma unroll
          for (int ni = 0; ni < NB; ++ni) ET<T>::mma(pv[ni], fv[kq][ni], fp[kq]);         // (P v)^T
        }
      }
      float rden = 1.f;
      if constexpr (NORM) {
        // the row sums of P (as rounded for P v), again the same sum in every row of the accumulator
        typename ET<T>::frag one8;
#pragma unroll
        for (int e = 0; e < 8; ++e) one8[e] = (bf16)1.f;
        f32x4 pz = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kq = 0; kq < CS; ++kq)
          if (2 * kq <= ow) ET<T>::mma(pz, one8, fp[kq]);
        const float dsum = (oz[0] * ebi + pz[0]) * a.scale + a.norm_eps;
        rden = a.normalize == 2 ? 1.f : 1.f / dsum;      // 2: den is handed out beside o, the caller divides
        if (vsl == 0 && l < 16 && 16 * ow + fr < len)
          ((float*)a.den.ptr)[row_off(a.den, sq.b, tok + 16 * ow + fr, h)] = dsum;
      }
      __builtin_amdgcn_sched_barrier(0);
      if (ow == 0) TR(2, c, 2);
      // lane: token 16 ow + fr, columns 16 ni + g4 .. + 3
      T* orow = row_ptr<T>(a.o, sq.b, tok + 16 * ow + fr, h) + v0 + g4;
      if (16 * ow + fr < len) {
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) {
          const f32x4 x = (ot[ni] * ebi + pv[ni]) * (NORM ? a.scale * rden : a.scale);
          bf16x4 y;
#pragma unroll
          for (int e = 0; e < 4; ++e) y[e] = (bf16)x[e];
          *(bf16x4*)(orow + 16 * ni) = y;
        }
      }
      if (ow == 0) TR(2, c, 4);
      if (c + 1 < sq.nchunks) {
        preread(c + 1);
        p_diag(c + 1);
      }
      if (ow == 0) TR(2, c, 6);
    }
    if (ow == 0) trace_out(2);
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
        for (int i = 0; i < 4; ++i)
          S[mi][ni][i] = h0[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)];
  }
  f32x4 Sz[NORM ? MB : 1];                  // NORM: the column of ones (every column of the tile holds the same sum)
#pragma unroll
  for (int mi = 0; mi < (NORM ? MB : 1); ++mi) Sz[mi] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto copy_state = [&](int c) {            // S at the start of chunk c -> LDS as S^T
    const int buf = c & 1;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(S[mi][ni], s_hT[buf], LDK, krow0 + 16 * mi, 16 * ni);
    if constexpr (NORM) {
      // z beside it, and (SAVE) to zs for the backward: from this team, which has no loads in flight that a store
      // could be made to wait for, and by every V slice (they hold the same sums bit for bit)
      if ((l & 15) == 0) {
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) {
          const int row = krow0 + 16 * mi + 4 * (l >> 4);
          *(f32x4*)&s_z[buf][row] = Sz[mi];
          if constexpr (SAVE) *(f32x4*)&a.zs[((int64_t)(sq.chunk0 + c) * a.H + h) * K + row] = Sz[mi];
        }
      }
    }
  };
  const int pti = wv == 0 ? 3 : wv == 1 ? 2 : wv == 2 ? 3 : 1, ptja = wv == 2 ? 2 : 0, pn = wv < 2 ? 2 : 1;
  copy_state(0);
  lds_barrier();                                                                         // chunks 0, 1 staged
  p_blocks(0, pti, ptja, 1, pn);
  // The operands of the state update of a chunk were staged two windows earlier: they are read (and the row scaling
  // e_d applied to the v' fragments) at the end of the window before, when the LDS is quiet; behind the barrier the
  // update is eight products on registers.
  typename ET<T>::frag af[CS][MB], bf[CS][NB];
  float dec;
  auto preread = [&](int c) {
    const int cb = c & 1;
#pragma unroll
    for (int kq = 0; kq < CS; ++kq) {
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) af[kq][mi] = ET<T>::load_frag_t(s_k[cb], LDK, 32 * kq, krow0 + 16 * mi);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) bf[kq][ni] = ET<T>::load_frag_t(s_u[cb], LDU, 32 * kq, 16 * ni);
    }
    dec = s_dec[cb];
#pragma unroll
    for (int kq = 0; kq < CS; ++kq)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) scale_frag<T>(bf[kq][ni], &s_ed[cb][32 * kq + 8 * (l >> 4)]);
  };
  preread(0);
  for (int c = 0; c < sq.nchunks; ++c) {
    if (wv == 0) TR(0, c, 0);
    lds_barrier();
    if (wv == 0) TR(0, c, 1);
    // S = e^{b_C} S + k^T (e_d v')
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) S[mi][ni] *= dec;
#pragma unroll
    for (int kq = 0; kq < CS; ++kq)
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(S[mi][ni], af[kq][mi], bf[kq][ni]);
    if constexpr (NORM) {                   // z += k^T 1 (ungated: no decay; rows past the end of a chunk are zero)
      typename ET<T>::frag one8;
#pragma unroll
      for (int e = 0; e < 8; ++e) one8[e] = (bf16)1.f;
#pragma unroll
      for (int kq = 0; kq < CS; ++kq)
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) ET<T>::mma(Sz[mi], af[kq][mi], one8);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (wv == 0) TR(0, c, 5);
    if (c + 1 < sq.nchunks) {
      copy_state(c + 1);
      if (wv == 0) TR(0, c, 6);
      p_blocks(c + 1, pti, ptja, 1, pn);
      if (wv == 0) TR(0, c, 2);
      preread(c + 1);
    }
    if (wv == 0) TR(0, c, 3);
  }
  if (wv == 0) trace_out(0);
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
