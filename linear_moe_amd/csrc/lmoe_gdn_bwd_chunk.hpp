// Gated delta rule, chunk-parallel part of the backward: everything that follows the reverse
// state pass, for one (chunk, head) at a time, in one kernel.
//
// Inputs per chunk: do, v' = v_new, du = dv_new, S^T and dS'^T (hs, dhs: [V][K]), q, k, v, Tinv, g,
// beta.  With b = cumulative gate inside the chunk, Gamma_ij = e^{b_i - b_j}, k_b = beta k,
// k_bg = k_b e^{b}:
//   stage 1 (loop over V-slices of width BVH, contraction over the slice's columns)
//     dP   += do v'^T            dq_i += do S^T         dk_d += v' dS'^T
//     dw   -= du S^T             dT_v += du v^T
//     dv_b  = Tinv^T du  (slice) -> dv = dv_b beta (stored),  dbeta += <dv_b, v>
//   stage 2
//     G    = scale (dP . Gamma) [i >= j]
//     dq   = scale e_b dq_i + G k                       (stored)
//     dk   = e_d dk_d + G^T q                           (the part that does not pass through w, u)
//     dT   = dT_v . beta_j + (dw k^T) . (beta_j e^{b_j})
//     dk_bg = Tinv^T dw
//     dL   = - strictlower(Tinv^T dT Tinv^T),   dM = dL . Gamma_s        (L = M . Gamma_s, M = k_b k^T)
//     dk_b = dM k + dk_bg e^{b}
//     dk  += dM^T k_b + dk_b beta                       (stored);   dbeta += <dk_b, k>
//     db_i = q_i.dq_i - k_i.dk_i(first part) + k_b.(dM k) - k.(dM^T k_b) + dk_bg.k_bg
//            (+ on the last row  sum_j (e_d dk_d . k)_j + e^{b_C} <S, dS'>),   dg = reverse cumsum of db
// Nothing but the final gradients leaves the chip: dw, the two parts of dk and the second read of
// du stay in registers / LDS.
//
// persistent: grid = one work-group per CU, item = (chunk, head).  Work-group = 12 waves on one
// barrier script: 8 compute waves and 4 loader waves.
//   Compute wave w owns chunk rows 16 (w % 4) .. + 15 and column half w / 4 of every product (half
//   of K for the K-wide ones, 32 of the 64 columns for the chunk x chunk ones).  The compute waves
//   touch only LDS and the matrix cores, apart from the 64 floats of dbeta and dg per item.
//   The loader waves own all other global traffic: they keep the next slice, the next q, k and the
//   next item's Tinv, g, beta in flight in registers (whole 128-byte lines per row), stage them into
//   LDS (slices into NBUF alternating buffers, two where LDS has the room, so that a slice is filled
//   while the previous one is consumed; the stage 2 tiles lie over the last buffer), and lift the
//   results (dv per slice, dq, dk) out of LDS and store them.  They also form <S, dS'> from the
//   registers they hold and the gate cumsum of the chunk.
//   Script per item (NS slices), three slice buffers:  D(0) .. D(NS-1) = A | b c d e f g h | E
//     (slice s is staged two windows before the compute team reaches it; slices 0, 1 of the next item
//     during f .. h of this one)
//   one slice buffer:  [R(0)] D(0) R(1) D(1) .. D(NS-1) | A | b c d e f g h | E | R(0) of the next item
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

// LDS bytes of k_gdn_bwd_chunk
template <typename T, int K, int BVH, int NBUF> struct GdnBwdChunkLds {
  static constexpr int LDV = BVH + LPAD, LDC = CH + LPAD, LDK = K + LPAD;
  static constexpr int A_END = 4 * CH * LDV + 2 * BVH * LDK;
  static constexpr int B_END = 2 * CH * LDK + CH * LDC + CH * LDK;
  static constexpr int NREG = (NBUF - 1) * A_END + (A_END > B_END ? A_END : B_END);
  static constexpr int NDV = NBUF == 3 ? 2 : 1;      // copies of the dv strip
  static constexpr int BYTES = (NREG + CH * LDC + NDV * CH * LDV) * (int)sizeof(T) + (12 * 64 + 16) * 4;
};

// gemm with a scheduling fence after every 32-deep step: at most one step's fragments are in flight,
// which keeps the register budget of a kernel with many live accumulators
template <typename T, int MB, int NB, bool AT, bool BT>
__device__ __forceinline__ void gemm_bounded(f32x4 (&acc)[MB][NB], const T* A, int lda, int a0,
                                             const T* B, int ldb, int b0, int k0, int k1, int l) {
#pragma unroll
  for (int kk = k0; kk < k1; kk += 32) {
    gemm<T, MB, NB, AT, BT>(acc, A, lda, a0, B, ldb, b0, kk, kk + 32, l);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// compile-time loop: f(IC<0>()), .., f(IC<N - 1>())
template <int I> struct IC { static constexpr int value = I; };
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(IC<I>());
    static_for<N, I + 1>(f);
  }
}

// Forces x to be computed here: without it the compiler moves a running sum's updates down to
// the sum's first use, and keeps every operand alive (spilled) until then.
__device__ __forceinline__ void pin(float& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin(float (&x)[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) pin(x[i]);
}

template <typename T, int K, int V, int BVH, int NBUF, int DEPTH>
__global__ __launch_bounds__(3 * NTHR) void k_gdn_bwd_chunk(const lmoe_args a) {
  typedef GdnBwdChunkLds<T, K, BVH, NBUF> L;
  constexpr int LDV = L::LDV, LDC = L::LDC, LDK = L::LDK;
  constexpr int NS = V / BVH;
  constexpr int KH = K / 2, NBK = KH / 16;     // columns / 16-wide tiles of a K-wide product per compute wave
  static_assert(V % BVH == 0 && BVH == 32, "V-slices: the 8 compute waves split a 64 x 32 slice product 4 x 2");
  static_assert(NBUF == 1 || NBUF == 3, "one slice buffer, or three in rotation");
  // tiles of one V-slice
  constexpr int A_DO = 0, A_VN = A_DO + CH * LDV, A_DVN = A_VN + CH * LDV, A_VV = A_DVN + CH * LDV,
                A_H = A_VV + CH * LDV, A_DH = A_H + BVH * LDK, A_END = L::A_END;
  // stage 2 tiles, laid over the last slice buffer: q (later dq, then dk, on their way out), k,
  // T0 = G^T then dT^T then (beta dM)^T, DW = dw (rows), later T1 = X1^T then dM^T in its first 64 x 64
  constexpr int SB = (NBUF - 1) * A_END;
  constexpr int B_Q = SB, B_K = B_Q + CH * LDK, B_T0 = B_K + CH * LDK, B_DW = B_T0 + CH * LDC, B_T1 = B_DW;
  __shared__ __attribute__((aligned(16))) T smem[L::NREG];
  __shared__ __attribute__((aligned(16))) T s_ti[CH * LDC];              // Tinv, whole item
  // dv of a slice on its way out; with three slice buffers no barrier separates the loaders' read of
  // slice s from the compute team's write of slice s + 1: two copies
  __shared__ __attribute__((aligned(16))) T s_dv[L::NDV][CH * LDV];
  // gate cumsum, its exponentials and beta: two copies, the loaders fill the next item's during stage 2
  __shared__ float s_gb[2][64], s_geb[2][64], s_ged[2][64], s_gbeta[2][64], s_db[2][64], s_dbeta[2][64], s_red[16];

  typedef TileIO<T, CH, BVH> IOV;
  typedef TileIO<T, BVH, K> IOH;
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, CH> IO64;
  const int nitems = a.NT * a.H;
  const int stride = gridDim.x;

  if (threadIdx.x >= 2 * NTHR) {
    // --------------------------------- loaders -------------------------------------------
    const int l = lane_id();
    // thread index inside the team, refreshed per item: the per-thread tile offsets are then recomputed
    // where they are used instead of held (and spilled) for the whole kernel
    int tid = threadIdx.x & (NTHR - 1);
    const int lw = wave_id() - 8;            // wave of the loader team
    // The bulk input of an item is a sequence of NU units: the NS slices, then q, then k.  Units go
    // through DEPTH register sets in rotation (unit u uses set u % DEPTH; NU is a multiple of DEPTH):
    // staging unit u into LDS frees its set for unit u + DEPTH, so DEPTH - 1 .. DEPTH units are in
    // flight at any time.  Every load is issued unconditionally (item index clamped to the last item):
    // a load that is skipped on some path would make the compiler drain all outstanding loads at
    // every use.
    constexpr int NU = NS + 2;
    constexpr int PV = IOV::PASSES, PH = IOH::PASSES, PK = IOK::PASSES;
    constexpr int NVEC = (4 * PV + 2 * PH) > PK ? (4 * PV + 2 * PH) : PK;
    static_assert(NU % DEPTH == 0, "units per item and register sets");
    typedef typename ET<T>::vec vec;
    struct Unit { vec v[NVEC]; int len; };
    Unit U[DEPTH];
    typename IO64::Regs rt;
    uint32_t graw, braw;
    int glen;
    float hdh = 0.f;   // partial <S, dS'> of the item whose slices are being staged
    // unit u counted from the first unit of item it (u >= NU: units of the item after it)
    auto issue = [&](auto uc, int it) {
      constexpr int u = decltype(uc)::value, unit = u % NU;
      Unit& R = U[u % DEPTH];
      it = __builtin_amdgcn_readfirstlane(min(it + (u / NU) * stride, nitems - 1));
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      R.len = ci.len;
      if constexpr (unit < NS) {
        constexpr int vv = unit * BVH;
        static_assert(BVH == SLICE_COLS, "a slice of this kernel is one block of vnew / dvnew");
        const lmoe_tensor* ts[4] = {&a.d_o, &a.vnew, &a.dvnew, &a.v};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          typename IOV::Regs r;
          // do, v: the caller's rows; vnew, dvnew: one contiguous block per (chunk, head, slice)
          if (t == 1 || t == 2) IOV::load_nomask(r, slice_ptr<T>(*ts[t], cid, h, a.H, V, vv), SLICE_COLS, ci.len, tid);
          else IOV::load_nomask(r, row_ptr<T>(*ts[t], ci.b, ci.tok, h) + vv, ts[t]->st, ci.len, tid);
#pragma unroll
          for (int p = 0; p < PV; ++p) R.v[t * PV + p] = r.v[p];
        }
        const T* hp[2] = {(const T*)a.hs, (const T*)a.dhs};
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          typename IOH::Regs r;
          IOH::load_nomask(r, hp[t] + ((int64_t)it * V + vv) * K, K, BVH, tid);         // it = cid * H + h
#pragma unroll
          for (int p = 0; p < PH; ++p) R.v[4 * PV + t * PH + p] = r.v[p];
        }
      } else {
        const lmoe_tensor& x = unit == NS ? a.q : a.k;
        typename IOK::Regs r;
        IOK::load_nomask(r, row_ptr<T>(x, ci.b, ci.tok, h), x.st, ci.len, tid);
#pragma unroll
        for (int p = 0; p < PK; ++p) R.v[p] = r.v[p];
      }
    };
    // unit u (u == NU: slice 0 of the next item) from its registers into LDS; slices go to buffer buf
    auto stage = [&](auto uc, int buf) {
      constexpr int u = decltype(uc)::value, unit = u % NU;
      Unit& R = U[u % DEPTH];
      if constexpr (unit < NS) {
        T* base = smem + buf * A_END;
        constexpr int off[4] = {A_DO, A_VN, A_DVN, A_VV};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          typename IOV::Regs r;
#pragma unroll
          for (int p = 0; p < PV; ++p) r.v[p] = R.v[t * PV + p];
          IOV::mask(r, R.len, tid);
          IOV::store_lds(r, base + off[t], LDV, tid);
        }
        typename IOH::Regs rh, rdh;
#pragma unroll
        for (int p = 0; p < PH; ++p) { rh.v[p] = R.v[4 * PV + p]; rdh.v[p] = R.v[4 * PV + PH + p]; }
#pragma unroll
        for (int p = 0; p < PH; ++p)
#pragma unroll
          for (int i = 0; i < IOH::VEC; ++i) hdh += ET<T>::to_f(rh.v[p][i]) * ET<T>::to_f(rdh.v[p][i]);
        IOH::store_lds(rh, base + A_H, LDK, tid);
        IOH::store_lds(rdh, base + A_DH, LDK, tid);
      } else {
        typename IOK::Regs r;
#pragma unroll
        for (int p = 0; p < PK; ++p) r.v[p] = R.v[p];
        IOK::mask(r, R.len, tid);
        IOK::store_lds(r, smem + (unit == NS ? B_Q : B_K), LDK, tid);
      }
    };
    // stage unit u of item it, then request the unit that takes over its registers
    auto advance = [&](auto uc, int it, int buf) {
      constexpr int u = decltype(uc)::value;
      stage(uc, buf);
      issue(IC<u + DEPTH>(), it);
    };
    auto issue_tinv = [&](int it) {
      it = min(it, nitems - 1);
      IO64::load_nomask(rt, (const T*)a.tinv + (int64_t)it * CH * CH, CH, CH, tid);     // it = cid * H + h
    };
    auto issue_gates = [&](int it) {
      it = __builtin_amdgcn_readfirstlane(min(it, nitems - 1));
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      glen = ci.len;
      graw = gate_prefetch(a, ci.b, ci.tok, ci.len, h);
      braw = load_scalar_raw(a.beta.ptr, a.beta_dtype, row_off(a.beta, ci.b, ci.tok + min(l, ci.len - 1), h));
    };
    // gate cumsum and beta of an item into copy par
    auto stage_gates = [&](int par) {
      gate_finish_wave(a, graw, glen, l, lw == 0, s_gb[par], s_geb[par], s_ged[par]);
      if (lw == 1) s_gbeta[par][l] = l < glen ? scalar_from_raw(braw, a.beta_dtype) : 0.f;
    };
    const int it0 = blockIdx.x;
    issue_tinv(it0);
    issue_gates(it0);
    issue(IC<0>(), it0);
    if constexpr (DEPTH == 2) issue(IC<1>(), it0);
    // the first loads may be ordered freely by the compiler; were they still pending at the loop
    // header, its wait-count analysis would carry that order into every iteration
    wait_all_loads();
    IO64::store_lds(rt, s_ti, LDC, tid);
    stage_gates(0);
    issue_gates(it0 + stride);
    advance(IC<0>(), it0, 0);
    if constexpr (NBUF == 3) advance(IC<1>(), it0, 1);
    int par = 0;
    auto store_dv = [&](const ChunkInfo& ci, int h, int s) {
      typename IOV::Regs r;
      IOV::load_lds_clamped(r, s_dv[s % L::NDV], LDV, ci.len, tid);
      IOV::template store_global_clamped<true>(r, row_ptr<T>(a.dv, ci.b, ci.tok, h) + s * BVH, a.dv.st, ci.len, tid);
    };
    auto close_hdh = [&]() {
      hdh = wave_sum(hdh);
      if (l == 0) s_red[lw] = hdh;
      hdh = 0.f;
    };
    lds_barrier();                                                                       // first slice staged
    for (int it = it0; it < nitems; it += stride) {
      tid = fresh_index(tid) & (NTHR - 1);
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      if constexpr (NBUF == 3) {
        // window w: the compute team works on slice w.  Slice s lives in buffer s % 3 and is staged two
        // windows ahead; q, k go to the third buffer's region in the last window.
        // In every window the loaders fill LDS first and meet the compute team at the barrier; the requests
        // that refill the freed registers follow the barrier.  Requests stall at the issue while the CU's
        // queue is full (32 KB take about a microsecond): issued before the barrier, that stall held up
        // the compute team in five windows of twelve (a quarter of the item, traced per barrier).
        static_for<NS>([&](auto wc) {
          constexpr int w = decltype(wc)::value;
          if constexpr (w >= 1) store_dv(ci, h, w - 1);
          if constexpr (w + 2 < NS) stage(IC<w + 2>(), (w + 2) % 3);
          if constexpr (w == NS - 1) {
            stage(IC<NS>(), 0);                                                          // q
            stage(IC<NS + 1>(), 0);                                                      // k
            close_hdh();
          }
          lds_barrier();                                                                 // D(w); the last one is A
          if constexpr (w + 2 < NS) issue(IC<w + 2 + DEPTH>(), it);
          if constexpr (w == NS - 1) issue(IC<NS + DEPTH>(), it);                        // slice 0 of the next item
        });
        store_dv(ci, h, NS - 1);
      } else {
        static_for<NS>([&](auto sc) {
          constexpr int s = decltype(sc)::value;
          if constexpr (s > 0) lds_barrier();                                            // R(s)
          lds_barrier();                                                                 // D(s)
          store_dv(ci, h, s);
          if constexpr (s + 1 < NS) advance(IC<s + 1>(), it, 0);
        });
        advance(IC<NS>(), it, 0);                                                        // q
        advance(IC<NS + 1>(), it, 0);                                                    // k
        close_hdh();
        lds_barrier();                                                                   // A
      }
      lds_barrier();                                                                     // b
      if constexpr (NBUF == 3) issue(IC<NS + 1 + DEPTH>(), it);                          // slice 1 of the next item
      issue_tinv(it + stride);
      stage_gates(par ^ 1);                                    // the next item's; its copy is idle since E of the last item
      issue_gates(it + 2 * stride);
      lds_barrier();                                                                     // c
      lds_barrier();                                                                     // d: dq lies in the q tile
      {
        typename IOK::Regs r;
        IOK::load_lds_clamped(r, smem + B_Q, LDK, ci.len, tid);
        IOK::template store_global_clamped<true>(r, row_ptr<T>(a.dq, ci.b, ci.tok, h), a.dq.st, ci.len, tid);
      }
      lds_barrier();                                                                     // e
      lds_barrier();                                                                     // f: Tinv of this item is dead
      IO64::store_lds(rt, s_ti, LDC, tid);
      if constexpr (NBUF == 3) stage(IC<NU>(), 0);             // slice 0 of the next item
      lds_barrier();                                                                     // g
      if constexpr (NBUF == 3) {
        issue(IC<NU + DEPTH>(), it);                           // slice 2 of the next item
        stage(IC<NU + 1>(), 1);                                // slice 1 of the next item
      }
      lds_barrier();                                                                     // h: dk lies in the q tile
      if constexpr (NBUF == 3) issue(IC<NU + 1 + DEPTH>(), it);                          // slice 3 of the next item
      {
        typename IOK::Regs r;
        IOK::load_lds_clamped(r, smem + B_Q, LDK, ci.len, tid);
        IOK::template store_global_clamped<true>(r, row_ptr<T>(a.dk, ci.b, ci.tok, h), a.dk.st, ci.len, tid);
      }
      lds_barrier();                                                                     // E
      if constexpr (NBUF == 1) {
        advance(IC<NU>(), it, 0);
        lds_barrier();                                                                   // R(0) of the next item
      }
      par ^= 1;
    }
    return;
  }

  // --------------------------------- compute ---------------------------------------------
  __builtin_amdgcn_s_setprio(3);           // compute waves before the loader wave of their SIMD
  const int wv = wave_id();
  const int r0 = 16 * (wv & 3);            // rows of this wave
  const int ch = wv >> 2;                  // column half
  const int c0 = 32 * ch;                  // first column in a chunk x chunk product
  const int k0 = KH * ch;                  // first column in a K-wide product
  const float scale = a.scale;
  int par = 0;
  lds_barrier();                                                                         // first slice staged
  for (int it = blockIdx.x; it < nitems; it += stride) {
    const float* s_b = s_gb[par]; const float* s_eb = s_geb[par]; const float* s_ed = s_ged[par];
    const float* s_beta = s_gbeta[par];
    // the lane index is refreshed per item: address arithmetic derived from it then stays inside
    // the iteration instead of living in registers for the whole kernel
    const int l = fresh_index(lane_id()) & 63;
    const int fr = l & 15, fg = 8 * (l >> 4);
    const int rb = r0 + 4 * (l >> 4);      // accumulator element i is row rb + i, column (tile) + fr
    f32x4 dP[1][2], dTv[1][2], dqi[1][NBK], dkd[1][NBK], dw[1][NBK];
    acc_zero(dP); acc_zero(dTv); acc_zero(dqi); acc_zero(dkd); acc_zero(dw);
    float dbt[4] = {0.f, 0.f, 0.f, 0.f};      // dbeta of rows rb + i (partial over lanes and column halves)
    // ---- stage 1 ----
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if constexpr (NBUF == 1) {
        if (s > 0) lds_barrier();                                                        // R(s)
      }
      const T* base = smem + (NBUF == 3 ? (s % 3) * A_END : 0);
      const T* DO = base + A_DO; const T* VN = base + A_VN; const T* DVN = base + A_DVN;
      const T* VV = base + A_VV; const T* HT = base + A_H; const T* DHT = base + A_DH;
#pragma unroll
      for (int kk = 0; kk < BVH; kk += 32) {
        const typename ET<T>::frag aDO = ET<T>::load_frag(DO + (r0 + fr) * LDV + kk + fg);
        const typename ET<T>::frag aVN = ET<T>::load_frag(VN + (r0 + fr) * LDV + kk + fg);
        const typename ET<T>::frag aDVN = ET<T>::load_frag(DVN + (r0 + fr) * LDV + kk + fg);
#pragma unroll
        for (int nj = 0; nj < 2; ++nj) {
          ET<T>::mma(dP[0][nj], aDO, ET<T>::load_frag(VN + (c0 + 16 * nj + fr) * LDV + kk + fg));
          ET<T>::mma(dTv[0][nj], aDVN, ET<T>::load_frag(VV + (c0 + 16 * nj + fr) * LDV + kk + fg));
        }
#pragma unroll
        for (int ni = 0; ni < NBK; ++ni) {
          const typename ET<T>::frag bH = ET<T>::load_frag_t(HT, LDK, kk, k0 + 16 * ni, l);
          ET<T>::mma(dqi[0][ni], aDO, bH);
          ET<T>::mma(dw[0][ni], aDVN, bH);
          ET<T>::mma(dkd[0][ni], aVN, ET<T>::load_frag_t(DHT, LDK, kk, k0 + 16 * ni, l));
        }
      }
      // dv_b = Tinv^T du for this slice: rows r0.., columns 16 ch .. + 15 of the slice
      f32x4 dvb[1][1];
      acc_zero(dvb);
      gemm<T, 1, 1, true, true>(dvb, s_ti, LDC, r0, DVN, LDV, 16 * ch, 0, CH, l);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dbt[i] += dvb[0][0][i] * ET<T>::to_f(VV[(rb + i) * LDV + 16 * ch + fr]);
        dvb[0][0][i] *= s_beta[rb + i];                                                  // final dv
      }
      acc_to_lds<T>(dvb[0][0], s_dv[s % L::NDV], LDV, r0, 16 * ch, l);
      pin(dbt);
      __builtin_amdgcn_sched_barrier(0);
      lds_barrier();                                                                     // D(s); with three buffers the last one is A
    }
    if constexpr (NBUF == 1) lds_barrier();                                              // A: q, k staged
    // ---- stage 2 ----
    T* Qt = smem + B_Q; T* Kt = smem + B_K; T* T0 = smem + B_T0; T* T1 = smem + B_T1; T* DW = smem + B_DW;
#pragma unroll
    for (int nj = 0; nj < 2; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = rb + i, cc = c0 + 16 * nj + fr;
        p[i] = (r >= cc) ? scale * dP[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds_t<T>(p, T0, LDC, r0, c0 + 16 * nj, l);                                  // G^T [j][i]
    }
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni) {
      f32x4 x;
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] = -dw[0][ni][i];                                  // dw = -du S^T
      acc_to_lds<T>(x, DW, LDK, r0, k0 + 16 * ni, l);
    }
    lds_barrier();                                                                       // b
    float dbp[4] = {0.f, 0.f, 0.f, 0.f};
    float kk = 0.f;
    f32x4 dq[1][NBK], dk[1][NBK], dkbg[1][NBK], dT[1][2];
    acc_zero(dq);
    gemm_bounded<T, 1, NBK, true, true>(dq, T0, LDC, r0, Kt, LDK, k0, 0, CH, l);         // G k
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = rb + i, cc = k0 + 16 * ni + fr;
        const float dqv = scale * s_eb[r] * dqi[0][ni][i] + dq[0][ni][i];
        dbp[i] += ET<T>::to_f(Qt[r * LDK + cc]) * dqv;
        dq[0][ni][i] = dqv;                                                              // final dq
      }
    pin(dbp);
    __builtin_amdgcn_sched_barrier(0);
    acc_zero(dk);
    gemm_bounded<T, 1, NBK, false, true>(dk, T0, LDC, r0, Qt, LDK, k0, 0, CH, l);        // G^T q
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = rb + i, cc = k0 + 16 * ni + fr;
        const float kv = ET<T>::to_f(Kt[r * LDK + cc]);
        const float dkdv = s_ed[r] * dkd[0][ni][i];
        const float dkv = dkdv + dk[0][ni][i];
        dbp[i] -= kv * dkv;
        kk += kv * dkdv;
        dk[0][ni][i] = dkv;                                                              // first part of dk
      }
    pin(dbp);
    pin(kk);
    __builtin_amdgcn_sched_barrier(0);
    {
      f32x4 t2[1][2];
      acc_zero(t2);
      gemm_bounded<T, 1, 2, false, false>(t2, DW, LDK, r0, Kt, LDK, c0, 0, K, l);        // dw k^T
#pragma unroll
      for (int nj = 0; nj < 2; ++nj) {
        const int cc = c0 + 16 * nj + fr;
        const float bj = s_beta[cc], bej = bj * s_eb[cc];
#pragma unroll
        for (int i = 0; i < 4; ++i) dT[0][nj][i] = dTv[0][nj][i] * bj + t2[0][nj][i] * bej;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    acc_zero(dkbg);
    gemm_bounded<T, 1, NBK, true, true>(dkbg, s_ti, LDC, r0, DW, LDK, k0, 0, CH, l);     // Tinv^T dw
    lds_barrier();                                                                       // c: G^T, DW, q read
#pragma unroll
    for (int nj = 0; nj < 2; ++nj) acc_to_lds_t<T>(dT[0][nj], T0, LDC, r0, c0 + 16 * nj, l);   // dT^T [n][i]
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni) acc_to_lds<T>(dq[0][ni], Qt, LDK, r0, k0 + 16 * ni, l);   // dq on its way out
    lds_barrier();                                                                       // d
    {
      // X1[j][n] = sum_i Tinv[i][j] dT[i][n]
      f32x4 x1[1][2];
      acc_zero(x1);
      gemm_bounded<T, 1, 2, true, false>(x1, s_ti, LDC, r0, T0, LDC, c0, 0, CH, l);
#pragma unroll
      for (int nj = 0; nj < 2; ++nj) acc_to_lds_t<T>(x1[0][nj], T1, LDC, r0, c0 + 16 * nj, l);   // X1^T [n][j]
    }
    lds_barrier();                                                                       // e
    {
      f32x4 dL[1][2];
      acc_zero(dL);
      // dL[j][m] = - sum_n X1[j][n] Tinv[m][n]
      gemm_bounded<T, 1, 2, true, false>(dL, T1, LDC, r0, s_ti, LDC, c0, 0, CH, l);
      lds_barrier();                                                                     // f: X1^T, dT^T, Tinv read
#pragma unroll
      for (int nj = 0; nj < 2; ++nj) {
        f32x4 p, pb;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = rb + i, cc = c0 + 16 * nj + fr;
          p[i] = (r > cc) ? -dL[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
          pb[i] = p[i] * s_beta[r];
        }
        acc_to_lds_t<T>(p, T1, LDC, r0, c0 + 16 * nj, l);                                // dM^T  [j][i]
        acc_to_lds_t<T>(pb, T0, LDC, r0, c0 + 16 * nj, l);                               // (diag(beta) dM)^T [j][i]
      }
    }
    lds_barrier();                                                                       // g
    {
      // dM k first: it closes dk_b (dbeta, the k_b.(dM k) term); then dM^T k_b
      // (k is re-read from LDS through an offset the compiler cannot see through: it would otherwise
      // keep the values read for the first part of dk in registers across phases c .. g)
      const T* Kr = Kt + fresh_index(0);
      f32x4 m[1][NBK];
      acc_zero(m);
      gemm_bounded<T, 1, NBK, true, true>(m, T1, LDC, r0, Kt, LDK, k0, 0, CH, l);
#pragma unroll
      for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = rb + i, cc = k0 + 16 * ni + fr;
          const float kv = ET<T>::to_f(Kr[r * LDK + cc]);
          const float bt = s_beta[r], eb = s_eb[r];
          const float kbv = kv * bt;
          const float dkb = m[0][ni][i] + dkbg[0][ni][i] * eb;
          dbt[i] += dkb * kv;
          dbp[i] += kbv * m[0][ni][i] + dkbg[0][ni][i] * kbv * eb;
          dk[0][ni][i] += dkb * bt;
        }
      pin(dbp);
      pin(dbt);
      __builtin_amdgcn_sched_barrier(0);
      const T* Kr2 = Kt + fresh_index(0);
      acc_zero(m);
      gemm_bounded<T, 1, NBK, false, true>(m, T0, LDC, r0, Kt, LDK, k0, 0, CH, l);
#pragma unroll
      for (int ni = 0; ni < NBK; ++ni) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = rb + i, cc = k0 + 16 * ni + fr;
          dbp[i] -= ET<T>::to_f(Kr2[r * LDK + cc]) * m[0][ni][i];
          dk[0][ni][i] += m[0][ni][i];                                                   // final dk
        }
        acc_to_lds<T>(dk[0][ni], Qt, LDK, r0, k0 + 16 * ni, l);                          // dk on its way out
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dbp[i] = group_sum<16>(dbp[i]);
      dbt[i] = group_sum<16>(dbt[i]);
    }
    if (fr == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        s_db[ch][rb + i] = dbp[i];
        s_dbeta[ch][rb + i] = dbt[i];
      }
    }
    kk = wave_sum(kk);
    if (l == 0) s_red[4 + wv] = kk;
    lds_barrier();                                                                       // h
    if (threadIdx.x < 64) {
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      // refreshed: the LDS addresses derived from it are otherwise hoisted out of the item loop and spilled
      const int j = fresh_index(threadIdx.x) & 63;
      float x = 0.f;
      if (j < ci.len) {
        ((float*)a.dbeta.ptr)[row_off(a.dbeta, ci.b, ci.tok + j, h)] = s_dbeta[0][j] + s_dbeta[1][j];
        x = s_db[0][j] + s_db[1][j];
        // last-row term; rows past the end of a partial chunk carry zero q, k, so the term may sit
        // on the last valid row without changing the reverse cumulative sum
        if (j == ci.len - 1) {
          float skk = 0.f, shd = 0.f;
#pragma unroll
          for (int w = 0; w < 8; ++w) skk += s_red[4 + w];
#pragma unroll
          for (int w = 0; w < 4; ++w) shd += s_red[w];
          x += skk + expf(s_b[CH - 1]) * shd;
        }
      }
      x = wave_rev_scan(x);
      if (j < ci.len) ((float*)a.dg.ptr)[row_off(a.dg, ci.b, ci.tok + j, h)] = x;
    }
    lds_barrier();           // E: the stage 2 region goes to the next item
    if constexpr (NBUF == 1) lds_barrier();                                              // R(0) of the next item
    par ^= 1;
  }
}

}  // namespace lmoe
