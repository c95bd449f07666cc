// Gated delta rule, chunk-parallel part of the backward: everything that follows the reverse
// state pass, for one (chunk, head) at a time, in one kernel.
//
// The WY form of a chunk is v_new = Tinv Z with Z = beta (v - e^{b} k S) and Tinv = (I + L)^{-1},
// L = strictlower((beta k k^T) . Gamma): v_new solves (I + L) v_new = Z.  Its backward needs no product
// with Tinv once dZ = Tinv^T dv_new is known (the reverse state pass writes dZ, not dv_new):
//     dv = beta dZ,   d(k beta e^{b}) = -dZ S^T,   dL = -strictlower(dZ v_new^T),   dS -= (k beta e^{b})^T dZ.
//
// Inputs per chunk: do, v' = v_new, dZ, S^T and dS'^T (hs, dhs: [V][K]), q, k, v, g, beta.  With
// b = cumulative gate inside the chunk, Gamma_ij = e^{b_i - b_j}, k_b = beta k, k_bg = k_b e^{b}:
//   stage 1 (loop over V-slices of width BVH, contraction over the slice's columns)
//     dP   += do v'^T            dq_i += do S^T         dk_d += v' dS'^T
//     dk_bg -= dZ S^T            dLf  += dZ v'^T
//     (loader waves, from the registers they stage:  dv = beta dZ, stored;  dbeta += <dZ, v>)
//   stage 2
//     G    = scale (dP . Gamma) [i >= j],     dM = -(dLf . Gamma) [i > j]       (L = M . Gamma_s, M = k_b k^T)
//     dq   = scale e_b dq_i + G k                       (stored)
//     dk   = e_d dk_d + G^T q                           (the part that does not pass through the WY form)
//     dk_b = dM k + dk_bg e^{b}
//     dk  += dM^T k_b + dk_b beta                       (stored);   dbeta += <dk_b, k>
//     db_i = q_i.dq_i - k_i.dk_i(first part) + k_b.(dM k) - k.(dM^T k_b) + dk_bg.k_bg
//            (+ on the last row  sum_j (e_d dk_d . k)_j + e^{b_C} <S, dS'>),   dg = reverse cumsum of db
// Nothing but the final gradients leaves the chip.
//
// persistent: grid = one work-group per CU, item = (chunk, head).  Work-group = 12 waves on one
// barrier script: 8 compute waves and 4 loader waves.
//   Compute wave w owns chunk rows 16 (w % 4) .. + 15 and column half w / 4 of every product (half
//   of K for the K-wide ones, 32 of the 64 columns for the chunk x chunk ones).  The compute waves
//   touch only LDS and the matrix cores, apart from the 64 floats of dbeta and dg per item.
//   The loader waves own all other global traffic: they keep the next slices, the next q and k and the
//   next item's g, beta in flight in registers (whole 128-byte lines per row), stage them into
//   LDS (slices into NBUF alternating buffers, q and k into tiles of their own; the three chunk x chunk
//   tiles of stage 2 lie over the last slice buffer), form dv and the value part of dbeta from the
//   registers on the way, and lift dq, dk out of LDS and store them.  They also form <S, dS'> from
//   the registers they hold and the gate cumsum of the chunk.
//   Script per item (NS = 4 slices), three slice buffers:   D0 D1 D2 A | b c d
//     window w: the compute team works on slice w (buffer w % 3); the loaders stage slice w + 2, then q
//     (window 2) and k (window 3), and slices 0, 1 of the next item during b .. d
//   one slice buffer:  [R(0)] D(0) R(1) D(1) .. D(NS-1) | A | b c d | R(0) of the next item
#pragma once
#include "lmoe_seq.hpp"

namespace lmoe {

// LDS bytes of k_gdn_bwd_chunk
template <typename T, int K, int BVH, int NBUF> struct GdnBwdChunkLds {
  static constexpr int LDV = BVH + LPAD, LDC = CH + LPAD, LDK = K + LPAD;
  static constexpr int A_END = 3 * CH * LDV + 2 * BVH * LDK;      // do, v_new, dZ; S^T, dS'^T of one slice
  static constexpr int T_END = 3 * CH * LDC;                      // G^T, dM^T, (beta dM)^T: over the last slice buffer
  static constexpr int S_END = (NBUF - 1) * A_END + (A_END > T_END ? A_END : T_END);   // slice buffers, the last one widened to hold the tiles
  static constexpr int NREG = S_END + 2 * CH * LDK;               // ..; q, k
  static constexpr int BYTES = NREG * (int)sizeof(T) + (13 * 64 + 16) * 4;
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

// QKACT: q and k as given are l2norm(silu(.)) of rows of a projection that the caller holds (lmoe_args.q_raw, k_raw):
// dq and dk leave as the gradients with respect to those rows - the backward of the L2 norm and of SiLU is applied to
// the dq, dk tiles on their way from LDS to memory, by the loader threads that store them, from the raw rows, which
// are requested when stage 2 begins.  (What it costs is those rows: 32 KB more per item through a request path that is
// full; the arithmetic, spread over the first windows of the next item or not, is a tenth of it.)
template <typename T, int K, int V, int BVH, int NBUF, int DEPTH, bool QKACT = false>
__global__ __launch_bounds__(3 * NTHR) void k_gdn_bwd_chunk(const lmoe_args a) {
  static_assert(!QKACT || (sizeof(T) == 2 && NBUF == 3), "the activation backward exists for 2-byte elements");
  typedef GdnBwdChunkLds<T, K, BVH, NBUF> L;
  constexpr int LDV = L::LDV, LDC = L::LDC, LDK = L::LDK;
  constexpr int NS = V / BVH;
  constexpr int KH = K / 2, NBK = KH / 16;     // columns / 16-wide tiles of a K-wide product per compute wave
  static_assert(V % BVH == 0 && BVH == 32, "V-slices: the 8 compute waves split a 64 x 32 slice product 4 x 2");
  static_assert(NBUF == 1 || NBUF == 3, "one slice buffer, or three in rotation");
  // tiles of one V-slice
  constexpr int A_DO = 0, A_VN = A_DO + CH * LDV, A_DZ = A_VN + CH * LDV,
                A_H = A_DZ + CH * LDV, A_DH = A_H + BVH * LDK, A_END = L::A_END;
  // stage 2: q (later dq on its way out) and k (later dk) in tiles of their own; T0 = G^T, T1 = dM^T,
  // T2 = (diag(beta) dM)^T over the last slice buffer
  constexpr int B_T0 = (NBUF - 1) * A_END, B_T1 = B_T0 + CH * LDC, B_T2 = B_T1 + CH * LDC;
  constexpr int B_Q = L::S_END, B_K = B_Q + CH * LDK;
  __shared__ __attribute__((aligned(16))) T smem[L::NREG];
  // gate cumsum, its exponentials and beta: two copies, the loaders fill the next item's during stage 2
  __shared__ float s_gb[2][64], s_geb[2][64], s_ged[2][64], s_gbeta[2][64], s_db[2][64], s_dbeta[2][64], s_dbv[64], s_red[16];

  typedef TileIO<T, CH, BVH> IOV;
  typedef TileIO<T, BVH, K> IOH;
  typedef TileIO<T, CH, K> IOK;
  const int nitems = num_chunks(a) * a.H;
  if (nitems <= 0) return;                   // (a chunk count read on the device may be zero)
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
    uint32_t graw, braw;
    int glen;
    float hdh = 0.f;   // partial <S, dS'> of the item whose slices are being staged
    float dbv[PV];     // partial <dZ, v> of this thread's rows of that item
#pragma unroll
    for (int p = 0; p < PV; ++p) dbv[p] = 0.f;
    // unit u counted from the first unit of item it (u >= NU: units of the item after it)
    auto issue = [&](auto uc, int it) {
      constexpr int u = decltype(uc)::value, unit = u % NU;
      Unit& R = U[u % DEPTH];
      it = __builtin_amdgcn_readfirstlane(min(it + (u / NU) * stride, nitems - 1));
      // with many slices per item the scalar addresses of all of them, formed at the top of the item, do not fit the
      // scalar registers: the item index is made opaque per unit, so that each unit's addresses are formed where it
      // is requested
      if constexpr (NS > 4) asm volatile("" : "+s"(it));
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
          // do, v: the caller's rows; vnew, dvnew (= dZ): one contiguous block per (chunk, head, slice)
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
    // dv of a slice on its way from the registers to memory
    struct DV { typename IOV::Regs r; };
    // unit u (u >= NU: of the next item) from its registers into LDS; slices go to buffer buf, and their dv = beta dZ
    // into d (gp = the copy of the gate arrays that holds the beta of the unit's item)
    auto stage = [&](auto uc, int buf, int gp, DV& d) {
      constexpr int u = decltype(uc)::value, unit = u % NU;
      Unit& R = U[u % DEPTH];
      if constexpr (unit < NS) {
        T* base = smem + buf * A_END;
        // dv and <dZ, v> first, from the registers as loaded: rows past the end of a partial chunk repeat its last row
        // there, which is what the branch-free store of dv rewrites
#pragma unroll
        for (int p = 0; p < PV; ++p) {
          int row, col; IOV::coords(p, row, col, tid);
          const float bt = s_gbeta[gp][min(row, R.len - 1)];
          const vec z = R.v[2 * PV + p], vv = R.v[3 * PV + p];
          vec o;
          float s = 0.f;
#pragma unroll
          for (int i = 0; i < IOV::VEC; ++i) {
            const float zf = ET<T>::to_f(z[i]);
            if (a.v_act) {
              // v as given is the argument of a SiLU: the op runs on silu(v) (rounded to the element type, as the
              // forward pass staged it) and dv is the gradient with respect to the argument
              const float vr = ET<T>::to_f(vv[i]);
              o[i] = ET<T>::from_f(zf * bt * silu_grad(vr));
              s += zf * ET<T>::to_f(ET<T>::from_f(silu_of(vr)));
            } else {
              o[i] = ET<T>::from_f(zf * bt);
              s += zf * ET<T>::to_f(vv[i]);
            }
          }
          d.r.v[p] = o;
          s = group_sum<IOV::VPR>(s);                   // the VPR lanes that hold one row are neighbours
          dbv[p] += row < R.len ? s : 0.f;
          pin(dbv[p]);
        }
        constexpr int off[3] = {A_DO, A_VN, A_DZ};
#pragma unroll
        for (int t = 0; t < 3; ++t) {
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
        pin(hdh);                                         // here, not where the item is closed (the tiles would stay live)
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
    auto store_dv = [&](const DV& d, const ChunkInfo& ci, int h, int s) {
      IOV::template store_global_clamped<true>(d.r, row_ptr<T>(a.dv, ci.b, ci.tok, h) + s * BVH, a.dv.st, ci.len, tid);
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
    // the sums of an item whose slices have all been staged
    auto close_item = [&]() {
      hdh = wave_sum(hdh);
      if (l == 0) s_red[lw] = hdh;
      hdh = 0.f;
#pragma unroll
      for (int p = 0; p < PV; ++p) {
        int row, col; IOV::coords(p, row, col, tid);
        if (col == 0) s_dbv[row] = dbv[p];
        dbv[p] = 0.f;
      }
    };
    // QKACT: the raw rows behind q and k of an item, and the backward of y = l2norm(silu(x)) on a tile of dy:
    //   s = silu(x), r = (|s|^2 + eps)^-1/2, dx = silu'(x) (dy r - (dy . s) r^3 s)
    // with the sums of a row over the VPR neighbouring lanes that hold it (the arithmetic, step for step, of the row
    // kernel that does the same in front of the op: the results agree bit for bit)
    typename IOK::Regs XQ, XK;
    auto issue_raw = [&](int it) __attribute__((always_inline)) {
      if constexpr (QKACT) {
        const int cid = it / a.H, h = it % a.H;
        const ChunkInfo ci = chunk_info(a, cid);
        IOK::load_nomask(XQ, row_ptr<T>(a.q_raw, ci.b, ci.tok, h), a.q_raw.st, ci.len, tid);
        IOK::load_nomask(XK, row_ptr<T>(a.k_raw, ci.b, ci.tok, h), a.k_raw.st, ci.len, tid);
      }
    };
    auto act_backward = [&](typename IOK::Regs& r, const typename IOK::Regs& X) __attribute__((always_inline)) {
      if constexpr (QKACT) {
#pragma unroll
        for (int p = 0; p < PK; ++p) {
          float sv[IOK::VEC], gv[IOK::VEC], fv[IOK::VEC], ss = 0.f, c = 0.f;
#pragma unroll
          for (int i = 0; i < IOK::VEC; ++i) {
            const float x = ET<T>::to_f(X.v[p][i]), sg = sigmoid_fast(x);
            sv[i] = x * sg;
            gv[i] = sg * (1.0f + x * (1.0f - sg));
            ss += sv[i] * sv[i];
          }
#pragma unroll
          for (int i = 0; i < IOK::VEC; ++i) { fv[i] = ET<T>::to_f(r.v[p][i]); c += fv[i] * sv[i]; }
          ss = group_sum<IOK::VPR>(ss);
          c = group_sum<IOK::VPR>(c);
          const float rn = 1.0f / sqrtf(ss + a.qk_eps);
          c = c * rn * rn * rn;
#pragma unroll
          for (int i = 0; i < IOK::VEC; ++i) r.v[p][i] = ET<T>::from_f((fv[i] * rn - c * sv[i]) * gv[i]);
        }
      }
    };
    // (a launch sized by an upper bound of the chunk count may hold work-groups without an item: they stage the last
    // item like every load past the end and skip the loop)
    const int it0 = min((int)blockIdx.x, nitems - 1);
    DV d0, d1;
    issue_gates(it0);
    static_for<DEPTH>([&](auto jc) { issue(jc, it0); });
    // the first loads may be ordered freely by the compiler; were they still pending at the loop
    // header, its wait-count analysis would carry that order into every iteration
    wait_all_loads();
    stage_gates(0);
    issue_gates(it0 + stride);
    lds_barrier();                                                                       // beta of the first item staged
    {
      const ChunkInfo ci = chunk_info(a, it0 / a.H);
      stage(IC<0>(), 0, 0, d0);
      issue(IC<DEPTH>(), it0);
      store_dv(d0, ci, it0 % a.H, 0);
      if constexpr (NBUF == 3) {
        stage(IC<1>(), 1, 0, d1);
        issue(IC<1 + DEPTH>(), it0);
        store_dv(d1, ci, it0 % a.H, 1);
      }
    }
    int par = 0;
    lds_barrier();                                                                       // first slice staged
    for (int it = blockIdx.x; it < nitems; it += stride) {
      tid = fresh_index(tid) & (NTHR - 1);
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      // the item after this one (past the end: the last item once more, see issue)
      const int itn = __builtin_amdgcn_readfirstlane(min(it + stride, nitems - 1));
      const int hn = itn % a.H;
      const ChunkInfo cin = chunk_info(a, itn / a.H);
      if constexpr (NBUF == 3) {
        // window w: the compute team works on slice w.  Slice s lives in buffer s % 3 and is staged two
        // windows ahead; q and k follow in windows 2 and 3.
        // In every window the loaders fill LDS first and meet the compute team at the barrier; the stores and the
        // requests that refill the freed registers follow the barrier.  Requests stall at the issue while the CU's
        // queue is full (32 KB take about a microsecond): issued before the barrier, that stall holds up the
        // compute team.
        static_for<NS>([&](auto wc) {
          constexpr int w = decltype(wc)::value, u = w + 2;    // u < NS: a slice (buffer u % 3), then q, then k
          stage(IC<u>(), u % 3, par, d0);
          if constexpr (w == NS - 1) close_item();
          lds_barrier();                                                                 // D(w); the last one is A
          if constexpr (u < NS) store_dv(d0, ci, h, u);
          if constexpr (w < NS - 1) issue(IC<u + DEPTH>(), it);                          // q, k, slice 0 of the next item
        });
        issue_raw(it);                                                                   // (QKACT) used behind d
        issue(IC<NS + 1 + DEPTH>(), it);                                                 // slice 1 of the next item
        stage_gates(par ^ 1);                                  // the next item's; its copy is idle since d of the last item
        issue_gates(it + 2 * stride);
        lds_barrier();                                                                   // b
        stage(IC<NU>(), 0, par ^ 1, d0);                       // slice 0 of the next item (buffer 0: slice 3 is done)
        lds_barrier();                                                                   // c
        store_dv(d0, cin, hn, 0);
        issue(IC<NU + DEPTH>(), it);                                                     // slice 2 of the next item
        stage(IC<NU + 1>(), 1, par ^ 1, d1);                   // slice 1 of the next item
        lds_barrier();                                                                   // d: dq, dk lie in the q, k tiles
        store_dv(d1, cin, hn, 1);
        issue(IC<NU + 1 + DEPTH>(), it);                                                 // slice 3 of the next item
      } else {
        static_for<NS>([&](auto sc) {
          constexpr int s = decltype(sc)::value;
          if constexpr (s > 0) lds_barrier();                                            // R(s)
          lds_barrier();                                                                 // D(s)
          if constexpr (s + 1 < NS) {
            stage(IC<s + 1>(), 0, par, d0);
            issue(IC<s + 1 + DEPTH>(), it);
            store_dv(d0, ci, h, s + 1);
          }
        });
        stage(IC<NS>(), 0, par, d0);                                                     // q
        issue(IC<NS + DEPTH>(), it);
        stage(IC<NS + 1>(), 0, par, d0);                                                 // k
        issue(IC<NS + 1 + DEPTH>(), it);
        close_item();
        lds_barrier();                                                                   // A
        stage_gates(par ^ 1);
        issue_gates(it + 2 * stride);
        lds_barrier();                                                                   // b
        lds_barrier();                                                                   // c
        lds_barrier();                                                                   // d
      }
      {
        typename IOK::Regs r;
        IOK::load_lds_clamped(r, smem + B_Q, LDK, ci.len, tid);
        act_backward(r, XQ);
        IOK::template store_global_clamped<true>(r, row_ptr<T>(a.dq, ci.b, ci.tok, h), a.dq.st, ci.len, tid);
        IOK::load_lds_clamped(r, smem + B_K, LDK, ci.len, tid);
        act_backward(r, XK);
        IOK::template store_global_clamped<true>(r, row_ptr<T>(a.dk, ci.b, ci.tok, h), a.dk.st, ci.len, tid);
      }
      if constexpr (NBUF == 1) {
        stage(IC<NU>(), 0, par ^ 1, d0);                       // slice 0 of the next item
        issue(IC<NU + DEPTH>(), it);
        store_dv(d0, cin, hn, 0);
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
  lds_barrier();                                                                         // beta of the first item staged
  lds_barrier();                                                                         // first slice staged
  for (int it = blockIdx.x; it < nitems; it += stride) {
    const float* s_b = s_gb[par]; const float* s_eb = s_geb[par]; const float* s_ed = s_ged[par];
    const float* s_beta = s_gbeta[par];
    // the lane index is refreshed per item: address arithmetic derived from it then stays inside
    // the iteration instead of living in registers for the whole kernel
    const int l = fresh_index(lane_id()) & 63;
    const int fr = l & 15, fg = 8 * (l >> 4);
    const int rb = r0 + 4 * (l >> 4);      // accumulator element i is row rb + i, column (tile) + fr
    f32x4 dP[1][2], dLf[1][2], dqi[1][NBK], dkd[1][NBK], dkbg[1][NBK];
    acc_zero(dP); acc_zero(dLf); acc_zero(dqi); acc_zero(dkd); acc_zero(dkbg);
    // ---- stage 1 ----
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if constexpr (NBUF == 1) {
        if (s > 0) lds_barrier();                                                        // R(s)
      }
      const T* base = smem + (NBUF == 3 ? (s % 3) * A_END : 0);
      const T* DO = base + A_DO; const T* VN = base + A_VN; const T* DZ = base + A_DZ;
      const T* HT = base + A_H; const T* DHT = base + A_DH;
#pragma unroll
      for (int kk = 0; kk < BVH; kk += 32) {
        const typename ET<T>::frag aDO = ET<T>::load_frag(DO + (r0 + fr) * LDV + kk + fg);
        const typename ET<T>::frag aVN = ET<T>::load_frag(VN + (r0 + fr) * LDV + kk + fg);
        const typename ET<T>::frag aDZ = ET<T>::load_frag(DZ + (r0 + fr) * LDV + kk + fg);
#pragma unroll
        for (int nj = 0; nj < 2; ++nj) {
          const typename ET<T>::frag bVN = ET<T>::load_frag(VN + (c0 + 16 * nj + fr) * LDV + kk + fg);
          ET<T>::mma(dP[0][nj], aDO, bVN);
          ET<T>::mma(dLf[0][nj], aDZ, bVN);
        }
#pragma unroll
        for (int ni = 0; ni < NBK; ++ni) {
          const typename ET<T>::frag bH = ET<T>::load_frag_t(HT, LDK, kk, k0 + 16 * ni, l);
          ET<T>::mma(dqi[0][ni], aDO, bH);
          ET<T>::mma(dkbg[0][ni], aDZ, bH);                                              // + dZ S^T: dk_bg is its negative
          ET<T>::mma(dkd[0][ni], aVN, ET<T>::load_frag_t(DHT, LDK, kk, k0 + 16 * ni, l));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      lds_barrier();                                                                     // D(s); with three buffers the last one is A
    }
    if constexpr (NBUF == 1) lds_barrier();                                              // A: q, k staged
    // ---- stage 2 ----
    T* Qt = smem + B_Q; T* Kt = smem + B_K; T* T0 = smem + B_T0; T* T1 = smem + B_T1; T* T2 = smem + B_T2;
#pragma unroll
    for (int nj = 0; nj < 2; ++nj) {
      f32x4 g, m, mb;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = rb + i, cc = c0 + 16 * nj + fr;
        const float e = (r >= cc) ? texp<T>(s_b[r] - s_b[cc]) : 0.f;
        g[i] = scale * dP[0][nj][i] * e;
        m[i] = (r > cc) ? -dLf[0][nj][i] * e : 0.f;
        mb[i] = m[i] * s_beta[r];
      }
      acc_to_lds_t<T>(g, T0, LDC, r0, c0 + 16 * nj, l);                                  // G^T [j][i]
      acc_to_lds_t<T>(m, T1, LDC, r0, c0 + 16 * nj, l);                                  // dM^T [j][i]
      acc_to_lds_t<T>(mb, T2, LDC, r0, c0 + 16 * nj, l);                                 // (diag(beta) dM)^T [j][i]
    }
    lds_barrier();                                                                       // b
    float dbp[4] = {0.f, 0.f, 0.f, 0.f};      // db of rows rb + i (partial over lanes and column halves)
    float dbt[4] = {0.f, 0.f, 0.f, 0.f};      // dbeta of rows rb + i, the part through k_b
    float kk = 0.f;
    f32x4 dq[1][NBK], dk[1][NBK];
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
      // dM k first: it closes dk_b (dbeta, the k_b.(dM k) term); then dM^T k_b
      // (k is re-read from LDS through an offset the compiler cannot see through: it would otherwise
      // keep the values read for the first part of dk in registers)
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
          const float dkbgv = -dkbg[0][ni][i];
          const float dkb = m[0][ni][i] + dkbgv * eb;
          dbt[i] += dkb * kv;
          dbp[i] += kbv * m[0][ni][i] + dkbgv * kbv * eb;
          dk[0][ni][i] += dkb * bt;
        }
      pin(dbp);
      pin(dbt);
      __builtin_amdgcn_sched_barrier(0);
      const T* Kr2 = Kt + fresh_index(0);
      acc_zero(m);
      gemm_bounded<T, 1, NBK, false, true>(m, T2, LDC, r0, Kt, LDK, k0, 0, CH, l);
#pragma unroll
      for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int r = rb + i, cc = k0 + 16 * ni + fr;
          dbp[i] -= ET<T>::to_f(Kr2[r * LDK + cc]) * m[0][ni][i];
          dk[0][ni][i] += m[0][ni][i];                                                   // final dk
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dbp[i] = group_sum<16>(dbp[i]);
      dbt[i] = group_sum<16>(dbt[i]);
    }
    kk = wave_sum(kk);
    lds_barrier();                                                                       // c: q, k, the chunk x chunk tiles read
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni) {
      acc_to_lds<T>(dq[0][ni], Qt, LDK, r0, k0 + 16 * ni, l);                            // dq, dk on their way out
      acc_to_lds<T>(dk[0][ni], Kt, LDK, r0, k0 + 16 * ni, l);
    }
    if (fr == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        s_db[ch][rb + i] = dbp[i];
        s_dbeta[ch][rb + i] = dbt[i];
      }
    }
    if (l == 0) s_red[4 + wv] = kk;
    lds_barrier();                                                                       // d
    if (threadIdx.x < 64) {
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      // refreshed: the LDS addresses derived from it are otherwise hoisted out of the item loop and spilled
      const int j = fresh_index(threadIdx.x) & 63;
      float x = 0.f;
      if (j < ci.len) {
        ((float*)a.dbeta.ptr)[row_off(a.dbeta, ci.b, ci.tok + j, h)] = s_dbeta[0][j] + s_dbeta[1][j] + s_dbv[j];
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
    if constexpr (NBUF == 1) lds_barrier();                                              // R(0) of the next item
    par ^= 1;
  }
}

}  // namespace lmoe
