// Backward kernels of chunk_simple_gla (one scalar log-decay per token and head).
// Notation per chunk: b = inclusive cumsum of g, e_b = e^{b}, e_d = e^{b_C - b},
// Gamma_ij = e^{b_i - b_j} [i >= j], P = (q k^T) . Gamma, S = state at chunk start,
// dS' = gradient w.r.t. the state at chunk end.
//
//   k_bwd_dv    : chunk-parallel   dv = scale P^T do + (k . e_d) dS'
//   k_state_bwd : reverse sequential pass over the chunks of one (sequence, head, V-slice):
//                 writes dS' of every chunk (dhs);  dS = e^{b_C} dS' + scale (q . e_b)^T do
//   k_bwd_dqk   : chunk-parallel   dq, dk, gate gradient
//                 db_i = q_i.dq_i - k_i.dk_i (+ on the last row sum_j (dk_d . k_d)_j + e^{b_C} <S, dS'>),
//                 dg = reverse cumsum of db.
//   k_bwd_dqkv  : k_bwd_dqk and k_bwd_dv in one kernel (2-byte elements; the fp32 path runs the two)
#pragma once
#include "lmoe_seq.hpp"
#include "lmoe_scalar_fwd.hpp"   // scale_frag

namespace lmoe {

// ------------------------------------------------------------------------- //
// dv' = scale P^T do + (k . e_d) dS'        grid = (NT, H, V / BV)
// (dhs holds dS'^T: [V][K])
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BV, bool LOCAL>
__global__ __launch_bounds__(NTHR) void k_bwd_dv(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDC = CH + LPAD, LDV = BV + LPAD;
  constexpr int NB = BV / 16;
  // One-shot work-groups: what hides their load latency is the number of them a CU holds, so LDS is used twice.
  //   region A: q (for P), then dS'^T;   region B: do, then the staging strips of the result;   k and P^T apart.
  // Every load is requested up front and waits in registers for its region.
  constexpr int RA = (CH * LDK > (LOCAL ? 8 : BV * LDK)) ? CH * LDK : BV * LDK;
  constexpr int RB = (CH * LDV > 4 * 16 * LDV) ? CH * LDV : 4 * 16 * LDV;
  __shared__ __attribute__((aligned(16))) T s_ra[RA];
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];
  __shared__ __attribute__((aligned(16))) T s_rb[RB];
  __shared__ __attribute__((aligned(16))) T s_PT[CH * LDC];
  __shared__ float s_b[64], s_ed[64];
  T* s_q = s_ra; T* s_dhT = s_ra;
  T* s_do = s_rb; T* s_stg = s_rb;

  const int cid = blockIdx.x, h = blockIdx.y, v0 = blockIdx.z * BV;
  if (cid >= num_chunks(a)) return;          // launch sized by an upper bound of the chunk count
  const ChunkInfo ci = chunk_info(a, cid);
  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, BV> IOV;
  typedef TileIO<T, BV, K> IOH;
  typename IOH::Regs rh;
  {
    typename IOK::Regs rq, rk;
    IOK::load(rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
    IOK::load(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
    typename IOV::Regs rd;
    IOV::load(rd, row_ptr<T>(a.d_o, ci.b, ci.tok, h) + v0, a.d_o.st, ci.len);
    if constexpr (!LOCAL) IOH::load(rh, (const T*)a.dhs + (((int64_t)cid * a.H + h) * V + v0) * K, K, BV);
    chunk_gate_cumsum(a, ci.b, ci.tok, ci.len, h, s_b, nullptr, s_ed);
    IOK::store_lds(rq, s_q, LDK);
    IOK::store_lds(rk, s_k, LDK);
    IOV::store_lds(rd, s_do, LDV);
  }
  lds_barrier();
  {
    // P^T stored as s_PT[j][i]; wave w computes rows i = 16w.. of P and writes them transposed
    f32x4 s[1][4];
    acc_zero(s);
    gemm<T, 1, 4, false, false>(s, s_q, LDK, 16 * wv, s_k, LDK, 0, 0, K);
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r >= cc) ? s[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds_t<T>(p, s_PT, LDC, 16 * wv, 16 * nj);
    }
  }
  lds_barrier();                                                                         // q is dead
  if constexpr (!LOCAL) IOH::store_lds(rh, s_dhT, LDK);
  f32x4 dv[1][NB];
  acc_zero(dv);
  gemm<T, 1, NB, false, true>(dv, s_PT, LDC, 16 * wv, s_do, LDV, 0, 0, CH);
#pragma unroll
  for (int ni = 0; ni < NB; ++ni) dv[0][ni] *= a.scale;
  lds_barrier();                                                                         // dS'^T staged; do is dead
  if constexpr (!LOCAL) {
    f32x4 t[1][NB];
    acc_zero(t);
    gemm<T, 1, NB, false, false>(t, s_k, LDK, 16 * wv, s_dhT, LDK, 0, 0, K);
#pragma unroll
    for (int ni = 0; ni < NB; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) dv[0][ni][i] = __builtin_fmaf(t[0][ni][i], s_ed[16 * wv + 4 * (l >> 4) + i], dv[0][ni][i]);
  }
  const lmoe_tensor& dst = LOCAL ? a.dvnew : a.dv;
  store_strip<T, NB>(dv, s_stg + wv * 16 * LDV, row_ptr<T>(dst, ci.b, ci.tok + 16 * wv, h) + v0, dst.st,
                     ci.len - 16 * wv, 1.0f);
}

// ------------------------------------------------------------------------- //
// reverse state pass: producer / consumer work-group of 512 threads (mirror of k_state_fwd)
//   grid = ceil(N*H / 8) * 8 * (V / BV) work-groups (1-D); V-slices of one (sequence, head)
//   share an XCD.  dS slice [K x BV] lives in fp32 MFMA accumulators of waves 0-3 (consumers):
//        dS' -> LDS | B1 | B2 | dS = e^{b_C} dS' + q^T (scale e_b do)
//   Waves 4-7 (loaders) keep the next chunks' q, do in flight, stage them unscaled and write
//   dhs (layout [V][K]).  Both teams meet at the same barriers.
// ------------------------------------------------------------------------- //
// NORM (ungated calls with the output normalised in the forward pass): d_o is the gradient of the normalised output
// o' = o / D, D = den + eps.  The pass then runs on do = d_o / D (folded into the row factor of the do fragments) and
// carries, beside dS, the gradient dz of the column of ones that forms den, whose "do" is dden_i = -(d_o_i . o'_i) / D_i.
// A V slice sees only its columns of d_o and o': it forms the partial row dots over those, and since everything
// downstream is linear in dden it carries the partial dz that belongs to them; the chunk-parallel kernel adds the
// partial sums of all slices.  Per chunk, head and 32 columns of V one row of norm_ws: [64] scale dden (partial),
// [K] dz at the end of the chunk (partial); a slice of 64 columns fills the first of its two rows and zeroes the other.
// NORM = 2: the forward handed out o undivided and den beside it (a caller that adds the den of several key blocks
// before it divides): d_o is the gradient of o as it stands and dden comes in as a tensor; it enters once, in the first
// V slice (the other slices carry zeros).
constexpr int NORM_SLOT_COLS = 32;
template <typename T, int K, int V, int BV, int NORM = 0>
__global__ __launch_bounds__(2 * NTHR) void k_state_bwd(const lmoe_args a) {
  constexpr int LDK = K + LPAD, LDU = BV + LPAD;
  constexpr int MB = K / 64, NB = BV / 16;
  static_assert(!NORM || sizeof(T) == 2, "the normalised pass exists for 2-byte elements");
  constexpr int WS_ROW = CH + K, WS_SLOTS = V / NORM_SLOT_COLS, SLOTS_PER_SLICE = BV / NORM_SLOT_COLS;
  // bf16: two operand buffers; fp32 (the parity path) has LDS for one and pays extra barriers
  constexpr int NBUF = sizeof(T) == 2 ? 2 : 1;
  __shared__ __attribute__((aligned(16))) T s_q[NBUF][CH * LDK];             // q       [64][K]
  __shared__ __attribute__((aligned(16))) T s_do[NBUF][CH * LDU];            // do      [64][BV]
  __shared__ __attribute__((aligned(16))) T s_dST[BV * LDK];                 // dS'^T   [BV][K]
  __shared__ __attribute__((aligned(16))) float s_b[NBUF][64], s_qs[NBUF][64], s_ed[NBUF][64];
  __shared__ float s_dec[NBUF];
  __shared__ __attribute__((aligned(16))) float s_dd[NORM ? NBUF : 1][NORM ? 64 : 4];    // NORM: scale dden (partial)

  constexpr int NVS = V / BV;
  const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
  const int vsl = jj % NVS, pair = (jj / NVS) * 8 + xcd;
  if (pair >= a.N * a.H) return;
  const int v0 = vsl * BV, h = pair % a.H, n = seq_at(a, pair / a.H);
  const SeqInfo sq = seq_info(a, n);
  const int l = lane_id();
  const int team = threadIdx.x / NTHR;      // 0: consumers, 1: loaders
  const bool producer = team == 1;
  // NORM: the rows of norm_ws of this slice in chunk c
  auto ws_row = [&](int c) {
    return a.norm_ws + (((int64_t)(sq.chunk0 + c) * a.H + h) * WS_SLOTS + vsl * SLOTS_PER_SLICE) * WS_ROW;
  };
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

  if (producer) {
    // ------------------------------- producers -------------------------------------------
    constexpr int PF = 2;
    // (NORM: the slice of the normalised output, D of the rows this thread holds of it and of row = lane; c = chunk)
    struct Pre { typename IOK::Regs rq; typename IOV::Regs rd, ro; float rD[IOV::PASSES], dl; uint32_t graw; int len, c; };
    Pre pre[PF];
    const int pw = wave_id() - 4;
    const bool gated = a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr;
    const void* gptr = gated ? a.g.ptr : a.k.ptr;
    const float scale = a.scale;
    // always issued, chunk index clamped (see k_state_fwd)
    auto issue = [&](Pre& P, int c) {
      c = max(c, 0);
      const int tok = sq.tok0 + c * CH;
      const int len = min(CH, sq.len - c * CH);
      IOK::load_nomask(P.rq, row_ptr<T>(a.q, sq.b, tok, h), a.q.st, len);
      IOV::load_nomask(P.rd, row_ptr<T>(a.d_o, sq.b, tok, h) + v0, a.d_o.st, len);
      P.len = len;
      P.graw = load_scalar_raw(gptr, a.g_dtype, gated ? row_off(a.g, sq.b, tok + min(l, len - 1), h) : 0);
      if constexpr (NORM == 1) {
        P.c = c;
        IOV::load_nomask(P.ro, row_ptr<T>(a.o, sq.b, tok, h) + v0, a.o.st, len);
        const float* den = (const float*)a.den.ptr;
#pragma unroll
        for (int p = 0; p < IOV::PASSES; ++p) {
          int row, col; IOV::coords(p, row, col);
          P.rD[p] = den[row_off(a.den, sq.b, tok + min(row, len - 1), h)];
        }
        P.dl = den[row_off(a.den, sq.b, tok + min(l, len - 1), h)];
      }
      if constexpr (NORM == 2) {
        P.c = c;
        P.dl = ((const float*)a.dden.ptr)[row_off(a.dden, sq.b, tok + min(l, len - 1), h)];
      }
    };
    auto stage = [&](Pre& P, int buf) {
      if constexpr (NORM == 2) {
        if (pw == 0) {                     // scale dden as given, once: in the first V slice
          float* ws = ws_row(P.c);
          const float dd = (vsl == 0 && l < P.len) ? scale * P.dl : 0.f;
          s_dd[buf][l] = dd;
          ws[l] = dd;
          if constexpr (SLOTS_PER_SLICE == 2) ws[WS_ROW + l] = 0.f;
        }
      }
      if constexpr (NORM == 1) {
        // partial row dots of d_o and o' over the columns of this slice -> scale dden (partial), for the consumers and
        // for the chunk-parallel kernel; from the registers as loaded (rows past the end of a partial chunk: zero)
        float* ws = ws_row(P.c);
#pragma unroll
        for (int p = 0; p < IOV::PASSES; ++p) {
          int row, col; IOV::coords(p, row, col);
          float sum = 0.f;
#pragma unroll
          for (int i = 0; i < IOV::VEC; ++i) sum += ET<T>::to_f(P.rd.v[p][i]) * ET<T>::to_f(P.ro.v[p][i]);
          sum = group_sum<IOV::VPR>(sum);               // the VPR lanes that hold one row are neighbours
          const float dd = row < P.len ? -scale * sum / P.rD[p] : 0.f;
          if (col == 0) {
            s_dd[buf][row] = dd;
            ws[row] = dd;
            if constexpr (SLOTS_PER_SLICE == 2) ws[WS_ROW + row] = 0.f;
          }
        }
      }
      IOK::mask(P.rq, P.len);
      IOV::mask(P.rd, P.len);
      IOK::store_lds(P.rq, s_q[buf], LDK);
      IOV::store_lds(P.rd, s_do[buf], LDU);
      if constexpr (NORM == 1) {
        if (pw == 0) {                     // ungated: the row factor of the do fragments is scale / D
          s_b[buf][l] = 0.f;
          s_qs[buf][l] = scale / P.dl;
          s_ed[buf][l] = 1.f;
          if (l == 0) s_dec[buf] = 1.f;
        }
      } else if (pw == 0) {
        const float x = wave_incl_scan((gated && l < P.len) ? scalar_from_raw(P.graw, a.g_dtype) : 0.f);
        const float xl = __shfl(x, 63, 64);
        s_b[buf][l] = x;
        s_qs[buf][l] = scale * expf(x);
        s_ed[buf][l] = expf(xl - x);
        if (l == 0) s_dec[buf] = expf(xl);
      }
    };
#pragma unroll
    for (int j = 0; j < PF; ++j) issue(pre[j], sq.nchunks - 1 - j);
    stage(pre[0], 0);
    issue(pre[0], sq.nchunks - 1 - PF);
    lds_barrier();                                   // P0: the first chunk's tiles are complete
    for (int it0 = 0; it0 < sq.nchunks; it0 += PF) {
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        const int it = it0 + j;
        if (it >= sq.nchunks) break;
        const int c = sq.nchunks - 1 - it;
        const int nb = NBUF == 2 ? ((it + 1) & 1) : 0;
        lds_barrier();                                                                   // B1
        IOHT::lds_to_global(s_dST, LDK, (T*)a.dhs + (((int64_t)(sq.chunk0 + c) * a.H + h) * V + v0) * K, K, BV);
        if constexpr (NBUF == 2) {
          if (c > 0) stage(pre[(j + 1) % PF], nb);
        }
        lds_barrier();                                                                   // B2
        if constexpr (NBUF == 1) {
          lds_barrier();                                                                 // B3: buffer read
          if (c > 0) stage(pre[(j + 1) % PF], 0);
          lds_barrier();                                                                 // B4: tiles complete
        }
        issue(pre[(j + 1) % PF], c - 1 - PF);
      }
    }
    return;
  }

  // --------------------------------- consumers -------------------------------------------
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
        for (int i = 0; i < 4; ++i)
          dS[mi][ni][i] = p[(int64_t)(krow0 + acc_row(mi, i)) * V + v0 + acc_col(ni)];
  }
  f32x4 dz[NORM ? MB : 1];                  // NORM: gradient of the column of ones (the same sum in every column)
#pragma unroll
  for (int mi = 0; mi < (NORM ? MB : 1); ++mi) dz[mi] = f32x4{0.f, 0.f, 0.f, 0.f};
  lds_barrier();                                     // P0
  for (int it = 0; it < sq.nchunks; ++it) {
    const int c = sq.nchunks - 1 - it;
    const int cur = NBUF == 2 ? (it & 1) : 0;
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) acc_to_lds_t<T>(dS[mi][ni], s_dST, LDK, krow0 + 16 * mi, 16 * ni);
    if constexpr (NORM) {
      // dz at the end of chunk c (partial): from this team, which has no loads in flight that a store could wait for
      if ((l & 15) == 0) {
        float* ws = ws_row(c) + CH;
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) {
          const int row = krow0 + 16 * mi + 4 * (l >> 4);
          *(f32x4*)&ws[row] = dz[mi];
          if constexpr (SLOTS_PER_SLICE == 2) *(f32x4*)&ws[WS_ROW + row] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
      }
    }
    lds_barrier();                                                                       // B1
    const float dec = s_dec[cur];
    f32x4 t[1][NB];
    acc_zero(t);
    lds_barrier();                                                                       // B2
#pragma unroll
    for (int mi = 0; mi < MB; ++mi)
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) dS[mi][ni] *= dec;
    // dS += q^T (scale e_b do): the row scaling is applied to the do fragments in registers
    for (int kk = 0; kk < CH; kk += 32) {
      typename ET<T>::frag af[MB], bf[NB];
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) af[mi] = ET<T>::load_frag_t(s_q[cur], LDK, kk, krow0 + 16 * mi);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        bf[ni] = ET<T>::load_frag_t(s_do[cur], LDU, kk, 16 * ni);
        scale_frag<T>(bf[ni], &s_qs[cur][kk + 8 * (l >> 4)]);
      }
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(dS[mi][ni], af[mi], bf[ni]);
      if constexpr (NORM) {                 // dz += q^T (scale dden): sixteen equal columns
        const f32x4 d0 = *(const f32x4*)&s_dd[cur][kk + 8 * (l >> 4)], d1 = *(const f32x4*)&s_dd[cur][kk + 8 * (l >> 4) + 4];
        typename ET<T>::frag fd;
#pragma unroll
        for (int e = 0; e < 4; ++e) { fd[e] = (bf16)d0[e]; fd[e + 4] = (bf16)d1[e]; }
#pragma unroll
        for (int mi = 0; mi < MB; ++mi) ET<T>::mma(dz[mi], af[mi], fd);
      }
    }
    if constexpr (NBUF == 1) {
      lds_barrier();                                                                     // B3
      lds_barrier();                                                                     // B4
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

// ------------------------------------------------------------------------- //
// dq, dk, gate gradient        persistent: one work-group per CU, one item = (chunk, head)
//   phase A: loop over V-slices of width BVH accumulating
//              dP = do v^T, dq_i = do S^T, dk_d = v dS'^T
//            (hs, dhs hold S^T, dS'^T: [V][K]; the slice tiles are [BVH][K])
//   phase B: dq = scale e_b dq_i + (scale dP . Gamma) k ; dk = e_d dk_d + (scale dP . Gamma)^T q
//            with one LDS copy of (scale dP . Gamma)^T and q, k stored as loaded
//   Work-group = 2 teams of 4 waves on one barrier script.  Team 0 (compute) reads LDS and drives
//   the matrix cores; wave w owns chunk rows 16 w .. 16 w + 15.  Team 1 (loaders) keeps the next
//   slice and the next q, k in flight in registers and stages them into two alternating slice
//   buffers, so a slice is being filled while the previous one is being consumed; the phase B
//   tiles lie over the second buffer.  It also forms <S, dS'> from the registers it holds and the
//   gate cumsum of the chunk.
//   Script per item (NS slices):  R(0) .. R(NS-1) | D | A | b | c | E
//     loaders : R(s): stage slice s+1 | D: stage q, k, gates | A: stage slice 0 of the next item
//     compute : R(s): products of slice s | D, A | (dP . Gamma)^T -> LDS | b | products, combine |
//               c | stores | E
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int BVH>
__global__ __launch_bounds__(2 * NTHR) void k_bwd_dqk(const lmoe_args a) {
  constexpr int LDV = BVH + LPAD, LDC = CH + LPAD, LDK = K + LPAD;
  constexpr int NBK = K / 16, NS = V / BVH;
  // tiles of one V-slice
  constexpr int A_DO = 0, A_V = A_DO + CH * LDV, A_H = A_V + CH * LDV, A_DH = A_H + BVH * LDK,
                A_END = A_DH + BVH * LDK;
  // phase B tiles (relative to the second slice buffer)
  constexpr int B_DPT = 0, B_K = B_DPT + CH * LDC, B_Q = B_K + CH * LDK, B_END = B_Q + CH * LDK;
  constexpr int BUF1 = A_END;
  constexpr int NELEM = BUF1 + (A_END > B_END ? A_END : B_END);
  __shared__ __attribute__((aligned(16))) T smem[NELEM];
  __shared__ float s_b[64], s_eb[64], s_ed[64], s_db[64], s_red[8];

  const int l = lane_id();
  const int team = threadIdx.x / NTHR;
  typedef TileIO<T, CH, BVH> IOV;
  typedef TileIO<T, BVH, K> IOH;
  typedef TileIO<T, CH, K> IOK;
  const lmoe_tensor& vs = a.v;
  const int nitems = num_chunks(a) * a.H;
  if (nitems <= 0) return;                   // (a chunk count read on the device may be zero)
  const int stride = gridDim.x;

  if (team == 1) {
    // --------------------------------- loaders -------------------------------------------
    struct SliceRegs { typename IOV::Regs rd, rv; typename IOH::Regs rh, rdh; int len; };
    struct QKRegs { typename IOK::Regs rq, rk; uint32_t graw; int len; };
    SliceRegs S;
    QKRegs Q;
    // Every prefetch is issued unconditionally (item index clamped to the last item): a load that
    // is skipped on some path would make the compiler drain all outstanding loads at every use.
    auto issue_slice = [&](int it, int vv) {
      it = min(it, nitems - 1);
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      S.len = ci.len;
      IOV::load_nomask(S.rd, row_ptr<T>(a.d_o, ci.b, ci.tok, h) + vv, a.d_o.st, ci.len);
      IOV::load_nomask(S.rv, row_ptr<T>(vs, ci.b, ci.tok, h) + vv, vs.st, ci.len);
      IOH::load_nomask(S.rh, (const T*)a.hs + (((int64_t)cid * a.H + h) * V + vv) * K, K, BVH);
      IOH::load_nomask(S.rdh, (const T*)a.dhs + (((int64_t)cid * a.H + h) * V + vv) * K, K, BVH);
    };
    auto issue_qk = [&](int it) {
      it = min(it, nitems - 1);
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      Q.len = ci.len;
      IOK::load_nomask(Q.rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
      IOK::load_nomask(Q.rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
      Q.graw = gate_prefetch(a, ci.b, ci.tok, ci.len, h);
    };
    float hdh = 0.f;   // partial <S, dS'> of the item whose slices are being staged
    auto stage_slice = [&](int buf) {
      T* base = smem + buf * BUF1;
#pragma unroll
      for (int p = 0; p < IOH::PASSES; ++p)
#pragma unroll
        for (int i = 0; i < IOH::VEC; ++i) hdh += ET<T>::to_f(S.rh.v[p][i]) * ET<T>::to_f(S.rdh.v[p][i]);
      IOV::mask(S.rd, S.len);
      IOV::mask(S.rv, S.len);
      IOV::store_lds(S.rd, base + A_DO, LDV);
      IOV::store_lds(S.rv, base + A_V, LDV);
      IOH::store_lds(S.rh, base + A_H, LDK);
      IOH::store_lds(S.rdh, base + A_DH, LDK);
    };
    // the slice after slice s of item it
    auto issue_next = [&](int it, int s) {
      if (s + 1 < NS) issue_slice(it, (s + 1) * BVH); else issue_slice(it + stride, 0);
    };
    const int it0 = blockIdx.x;
    issue_slice(it0, 0);
    issue_qk(it0);
    // the first loads may be ordered freely by the compiler; were they still pending at the loop
    // header, its wait-count analysis would carry that order into every iteration
    wait_all_loads();
    stage_slice(0);
    issue_next(it0, 0);
    for (int it = it0; it < nitems; it += stride) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        lds_barrier();                                                                   // R(s)
        if (s + 1 < NS) {
          stage_slice((s + 1) & 1);        // its buffer was left when the compute team passed R(s)
          issue_next(it, s + 1);
        }
      }
      lds_barrier();                                                                     // D
      gate_finish_wave(a, Q.graw, Q.len, l, wave_id() == 4, s_b, s_eb, s_ed);
      IOK::mask(Q.rq, Q.len);
      IOK::mask(Q.rk, Q.len);
      IOK::store_lds(Q.rq, smem + BUF1 + B_Q, LDK);
      IOK::store_lds(Q.rk, smem + BUF1 + B_K, LDK);
      hdh = wave_sum(hdh);
      if (l == 0) s_red[wave_id() - 4] = hdh;
      hdh = 0.f;
      lds_barrier();                                                                     // A
      issue_qk(it + stride);
      stage_slice(0);                      // slice 0 of the next item (buffer 0 is idle in phase B)
      issue_next(it + stride, 0);
      lds_barrier();                                                                     // b
      lds_barrier();                                                                     // c
      lds_barrier();                                                                     // E
    }
    return;
  }

  // --------------------------------- compute ---------------------------------------------
  const int wv = wave_id();
  const int fr = l & 15, fg = 8 * (l >> 4);
  for (int it = blockIdx.x; it < nitems; it += stride) {
    const int cid = it / a.H, h = it % a.H;
    const ChunkInfo ci = chunk_info(a, cid);
    f32x4 dP[1][4], dqi[1][NBK], dkd[1][NBK];
    acc_zero(dP); acc_zero(dqi); acc_zero(dkd);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      lds_barrier();                                                                     // R(s)
      const T* base = smem + (s & 1) * BUF1;
      const T* DO = base + A_DO; const T* VN = base + A_V;
      const T* HT = base + A_H; const T* DHT = base + A_DH;
#pragma unroll
      for (int kk = 0; kk < BVH; kk += 32) {
        const typename ET<T>::frag aDO = ET<T>::load_frag(DO + (16 * wv + fr) * LDV + kk + fg);
        const typename ET<T>::frag aVN = ET<T>::load_frag(VN + (16 * wv + fr) * LDV + kk + fg);
#pragma unroll
        for (int nj = 0; nj < 4; ++nj)
          ET<T>::mma(dP[0][nj], aDO, ET<T>::load_frag(VN + (16 * nj + fr) * LDV + kk + fg));
        __builtin_amdgcn_sched_barrier(0);     // bounds the fragments in flight (register budget)
#pragma unroll
        for (int ni = 0; ni < NBK; ++ni) {
          const typename ET<T>::frag bH = ET<T>::load_frag_t(HT, LDK, kk, 16 * ni);
          ET<T>::mma(dqi[0][ni], aDO, bH);
          ET<T>::mma(dkd[0][ni], aVN, ET<T>::load_frag_t(DHT, LDK, kk, 16 * ni));
          if (ni % 4 == 3) __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    lds_barrier();                                                                       // D
    lds_barrier();                                                                       // A
    T* PB = smem + BUF1;
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * nj + (l & 15);
        p[i] = (r >= cc) ? a.scale * dP[0][nj][i] * texp<T>(s_b[r] - s_b[cc]) : 0.f;
      }
      acc_to_lds_t<T>(p, PB + B_DPT, LDC, 16 * wv, 16 * nj);      // [j][i]
    }
    lds_barrier();                                                                       // b
    f32x4 dq[1][NBK], dk[1][NBK];
    acc_zero(dq); acc_zero(dk);
    // dq_intra[i][c] = sum_j dPG[i][j] k[j][c] : A = dPG^T stored [j][i] (contraction along rows)
    gemm<T, 1, NBK, true, true>(dq, PB + B_DPT, LDC, 16 * wv, PB + B_K, LDK, 0, 0, CH);
    __builtin_amdgcn_sched_barrier(0);
    // dk_intra[j][c] = sum_i dPG[i][j] q[i][c] : A = dPG^T rows j (contraction along columns)
    gemm<T, 1, NBK, false, true>(dk, PB + B_DPT, LDC, 16 * wv, PB + B_Q, LDK, 0, 0, CH);
    __builtin_amdgcn_sched_barrier(0);
    // combine and form db_i = q_i.dq_i - k_i.dk_i ; kk = sum_j (dk_d . k_d)_j
    float dbp[4] = {0.f, 0.f, 0.f, 0.f};
    float kk = 0.f;
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * (l >> 4) + i, cc = 16 * ni + (l & 15);
        const float qv = ET<T>::to_f(PB[B_Q + r * LDK + cc]);
        const float kv = ET<T>::to_f(PB[B_K + r * LDK + cc]);
        const float dqv = a.scale * s_eb[r] * dqi[0][ni][i] + dq[0][ni][i];
        const float dkdv = s_ed[r] * dkd[0][ni][i];
        const float dkv = dkdv + dk[0][ni][i];
        dbp[i] += qv * dqv - kv * dkv;
        kk += kv * dkdv;
        dq[0][ni][i] = dqv;
        dk[0][ni][i] = dkv;
      }
    // reduce db over the 16 lanes that share a row group, kk over the whole team
#pragma unroll
    for (int i = 0; i < 4; ++i) dbp[i] = group_sum<16>(dbp[i]);
    if ((l & 15) == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) s_db[16 * wv + 4 * (l >> 4) + i] = dbp[i];
    }
    kk = wave_sum(kk);
    if (l == 0) s_red[4 + wv] = kk;
    lds_barrier();     // c: q, k tiles are dead from here: wave-private slices become store staging
    {
      T* stg = PB + B_K + wv * 16 * LDK;    // this wave's 16 rows of the k tile, then of the q tile
      store_strip<T, NBK>(dq, stg, row_ptr<T>(a.dq, ci.b, ci.tok + 16 * wv, h), a.dq.st, ci.len - 16 * wv, 1.0f);
      T* stg2 = PB + B_Q + wv * 16 * LDK;
      store_strip<T, NBK>(dk, stg2, row_ptr<T>(a.dk, ci.b, ci.tok + 16 * wv, h), a.dk.st, ci.len - 16 * wv, 1.0f);
    }
    if (threadIdx.x < 64) {
      const int j = threadIdx.x;
      float x = s_db[j];
      // last-row term; rows past the end of a partial chunk carry zero q, k, so the term may sit
      // on the last valid row without changing the reverse cumulative sum
      const float hsum = s_red[0] + s_red[1] + s_red[2] + s_red[3];
      const float ksum = s_red[4] + s_red[5] + s_red[6] + s_red[7];
      if (j == ci.len - 1) x += ksum + expf(s_b[63]) * hsum;
      x = wave_rev_scan(x);   // dg
      if (a.dg.ptr && j < ci.len) ((float*)a.dg.ptr)[row_off(a.dg, ci.b, ci.tok + j, h)] = x;
    }
    lds_barrier();     // E: the second buffer and the gate arrays go to the next item
  }
}

// ------------------------------------------------------------------------- //
// dq, dk, dv, gate gradient in one kernel (2-byte elements)     persistent: one work-group per CU,
// one item = (chunk, head).  k_bwd_dqk with the work of k_bwd_dv folded in: the do, dS'^T, q and k tiles that dv
// needs lie in LDS for dq and dk anyway, so dv costs this kernel no load, and q, k, do and dhs are not fetched a
// second time by a kernel of their own.
//   start of an item : wave w forms columns 16 w .. of P = (q k^T) . Gamma transposed (lane: four consecutive rows i
//                      of one column j, 8-byte writes into its own rows of the P^T tile) and keeps those rows and
//                      its k rows as matrix operands in registers
//   slice s          : dP, dq_i, dk_d as in k_bwd_dqk, and  dv^T = scale do^T P + dS'^T (k . e_d)^T  formed
//                      transposed, so that a lane holds four consecutive columns of one token: 8-byte stores
//                      straight from the accumulators
//   phase B          : as in k_bwd_dqk; (scale dP . Gamma)^T takes the place of P^T
//   q, k and the gate arrays of an item are staged while the item before stores its results (its own staging strips
//   lie in the slice buffer that is idle then); the gate arrays alternate between two sets.
//   Script per item (NS slices):  [slice 0] R(1) .. R(NS-1) | D | A | b | c | E
//     loaders : R(s): stage slice s+1 | D: <S, dS'> | A: stage slice 0 of the next item | c: stage q, k, gates of
//               the next item, request those of the one after
//     compute : P^T strip | products of slice s, dv stores | D, A | (dP . Gamma)^T -> LDS | b | products, combine |
//               c | stores | E
// Every sum is formed in the order of k_bwd_dv and k_bwd_dqk: the results are theirs bit for bit.
// ------------------------------------------------------------------------- //
// NORM (see k_state_bwd): d_o is the gradient of the normalised output.  With rD = 1 / D, dd = scale dden (the sum of
// the partial rows of norm_ws), z = the sum of the keys before the chunk (zs) and dz = the gradient of the column of
// ones at the end of the chunk (the sum of the partial rows of norm_ws), ungated:
//   dv: P^T formed with its rows i scaled by rD_i;   dP_ij -> scale dP_ij rD_i + dd_i;
//   dq_i = scale rD_i dq_i,inter + dd_i z + (dP k)_i;   dk_j = dk_d,j + dz + (dP^T q)_j
// i.e. row and column factors on sums the kernel forms anyway; d_o itself is staged as it is.
// NORM = 2 (o undivided, den beside it, see k_state_bwd): rD = 1 and dd, dz come from the rows of norm_ws alone.
template <typename T, int K, int V, int BVH, int NORM = 0>
__global__ __launch_bounds__(2 * NTHR) void k_bwd_dqkv(const lmoe_args a) {
  static_assert(sizeof(T) == 2, "2-byte elements");
  constexpr int WS_ROW = CH + K, WS_SLOTS = V / NORM_SLOT_COLS;
  static_assert(CH + K <= NTHR, "one loader thread per entry of a row of norm_ws");
  constexpr int LDV = BVH + LPAD, LDC = CH + LPAD, LDK = K + LPAD;
  constexpr int NBK = K / 16, NS = V / BVH, NBV = BVH / 16, KS = K / 32, CS = CH / 32;
  // tiles of one V-slice (two buffers)
  constexpr int A_DO = 0, A_V = A_DO + CH * LDV, A_H = A_V + CH * LDV, A_DH = A_H + BVH * LDK,
                A_END = A_DH + BVH * LDK;
  constexpr int BUF1 = A_END;
  // tiles of the item
  constexpr int B_PT = 2 * A_END, B_K = B_PT + CH * LDC, B_Q = B_K + CH * LDK, NELEM = B_Q + CH * LDK;
  static_assert(2 * 4 * 16 * LDK <= A_END, "the store staging strips fit the idle slice buffer");
  __shared__ __attribute__((aligned(16))) T smem[NELEM];
  __shared__ __attribute__((aligned(16))) float s_b[2][64], s_eb[2][64], s_ed[2][64];
  __shared__ float s_db[64], s_red[8];
  // NORM: rD and dd per row, z and dz per key column (two sets, like the gate arrays)
  __shared__ __attribute__((aligned(16))) float s_rD[NORM ? 2 : 1][NORM ? 64 : 4], s_dd[NORM ? 2 : 1][NORM ? 64 : 4];
  __shared__ __attribute__((aligned(16))) float s_z[NORM ? 2 : 1][NORM ? K : 4], s_dz[NORM ? 2 : 1][NORM ? K : 4];

  const int l = lane_id();
  const int team = threadIdx.x / NTHR;
  typedef TileIO<T, CH, BVH> IOV;
  typedef TileIO<T, BVH, K> IOH;
  typedef TileIO<T, CH, K> IOK;
  const int nitems = num_chunks(a) * a.H;
  if (nitems <= 0) return;                   // (a chunk count read on the device may be zero)
  const int stride = gridDim.x;

  if (team == 1) {
    // --------------------------------- loaders -------------------------------------------
    struct SliceRegs { typename IOV::Regs rd, rv; typename IOH::Regs rh, rdh; int len; };
    // (NORM: thread e < 64 + K holds entry e of the rows of norm_ws and D of row e or z of column e - 64)
    struct QKRegs { typename IOK::Regs rq, rk; uint32_t graw; int len; float ws[NORM ? WS_SLOTS : 1], x; };
    SliceRegs S;
    QKRegs Q;
    const int e_norm = min((int)(threadIdx.x & (NTHR - 1)), WS_ROW - 1);
    // Every prefetch is issued unconditionally (item index clamped to the last item): a load that
    // is skipped on some path would make the compiler drain all outstanding loads at every use.
    auto issue_slice = [&](int it, int vv) {
      it = min(it, nitems - 1);
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      S.len = ci.len;
      IOV::load_nomask(S.rd, row_ptr<T>(a.d_o, ci.b, ci.tok, h) + vv, a.d_o.st, ci.len);
      IOV::load_nomask(S.rv, row_ptr<T>(a.v, ci.b, ci.tok, h) + vv, a.v.st, ci.len);
      IOH::load_nomask(S.rh, (const T*)a.hs + (((int64_t)cid * a.H + h) * V + vv) * K, K, BVH);
      IOH::load_nomask(S.rdh, (const T*)a.dhs + (((int64_t)cid * a.H + h) * V + vv) * K, K, BVH);
    };
    auto issue_qk = [&](int it) {
      it = min(it, nitems - 1);
      const int cid = it / a.H, h = it % a.H;
      const ChunkInfo ci = chunk_info(a, cid);
      Q.len = ci.len;
      IOK::load_nomask(Q.rq, row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, ci.len);
      IOK::load_nomask(Q.rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len);
      Q.graw = gate_prefetch(a, ci.b, ci.tok, ci.len, h);
      if constexpr (NORM) {
        const float* ws = a.norm_ws + (int64_t)it * WS_SLOTS * WS_ROW + e_norm;          // it = cid * H + h
#pragma unroll
        for (int sl = 0; sl < WS_SLOTS; ++sl) Q.ws[sl] = ws[sl * WS_ROW];
        const lmoe_tensor& dt = NORM == 1 ? a.den : a.dden;               // (NORM = 2: read, not used, for rows)
        const float* den = (const float*)dt.ptr + row_off(dt, ci.b, ci.tok + min(e_norm, ci.len - 1), h);
        const float* zc = a.zs + (int64_t)it * K + max(e_norm - CH, 0);
        Q.x = *(e_norm < CH ? den : zc);
      }
    };
    float hdh = 0.f;   // partial <S, dS'> of the item whose slices are being staged
    auto stage_slice = [&](int buf) {
      T* base = smem + buf * BUF1;
#pragma unroll
      for (int p = 0; p < IOH::PASSES; ++p)
#pragma unroll
        for (int i = 0; i < IOH::VEC; ++i) hdh += ET<T>::to_f(S.rh.v[p][i]) * ET<T>::to_f(S.rdh.v[p][i]);
      IOV::mask(S.rd, S.len);
      IOV::mask(S.rv, S.len);
      IOV::store_lds(S.rd, base + A_DO, LDV);
      IOV::store_lds(S.rv, base + A_V, LDV);
      IOH::store_lds(S.rh, base + A_H, LDK);
      IOH::store_lds(S.rdh, base + A_DH, LDK);
    };
    auto stage_qk = [&](int par) {
      if constexpr (NORM) {
        float sum = 0.f;
#pragma unroll
        for (int sl = 0; sl < WS_SLOTS; ++sl) sum += Q.ws[sl];
        const int e = threadIdx.x & (NTHR - 1);
        if (e < CH) {
          s_dd[par][e] = sum;                                // (zero past the end of a partial chunk)
          s_rD[par][e] = e < Q.len ? (NORM == 1 ? 1.f / Q.x : 1.f) : 0.f;
        } else if (e < WS_ROW) {
          s_dz[par][e - CH] = sum;
          s_z[par][e - CH] = Q.x;
        }
      }
      gate_finish_wave(a, Q.graw, Q.len, l, wave_id() == 4, s_b[par], s_eb[par], s_ed[par]);
      IOK::mask(Q.rq, Q.len);
      IOK::mask(Q.rk, Q.len);
      IOK::store_lds(Q.rq, smem + B_Q, LDK);
      IOK::store_lds(Q.rk, smem + B_K, LDK);
    };
    // the slice after slice s of item it
    auto issue_next = [&](int it, int s) {
      if (s + 1 < NS) issue_slice(it, (s + 1) * BVH); else issue_slice(it + stride, 0);
    };
    const int it0 = blockIdx.x;
    issue_slice(it0, 0);
    issue_qk(it0);
    // the first loads may be ordered freely by the compiler; were they still pending at the loop
    // header, its wait-count analysis would carry that order into every iteration
    wait_all_loads();
    stage_slice(0);
    stage_qk(0);
    issue_qk(it0 + stride);
    issue_next(it0, 0);
    lds_barrier();                                                                       // first item staged
    int par = 0;
    for (int it = it0; it < nitems; it += stride, par ^= 1) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        if (s > 0) lds_barrier();                                                        // R(s)
        if (s + 1 < NS) {
          stage_slice((s + 1) & 1);        // its buffer was left when the compute team passed R(s) (s = 0: E)
          issue_next(it, s + 1);
        }
      }
      lds_barrier();                                                                     // D
      hdh = wave_sum(hdh);
      if (l == 0) s_red[wave_id() - 4] = hdh;
      hdh = 0.f;
      lds_barrier();                                                                     // A
      stage_slice(0);                      // slice 0 of the next item (buffer 0 is idle in phase B)
      issue_next(it + stride, 0);
      lds_barrier();                                                                     // b
      lds_barrier();                                                                     // c
      stage_qk(par ^ 1);                   // q, k of this item were read for the last time before c
      issue_qk(it + 2 * stride);
      lds_barrier();                                                                     // E
    }
    return;
  }

  // --------------------------------- compute ---------------------------------------------
  const int wv = wave_id();
  const T* QT = smem + B_Q;
  const T* KT = smem + B_K;
  T* PT = smem + B_PT;
  lds_barrier();                                                                         // first item staged
  int par = 0;
  for (int it = blockIdx.x; it < nitems; it += stride, par ^= 1) {
    const int cid = it / a.H, h = it % a.H;
    const ChunkInfo ci = chunk_info(a, cid);
    // (the lane index refreshed per item: what derives from it is recomputed where it is used instead of being kept,
    // and spilled, for the whole kernel)
    const int lf = fresh_index(l);
    const int fr = lf & 15, g = lf >> 4, fg = 8 * g;
    const int j = 16 * wv + fr;            // the token of this lane in transposed products
    // rows j = 16 wv .. of P^T (zero where i < j), written by and for this wave only
    typename ET<T>::frag fk[KS], fpt[CS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) fk[ks] = ET<T>::load_frag(KT + j * LDK + 32 * ks + fg);
    const float bj = s_b[par][j], edj = s_ed[par][j];
#pragma unroll
    for (int ib = 0; ib < 4; ++ib) {
      bf16x4 y = {(bf16)0.f, (bf16)0.f, (bf16)0.f, (bf16)0.f};
      if (ib >= wv) {
        typename ET<T>::frag fq[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fq[ks] = ET<T>::load_frag(QT + (16 * ib + fr) * LDK + 32 * ks + fg);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ET<T>::mma(acc, fq[ks], fk[ks]);
        const f32x4 bi = *(const f32x4*)&s_b[par][16 * ib + 4 * g];
        if constexpr (NORM) {
          const f32x4 rdi = *(const f32x4*)&s_rD[par][16 * ib + 4 * g];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] *= rdi[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = (bf16)((16 * ib + 4 * g + e >= j) ? acc[e] * texp<T>(bi[e] - bj) : 0.f);
      }
      *(bf16x4*)(PT + j * LDC + 16 * ib + 4 * g) = y;
    }
#pragma unroll
    for (int kq = 0; kq < CS; ++kq) fpt[kq] = ET<T>::load_frag(PT + j * LDC + 32 * kq + fg);

    f32x4 dP[1][4], dqi[1][NBK], dkd[1][NBK];
    acc_zero(dP); acc_zero(dqi); acc_zero(dkd);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      if (s > 0) lds_barrier();                                                          // R(s)
      const T* base = smem + (s & 1) * BUF1;
      const T* DO = base + A_DO; const T* VN = base + A_V;
      const T* HT = base + A_H; const T* DHT = base + A_DH;
#pragma unroll
      for (int kk = 0; kk < BVH; kk += 32) {
        const typename ET<T>::frag aDO = ET<T>::load_frag(DO + (16 * wv + fr) * LDV + kk + fg);
        const typename ET<T>::frag aVN = ET<T>::load_frag(VN + (16 * wv + fr) * LDV + kk + fg);
#pragma unroll
        for (int nj = 0; nj < 4; ++nj)
          ET<T>::mma(dP[0][nj], aDO, ET<T>::load_frag(VN + (16 * nj + fr) * LDV + kk + fg));
        __builtin_amdgcn_sched_barrier(0);     // bounds the fragments in flight (register budget)
#pragma unroll
        for (int ni = 0; ni < NBK; ++ni) {
          const typename ET<T>::frag bH = ET<T>::load_frag_t(HT, LDK, kk, 16 * ni, lf);
          ET<T>::mma(dqi[0][ni], aDO, bH);
          ET<T>::mma(dkd[0][ni], aVN, ET<T>::load_frag_t(DHT, LDK, kk, 16 * ni, lf));
          if (ni % 4 == 3) __builtin_amdgcn_sched_barrier(0);
        }
      }
      // dv^T of the slice: lane = token j, columns 16 ni + 4 g .. + 3
      f32x4 t1[NBV], t2[NBV];
#pragma unroll
      for (int ni = 0; ni < NBV; ++ni) t1[ni] = t2[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kq = 0; kq < CS; ++kq) {
        if (2 * kq + 1 >= wv) {            // rows i < 32 of P^T are zero for the waves 2, 3
#pragma unroll
          for (int ni = 0; ni < NBV; ++ni) ET<T>::mma(t1[ni], ET<T>::load_frag_t(DO, LDV, 32 * kq, 16 * ni, lf), fpt[kq]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int ni = 0; ni < NBV; ++ni)
          ET<T>::mma(t2[ni], ET<T>::load_frag(DHT + (16 * ni + fr) * LDK + 32 * ks + fg), fk[ks]);
        if (ks % 2 == 1) __builtin_amdgcn_sched_barrier(0);     // bounds the fragments in flight (register budget)
      }
      if (j < ci.len) {
        T* drow = row_ptr<T>(a.dv, ci.b, ci.tok + j, h) + s * BVH + 4 * g;
#pragma unroll
        for (int ni = 0; ni < NBV; ++ni) {
          bf16x4 y;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // (the rounding steps of k_bwd_dv: the product with the scale rounded, then one fused multiply-add)
            y[e] = (bf16)__builtin_fmaf(t2[ni][e], edj, __fmul_rn(t1[ni][e], a.scale));
          }
          *(bf16x4*)(drow + 16 * ni) = y;
        }
      }
    }
    lds_barrier();                                                                       // D
    lds_barrier();                                                                       // A
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 p;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * g + i, cc = 16 * nj + fr;
        if constexpr (NORM) p[i] = (r >= cc) ? a.scale * dP[0][nj][i] * s_rD[par][r] + s_dd[par][r] : 0.f;
        else p[i] = (r >= cc) ? a.scale * dP[0][nj][i] * texp<T>(s_b[par][r] - s_b[par][cc]) : 0.f;
      }
      acc_to_lds_t<T>(p, PT, LDC, 16 * wv, 16 * nj, lf);      // [j][i]
    }
    lds_barrier();                                                                       // b
    f32x4 dq[1][NBK], dk[1][NBK];
    acc_zero(dq); acc_zero(dk);
    // dq_intra[i][c] = sum_j dPG[i][j] k[j][c] : A = dPG^T stored [j][i] (contraction along rows)
    gemm<T, 1, NBK, true, true>(dq, PT, LDC, 16 * wv, KT, LDK, 0, 0, CH, lf);
    __builtin_amdgcn_sched_barrier(0);
    // dk_intra[j][c] = sum_i dPG[i][j] q[i][c] : A = dPG^T rows j (contraction along columns)
    gemm<T, 1, NBK, false, true>(dk, PT, LDC, 16 * wv, QT, LDK, 0, 0, CH, lf);
    __builtin_amdgcn_sched_barrier(0);
    // combine and form db_i = q_i.dq_i - k_i.dk_i ; kk = sum_j (dk_d . k_d)_j
    float dbp[4] = {0.f, 0.f, 0.f, 0.f};
    float kk = 0.f;
#pragma unroll
    for (int ni = 0; ni < NBK; ++ni)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = 16 * wv + 4 * g + i, cc = 16 * ni + fr;
        const float qv = ET<T>::to_f(QT[r * LDK + cc]);
        const float kv = ET<T>::to_f(KT[r * LDK + cc]);
        float dqv, dkdv;
        if constexpr (NORM) {
          dqv = a.scale * s_rD[par][r] * dqi[0][ni][i] + s_dd[par][r] * s_z[par][cc] + dq[0][ni][i];
          dkdv = dkd[0][ni][i] + s_dz[par][cc];
        } else {
          dqv = a.scale * s_eb[par][r] * dqi[0][ni][i] + dq[0][ni][i];
          dkdv = s_ed[par][r] * dkd[0][ni][i];
        }
        const float dkv = dkdv + dk[0][ni][i];
        dbp[i] += qv * dqv - kv * dkv;
        kk += kv * dkdv;
        dq[0][ni][i] = dqv;
        dk[0][ni][i] = dkv;
      }
    // reduce db over the 16 lanes that share a row group, kk over the whole team
#pragma unroll
    for (int i = 0; i < 4; ++i) dbp[i] = group_sum<16>(dbp[i]);
    if (fr == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) s_db[16 * wv + 4 * g + i] = dbp[i];
    }
    kk = wave_sum(kk);
    if (lf == 0) s_red[4 + wv] = kk;
    lds_barrier();     // c: the q, k tiles go to the next item; the idle slice buffer is the store staging
    {
      T* stg = smem + BUF1 + wv * 16 * LDK;
      store_strip<T, NBK>(dq, stg, row_ptr<T>(a.dq, ci.b, ci.tok + 16 * wv, h), a.dq.st, ci.len - 16 * wv, 1.0f, lf);
      T* stg2 = smem + BUF1 + (4 + wv) * 16 * LDK;
      store_strip<T, NBK>(dk, stg2, row_ptr<T>(a.dk, ci.b, ci.tok + 16 * wv, h), a.dk.st, ci.len - 16 * wv, 1.0f, lf);
    }
    if (threadIdx.x < 64) {
      const int t = threadIdx.x;
      float x = s_db[t];
      // last-row term; rows past the end of a partial chunk carry zero q, k, so the term may sit
      // on the last valid row without changing the reverse cumulative sum
      const float hsum = s_red[0] + s_red[1] + s_red[2] + s_red[3];
      const float ksum = s_red[4] + s_red[5] + s_red[6] + s_red[7];
      if (t == ci.len - 1) x += ksum + expf(s_b[par][63]) * hsum;
      x = wave_rev_scan(x);   // dg
      if (a.dg.ptr && t < ci.len) ((float*)a.dg.ptr)[row_off(a.dg, ci.b, ci.tok + t, h)] = x;
    }
    lds_barrier();     // E: the staging strips and the P^T tile go to the next item
  }
}

}  // namespace lmoe
