// Gated delta rule, chunk-parallel WY / UT preparation (forward):
//   L = strictlower( diag(beta) (k k^T) . Gamma ),  Gamma_ij = e^{b_i - b_j}
//   Tinv = (I + L)^-1            (unit lower triangular, fp32)
//   w = Tinv (k . beta e^{b}),   u = Tinv (v . beta)
// and the intra-chunk attention matrix the two sequential passes consume,
//   P = (q k^T) . Gamma  (lower triangle incl. the diagonal)
// (not in the lean form below: the register-resident forward pass forms P itself and q is not read here).
// persistent: grid = a few work-groups of 256 threads per CU, item = (chunk, head).  The inputs of
// the next item (q rows as fragments, k, v tiles, gate, beta) are requested at the top of an item and
// stay in flight behind its LDS-only barriers.  Writes w, u, Tinv and P (element type T) and the
// chunk's decay table e^{b}, e^{b_C - b} (fp32).
#pragma once
#include <type_traits>
#include "lmoe_seq.hpp"

namespace lmoe {

// In-LDS inverse of the unit lower triangular matrix I + L (64 x 64, fp32).
//   sL : strictly lower part L (upper part and diagonal must be 0), leading dimension ldl
//   sX : receives (I + L)^-1, leading dimension ldx
//   sY : scratch, one 16 x 17 fp32 block per wave (4 * 272 floats)
// Block forward substitution with 16 x 16 blocks.  The four diagonal blocks are inverted by the
// four waves on the vector ALU (one column per lane).  The off-diagonal blocks follow by block
// distance d = I - J, one block per wave, on the matrix cores in fp32 (v_mfma_f32_16x16x4_f32):
//   Y = sum_{M = J}^{I-1} L_IM X_MJ   (4 d instructions),   X_IJ = - X_II Y   (4 instructions),
// with Y passed through the wave's own scratch block, so a round needs one work-group barrier.
// Must be called by all 256 threads (l, tid: lane and thread index); sL must be complete and sX free
// (barrier before the call).
__device__ __forceinline__ void tri_inverse_64(const float* sL, int ldl, float* sX, int ldx, float* sY, int l, int tid) {
  const int wv = wave_id();
  // clear X (upper blocks stay zero)
  // the six blocks above the diagonal are zero; nothing else writes them, so no barrier before the rest
  {
    const int r = tid >> 4, c = tid & 15;
#pragma unroll
    for (int I = 0; I < 3; ++I)
#pragma unroll
      for (int J = I + 1; J < 4; ++J) sX[(16 * I + r) * ldx + 16 * J + c] = 0.f;
  }
  if (l < 16) {
    // lane c solves column c by forward substitution; every lane reads the same coefficients (broadcast
    // reads of whole rows).  The rows are requested in three batches ahead of their use: reading each
    // coefficient where it is used cost one LDS round trip per row (1.3 us of an 11 us item)
    const float* lb = sL + 16 * wv * ldl + 16 * wv;
    f32x4 c[16][4];
    auto rows = [&](auto i0, auto i1) {
#pragma unroll
      for (int i = decltype(i0)::value; i < decltype(i1)::value; ++i)
#pragma unroll
        for (int j = 0; j < (i + 3) / 4; ++j) c[i][j] = *(const f32x4*)(lb + i * ldl + 4 * j);
    };
    float x[16];
    auto solve = [&](auto i0, auto i1) {
#pragma unroll
      for (int i = decltype(i0)::value; i < decltype(i1)::value; ++i) {
        float s = (i == l) ? 1.f : 0.f;
#pragma unroll
        for (int m = 0; m < i; ++m) s -= c[i][m >> 2][m & 3] * x[m];
        x[i] = s;
      }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 8> I8;
    typedef std::integral_constant<int, 12> I12;
    typedef std::integral_constant<int, 16> I16;
    rows(I0(), I8());
    __builtin_amdgcn_sched_barrier(0);
    rows(I8(), I12());
    __builtin_amdgcn_sched_barrier(0);
    solve(I0(), I8());
    __builtin_amdgcn_sched_barrier(0);
    rows(I12(), I16());
    __builtin_amdgcn_sched_barrier(0);
    solve(I8(), I12());
    __builtin_amdgcn_sched_barrier(0);
    solve(I12(), I16());
#pragma unroll
    for (int i = 0; i < 16; ++i) sX[(16 * wv + i) * ldx + 16 * wv + l] = x[i];
  }
  lds_barrier();
  // operand layout of the 16 x 16 x 4 instruction: A[m = l % 16][k = l / 16], B[k = l / 16][n = l % 16],
  // result rows 4 (l / 16) + i of column l % 16
  const int r16 = l & 15, k4 = l >> 4;
  float* yb = sY + wv * 272;
#pragma unroll
  for (int d = 1; d < 4; ++d) {
    if (wv + d < 4) {                      // wave-uniform: block (I, J) = (wv + d, wv)
      const int J = wv, I = wv + d;
      // every operand of the round is requested before the first product (one LDS round trip instead of
      // one per instruction)
      float la[12], xb[12], xd[4];
#pragma unroll
      for (int t = 0; t < 4 * d; ++t) {
        la[t] = sL[(16 * I + r16) * ldl + 16 * J + 4 * t + k4];
        xb[t] = sX[(16 * J + 4 * t + k4) * ldx + 16 * J + r16];
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) xd[t] = sX[(16 * I + r16) * ldx + 16 * I + 4 * t + k4];
      __builtin_amdgcn_sched_barrier(0);
      f32x4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < 4 * d; ++t) y = __builtin_amdgcn_mfma_f32_16x16x4f32(la[t], xb[t], y, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) yb[(4 * k4 + i) * 17 + r16] = y[i];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      float yv[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) yv[t] = yb[(4 * t + k4) * 17 + r16];
      __builtin_amdgcn_sched_barrier(0);
      f32x4 x = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < 4; ++t) x = __builtin_amdgcn_mfma_f32_16x16x4f32(xd[t], yv[t], x, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) sX[(16 * I + 4 * k4 + i) * ldx + 16 * J + r16] = -x[i];
    }
    lds_barrier();
  }
}

// SAVE = false (no Tinv buffer given): Tinv is not written.  With Tinv written and 2-byte elements the
// sequential passes form w and u on the chip from Tinv, k, v (LEAN below): neither is formed or written here and v
// is not read; the forward pass (k_gdn_state_fwd_reg) also forms P from q, k and the gate table, so P is not formed
// and q is not read here either: a lean item reads k, g, beta and writes Tinv and the gate table.
template <typename T, int K, int V, bool SAVE>
__global__ __launch_bounds__(NTHR, (sizeof(T) == 2 ? (SAVE ? 3 : 2) : 1)) void k_gdn_wy_fwd(const lmoe_args a) {
  constexpr bool LEAN = SAVE && sizeof(T) == 2;
  // lean: three work-groups per CU (53 KB of LDS each: fp32 tiles padded by 4 instead of 8, the inverse's
  // scratch in the k tile, which is dead by then)
  constexpr int LDK = K + LPAD, LDV = V + LPAD, LDC = CH + (LEAN ? 4 : LPAD), LDP = CH + LPAD;
  constexpr int NBK = K / 16, NBV = V / 16;
  // k (raw, for k k^T), then overwritten in place by k beta e^{b}; v beta; both stored [64][D]
  __shared__ __attribute__((aligned(16))) T s_k[CH * LDK];
  __shared__ __attribute__((aligned(16))) T s_vb[CH * LDV];
  __shared__ __attribute__((aligned(16))) float s_L[CH * LDC];   // L, later Tinv in element type T
  __shared__ __attribute__((aligned(16))) float s_X[CH * LDC];
  __shared__ float s_Yown[LEAN ? 4 : 4 * 272];
  float* s_Y = LEAN ? (float*)s_k : s_Yown;
  __shared__ __attribute__((aligned(16))) float s_b[64];
  __shared__ float s_beta[64], s_beb[64];
  // Tinv as an MFMA operand: fp32 uses s_X in place, bf16 a copy in the (dead) L tile
  T* s_Tm = sizeof(T) == 4 ? (T*)s_X : (T*)s_L;

  const int wv = wave_id(), l = lane_id();
  typedef TileIO<T, CH, K> IOK;
  typedef TileIO<T, CH, V> IOV;
  typedef TileIO<T, CH, CH> IO64;
  const int nitems = num_chunks(a) * a.H;
  if (nitems <= 0) return;                   // (a chunk count read on the device may be zero)
  // Inputs of an item: one register set, refilled for the next item of this work-group as soon as the
  // current item has consumed a part (v after it is staged, q after q k^T, k after its second staging, gate
  // and beta after the gate phase), so the requests are spread over the item instead of arriving as one
  // burst: a burst of 48 KB per work-group fills the CU's queue of outstanding requests and the waves
  // stall at the issue (measured: 1.4 us of an 11 us item).  Always requested, item index clamped: a load
  // that is skipped on some path would make the compiler drain all outstanding loads at every use.
  typename IOK::Regs rk;
  typename IOV::Regs rv;
  RowFrags<T, K> fq;
  uint32_t graw, braw;
  auto item_of = [&](int it, int& h) {
    it = min(it, nitems - 1);
    h = it % a.H;
    return chunk_info(a, it / a.H);
  };
  // q enters only as the A operand of q k^T: each wave takes its 16 rows straight into fragments
  auto issue_q = [&](int it) { if constexpr (LEAN) return; int h; const ChunkInfo ci = item_of(it, h); fq.load(row_ptr<T>(a.q, ci.b, ci.tok, h), a.q.st, 16 * wv, ci.len - 1); };
  auto issue_k = [&](int it) { int h; const ChunkInfo ci = item_of(it, h); IOK::load_nomask(rk, row_ptr<T>(a.k, ci.b, ci.tok, h), a.k.st, ci.len); };
  auto issue_v = [&](int it) {
    if constexpr (!LEAN) { int h; const ChunkInfo ci = item_of(it, h); IOV::load_nomask(rv, row_ptr<T>(a.v, ci.b, ci.tok, h), a.v.st, ci.len); }
  };
  auto issue_gb = [&](int it) {
    int h; const ChunkInfo ci = item_of(it, h);
    graw = gate_prefetch(a, ci.b, ci.tok, ci.len, h);
    braw = load_scalar_raw(a.beta.ptr, a.beta_dtype, row_off(a.beta, ci.b, ci.tok + min(l, ci.len - 1), h));
  };
  issue_q(blockIdx.x);
  issue_k(blockIdx.x);
  issue_v(blockIdx.x);
  issue_gb(blockIdx.x);
  wait_all_loads();   // the first loads may be ordered freely; the loop's waits must not inherit that order
  for (int it = blockIdx.x; it < nitems; it += gridDim.x) {
  // lane / thread index refreshed per item: the address arithmetic derived from them stays inside the
  // iteration instead of living in registers for the whole kernel
  const int l = fresh_index(lane_id()) & 63;
  const int tid = fresh_index((int)threadIdx.x) & (NTHR - 1);
  const int cid = it / a.H, h = it % a.H;
  const ChunkInfo ci = chunk_info(a, cid);
  const int nxt = it + gridDim.x;
  IOK::mask(rk, ci.len, tid);
  if constexpr (!LEAN) IOV::mask(rv, ci.len, tid);
  lds_barrier();      // the previous item has left every tile
  // Every wave holds the gates and beta of all 64 tokens (lane = token) and forms the cumulative gate for
  // itself: the staging below needs no value from another wave, so one barrier covers gate and staging
  const bool gated = a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr;
  const float bl = l < ci.len ? scalar_from_raw(braw, a.beta_dtype) : 0.f;
  const float xb = wave_incl_scan((gated && l < ci.len) ? scalar_from_raw(graw, a.g_dtype) : 0.f);
  const float eb = expf(xb), ed = expf(__shfl(xb, 63, 64) - xb);
  issue_gb(nxt);
  if (wv == 0) {
    s_b[l] = xb;
    s_beta[l] = bl;
    s_beb[l] = bl * eb;
  }
  {
    // gate table of the chunk for the sequential passes: e^{b_j}, e^{b_C - b_j}, beta_j, beta_j e^{b_j}, b_j.  Every global store of
    // this loop is issued by all threads on every path (here two waves write each entry), so that the
    // compiler can count the operations behind the prefetches exactly: a store under a condition made
    // the wait for the next item's inputs a wait for this item's last stores as well
    // (rows 2, 3: beta and beta e^{b}, zero past the end of the chunk -- the sequential passes then read no beta,
    // whose run-time element type would put a load behind a branch in their prefetch loops)
    float* gc = a.gcum + ((int64_t)cid * a.H + h) * GATE_ROWS * CH;
    const int row = tid >> 6;
    gc[tid] = row == 0 ? eb : row == 1 ? ed : row == 2 ? bl : bl * eb;
    gc[4 * CH + l] = xb;       // (all four waves, the same bytes)
  }
  IOK::store_lds(rk, s_k, LDK, tid);
  if constexpr (!LEAN) {
#pragma unroll
    for (int p = 0; p < IOV::PASSES; ++p) {       // v beta, beta of the row from the lane that holds it
      int row, col;
      IOV::coords(p, row, col, tid);
      const float sc = __shfl(bl, row & 63, 64);
      typename IOV::vec o;
#pragma unroll
      for (int i = 0; i < IOV::VEC; ++i) o[i] = ET<T>::from_f(ET<T>::to_f(rv.v[p][i]) * sc);
      *(typename IOV::vec*)(s_vb + row * LDV + col) = o;
    }
  }
  issue_v(nxt);
  lds_barrier();
  {
    // L (from k k^T) and P = (q k^T) . Gamma over the same k fragments; the blocks above the diagonal are
    // zero and skipped (wave-uniform), and one exponential per element serves both.  P goes to global
    // memory, staged through the (still unused) X tile
    T* s_P = (T*)s_X;
    T* pg = (T*)a.pmat + ((int64_t)cid * a.H + h) * CH * CH;
    f32x4 m[4], pm[4];
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) { m[nj] = f32x4{0.f, 0.f, 0.f, 0.f}; pm[nj] = m[nj]; }
    if constexpr (!LEAN) fq.mask(16 * wv, ci.len);
    const int fr = l & 15, fg = 8 * (l >> 4);
#pragma unroll
    for (int ks = 0; ks < K / 32; ++ks) {
      const typename ET<T>::frag ak = ET<T>::load_frag(s_k + (16 * wv + fr) * LDK + 32 * ks + fg);
#pragma unroll
      for (int nj = 0; nj < 4; ++nj) {
        if (nj <= wv) {
          const typename ET<T>::frag bk = ET<T>::load_frag(s_k + (16 * nj + fr) * LDK + 32 * ks + fg);
          ET<T>::mma(m[nj], bk, ak);          // transposed: a lane holds four consecutive columns of one row
          if constexpr (!LEAN) ET<T>::mma(pm[nj], bk, fq.f[ks]);
        }
      }
    }
    issue_q(nxt);
    const int r = 16 * wv + fr;
    const float br = s_b[r], betar = s_beta[r];
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      f32x4 pl = {0.f, 0.f, 0.f, 0.f}, pp = {0.f, 0.f, 0.f, 0.f};
      if (nj <= wv) {
        const int cc0 = 16 * nj + 4 * (l >> 4);
        const f32x4 bc = *(const f32x4*)(s_b + cc0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = texp<T>(br - bc[i]);
          pl[i] = (r > cc0 + i) ? betar * m[nj][i] * e : 0.f;
          pp[i] = (r >= cc0 + i) ? pm[nj][i] * e : 0.f;
        }
      }
      acc_to_lds_t<float>(pl, s_L, LDC, 16 * nj, 16 * wv, l);      // s_L[r][cc0 ..]: one 16-byte write
      if constexpr (!LEAN) acc_to_lds_t<T>(pp, s_P, LDP, 16 * nj, 16 * wv, l);
    }
    if constexpr (!LEAN) {
      lds_barrier();
      IO64::template lds_to_global<true>(s_P, LDP, pg, CH, CH, tid);
    }
  }
  // k is dead as an operand of k k^T and q k^T: scale it in place to k beta e^{b} (from the registers)
  if constexpr (!LEAN) IOK::store_lds_scaled(rk, s_k, LDK, s_beb, tid);
  issue_k(nxt);
  lds_barrier();   // L is complete, the P staging has been read: the inverse may overwrite X
  tri_inverse_64(s_L, LDC, s_X, LDC, s_Y, l, tid);       // barriers inside; s_L is dead afterwards
  {
    T* tg = (T*)a.tinv + ((int64_t)cid * a.H + h) * CH * CH;
#pragma unroll
    for (int p = 0; p < CH * CH / 4 / NTHR; ++p) {      // fixed trip count: see the decay table above
      const int idx = p * NTHR + tid;
      const int r = idx >> 4, c = (idx & 15) * 4;
      const f32x4 x = *(const f32x4*)(s_X + r * LDC + c);
      if constexpr (sizeof(T) == 2) {
        bf16x4 y; y[0] = (bf16)x[0]; y[1] = (bf16)x[1]; y[2] = (bf16)x[2]; y[3] = (bf16)x[3];
        if constexpr (!LEAN) *(bf16x4*)(s_Tm + r * LDC + c) = y;
        if constexpr (SAVE) __builtin_nontemporal_store(y, (bf16x4*)(tg + r * CH + c));
      } else {
        if constexpr (SAVE) __builtin_nontemporal_store(x, (f32x4*)(tg + r * CH + c));
      }
    }
  }
  if constexpr (!LEAN) {
  lds_barrier();
  // w = Tinv (k beta e^{b}),  u = Tinv (v beta): contraction over the rows of the [64][D] tiles.  Formed
  // transposed (the tile as the A operand through transposing LDS reads, Tinv rows as B), so that a lane
  // holds four consecutive columns of one token and the results go back to LDS as 8-byte writes.  Tinv is
  // lower triangular: the second half of the contraction is zero for the first 32 tokens
  f32x4 w[NBK], u[NBV];
#pragma unroll
  for (int ni = 0; ni < NBK; ++ni) w[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ni = 0; ni < NBV; ++ni) u[ni] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < CH / 32; ++ks) {
    if (ks == 0 || wv >= 2) {
      const typename ET<T>::frag bt = ET<T>::load_frag(s_Tm + (16 * wv + (l & 15)) * LDC + 32 * ks + 8 * (l >> 4));
#pragma unroll
      for (int ni = 0; ni < NBK; ++ni) ET<T>::mma(w[ni], ET<T>::load_frag_t(s_k, LDK, 32 * ks, 16 * ni), bt);
#pragma unroll
      for (int ni = 0; ni < NBV; ++ni) ET<T>::mma(u[ni], ET<T>::load_frag_t(s_vb, LDV, 32 * ks, 16 * ni), bt);
    }
  }
  lds_barrier();   // k, v tiles are dead: they stage the stores
#pragma unroll
  for (int ni = 0; ni < NBK; ++ni) acc_to_lds_t<T>(w[ni], s_k, LDK, 16 * ni, 16 * wv, l);
#pragma unroll
  for (int ni = 0; ni < NBV; ++ni) acc_to_lds_t<T>(u[ni], s_vb, LDV, 16 * ni, 16 * wv, l);
  lds_barrier();
  {
    // branch-free (rows past the end of a partial chunk rewrite its last row with the same bytes)
    typename IOK::Regs ow;
    typename IOV::Regs ou;
    IOK::load_lds_clamped(ow, s_k, LDK, ci.len, tid);
    IOV::load_lds_clamped(ou, s_vb, LDV, ci.len, tid);
    IOK::template store_global_clamped<true>(ow, row_ptr<T>(a.w, ci.b, ci.tok, h), a.w.st, ci.len, tid);
    IOV::template store_global_clamped<true>(ou, row_ptr<T>(a.u, ci.b, ci.tok, h), a.u.st, ci.len, tid);
  }
  }
  }   // items
}

}  // namespace lmoe
