// What the gated-delta-rule token mixer does to its projections on either side of the chunk op, one pass each.
//
//  * prologue (linear_moe/sequence_modeling/linear_attention.py:159-163 the q / k / v split of the fused
//    projection; gated_deltanet/gated_deltanet.py:99 'n b h d -> b n h d', :101 SiLU on q, k, v, :105-106 the L2
//    norm of q and k): reads the fused projection [T, B, H, 3 D] once and writes
//        q^ = l2norm(silu(q)),  k^ = l2norm(silu(k)),  v~ = silu(v)          each [B, T, H, D],
//    the layout the op reads.  The eager chain makes three strided copies, runs two row kernels and one
//    elementwise kernel: 9 D elements read and 9 D written per row instead of 3 D and 3 D.
//    Backward: from dq^, dk^, dv~ and the projection, d(projection) [T, B, H, 3 D] in one pass.
//  * epilogue (gated_deltanet.py:114 'b n h d -> n b (h d)', linear_attention.py:255 o * swish(o_gate)):
//        y[t, b, :] = o[b, t, :] * o_gate[t, b, :] * sigmoid(o_gate[t, b, :])
//    and its backward (do in the op's layout, do_gate in the projection's).
// fp32 math, one 16-byte vector per lane and tensor, grid-stride, HBM-bound.
#include "lmoe_launch.hpp"
#include "lmoe_seq.hpp"

namespace lmoe {

namespace {
__device__ __forceinline__ float sigm(float z) { return sigmoid_fast(z); }
// sum over the LPR neighbouring lanes that hold one row
template <int LPR> __device__ __forceinline__ float row_sum(float x) {
  if constexpr (LPR <= 16) {
    return group_sum<LPR>(x);
  } else {
#pragma unroll
    for (int d = 1; d < LPR; d <<= 1) x += __shfl_xor(x, d, 64);
    return x;
  }
}

// rows are (t, b, h) in the projection and (b, t, h) in the op's tensors
// WITH_V = false: v is left to the op (which then applies SiLU to the column block of the projection itself and writes
// its gradient into that block of d(projection)): q^ and k^ only; the backward leaves the v block of d(projection) alone
template <typename T, int D, bool BWD, bool WITH_V>
__global__ __launch_bounds__(NTHR) void k_gdn_qkv_prologue(const T* __restrict__ qkv, const T* __restrict__ dq,
                                                           const T* __restrict__ dk, const T* __restrict__ dv,
                                                           T* __restrict__ o0, T* __restrict__ o1, T* __restrict__ o2,
                                                           int Tn, int Bn, int H, float eps) {
  constexpr int VEC = ET<T>::VEC, LPR = D / VEC, RPB = NTHR / LPR;
  typedef typename ET<T>::vec vec;
  const int lr = threadIdx.x % LPR, rb = threadIdx.x / LPR;
  const int64_t rows = (int64_t)Tn * Bn * H;
  for (int64_t r = (int64_t)blockIdx.x * RPB + rb; r < rows; r += (int64_t)gridDim.x * RPB) {
    // r counts the rows of the op's layout: r = (b T + t) H + h
    const int h = (int)(r % H);
    const int64_t bt = r / H;
    const int t = (int)(bt % Tn), b = (int)(bt / Tn);
    const T* src = qkv + (((int64_t)t * Bn + b) * H + h) * (3 * D) + lr * VEC;
    const vec xq = *(const vec*)src, xk = *(const vec*)(src + D);
    float sq[VEC], sk[VEC], gq[VEC], gk[VEC], ssq = 0.f, ssk = 0.f;
    vec ov;
    if constexpr (WITH_V) {
      const vec xv = *(const vec*)(src + 2 * D);
      vec dvv;
      if constexpr (BWD) dvv = *(const vec*)(dv + r * D + lr * VEC);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float zv = ET<T>::to_f(xv[i]), av = sigm(zv);
        if constexpr (BWD) ov[i] = ET<T>::from_f(ET<T>::to_f(dvv[i]) * av * (1.0f + zv * (1.0f - av)));
        else ov[i] = ET<T>::from_f(zv * av);
      }
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float zq = ET<T>::to_f(xq[i]), zk = ET<T>::to_f(xk[i]);
      const float aq = sigm(zq), ak = sigm(zk);
      sq[i] = zq * aq; sk[i] = zk * ak;
      gq[i] = aq * (1.0f + zq * (1.0f - aq));       // silu'(z)
      gk[i] = ak * (1.0f + zk * (1.0f - ak));
      ssq += sq[i] * sq[i]; ssk += sk[i] * sk[i];
    }
    ssq = row_sum<LPR>(ssq); ssk = row_sum<LPR>(ssk);
    const float rq = 1.0f / sqrtf(ssq + eps), rk = 1.0f / sqrtf(ssk + eps);
    vec oq, ok;
    if constexpr (BWD) {
      const vec dqv = *(const vec*)(dq + r * D + lr * VEC), dkv = *(const vec*)(dk + r * D + lr * VEC);
      float fq[VEC], fk[VEC], cq = 0.f, ck = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        fq[i] = ET<T>::to_f(dqv[i]); fk[i] = ET<T>::to_f(dkv[i]);
        cq += fq[i] * sq[i]; ck += fk[i] * sk[i];
      }
      cq = row_sum<LPR>(cq) * rq * rq * rq; ck = row_sum<LPR>(ck) * rk * rk * rk;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        oq[i] = ET<T>::from_f((fq[i] * rq - cq * sq[i]) * gq[i]);
        ok[i] = ET<T>::from_f((fk[i] * rk - ck * sk[i]) * gk[i]);
      }
      T* dst = o0 + (((int64_t)t * Bn + b) * H + h) * (3 * D) + lr * VEC;       // d(projection)
      *(vec*)dst = oq; *(vec*)(dst + D) = ok;
      if constexpr (WITH_V) *(vec*)(dst + 2 * D) = ov;
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) { oq[i] = ET<T>::from_f(sq[i] * rq); ok[i] = ET<T>::from_f(sk[i] * rk); }
      *(vec*)(o0 + r * D + lr * VEC) = oq;
      *(vec*)(o1 + r * D + lr * VEC) = ok;
      if constexpr (WITH_V) *(vec*)(o2 + r * D + lr * VEC) = ov;
    }
  }
}

// rows of W = H D elements: (b, t) in the op's output, (t, b) in the gate and the result
template <typename T, bool BWD>
__global__ __launch_bounds__(NTHR) void k_swish_gate_relayout(const T* __restrict__ o, const T* __restrict__ gate,
                                                              const T* __restrict__ dy, T* __restrict__ out,
                                                              T* __restrict__ dgate, int Tn, int Bn, int W) {
  constexpr int VEC = ET<T>::VEC;
  typedef typename ET<T>::vec vec;
  const int vpr = W / VEC;
  const int64_t nvec = (int64_t)Tn * Bn * vpr;
  for (int64_t i = (int64_t)blockIdx.x * NTHR + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * NTHR) {
    // i counts the vectors of the (t, b) layout
    const int c = (int)(i % vpr) * VEC;
    const int64_t tb = i / vpr;
    const int b = (int)(tb % Bn), t = (int)(tb / Bn);
    const int64_t io = ((int64_t)b * Tn + t) * W + c, ig = tb * W + c;
    const vec ov = *(const vec*)(o + io), gv = *(const vec*)(gate + ig);
    vec r0, r1;
    vec dv;
    if constexpr (BWD) dv = *(const vec*)(dy + ig);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float z = ET<T>::to_f(gv[j]), s = sigm(z), x = ET<T>::to_f(ov[j]);
      if constexpr (BWD) {
        const float d = ET<T>::to_f(dv[j]);
        r0[j] = ET<T>::from_f(d * z * s);                                 // do
        r1[j] = ET<T>::from_f(d * x * s * (1.0f + z * (1.0f - s)));       // do_gate
      } else {
        r0[j] = ET<T>::from_f(x * z * s);
      }
    }
    if constexpr (BWD) { *(vec*)(out + io) = r0; *(vec*)(dgate + ig) = r1; }
    else *(vec*)(out + ig) = r0;
  }
}

template <typename T, int D>
void prologue_t(const void* qkv, const void* dq, const void* dk, const void* dv, void* o0, void* o1, void* o2, int Tn,
                int Bn, int H, float eps, bool bwd, hipStream_t st) {
  constexpr int RPB = NTHR / (D / ET<T>::VEC);
  const int64_t rows = (int64_t)Tn * Bn * H, blocks = (rows + RPB - 1) / RPB, cap = (int64_t)cu_count() * 8;
  const int grid = (int)(blocks < cap ? blocks : cap);
  // v handed in (forward: o2, backward: dv) or left to the op
  const bool with_v = bwd ? dv != nullptr : o2 != nullptr;
#define LMOE_P(BWD, WV)                                                                                                  \
  hipLaunchKernelGGL((k_gdn_qkv_prologue<T, D, BWD, WV>), dim3(grid), dim3(NTHR), 0, st, (const T*)qkv, (const T*)dq,    \
                     (const T*)dk, (const T*)dv, (T*)o0, (T*)o1, (T*)o2, Tn, Bn, H, eps)
  if (bwd) { if (with_v) LMOE_P(true, true); else LMOE_P(true, false); }
  else { if (with_v) LMOE_P(false, true); else LMOE_P(false, false); }
#undef LMOE_P
}
}  // namespace

void launch_gdn_qkv_prologue(int dtype, int D, const void* qkv, const void* dq, const void* dk, const void* dv, void* o0,
                             void* o1, void* o2, int Tn, int Bn, int H, float eps, bool bwd, hipStream_t st) {
#define LMOE_D(T)                                                                       \
  if (D == 64) prologue_t<T, 64>(qkv, dq, dk, dv, o0, o1, o2, Tn, Bn, H, eps, bwd, st);  \
  else prologue_t<T, 128>(qkv, dq, dk, dv, o0, o1, o2, Tn, Bn, H, eps, bwd, st);
  if (dtype == LMOE_BF16) { LMOE_D(bf16) } else { LMOE_D(float) }
#undef LMOE_D
}

void launch_swish_gate_relayout(int dtype, const void* o, const void* gate, const void* dy, void* out, void* dgate, int Tn,
                                int Bn, int W, bool bwd, hipStream_t st) {
  const int vec = dtype == LMOE_BF16 ? 8 : 4;
  const int64_t nvec = (int64_t)Tn * Bn * (W / vec), blocks = (nvec + NTHR - 1) / NTHR, cap = (int64_t)cu_count() * 16;
  const int grid = (int)(blocks < cap ? blocks : cap);
#define LMOE_L(T)                                                                                                          \
  if (bwd) hipLaunchKernelGGL((k_swish_gate_relayout<T, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)o, (const T*)gate, \
                              (const T*)dy, (T*)out, (T*)dgate, Tn, Bn, W);                                                \
  else hipLaunchKernelGGL((k_swish_gate_relayout<T, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)o, (const T*)gate,   \
                          (const T*)nullptr, (T*)out, (T*)nullptr, Tn, Bn, W);
  if (dtype == LMOE_BF16) { LMOE_L(bf16) } else { LMOE_L(float) }
#undef LMOE_L
}

}  // namespace lmoe
