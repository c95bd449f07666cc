// Token-by-token (recurrent) forward of the three ops, for decoding and short sequences: the state
// lives in registers for the whole sequence, nothing but q, k, v, the gates and o moves per token.
//   simple_gla :  S = e^{g_t} S + k_t^T v_t
//   gla        :  S = diag(e^{g_t}) S + k_t^T v_t
//   delta rule :  S = e^{g_t} S;  S += k_t^T beta_t (v_t - k_t S)
//   o_t = scale q_t S
// (the `fused_recurrent_*` callables the reference selects with la_mode = 'fused_recurrent':
// linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:72-73, gla/gla.py:58-59,
// deltanet/deltanet.py:81-82, basic_linear_attention/basic_linear_attention.py:99-100).
//
// grid = N * H * (V / 32) work-groups of 256 threads.  A work-group owns the [K x 32] slice of the state
// of one (sequence, head): thread (c, kg) = (tid / 8, tid % 8) holds rows kg, kg + 8, .. of column c in
// fp32 registers, so a contraction over K is K / 8 multiply-adds per thread and three lane exchanges
// inside a group of 8 adjacent lanes.  q, k (, the vector gate) of a block of 16 tokens are staged in
// LDS as fp32; v, the scalar gate and beta are read by the threads that need them.  HBM-bound for
// decoding (T = 1: the state is read and written once), latency-bound per token otherwise.
#include "lmoe_launch.hpp"
#include "lmoe_seq.hpp"

namespace lmoe {

constexpr int RBV = 32;     // V columns per work-group
constexpr int RTB = 16;     // tokens staged per block

__device__ __forceinline__ float group8_sum(float x) {
  x += __shfl_xor(x, 1, 64);
  x += __shfl_xor(x, 2, 64);
  x += __shfl_xor(x, 4, 64);
  return x;
}

template <typename T, int K, int V, int GATE, bool DELTA>
__global__ __launch_bounds__(NTHR) void k_recurrent_fwd(const lmoe_args a) {
  constexpr int KR = K / 8;                 // state rows per thread
  __shared__ float s_q[RTB][K], s_k[RTB][K], s_g[GATE == LMOE_GATE_VECTOR ? RTB : 1][K];
  const int nvs = V / RBV;
  const int vsl = blockIdx.x % nvs, pair = blockIdx.x / nvs;
  const int h = pair % a.H, n = pair / a.H;
  const SeqInfo sq = seq_info(a, n);
  const int c = threadIdx.x >> 3, kg = threadIdx.x & 7;
  const int vcol = vsl * RBV + c;
  float S[KR];
#pragma unroll
  for (int j = 0; j < KR; ++j) S[j] = 0.f;
  if (a.h0) {
    const float* h0 = a.h0 + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int j = 0; j < KR; ++j) S[j] = h0[(int64_t)(kg + 8 * j) * V + vcol];
  }
  const float scale = a.scale;
  for (int t0 = 0; t0 < sq.len; t0 += RTB) {
    const int nt = min(RTB, sq.len - t0);
    __syncthreads();                        // the previous block has been consumed
    for (int idx = threadIdx.x; idx < nt * K; idx += NTHR) {
      const int tt = idx / K, kk = idx % K;
      const int64_t ro = row_off(a.q, sq.b, sq.tok0 + t0 + tt, h);
      s_q[tt][kk] = ET<T>::to_f(((const T*)a.q.ptr)[ro + kk]);
      s_k[tt][kk] = ET<T>::to_f(((const T*)a.k.ptr)[row_off(a.k, sq.b, sq.tok0 + t0 + tt, h) + kk]);
      if constexpr (GATE == LMOE_GATE_VECTOR)
        s_g[tt][kk] = __expf(load_scalar(a.g.ptr, a.g_dtype, row_off(a.g, sq.b, sq.tok0 + t0 + tt, h) + kk));
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const int tok = sq.tok0 + t0 + tt;
      const float vt = ET<T>::to_f(((const T*)a.v.ptr)[row_off(a.v, sq.b, tok, h) + vcol]);
      if constexpr (GATE == LMOE_GATE_SCALAR) {
        const float eg = __expf(load_scalar(a.g.ptr, a.g_dtype, row_off(a.g, sq.b, tok, h)));
#pragma unroll
        for (int j = 0; j < KR; ++j) S[j] *= eg;
      } else if constexpr (GATE == LMOE_GATE_VECTOR) {
#pragma unroll
        for (int j = 0; j < KR; ++j) S[j] *= s_g[tt][kg + 8 * j];
      }
      float upd = vt;
      if constexpr (DELTA) {
        float p = 0.f;
#pragma unroll
        for (int j = 0; j < KR; ++j) p += s_k[tt][kg + 8 * j] * S[j];
        p = group8_sum(p);
        const float bt = load_scalar(a.beta.ptr, a.beta_dtype, row_off(a.beta, sq.b, tok, h));
        upd = bt * (vt - p);
      }
      float oacc = 0.f;
#pragma unroll
      for (int j = 0; j < KR; ++j) {
        S[j] += s_k[tt][kg + 8 * j] * upd;
        oacc += s_q[tt][kg + 8 * j] * S[j];
      }
      oacc = group8_sum(oacc);
      if (kg == 0) ((T*)a.o.ptr)[row_off(a.o, sq.b, tok, h) + vcol] = ET<T>::from_f(oacc * scale);
    }
  }
  if (a.ht) {
    float* ht = a.ht + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int j = 0; j < KR; ++j) ht[(int64_t)(kg + 8 * j) * V + vcol] = S[j];
  }
}

// ------------------------------------------------------------------------- //
// The same recurrence for decoding steps (a few tokens per sequence): the time goes into reading and writing
// the fp32 state once, so the state moves in 16-byte accesses.  Thread (cq, kg) = (tid % 8, tid / 8) holds rows
// kg, kg + 32, .. of the four columns 4 cq .. 4 cq + 3: eight adjacent lanes cover one 128-byte row piece.  A
// contraction over K is then a sum over the 32 row groups: three lane exchanges inside a wave, the four waves
// through LDS (one work-group barrier per contraction, i.e. one or two per token).
// ------------------------------------------------------------------------- //
template <typename T, int K, int V, int GATE, bool DELTA>
__global__ __launch_bounds__(NTHR) void k_recurrent_step(const lmoe_args a) {
  constexpr int KR = K / 32;                // state rows per thread
  __shared__ __attribute__((aligned(16))) float s_red[2][4][RBV];   // [contraction][wave][column]
  const int nvs = V / RBV;
  const int vsl = blockIdx.x % nvs, pair = blockIdx.x / nvs;
  const int h = pair % a.H, n = pair / a.H;
  const SeqInfo sq = seq_info(a, n);
  const int cq = threadIdx.x & 7, kg = threadIdx.x >> 3, wv = threadIdx.x >> 6;
  const int vcol = vsl * RBV + 4 * cq;
  f32x4 S[KR];
#pragma unroll
  for (int j = 0; j < KR; ++j) S[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  if (a.h0) {
    const float* h0 = a.h0 + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int j = 0; j < KR; ++j) S[j] = *(const f32x4*)(h0 + (int64_t)(kg + 32 * j) * V + vcol);
  }
  const float scale = a.scale;
  // sum over the 32 row groups of four per-thread partials; every thread receives the four totals
  auto reduce_rows = [&](f32x4 x, int which) {
#pragma unroll
    for (int d = 8; d < 64; d <<= 1)
#pragma unroll
      for (int c = 0; c < 4; ++c) x[c] += __shfl_xor(x[c], d, 64);
    if ((threadIdx.x & 63) < 8) *(f32x4*)&s_red[which][wv][4 * cq] = x;
    __syncthreads();
    f32x4 t = *(const f32x4*)&s_red[which][0][4 * cq];
#pragma unroll
    for (int w = 1; w < 4; ++w) t += *(const f32x4*)&s_red[which][w][4 * cq];
    return t;
  };
  for (int t = 0; t < sq.len; ++t) {
    const int tok = sq.tok0 + t;
    const T* qp = (const T*)a.q.ptr + row_off(a.q, sq.b, tok, h);
    const T* kp = (const T*)a.k.ptr + row_off(a.k, sq.b, tok, h);
    float qv[KR], kv[KR];
#pragma unroll
    for (int j = 0; j < KR; ++j) {
      qv[j] = ET<T>::to_f(qp[kg + 32 * j]);
      kv[j] = ET<T>::to_f(kp[kg + 32 * j]);
    }
    const typename ET<T>::vec4 vraw = *(const typename ET<T>::vec4*)((const T*)a.v.ptr + row_off(a.v, sq.b, tok, h) + vcol);
    f32x4 vt;
#pragma unroll
    for (int c = 0; c < 4; ++c) vt[c] = ET<T>::to_f(vraw[c]);
    if constexpr (GATE == LMOE_GATE_SCALAR) {
      const float eg = __expf(load_scalar(a.g.ptr, a.g_dtype, row_off(a.g, sq.b, tok, h)));
#pragma unroll
      for (int j = 0; j < KR; ++j) S[j] *= eg;
    } else if constexpr (GATE == LMOE_GATE_VECTOR) {
#pragma unroll
      for (int j = 0; j < KR; ++j)
        S[j] *= __expf(load_scalar(a.g.ptr, a.g_dtype, row_off(a.g, sq.b, tok, h) + kg + 32 * j));
    }
    f32x4 upd = vt;
    if constexpr (DELTA) {
      f32x4 p = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < KR; ++j) p += kv[j] * S[j];
      p = reduce_rows(p, 0);
      const float bt = load_scalar(a.beta.ptr, a.beta_dtype, row_off(a.beta, sq.b, tok, h));
      upd = bt * (vt - p);
    }
    f32x4 oacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < KR; ++j) {
      S[j] += kv[j] * upd;
      oacc += qv[j] * S[j];
    }
    // without the delta rule there is one barrier per token: alternate the buffer so that a fast wave's next
    // partials cannot overtake a slow wave's reads
    oacc = reduce_rows(oacc, DELTA ? 1 : (t & 1));
    if (threadIdx.x < 8) {
      typename ET<T>::vec4 ov;
#pragma unroll
      for (int c = 0; c < 4; ++c) ov[c] = ET<T>::from_f(oacc[c] * scale);
      *(typename ET<T>::vec4*)((T*)a.o.ptr + row_off(a.o, sq.b, tok, h) + vcol) = ov;
    }
  }
  if (a.ht) {
    float* ht = a.ht + ((int64_t)n * a.H + h) * K * V;
#pragma unroll
    for (int j = 0; j < KR; ++j) *(f32x4*)(ht + (int64_t)(kg + 32 * j) * V + vcol) = S[j];
  }
}

template <int GATE, bool DELTA> struct Recurrent {
  template <typename T, int K, int V> struct F {
    static void run(const lmoe_args& a, hipStream_t st) {
      const int grid = a.N * a.H * (V / RBV);
      // decoding steps (at most four tokens per sequence on average): the kernel built around the state traffic
      if ((int64_t)a.B * a.T <= 4 * (int64_t)a.N)
        hipLaunchKernelGGL((k_recurrent_step<T, K, V, GATE, DELTA>), dim3(grid), dim3(NTHR), 0, st, a);
      else
        hipLaunchKernelGGL((k_recurrent_fwd<T, K, V, GATE, DELTA>), dim3(grid), dim3(NTHR), 0, st, a);
    }
  };
};

void launch_recurrent(const lmoe_args& a, bool delta, hipStream_t st) {
  if (delta) {
    if (a.gate == LMOE_GATE_NONE || !a.g.ptr) dispatch<Recurrent<LMOE_GATE_NONE, true>::F>(a, st);
    else dispatch<Recurrent<LMOE_GATE_SCALAR, true>::F>(a, st);
  } else if (a.gate == LMOE_GATE_VECTOR) {
    dispatch<Recurrent<LMOE_GATE_VECTOR, false>::F>(a, st);
  } else if (a.gate == LMOE_GATE_NONE || !a.g.ptr) {
    dispatch<Recurrent<LMOE_GATE_NONE, false>::F>(a, st);
  } else {
    dispatch<Recurrent<LMOE_GATE_SCALAR, false>::F>(a, st);
  }
}

}  // namespace lmoe
