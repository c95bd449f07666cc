// Row routing for mixture-of-memories layers: pack the tokens routed to each (memory, batch row) into one
// variable-length batch, and combine the per-memory results back per token.
// Replaces the pad-to-capacity `transform` / `reconstruct` pair of the reference
// (linear_moe/sequence_modeling/mom_linear_attention.py:15-77, :79-120), whose output feeds one op call per
// memory (:369-409): the packed rows feed ONE call of the variable-length kernels instead.
//   gather :  out[i]  = scale[i] * src[idx[i]]                    (idx < 0: zeros; scale may be null)
//   combine:  out[t]  = sum_k w[t][k] * src[idx[t][k]]            (idx < 0: skipped; w null: 1)
//   rowdot :  dw[t][k] = < g[t], src[idx[t][k]] >                 (idx < 0: 0)
// Rows of D elements (D a multiple of 8, 16-byte aligned), fp32 math, one 16-byte vector per lane per
// step, no atomics: every output row is written by one work-group slice.  HBM-bound.
#include "lmoe_launch.hpp"
#include "lmoe_seq.hpp"

namespace lmoe {

constexpr int MOM_LPR = 64;                 // lanes (one wave) per row
constexpr int MOM_RPB = NTHR / MOM_LPR;     // rows per work-group pass

template <typename T>
__global__ __launch_bounds__(NTHR) void k_gather_rows(const T* __restrict__ src, const int32_t* __restrict__ idx,
                                                      const T* __restrict__ scale, T* __restrict__ out, int64_t nout, int D) {
  constexpr int VEC = ET<T>::VEC;
  typedef typename ET<T>::vec vec;
  const int lr = threadIdx.x % MOM_LPR, rb = threadIdx.x / MOM_LPR;
  for (int64_t r = (int64_t)blockIdx.x * MOM_RPB + rb; r < nout; r += (int64_t)gridDim.x * MOM_RPB) {
    const int s = idx[r];
    const float sc = (scale && s >= 0) ? ET<T>::to_f(scale[r]) : 1.0f;
    for (int c = lr * VEC; c < D; c += MOM_LPR * VEC) {
      vec o;
      if (s >= 0) {
        const vec v = *(const vec*)(src + (int64_t)s * D + c);
#pragma unroll
        for (int i = 0; i < VEC; ++i) o[i] = scale ? ET<T>::from_f(ET<T>::to_f(v[i]) * sc) : v[i];
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(0.f);
      }
      *(vec*)(out + r * D + c) = o;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NTHR) void k_combine_rows(const T* __restrict__ src, const int32_t* __restrict__ idx,
                                                       const T* __restrict__ w, T* __restrict__ out, int64_t ntok, int topk,
                                                       int D) {
  constexpr int VEC = ET<T>::VEC;
  typedef typename ET<T>::vec vec;
  const int lr = threadIdx.x % MOM_LPR, rb = threadIdx.x / MOM_LPR;
  for (int64_t t = (int64_t)blockIdx.x * MOM_RPB + rb; t < ntok; t += (int64_t)gridDim.x * MOM_RPB) {
    for (int c = lr * VEC; c < D; c += MOM_LPR * VEC) {
      float acc[VEC];
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
      for (int k = 0; k < topk; ++k) {
        const int s = idx[t * topk + k];
        if (s < 0) continue;
        const float wk = w ? ET<T>::to_f(w[t * topk + k]) : 1.0f;
        const vec v = *(const vec*)(src + (int64_t)s * D + c);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] += wk * ET<T>::to_f(v[i]);
      }
      vec o;
#pragma unroll
      for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(acc[i]);
      *(vec*)(out + t * D + c) = o;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(NTHR) void k_rowdot(const T* __restrict__ src, const int32_t* __restrict__ idx,
                                                 const T* __restrict__ g, T* __restrict__ dw, int64_t ntok, int topk, int D) {
  constexpr int VEC = ET<T>::VEC;
  typedef typename ET<T>::vec vec;
  const int lr = threadIdx.x % MOM_LPR, rb = threadIdx.x / MOM_LPR;
  for (int64_t t = (int64_t)blockIdx.x * MOM_RPB + rb; t < ntok; t += (int64_t)gridDim.x * MOM_RPB) {
    for (int k = 0; k < topk; ++k) {
      const int s = idx[t * topk + k];
      float acc = 0.f;
      if (s >= 0) {
        for (int c = lr * VEC; c < D; c += MOM_LPR * VEC) {
          const vec v = *(const vec*)(src + (int64_t)s * D + c);
          const vec gv = *(const vec*)(g + t * D + c);
#pragma unroll
          for (int i = 0; i < VEC; ++i) acc += ET<T>::to_f(v[i]) * ET<T>::to_f(gv[i]);
        }
      }
      acc = wave_sum(acc);
      if (lr == 0) dw[t * topk + k] = ET<T>::from_f(acc);
    }
  }
}

static int mom_grid(int64_t rows) {
  const int64_t blocks = (rows + MOM_RPB - 1) / MOM_RPB, cap = (int64_t)cu_count() * 8;
  return (int)(blocks < cap ? blocks : cap);
}

void launch_mom_gather(int dtype, const void* src, const int32_t* idx, const void* scale, void* out, int64_t nout, int D,
                       hipStream_t st) {
  const int grid = mom_grid(nout);
  if (dtype == LMOE_BF16) hipLaunchKernelGGL(k_gather_rows<bf16>, dim3(grid), dim3(NTHR), 0, st, (const bf16*)src, idx, (const bf16*)scale, (bf16*)out, nout, D);
  else hipLaunchKernelGGL(k_gather_rows<float>, dim3(grid), dim3(NTHR), 0, st, (const float*)src, idx, (const float*)scale, (float*)out, nout, D);
}
void launch_mom_combine(int dtype, const void* src, const int32_t* idx, const void* w, void* out, int64_t ntok, int topk,
                        int D, hipStream_t st) {
  const int grid = mom_grid(ntok);
  if (dtype == LMOE_BF16) hipLaunchKernelGGL(k_combine_rows<bf16>, dim3(grid), dim3(NTHR), 0, st, (const bf16*)src, idx, (const bf16*)w, (bf16*)out, ntok, topk, D);
  else hipLaunchKernelGGL(k_combine_rows<float>, dim3(grid), dim3(NTHR), 0, st, (const float*)src, idx, (const float*)w, (float*)out, ntok, topk, D);
}
void launch_mom_rowdot(int dtype, const void* src, const int32_t* idx, const void* g, void* dw, int64_t ntok, int topk,
                       int D, hipStream_t st) {
  const int grid = mom_grid(ntok);
  if (dtype == LMOE_BF16) hipLaunchKernelGGL(k_rowdot<bf16>, dim3(grid), dim3(NTHR), 0, st, (const bf16*)src, idx, (const bf16*)g, (bf16*)dw, ntok, topk, D);
  else hipLaunchKernelGGL(k_rowdot<float>, dim3(grid), dim3(NTHR), 0, st, (const float*)src, idx, (const float*)g, (float*)dw, ntok, topk, D);
}

}  // namespace lmoe
