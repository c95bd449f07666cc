// Row-wise L2 normalisation y = x / sqrt(sum x^2 + eps) and its backward
//   dx = dy rstd - (sum dy x) rstd^3 x,
// the operation the reference applies to q and k in front of the delta-rule ops
// (linear_moe/model/common_modules/l2norm.py:22-45 forward, :64-95 backward).  fp32 math, one
// 16-byte vector per lane, D / VEC lanes per row, grid-stride over the rows: HBM-bound.
#include "lmoe_launch.hpp"
#include "lmoe_seq.hpp"

namespace lmoe {

template <int LPR> __device__ __forceinline__ float row_sum(float x) {
#pragma unroll
  for (int d = 1; d < LPR; d <<= 1) x += __shfl_xor(x, d, 64);
  return x;
}

template <typename T, int D, bool BWD>
__global__ __launch_bounds__(NTHR) void k_l2norm(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ out,
                                                 int64_t rows, float eps) {
  constexpr int VEC = ET<T>::VEC, LPR = D / VEC, RPB = NTHR / LPR;
  static_assert(LPR <= 64 && (LPR & (LPR - 1)) == 0, "a row is shared by a power-of-two group of lanes");
  typedef typename ET<T>::vec vec;
  const int lr = threadIdx.x % LPR, rb = threadIdx.x / LPR;
  for (int64_t r = (int64_t)blockIdx.x * RPB + rb; r < rows; r += (int64_t)gridDim.x * RPB) {
    const vec xv = *(const vec*)(x + r * D + lr * VEC);
    float xf[VEC], ss = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) { xf[i] = ET<T>::to_f(xv[i]); ss += xf[i] * xf[i]; }
    ss = row_sum<LPR>(ss);
    const float rstd = 1.0f / sqrtf(ss + eps);
    vec o;
    if constexpr (BWD) {
      const vec dv = *(const vec*)(dy + r * D + lr * VEC);
      float df[VEC], sd = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; ++i) { df[i] = ET<T>::to_f(dv[i]); sd += df[i] * xf[i]; }
      sd = row_sum<LPR>(sd);
      const float c = sd * rstd * rstd * rstd;
#pragma unroll
      for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(df[i] * rstd - c * xf[i]);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(xf[i] * rstd);
    }
    *(vec*)(out + r * D + lr * VEC) = o;
  }
}

template <typename T, int D>
static void launch_t(const void* x, const void* dy, void* out, int64_t rows, float eps, bool bwd, hipStream_t st) {
  constexpr int RPB = NTHR / (D / ET<T>::VEC);
  int64_t blocks = (rows + RPB - 1) / RPB;
  const int64_t cap = (int64_t)cu_count() * 8;
  const int grid = (int)(blocks < cap ? blocks : cap);
  if (bwd) hipLaunchKernelGGL((k_l2norm<T, D, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)dy, (T*)out, rows, eps);
  else hipLaunchKernelGGL((k_l2norm<T, D, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)nullptr, (T*)out, rows, eps);
}

void launch_l2norm(int dtype, int D, const void* x, const void* dy, void* out, int64_t rows, float eps, bool bwd,
                   hipStream_t st) {
#define LMOE_D(T)                                                        \
  if (D == 64) launch_t<T, 64>(x, dy, out, rows, eps, bwd, st);          \
  else if (D == 128) launch_t<T, 128>(x, dy, out, rows, eps, bwd, st);   \
  else launch_t<T, 256>(x, dy, out, rows, eps, bwd, st);
  if (dtype == LMOE_BF16) { LMOE_D(bf16) } else { LMOE_D(float) }
#undef LMOE_D
}

}  // namespace lmoe
