// Row-wise epilogue / prologue kernels around the chunk ops.  All of them: fp32 math, one 16-byte
// vector per lane, D / VEC lanes per row, grid-stride over the rows, HBM-bound.
//
//  * RMS norm of the op's output rows, optionally times a swish gate:
//        y = x rstd w  [* gate sigmoid(gate)],   rstd = 1 / sqrt(mean(x^2) + eps)
//    (linear_moe/model/common_modules/layernorm.py:69-132 with IS_RMS_NORM, no bias / residual:
//    forward; :212-300 backward; the gate product is linear_moe/sequence_modeling/linear_attention.py:255).
//    Backward, with x^ = x rstd, s = swish(gate) (1 without a gate), u = dy s:
//        dx = rstd (u w - x^ mean(u w x^)),  dw = sum_rows u x^,  dgate = dy (x^ w) swish'(gate).
//    dw: every work-group sums its rows in registers, reduces its row groups through LDS and writes
//    one fp32 partial row; k_colsum adds the partial rows in a fixed order (bit-reproducible).
//  * SiLU followed by the L2 norm of q and k rows:  y = silu(x) / sqrt(sum silu(x)^2 + eps)
//    (linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:101-106) and its backward.
#include <mutex>

#include "lmoe_launch.hpp"
#include "lmoe_seq.hpp"

namespace lmoe {

template <int LPR> __device__ __forceinline__ float lanes_sum(float x) {
#pragma unroll
  for (int d = 1; d < LPR; d <<= 1) x += __shfl_xor(x, d, 64);
  return x;
}
__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + __expf(-z)); }

// ------------------------------------------------------------------------- //
// RMS norm (+ swish gate)
// ------------------------------------------------------------------------- //
template <typename T, int D, bool GATE>
__global__ __launch_bounds__(NTHR) void k_rmsnorm_fwd(const T* __restrict__ x, const T* __restrict__ w,
                                                      const T* __restrict__ gate, T* __restrict__ y,
                                                      float* __restrict__ rstd_out, int64_t rows, float eps) {
  constexpr int VEC = ET<T>::VEC, LPR = D / VEC, RPB = NTHR / LPR;
  typedef typename ET<T>::vec vec;
  const int lr = threadIdx.x % LPR, rb = threadIdx.x / LPR;
  float wf[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) wf[i] = w ? ET<T>::to_f(w[lr * VEC + i]) : 1.0f;
  for (int64_t r = (int64_t)blockIdx.x * RPB + rb; r < rows; r += (int64_t)gridDim.x * RPB) {
    const vec xv = *(const vec*)(x + r * D + lr * VEC);
    vec gv;
    if constexpr (GATE) gv = *(const vec*)(gate + r * D + lr * VEC);
    float xf[VEC], ss = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) { xf[i] = ET<T>::to_f(xv[i]); ss += xf[i] * xf[i]; }
    ss = lanes_sum<LPR>(ss);
    const float rstd = 1.0f / sqrtf(ss * (1.0f / D) + eps);
    vec o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float v = xf[i] * rstd * wf[i];
      if constexpr (GATE) { const float z = ET<T>::to_f(gv[i]); v *= z * sigmoidf_(z); }
      o[i] = ET<T>::from_f(v);
    }
    *(vec*)(y + r * D + lr * VEC) = o;
    if (rstd_out && lr == 0) rstd_out[r] = rstd;
  }
}

template <typename T, int D, bool GATE>
__global__ __launch_bounds__(NTHR) void k_rmsnorm_bwd(const T* __restrict__ x, const T* __restrict__ w,
                                                      const T* __restrict__ gate, const T* __restrict__ dy,
                                                      T* __restrict__ dx, T* __restrict__ dgate,
                                                      float* __restrict__ dw_part, int64_t rows, float eps) {
  constexpr int VEC = ET<T>::VEC, LPR = D / VEC, RPB = NTHR / LPR;
  typedef typename ET<T>::vec vec;
  __shared__ float s_dw[RPB][D];
  const int lr = threadIdx.x % LPR, rb = threadIdx.x / LPR;
  float wf[VEC], dwacc[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) { wf[i] = w ? ET<T>::to_f(w[lr * VEC + i]) : 1.0f; dwacc[i] = 0.f; }
  for (int64_t r = (int64_t)blockIdx.x * RPB + rb; r < rows; r += (int64_t)gridDim.x * RPB) {
    const vec xv = *(const vec*)(x + r * D + lr * VEC);
    const vec dv = *(const vec*)(dy + r * D + lr * VEC);
    vec gv;
    if constexpr (GATE) gv = *(const vec*)(gate + r * D + lr * VEC);
    float xf[VEC], uf[VEC], ss = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) { xf[i] = ET<T>::to_f(xv[i]); ss += xf[i] * xf[i]; }
    ss = lanes_sum<LPR>(ss);
    const float rstd = 1.0f / sqrtf(ss * (1.0f / D) + eps);
    vec og;
    float c = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float xh = xf[i] * rstd, d = ET<T>::to_f(dv[i]);
      float u = d;
      if constexpr (GATE) {
        const float z = ET<T>::to_f(gv[i]), sg = sigmoidf_(z);
        u = d * z * sg;
        og[i] = ET<T>::from_f(d * xh * wf[i] * sg * (1.0f + z * (1.0f - sg)));
      }
      dwacc[i] += u * xh;
      uf[i] = u * wf[i];
      c += uf[i] * xh;
      xf[i] = xh;
    }
    c = lanes_sum<LPR>(c) * (1.0f / D);
    vec o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(rstd * (uf[i] - xf[i] * c));
    *(vec*)(dx + r * D + lr * VEC) = o;
    if constexpr (GATE) *(vec*)(dgate + r * D + lr * VEC) = og;
  }
  if (dw_part) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) s_dw[rb][lr * VEC + i] = dwacc[i];
    __syncthreads();
    for (int c = threadIdx.x; c < D; c += NTHR) {
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < RPB; ++j) s += s_dw[j][c];
      dw_part[(int64_t)blockIdx.x * D + c] = s;
    }
  }
}

// out[c] = sum_b part[b][c]  (fixed order)
__global__ __launch_bounds__(NTHR) void k_colsum(const float* __restrict__ part, float* __restrict__ out, int nb, int D) {
  __shared__ float s_p[NTHR];
  const int c = blockIdx.x, t = threadIdx.x;
  float s = 0.f;
  for (int b = t; b < nb; b += NTHR) s += part[(int64_t)b * D + c];
  s_p[t] = s;
  __syncthreads();
  for (int d = NTHR / 2; d > 0; d >>= 1) {
    if (t < d) s_p[t] += s_p[t + d];
    __syncthreads();
  }
  if (t == 0) out[c] = s_p[0];
}

template <typename T, int D> static int rows_grid(int64_t rows) {
  constexpr int RPB = NTHR / (D / ET<T>::VEC);
  const int64_t blocks = (rows + RPB - 1) / RPB, cap = (int64_t)cu_count() * 8;
  return (int)(blocks < cap ? blocks : cap);
}

template <typename T, int D>
static void rmsnorm_t(const void* x, const void* w, const void* gate, const void* dy, void* out, void* dgate,
                      float* rstd, float* dw_part, float* dw, int64_t rows, float eps, bool bwd, hipStream_t st) {
  const int grid = rows_grid<T, D>(rows);
  if (!bwd) {
    if (gate) hipLaunchKernelGGL((k_rmsnorm_fwd<T, D, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)w, (const T*)gate, (T*)out, rstd, rows, eps);
    else hipLaunchKernelGGL((k_rmsnorm_fwd<T, D, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)w, (const T*)nullptr, (T*)out, rstd, rows, eps);
  } else {
    if (gate) hipLaunchKernelGGL((k_rmsnorm_bwd<T, D, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)w, (const T*)gate, (const T*)dy, (T*)out, (T*)dgate, dw_part, rows, eps);
    else hipLaunchKernelGGL((k_rmsnorm_bwd<T, D, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)w, (const T*)nullptr, (const T*)dy, (T*)out, (T*)nullptr, dw_part, rows, eps);
    if (dw_part) hipLaunchKernelGGL(k_colsum, dim3(D), dim3(NTHR), 0, st, (const float*)dw_part, dw, grid, D);
  }
}

// Library-owned scratch of the allocation-free backward entry point: the fp32 partial rows of dw for the largest grid
// this file launches on a 256-CU GPU (8 work-groups per CU) at the widest row, 2 MiB per GPU, held until the process
// ends.  The array's name is a host-side handle, not a device address: host code only ever uses the address that
// hipGetSymbolAddress returns for the current device (each GPU holds its own copy).
constexpr int64_t RMS_SCRATCH_FLOATS = 2048 * 256;
static __device__ __align__(256) float scratch[RMS_SCRATCH_FLOATS];

int rmsnorm_scratch(float** out, int64_t* capacity_floats) {
  constexpr int MAXDEV = 64;
  static float* ptrs[MAXDEV] = {};
  static std::mutex mu;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAXDEV) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  *capacity_floats = RMS_SCRATCH_FLOATS;
  return 0;
}

// number of fp32 partial rows k_rmsnorm_bwd writes (the caller sizes dw_part with it)
int rmsnorm_partials(int dtype, int D, int64_t rows) {
#define LMOE_D(T) (D == 64 ? rows_grid<T, 64>(rows) : D == 128 ? rows_grid<T, 128>(rows) : rows_grid<T, 256>(rows))
  return dtype == LMOE_BF16 ? LMOE_D(bf16) : LMOE_D(float);
#undef LMOE_D
}

void launch_rmsnorm(int dtype, int D, const void* x, const void* w, const void* gate, const void* dy, void* out,
                    void* dgate, float* rstd, float* dw_part, float* dw, int64_t rows, float eps, bool bwd, hipStream_t st) {
#define LMOE_D(T)                                                                                          \
  if (D == 64) rmsnorm_t<T, 64>(x, w, gate, dy, out, dgate, rstd, dw_part, dw, rows, eps, bwd, st);          \
  else if (D == 128) rmsnorm_t<T, 128>(x, w, gate, dy, out, dgate, rstd, dw_part, dw, rows, eps, bwd, st);   \
  else rmsnorm_t<T, 256>(x, w, gate, dy, out, dgate, rstd, dw_part, dw, rows, eps, bwd, st);
  if (dtype == LMOE_BF16) { LMOE_D(bf16) } else { LMOE_D(float) }
#undef LMOE_D
}

// ------------------------------------------------------------------------- //
// SiLU + L2 norm
// ------------------------------------------------------------------------- //
template <typename T, int D, bool BWD>
__global__ __launch_bounds__(NTHR) void k_silu_l2norm(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ out,
                                                      int64_t rows, float eps) {
  constexpr int VEC = ET<T>::VEC, LPR = D / VEC, RPB = NTHR / LPR;
  typedef typename ET<T>::vec vec;
  const int lr = threadIdx.x % LPR, rb = threadIdx.x / LPR;
  for (int64_t r = (int64_t)blockIdx.x * RPB + rb; r < rows; r += (int64_t)gridDim.x * RPB) {
    const vec xv = *(const vec*)(x + r * D + lr * VEC);
    float sf[VEC], ds[VEC], ss = 0.f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const float z = ET<T>::to_f(xv[i]), sg = sigmoidf_(z);
      sf[i] = z * sg;
      ds[i] = sg * (1.0f + z * (1.0f - sg));       // silu'(z)
      ss += sf[i] * sf[i];
    }
    ss = lanes_sum<LPR>(ss);
    const float rstd = 1.0f / sqrtf(ss + eps);
    vec o;
    if constexpr (BWD) {
      const vec dv = *(const vec*)(dy + r * D + lr * VEC);
      float df[VEC], sd = 0.f;
#pragma unroll
      for (int i = 0; i < VEC; ++i) { df[i] = ET<T>::to_f(dv[i]); sd += df[i] * sf[i]; }
      sd = lanes_sum<LPR>(sd);
      const float c = sd * rstd * rstd * rstd;
#pragma unroll
      for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f((df[i] * rstd - c * sf[i]) * ds[i]);
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(sf[i] * rstd);
    }
    *(vec*)(out + r * D + lr * VEC) = o;
  }
}

template <typename T, int D>
static void silu_l2norm_t(const void* x, const void* dy, void* out, int64_t rows, float eps, bool bwd, hipStream_t st) {
  const int grid = rows_grid<T, D>(rows);
  if (bwd) hipLaunchKernelGGL((k_silu_l2norm<T, D, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)dy, (T*)out, rows, eps);
  else hipLaunchKernelGGL((k_silu_l2norm<T, D, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)nullptr, (T*)out, rows, eps);
}

void launch_silu_l2norm(int dtype, int D, const void* x, const void* dy, void* out, int64_t rows, float eps, bool bwd,
                        hipStream_t st) {
#define LMOE_D(T)                                                            \
  if (D == 64) silu_l2norm_t<T, 64>(x, dy, out, rows, eps, bwd, st);         \
  else if (D == 128) silu_l2norm_t<T, 128>(x, dy, out, rows, eps, bwd, st);  \
  else silu_l2norm_t<T, 256>(x, dy, out, rows, eps, bwd, st);
  if (dtype == LMOE_BF16) { LMOE_D(bf16) } else { LMOE_D(float) }
#undef LMOE_D
}

}  // namespace lmoe
