// Gate construction in front of the chunk ops (elementwise, HBM-bound, fp32 math).
//
//  * gated delta rule (linear_moe/sequence_modeling/linear_attention.py:153-154):
//        beta = sigmoid(b),    g = -exp(A_log[h]) * softplus(a + dt_bias[h])    (g in fp32)
//    for a, b of shape [rows][H].  Backward:
//        db = dbeta beta (1 - beta),   da = dg * (-exp(A_log)) * sigmoid(a + dt_bias),
//        dA_log[h] = sum_rows dg g,    ddt_bias[h] = sum_rows da.
//    The two parameter gradients: every thread keeps one head (the grid stride is a multiple of H),
//    a work-group reduces its threads through LDS and writes one fp32 partial row [2][H]; k_colsum2
//    adds the partial rows in a fixed order.
//  * chunk_gla (linear_moe/sequence_modeling/gla/gla.py:85, :90-91):
//        gk = max(logsigmoid(x) / normalizer, clamp_min),   dx = dy (1 - sigmoid(x)) / normalizer [gk > clamp_min]
//  * HGRN2 (linear_moe/sequence_modeling/linear_rnn.py:327-335): from the forget projection f, in fp32,
//        k = 1 - sigmoid(f),  g = logsigmoid(f)                                   (no lower bound)
//        G = lb + (1 - lb) sigmoid(f),  k = 1 - G,  g = log G                     (lower bound lb[col])
//    k in the dtype of f, g in fp32.  Backward, with s = sigmoid(f) (lb = 0, G = s without a bound):
//        df = (dg / G - dk) (1 - lb) s (1 - s)
#include "lmoe_launch.hpp"
#include "lmoe_seq.hpp"

namespace lmoe {

__device__ __forceinline__ float sigm(float z) { return 1.0f / (1.0f + __expf(-z)); }
// torch's softplus (beta 1, threshold 20)
// (1 + e^z is formed in fp32: absolute error <= 6e-8, far inside the fp32 parity tolerance)
__device__ __forceinline__ float softplusf_(float z) { return z > 20.0f ? z : __logf(1.0f + __expf(z)); }
// logsigmoid(z) = min(z, 0) - log1p(exp(-|z|))
__device__ __forceinline__ float logsigmoidf_(float z) { return fminf(z, 0.0f) - __logf(1.0f + __expf(-fabsf(z))); }

template <typename T, bool BWD>
__global__ __launch_bounds__(NTHR) void k_gdn_gates(const T* __restrict__ a, const T* __restrict__ b,
                                                    const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                    float* __restrict__ g, T* __restrict__ beta,
                                                    const float* __restrict__ dg, const T* __restrict__ dbeta,
                                                    T* __restrict__ da, T* __restrict__ db, float* __restrict__ part,
                                                    int64_t n, int H) {
  __shared__ float s_red[2][NTHR];
  // blockDim.x is a multiple of H, so is the grid stride: a thread stays with one head
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int h = (int)(i0 % H);
  const float negA = -__expf(A_log[h]), bias = dt_bias[h];
  float sA = 0.f, sB = 0.f;
  for (int64_t i = i0; i < n; i += stride) {
    const float z = ET<T>::to_f(a[i]) + bias;
    const float bt = sigm(ET<T>::to_f(b[i]));
    if constexpr (!BWD) {
      g[i] = negA * softplusf_(z);
      beta[i] = ET<T>::from_f(bt);
    } else {
      const float d = dg[i];
      const float dz = d * negA * (z > 20.0f ? 1.0f : sigm(z));
      da[i] = ET<T>::from_f(dz);
      db[i] = ET<T>::from_f(ET<T>::to_f(dbeta[i]) * bt * (1.0f - bt));
      sA += d * negA * softplusf_(z);
      sB += dz;
    }
  }
  if constexpr (BWD) {
    s_red[0][threadIdx.x] = sA;
    s_red[1][threadIdx.x] = sB;
    __syncthreads();
    if ((int)threadIdx.x < H) {
      float ta = 0.f, tb = 0.f;
      for (int t = threadIdx.x; t < (int)blockDim.x; t += H) { ta += s_red[0][t]; tb += s_red[1][t]; }
      part[(int64_t)blockIdx.x * 2 * H + threadIdx.x] = ta;
      part[(int64_t)blockIdx.x * 2 * H + H + threadIdx.x] = tb;
    }
  }
}

// out[c] = sum_b part[b][c], c < ncol  (fixed order)
__global__ __launch_bounds__(NTHR) void k_colsum2(const float* __restrict__ part, float* __restrict__ out, int nb, int ncol) {
  __shared__ float s_p[NTHR];
  const int c = blockIdx.x, t = threadIdx.x;
  float s = 0.f;
  for (int b = t; b < nb; b += NTHR) s += part[(int64_t)b * ncol + c];
  s_p[t] = s;
  __syncthreads();
  for (int d = NTHR / 2; d > 0; d >>= 1) {
    if (t < d) s_p[t] += s_p[t + d];
    __syncthreads();
  }
  if (t == 0) out[c] = s_p[0];
}

static int gates_block(int H) { return (NTHR / H) * H; }
int gdn_gates_partials(int64_t rows, int H) {
  const int bd = gates_block(H);
  const int64_t n = rows * H, blocks = (n + bd - 1) / bd, cap = (int64_t)cu_count() * 8;
  return (int)(blocks < cap ? blocks : cap);
}

void launch_gdn_gates(int dtype, const void* a, const void* b, const float* A_log, const float* dt_bias, float* g,
                      void* beta, const float* dg, const void* dbeta, void* da, void* db, float* part, float* dparams,
                      int64_t rows, int H, bool bwd, hipStream_t st) {
  const int bd = gates_block(H), grid = gdn_gates_partials(rows, H);
  const int64_t n = rows * H;
#define LMOE_G(T)                                                                                                       \
  if (bwd) hipLaunchKernelGGL((k_gdn_gates<T, true>), dim3(grid), dim3(bd), 0, st, (const T*)a, (const T*)b, A_log, dt_bias, \
                              g, (T*)beta, dg, (const T*)dbeta, (T*)da, (T*)db, part, n, H);                              \
  else hipLaunchKernelGGL((k_gdn_gates<T, false>), dim3(grid), dim3(bd), 0, st, (const T*)a, (const T*)b, A_log, dt_bias, \
                          g, (T*)beta, dg, (const T*)dbeta, (T*)da, (T*)db, part, n, H);
  if (dtype == LMOE_BF16) { LMOE_G(bf16) } else { LMOE_G(float) }
#undef LMOE_G
  if (bwd) hipLaunchKernelGGL(k_colsum2, dim3(2 * H), dim3(NTHR), 0, st, (const float*)part, dparams, grid, 2 * H);
}

template <typename T, bool BWD>
__global__ __launch_bounds__(NTHR) void k_gla_gate(const T* __restrict__ x, const T* __restrict__ dy, T* __restrict__ out,
                                                   int64_t nvec, float inv_norm, float clamp_min) {
  constexpr int VEC = ET<T>::VEC;
  typedef typename ET<T>::vec vec;
  for (int64_t i = (int64_t)blockIdx.x * NTHR + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * NTHR) {
    const vec xv = *(const vec*)(x + i * VEC);
    vec dv, o;
    if constexpr (BWD) dv = *(const vec*)(dy + i * VEC);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float z = ET<T>::to_f(xv[j]);
      const float y = logsigmoidf_(z) * inv_norm;
      if constexpr (BWD) o[j] = ET<T>::from_f(y > clamp_min ? ET<T>::to_f(dv[j]) * (1.0f - sigm(z)) * inv_norm : 0.0f);
      else o[j] = ET<T>::from_f(fmaxf(y, clamp_min));
    }
    *(vec*)(out + i * VEC) = o;
  }
}

template <typename T, bool BWD>
__global__ __launch_bounds__(NTHR) void k_hgrn2_gate(const T* __restrict__ f, const float* __restrict__ lb,
                                                     T* __restrict__ k, float* __restrict__ g, const T* __restrict__ dk,
                                                     const float* __restrict__ dg, T* __restrict__ df, int64_t nvec, int D) {
  constexpr int VEC = ET<T>::VEC;
  typedef typename ET<T>::vec vec;
  for (int64_t i = (int64_t)blockIdx.x * NTHR + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * NTHR) {
    const vec fv = *(const vec*)(f + i * VEC);
    const int col = (int)((i * VEC) % D);
    float lo[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) lo[j] = lb ? lb[col + j] : 0.0f;
    if constexpr (BWD) {
      const vec dkv = *(const vec*)(dk + i * VEC);
      float dgv[VEC];
#pragma unroll
      for (int j = 0; j < VEC; j += 4) {
        const f32x4 t = *(const f32x4*)(dg + i * VEC + j);
        dgv[j] = t[0], dgv[j + 1] = t[1], dgv[j + 2] = t[2], dgv[j + 3] = t[3];
      }
      vec o;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float z = ET<T>::to_f(fv[j]), s = sigm(z), G = lo[j] + (1.0f - lo[j]) * s;
        // dg / G: for lb = 0 this is dg / s, and (1 / s) s (1 - s) = 1 - s stays finite as s -> 0
        const float dgG = lb ? dgv[j] / G * s : dgv[j];
        o[j] = ET<T>::from_f((dgG - ET<T>::to_f(dkv[j]) * s) * (1.0f - lo[j]) * (1.0f - s));
      }
      *(vec*)(df + i * VEC) = o;
    } else {
      vec kv;
      float lgv[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float z = ET<T>::to_f(fv[j]);
        float G, lg;
        if (lb) {
          G = lo[j] + (1.0f - lo[j]) * sigm(z);
          lg = __logf(G);
        } else {
          G = sigm(z);
          lg = logsigmoidf_(z);
        }
        kv[j] = ET<T>::from_f(1.0f - G);
        lgv[j] = lg;
      }
      *(vec*)(k + i * VEC) = kv;
#pragma unroll
      for (int j = 0; j < VEC; j += 4) *(f32x4*)(g + i * VEC + j) = f32x4{lgv[j], lgv[j + 1], lgv[j + 2], lgv[j + 3]};
    }
  }
}

void launch_hgrn2_gate(int dtype, const void* f, const float* lb, void* k, float* g, const void* dk, const float* dg,
                       void* df, int64_t n, int D, bool bwd, hipStream_t st) {
#define LMOE_G(T)                                                                                                     \
  {                                                                                                                   \
    const int64_t nvec = n / ET<T>::VEC, blocks = (nvec + NTHR - 1) / NTHR, cap = (int64_t)cu_count() * 8;            \
    const int grid = (int)(blocks < cap ? blocks : cap);                                                              \
    if (bwd) hipLaunchKernelGGL((k_hgrn2_gate<T, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)f, lb, (T*)nullptr, (float*)nullptr, (const T*)dk, dg, (T*)df, nvec, D); \
    else hipLaunchKernelGGL((k_hgrn2_gate<T, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)f, lb, (T*)k, g, (const T*)nullptr, (const float*)nullptr, (T*)nullptr, nvec, D); \
  }
  if (dtype == LMOE_BF16) LMOE_G(bf16) else LMOE_G(float)
#undef LMOE_G
}

void launch_gla_gate(int dtype, const void* x, const void* dy, void* out, int64_t n, float normalizer, float clamp_min,
                     bool bwd, hipStream_t st) {
#define LMOE_G(T)                                                                                                     \
  {                                                                                                                   \
    const int64_t nvec = n / ET<T>::VEC, blocks = (nvec + NTHR - 1) / NTHR, cap = (int64_t)cu_count() * 8;            \
    const int grid = (int)(blocks < cap ? blocks : cap);                                                              \
    if (bwd) hipLaunchKernelGGL((k_gla_gate<T, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)dy, (T*)out, nvec, 1.0f / normalizer, clamp_min); \
    else hipLaunchKernelGGL((k_gla_gate<T, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (const T*)nullptr, (T*)out, nvec, 1.0f / normalizer, clamp_min); \
  }
  if (dtype == LMOE_BF16) LMOE_G(bf16) else LMOE_G(float)
#undef LMOE_G
}

}  // namespace lmoe
