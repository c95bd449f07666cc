// Quadratic feature maps in front of chunk_linear_attn (HBM-bound: D inputs, about D^2/2 outputs per row).
//
// For a row x of D numbers the map is the concatenation
//      [ c0 (one entry, only if c0 != 0) | c1 x_i (D, only if c1 != 0) | cd x_i^2 (D) | co x_i x_j, i < j (D(D-1)/2) ]
// with the pairs (i, j) in row-major order of the strict upper triangle.  The Taylor map of Based
// (linear_moe/model/common_modules/feature_map.py:190-203: c0 = 1, c1 = D^-1/4, cd = (2D)^-1/2, co = D^-1/2, so
// that phi(q).phi(k) = 1 + s + s^2/2 with s = q.k/sqrt(D)) and the flattened map of ReBased (:206-246 after its
// layer norm: c0 = c1 = 0, cd = D^-1/2, co = (2/D)^1/2, phi(q).phi(k) = (q.k)^2/D) are both of this form.
//
// The F features are padded with zeros to Kp (a multiple of 64) and written as key blocks of 128 columns (the last
// one may have 64): block b is a contiguous [rows][width_b] matrix at element offset rows * 128 * b, which is the
// layout the chunk kernels take (head dimension 64 or 128); linear attention without decay is a sum over key
// blocks.  Backward:   dx_i = c1 dy_lin(i) + 2 cd x_i dy_diag(i) + co sum_{j != i} x_j dy_off(i, j).
#include "lmoe_launch.hpp"
#include "lmoe_seq.hpp"

namespace lmoe {

// element offset of feature f of row r in the blocked layout
__device__ __forceinline__ int64_t feat_offset(int64_t rows, int64_t r, int f, int Kp) {
  const int b = f >> 7, width = (Kp - 128 * b) >= 128 ? 128 : 64;
  return rows * 128 * b + r * width + (f & 127);
}

template <typename T, int D, int ROWS, bool BWD>
__global__ __launch_bounds__(NTHR) void k_quad_featmap(const T* __restrict__ x, T* __restrict__ y, const T* __restrict__ dy,
                                                       T* __restrict__ dx, int64_t rows, int Kp, float c0, float c1,
                                                       float cd, float co) {
  constexpr int NOFF = D * (D - 1) / 2;
  constexpr int VEC = ET<T>::VEC;
  typedef typename ET<T>::vec vec;
  constexpr int KPMAX = (1 + D + D * (D + 1) / 2 + 63) / 64 * 64, LDY = KPMAX + VEC;
  static_assert(KPMAX / VEC <= NTHR, "one thread per 16-byte feature group");
  __shared__ float s_x[ROWS * (D + 1)];
  __shared__ __attribute__((aligned(16))) T s_dy[BWD ? ROWS * LDY : VEC];   // backward: the dy rows of the tile
  __shared__ uint8_t s_pi[NOFF], s_pj[NOFF];
  const int tid = threadIdx.x;
  const int n0 = c0 != 0.0f ? 1 : 0, n1 = c1 != 0.0f ? D : 0;
  const int f_diag = n0 + n1, f_off = f_diag + D, F = f_off + NOFF;
  for (int i = tid; i < D; i += NTHR) {
    int o = i * D - i * (i + 1) / 2 - i - 1;       // pair (i, j) sits at o + j
    for (int j = i + 1; j < D; ++j) {
      s_pi[o + j] = (uint8_t)i;
      s_pj[o + j] = (uint8_t)j;
    }
  }
  // forward: the feature group of this thread and its factors
  const int gpr = Kp / VEC, rstep = NTHR / gpr > 0 ? NTHR / gpr : 1;
  int my_r0 = tid / gpr, my_f0 = (tid % gpr) * VEC;
  if (my_r0 >= rstep) my_r0 = ROWS;                 // threads beyond rstep * gpr idle in the forward
  int fa[VEC], fb[VEC];
  float fc[VEC];
  if constexpr (!BWD) {
    __syncthreads();                                // the pair table
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const int f = my_f0 + j;
      fa[j] = fb[j] = D;
      fc[j] = 0.0f;
      if (f < n0) fc[j] = c0;
      else if (f < f_diag) fc[j] = c1, fa[j] = f - n0;
      else if (f < f_off) fc[j] = cd, fa[j] = fb[j] = f - f_diag;
      else if (f < F) fc[j] = co, fa[j] = s_pi[f - f_off], fb[j] = s_pj[f - f_off];
    }
  }
  const int64_t ntiles = (rows + ROWS - 1) / ROWS;
  for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const int64_t r0 = tile * ROWS;
    const int nr = (int)(rows - r0 < ROWS ? rows - r0 : ROWS);
    __syncthreads();
    for (int e = tid; e < ROWS * D; e += NTHR) {
      const int r = e / D, c = e % D;
      s_x[r * (D + 1) + c] = r < nr ? ET<T>::to_f(x[(r0 + r) * D + c]) : 0.0f;
    }
    for (int r = tid; r < ROWS; r += NTHR) s_x[r * (D + 1) + D] = 1.0f;
    __syncthreads();
    if constexpr (!BWD) {
      // a thread keeps one 16-byte group of features for the whole kernel (its factors sit in registers) and
      // walks down the rows of the tile: value = coefficient * x[a] * x[b], with x[D] = 1 for the constant and
      // linear features
      for (int r = my_r0; r < nr; r += rstep) {
        const float* xr = s_x + r * (D + 1);
        vec o;
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[j] = ET<T>::from_f(fc[j] * xr[fa[j]] * xr[fb[j]]);
        *(vec*)(y + feat_offset(rows, r0 + r, my_f0, Kp)) = o;
      }
    } else {
      const int gpr = Kp / VEC;
      for (int e = tid; e < nr * gpr; e += NTHR) {
        const int r = e / gpr, f0 = (e % gpr) * VEC;
        *(vec*)(s_dy + r * LDY + f0) = *(const vec*)(dy + feat_offset(rows, r0 + r, f0, Kp));
      }
      __syncthreads();
      for (int e = tid; e < nr * D; e += NTHR) {
        const int r = e / D, i = e % D;
        const float* xr = s_x + r * (D + 1);
        const T* dr = s_dy + r * LDY;
        float acc = 0.0f;
        if (n1) acc += c1 * ET<T>::to_f(dr[n0 + i]);
        acc += 2.0f * cd * xr[i] * ET<T>::to_f(dr[f_diag + i]);
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < D; ++j) {
          if (j == i) continue;
          const int a = j < i ? j : i, b = j < i ? i : j;
          const int p = a * D - a * (a + 1) / 2 - a - 1 + b;
          t += xr[j] * ET<T>::to_f(dr[f_off + p]);
        }
        dx[(r0 + r) * D + i] = ET<T>::from_f(acc + co * t);
      }
    }
  }
}

int quad_featmap_features(int D, float c0, float c1) { return (c0 != 0.0f ? 1 : 0) + (c1 != 0.0f ? D : 0) + D + D * (D - 1) / 2; }

template <typename T, int D>
static void launch_fm(const void* x, void* y, const void* dy, void* dx, int64_t rows, int Kp, float c0, float c1,
                      float cd, float co, bool bwd, hipStream_t st) {
  constexpr int ROWS = D <= 16 ? 64 : (sizeof(T) == 2 ? 32 : 16);    // backward LDS: ROWS x (Kp + pad) elements
  const int64_t tiles = (rows + ROWS - 1) / ROWS, cap = (int64_t)cu_count() * 8;
  const int grid = (int)(tiles < cap ? tiles : cap);
  if (bwd)
    hipLaunchKernelGGL((k_quad_featmap<T, D, ROWS, true>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (T*)nullptr,
                       (const T*)dy, (T*)dx, rows, Kp, c0, c1, cd, co);
  else
    hipLaunchKernelGGL((k_quad_featmap<T, D, ROWS, false>), dim3(grid), dim3(NTHR), 0, st, (const T*)x, (T*)y,
                       (const T*)nullptr, (T*)nullptr, rows, Kp, c0, c1, cd, co);
}

void launch_quad_featmap(int dtype, const void* x, void* y, const void* dy, void* dx, int64_t rows, int D, int Kp,
                         float c0, float c1, float cd, float co, bool bwd, hipStream_t st) {
#define LMOE_FM(T)                                                                        \
  {                                                                                       \
    if (D == 8) launch_fm<T, 8>(x, y, dy, dx, rows, Kp, c0, c1, cd, co, bwd, st);         \
    else if (D == 16) launch_fm<T, 16>(x, y, dy, dx, rows, Kp, c0, c1, cd, co, bwd, st);  \
    else launch_fm<T, 32>(x, y, dy, dx, rows, Kp, c0, c1, cd, co, bwd, st);               \
  }
  if (dtype == LMOE_BF16) LMOE_FM(bf16) else LMOE_FM(float)
#undef LMOE_FM
}

}  // namespace lmoe
