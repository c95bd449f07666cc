// Device toolkit shared by all chunk kernels (gfx950 / CDNA4, wave64).
//
// Conventions used by every kernel in this directory:
//  * a team is 256 threads = 4 wavefronts (a work-group is one to three teams); a chunk is 64 tokens;
//  * an LDS tile lies as it lies in memory: element (r, c) at tile[r * ld + c].  A product that
//    contracts along the tile columns reads its fragments row-wise (gemm_nt, load_frag); one that
//    contracts along the tile rows reads them through the transposing LDS read (gemm with AT / BT,
//    load_frag_t), so no operand is stored twice;
//  * MFMA shape: v_mfma_f32_16x16x32_bf16 for bf16 operands and
//    8 x v_mfma_f32_16x16x4_f32 for fp32 operands, behind the same fragment
//    layout (lane l holds row l%16, contraction elements 8*(l/16) .. +7);
//  * accumulator layout of one 16x16 block: lane l holds rows 4*(l/16)+i
//    (i = 0..3) of column l%16;
//  * helpers that index by lane / thread take that index as a last, defaulted argument: a
//    persistent kernel passes a value it refreshes per item (fresh_index), which keeps the
//    address arithmetic inside the iteration instead of hoisted into registers for the whole
//    kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lmoe {

typedef __bf16 bf16;
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int CH = 64;        // chunk length (tokens)
constexpr int GATE_ROWS = 5;  // rows of the gated delta rule's per-chunk gate table (e^b, e^{b_C - b}, beta, beta e^b, b)
constexpr int NTHR = 256;     // threads per work-group
constexpr int LPAD = 8;       // LDS row padding in elements (16 B for bf16, 32 B for fp32)

// Work-group barrier that orders LDS traffic only: waits for this wave's outstanding LDS
// operations, not for its global loads, so register prefetches issued before the barrier stay
// in flight across it (__syncthreads() would drain them).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// s_waitcnt vmcnt(0): every global load / store this wave has issued so far has completed (the
// scheduling barriers keep later loads behind it and earlier ones in front of it)
__device__ __forceinline__ void wait_all_loads() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __builtin_amdgcn_sched_barrier(0);
}

// x, in a form the compiler cannot prove loop-invariant
__device__ __forceinline__ int fresh_index(int x) {
  asm volatile("" : "+v"(x));
  return x;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }
// (uniform over the wave by construction; said to the compiler, so that what derives from it lives in scalar
// registers and the branches on it are scalar branches)
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); }

// ------------------------------------------------------------------------- //
// element traits
// ------------------------------------------------------------------------- //
template <typename T> struct ET;

template <> struct ET<bf16> {
  static constexpr int VEC = 8;                       // elements per 16-byte vector
  typedef bf16x8 vec;
  typedef bf16x4 vec4;      // four consecutive elements (one accumulator column group)
  typedef bf16x8 frag;
  static __device__ __forceinline__ vec zero() { vec z; for (int i = 0; i < 8; ++i) z[i] = (bf16)0.0f; return z; }
  static __device__ __forceinline__ float to_f(bf16 x) { return (float)x; }
  static __device__ __forceinline__ bf16 from_f(float x) { return (bf16)x; }
  static __device__ __forceinline__ frag load_frag(const bf16* p) { return *(const bf16x8*)p; }
  // Fragment of an operand stored with the contraction index along the ROWS of the tile:
  // lane (c = l%16, g = l/16) receives tile[k0 + 8g + i][n0 + c], i = 0..7, through two
  // ds_read_b64_tr_b16: inside each group of 16 lanes, lane s points at the 4 elements
  // tile[row + s/4][n0 + 4 (s%4) ..] and receives element (s%4) of the lanes 4j + s/4, j = 0..3,
  // i.e. the four rows row..row+3 of its own column.
  static __device__ __forceinline__ frag load_frag_t(const bf16* tile, int ld, int k0, int n0, int l = threadIdx.x & 63) {
    const int s = l & 15;
    const bf16* p = tile + (k0 + 8 * (l >> 4) + (s >> 2)) * ld + n0 + 4 * (s & 3);
    typedef __attribute__((address_space(3))) bf16x4 lds_b4;
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_b4*)p);
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_b4*)(p + 4 * ld));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
  static __device__ __forceinline__ void mma(f32x4& c, const frag& a, const frag& b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

struct f32frag { f32x4 lo, hi; };

template <> struct ET<float> {
  static constexpr int VEC = 4;
  typedef f32x4 vec;
  typedef f32x4 vec4;
  typedef f32frag frag;
  static __device__ __forceinline__ vec zero() { vec z = {0.f, 0.f, 0.f, 0.f}; return z; }
  static __device__ __forceinline__ float to_f(float x) { return x; }
  static __device__ __forceinline__ float from_f(float x) { return x; }
  static __device__ __forceinline__ frag load_frag(const float* p) {
    frag f; f.lo = *(const f32x4*)p; f.hi = *(const f32x4*)(p + 4); return f;
  }
  // contraction index along the rows of the tile: plain strided reads (fp32 is the parity path)
  static __device__ __forceinline__ frag load_frag_t(const float* tile, int ld, int k0, int n0, int l = threadIdx.x & 63) {
    const float* p = tile + (k0 + 8 * (l >> 4)) * ld + n0 + (l & 15);
    frag f;
#pragma unroll
    for (int i = 0; i < 4; ++i) { f.lo[i] = p[i * ld]; f.hi[i] = p[(i + 4) * ld]; }
    return f;
  }
  static __device__ __forceinline__ void mma(f32x4& c, const frag& a, const frag& b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.lo[i], b.lo[i], c, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.hi[i], b.hi[i], c, 0, 0, 0);
  }
};

// SiLU and its derivative in the form every kernel that applies them shares (the results agree bit for bit between
// the row kernels in front of the op and the op's own staging)
__device__ __forceinline__ float sigmoid_fast(float z) { return 1.0f / (1.0f + __expf(-z)); }
__device__ __forceinline__ float silu_of(float z) { return z * sigmoid_fast(z); }
__device__ __forceinline__ float silu_grad(float z) { const float a = sigmoid_fast(z); return a * (1.0f + z * (1.0f - a)); }

// e^x for the pairwise decay factors: library expf on the fp32 path (keeps 1e-5 parity),
// the hardware exp2 path for bf16 operands
template <typename T> __device__ __forceinline__ float texp(float x) {
  if constexpr (sizeof(T) == 4) return expf(x); else return __expf(x);
}
// The same with the argument scaled once up front: e^x = texp_scaled(x * TEXP_PRESCALE<T>); on the bf16 path the
// scale is log2(e) and the call is the bare hardware exp2, which saves a multiply per exponential in loops that
// form many exponentials of differences of the same few values.
template <typename T> constexpr float TEXP_PRESCALE = sizeof(T) == 4 ? 1.0f : 1.4426950408889634f;
template <typename T> __device__ __forceinline__ float texp_scaled(float x) {
  if constexpr (sizeof(T) == 4) return expf(x); else return __builtin_amdgcn_exp2f(x);
}

// ------------------------------------------------------------------------- //
// gemm_nt: acc[mi][ni] += A[arow0 + 16 mi + r][k] * B[brow0 + 16 ni + c][k], k in [k0, k1)
// (k0, k1 multiples of 32).  A, B: LDS tiles with leading dimensions lda, ldb.
// ------------------------------------------------------------------------- //
// PIPE (2-byte elements only): the fragments of step kk + 32 are requested before the products of step kk are
// issued (left to the compiler, every read is waited for right where it is used: a chain of LDS round trips).
// It costs a second set of fragment registers: for kernels whose latency is on a dependency chain, not for the
// one-shot kernels that live on occupancy.  The callers pass constant bounds, so the loop unrolls and the two
// fragment sets stay in registers.
template <typename T, int MB, int NB, bool PIPE = false>
__device__ __forceinline__ void gemm_nt(f32x4 (&acc)[MB][NB], const T* A, int lda, int arow0,
                                        const T* B, int ldb, int brow0, int k0, int k1, int l = threadIdx.x & 63) {
  const int r = l & 15, kg = (l >> 4) * 8;
  if constexpr (sizeof(T) == 2 && PIPE) {
    typename ET<T>::frag a[2][MB], b[2][NB];
    auto fetch = [&](int kk, int buf) {
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) a[buf][mi] = ET<T>::load_frag(A + (arow0 + 16 * mi + r) * lda + kk + kg);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) b[buf][ni] = ET<T>::load_frag(B + (brow0 + 16 * ni + r) * ldb + kk + kg);
    };
    fetch(k0, 0);
#pragma unroll
    for (int kk = k0, it = 0; kk < k1; kk += 32, ++it) {
      if (kk + 32 < k1) fetch(kk + 32, (it + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(acc[mi][ni], a[it & 1][mi], b[it & 1][ni]);
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
    for (int kk = k0; kk < k1; kk += 32) {
      typename ET<T>::frag a[MB], b[NB];
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) a[mi] = ET<T>::load_frag(A + (arow0 + 16 * mi + r) * lda + kk + kg);
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) b[ni] = ET<T>::load_frag(B + (brow0 + 16 * ni + r) * ldb + kk + kg);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(acc[mi][ni], a[mi], b[ni]);
    }
  }
}

// gemm: like gemm_nt, but either operand may be stored with the contraction index along the
// rows of its tile (AT / BT = true):  AT = false: A[a0 + m][k]   AT = true: A[k][a0 + m]
//                                     BT = false: B[b0 + n][k]   BT = true: B[k][b0 + n]
template <typename T, int MB, int NB, bool AT, bool BT, bool PIPE = false>
__device__ __forceinline__ void gemm(f32x4 (&acc)[MB][NB], const T* A, int lda, int a0,
                                     const T* B, int ldb, int b0, int k0, int k1, int l = threadIdx.x & 63) {
  const int r = l & 15, kg = (l >> 4) * 8;
  if constexpr (sizeof(T) == 2 && PIPE) {
    // fragments one step ahead of the products, as in gemm_nt
    typename ET<T>::frag a[2][MB], b[2][NB];
    auto fetch = [&](int kk, int buf) {
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) {
        if constexpr (AT) a[buf][mi] = ET<T>::load_frag_t(A, lda, kk, a0 + 16 * mi, l);
        else a[buf][mi] = ET<T>::load_frag(A + (a0 + 16 * mi + r) * lda + kk + kg);
      }
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        if constexpr (BT) b[buf][ni] = ET<T>::load_frag_t(B, ldb, kk, b0 + 16 * ni, l);
        else b[buf][ni] = ET<T>::load_frag(B + (b0 + 16 * ni + r) * ldb + kk + kg);
      }
    };
    fetch(k0, 0);
#pragma unroll
    for (int kk = k0, it = 0; kk < k1; kk += 32, ++it) {
      if (kk + 32 < k1) fetch(kk + 32, (it + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(acc[mi][ni], a[it & 1][mi], b[it & 1][ni]);
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
    for (int kk = k0; kk < k1; kk += 32) {
      typename ET<T>::frag a[MB], b[NB];
#pragma unroll
      for (int mi = 0; mi < MB; ++mi) {
        if constexpr (AT) a[mi] = ET<T>::load_frag_t(A, lda, kk, a0 + 16 * mi, l);
        else a[mi] = ET<T>::load_frag(A + (a0 + 16 * mi + r) * lda + kk + kg);
      }
#pragma unroll
      for (int ni = 0; ni < NB; ++ni) {
        if constexpr (BT) b[ni] = ET<T>::load_frag_t(B, ldb, kk, b0 + 16 * ni, l);
        else b[ni] = ET<T>::load_frag(B + (b0 + 16 * ni + r) * ldb + kk + kg);
      }
#pragma unroll
      for (int mi = 0; mi < MB; ++mi)
#pragma unroll
        for (int ni = 0; ni < NB; ++ni) ET<T>::mma(acc[mi][ni], a[mi], b[ni]);
    }
  }
}

template <int MB, int NB>
__device__ __forceinline__ void acc_zero(f32x4 (&acc)[MB][NB]) {
#pragma unroll
  for (int mi = 0; mi < MB; ++mi)
#pragma unroll
    for (int ni = 0; ni < NB; ++ni) acc[mi][ni] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// row / column of accumulator element i of block (mi, ni)
__device__ __forceinline__ int acc_row(int mi, int i) { return 16 * mi + 4 * (lane_id() >> 4) + i; }
__device__ __forceinline__ int acc_col(int ni) { return 16 * ni + (lane_id() & 15); }

// store one 16x16 accumulator block to an LDS tile as tile[row][col] (row = M index)
template <typename T>
__device__ __forceinline__ void acc_to_lds(const f32x4& a, T* tile, int ld, int row0, int col0, int l = threadIdx.x & 63) {
  const int r = row0 + 4 * (l >> 4), c = col0 + (l & 15);
#pragma unroll
  for (int i = 0; i < 4; ++i) tile[(r + i) * ld + c] = ET<T>::from_f(a[i]);
}
// store transposed: tile[col][row] -- the lane's 4 values are contiguous
template <typename T>
__device__ __forceinline__ void acc_to_lds_t(const f32x4& a, T* tile, int ld, int row0, int col0, int l = threadIdx.x & 63) {
  const int r = row0 + 4 * (l >> 4), c = col0 + (l & 15);
  T* p = tile + c * ld + r;
  if constexpr (sizeof(T) == 2) {
    bf16x4 v; v[0] = (bf16)a[0]; v[1] = (bf16)a[1]; v[2] = (bf16)a[2]; v[3] = (bf16)a[3];
    *(bf16x4*)p = v;
  } else {
    *(f32x4*)p = a;
  }
}

// Store the 16-row strip a wave holds in accumulators (NB*16 columns) to global memory with
// 16-byte vector stores, through a wave-private LDS staging area stg[16][NB*16 + LPAD].
// gdst points at row 0 / column 0 of the strip; rows >= nvalid are not written.  Only the
// calling wave touches stg, so no work-group barrier is involved.  With ADD the strip is added
// to what the destination already holds (read with the same 16-byte vectors).
template <typename T, int NB, bool ADD = false>
__device__ __forceinline__ void store_strip(const f32x4 (&acc)[1][NB], T* stg, T* __restrict__ gdst,
                                            int64_t row_stride, int nvalid, float mul, int l = threadIdx.x & 63) {
  constexpr int W = NB * 16, LD = W + LPAD, VEC = ET<T>::VEC, VPR = W / VEC;
  typedef typename ET<T>::vec vec;
#pragma unroll
  for (int ni = 0; ni < NB; ++ni)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      stg[(4 * (l >> 4) + i) * LD + 16 * ni + (l & 15)] = ET<T>::from_f(acc[0][ni][i] * mul);
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int idx = l; idx < 16 * VPR; idx += 64) {
    const int r = idx / VPR, c = (idx % VPR) * VEC;
    if (r < nvalid) {
      T* g = gdst + (int64_t)r * row_stride + c;
      if constexpr (ADD) {
        vec o = *(const vec*)g;
        const vec x = *(const vec*)(stg + r * LD + c);
#pragma unroll
        for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(ET<T>::to_f(o[i]) + ET<T>::to_f(x[i]));
        *(vec*)g = o;
      } else {
        *(vec*)g = *(const vec*)(stg + r * LD + c);
      }
    }
  }
}

// The same for a strip held transposed (acc[ni]: rows = columns 16 ni + 4 (l / 16) + e of the strip, column = row l % 16
// of the strip, i.e. a lane holds four consecutive columns of one row): 8-byte writes into the staging area.
template <typename T, int NB>
__device__ __forceinline__ void store_strip_t(const f32x4 (&acc)[NB], T* stg, T* __restrict__ gdst,
                                              int64_t row_stride, int nvalid, float mul, int l = threadIdx.x & 63) {
  constexpr int W = NB * 16, LD = W + LPAD, VEC = ET<T>::VEC, VPR = W / VEC;
  typedef typename ET<T>::vec vec;
#pragma unroll
  for (int ni = 0; ni < NB; ++ni) {
    const f32x4 x = acc[ni] * mul;
    acc_to_lds_t<T>(x, stg, LD, 16 * ni, 0, l);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int idx = l; idx < 16 * VPR; idx += 64) {
    const int r = idx / VPR, c = (idx % VPR) * VEC;
    if (r < nvalid) *(vec*)(gdst + (int64_t)r * row_stride + c) = *(const vec*)(stg + r * LD + c);
  }
}

// Operands that never leave the registers.  A pair of 16-wide accumulator blocks of a transposed product lies in a
// lane as elements e = 0..3 of block 2s (contraction index 32 s + 4 g + e, g = l / 16) and of block 2s + 1
// (32 s + 16 + 4 g + e); frag_of_blocks packs them into an MFMA operand in that numbering, and
// load_frag_t_blocks reads the other operand (a tile with the contraction index along its rows) in the same
// numbering through the transposing LDS read: lane (c = l % 16, g) receives tile[k0 + 4 g + e][n0 + c] and
// tile[k0 + 16 + 4 g + e][n0 + c].  The contraction index may be numbered freely as long as both operands agree.
__device__ __forceinline__ bf16x8 frag_of_blocks(const f32x4& a, const f32x4& b) {
  bf16x8 f;
#pragma unroll
  for (int i = 0; i < 4; ++i) { f[i] = (bf16)a[i]; f[4 + i] = (bf16)b[i]; }
  return f;
}
__device__ __forceinline__ bf16x8 load_frag_t_blocks(const bf16* tile, int ld, int k0, int n0, int l = threadIdx.x & 63) {
  const int s = l & 15;
  const bf16* p = tile + (k0 + 4 * (l >> 4) + (s >> 2)) * ld + n0 + 4 * (s & 3);
  typedef __attribute__((address_space(3))) bf16x4 lds_b4;
  const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_b4*)p);
  const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_b4*)(p + 16 * ld));
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// ------------------------------------------------------------------------- //
// fragments held in registers
// ------------------------------------------------------------------------- //
// multiply the 8 contraction elements a lane holds by s8[0..7]
template <typename T> __device__ __forceinline__ void scale_frag8(typename ET<T>::frag& f, const float* s8) {
  const f32x4 s0 = *(const f32x4*)s8, s1 = *(const f32x4*)(s8 + 4);
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { f[i] = (bf16)((float)f[i] * s0[i]); f[i + 4] = (bf16)((float)f[i + 4] * s1[i]); }
  } else {
    f.lo *= s0; f.hi *= s1;
  }
}

// f = -f
__device__ __forceinline__ void frag_negate(bf16x8& f) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  u32x4 w = __builtin_bit_cast(u32x4, f);
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] ^= 0x80008000u;
  f = __builtin_bit_cast(bf16x8, w);
}
__device__ __forceinline__ void frag_negate(f32frag& f) { f.lo = -f.lo; f.hi = -f.hi; }
__device__ __forceinline__ void frag_keep_if(bf16x8& f, bool ok) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  u32x4 w = __builtin_bit_cast(u32x4, f);
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = ok ? w[i] : 0u;
  f = __builtin_bit_cast(bf16x8, w);
}
__device__ __forceinline__ void frag_keep_if(f32frag& f, bool ok) {
#pragma unroll
  for (int i = 0; i < 4; ++i) { f.lo[i] = ok ? f.lo[i] : 0.f; f.hi[i] = ok ? f.hi[i] : 0.f; }
}

// MFMA A-fragments of one 16-row strip of a row-major matrix with D columns, loaded straight from
// global memory: lane (r = l%16, g = l/16) holds, for contraction step j, the 8 elements
// [row0 + r][32 j + 8 g ..].  Rows beyond `last` re-read row `last` (branch-free, so a prefetch
// stays in flight); mask() zeroes the rows >= nvalid when the strip is consumed.
template <typename T, int D> struct RowFrags {
  static constexpr int KS = D / 32;
  typename ET<T>::frag f[KS];
  __device__ __forceinline__ void load(const T* __restrict__ base, int64_t row_stride, int row0, int last, int l = threadIdx.x & 63) {
    int r = row0 + (l & 15);
    r = r < last ? r : last;
    const T* p = base + (int64_t)r * row_stride + 8 * (l >> 4);
#pragma unroll
    for (int j = 0; j < KS; ++j) f[j] = ET<T>::load_frag(p + 32 * j);
  }
  __device__ __forceinline__ void mask(int row0, int nvalid) {
    if (row0 + 16 <= nvalid) return;            // uniform: full strips (the common case) skip it
    const bool ok = row0 + (lane_id() & 15) < nvalid;
#pragma unroll
    for (int j = 0; j < KS; ++j) frag_keep_if(f[j], ok);
  }
};

// ------------------------------------------------------------------------- //
// cooperative global <-> LDS tile movement (all 256 threads)
//   a tile is ROWS x COLS elements, source rows `row_stride` elements apart;
//   rows >= nvalid read as zero / are not written.
// ------------------------------------------------------------------------- //
template <typename T, int ROWS, int COLS> struct TileIO {
  static constexpr int VEC = ET<T>::VEC;
  static constexpr int VPR = COLS / VEC;                 // vectors per row
  static constexpr int NVEC = ROWS * VPR;                // vectors in the tile
  static constexpr int PASSES = (NVEC + NTHR - 1) / NTHR;
  typedef typename ET<T>::vec vec;
  struct Regs { vec v[PASSES]; };

  // thread index inside a team of 256: work-groups of 512 threads use two teams (waves 0-3 and
  // 4-7) that each move whole tiles
  static __device__ __forceinline__ void coords(int p, int& row, int& col, int tid = threadIdx.x & (NTHR - 1)) {
    const int idx = p * NTHR + tid;
    row = idx / VPR; col = (idx % VPR) * VEC;
  }
  // Branch-free loads: rows >= nvalid (nvalid >= 1) re-read the last valid row, so that no load
  // sits behind a branch and the compiler can count outstanding loads exactly (prefetches stay in
  // flight across barriers).  mask() then zeroes the rows >= nvalid; software-pipelined kernels
  // call load_nomask() when they issue a prefetch and mask() when they consume it.
  static __device__ __forceinline__ void load_nomask(Regs& r, const T* __restrict__ src, int64_t row_stride, int nvalid, int tid = threadIdx.x & (NTHR - 1)) {
    const int last = (nvalid < ROWS ? nvalid : ROWS) - 1;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      row = row < last ? row : last;
      r.v[p] = *(const vec*)(src + (int64_t)row * row_stride + col);
    }
  }
  static __device__ __forceinline__ void mask(Regs& r, int nvalid, int tid = threadIdx.x & (NTHR - 1)) {
    if (nvalid >= ROWS) return;                 // uniform: full tiles (the common case) skip it
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      const bool ok = row < nvalid;
      u32x4 w = __builtin_bit_cast(u32x4, r.v[p]);
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = ok ? w[i] : 0u;
      r.v[p] = __builtin_bit_cast(vec, w);
    }
  }
  static __device__ __forceinline__ void load(Regs& r, const T* __restrict__ src, int64_t row_stride, int nvalid) {
    load_nomask(r, src, row_stride, nvalid);
    mask(r, nvalid);
  }
  // tile[row][col] = x
  static __device__ __forceinline__ void store_lds(const Regs& r, T* tile, int ld, int tid = threadIdx.x & (NTHR - 1)) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      if (row < ROWS) *(vec*)(tile + row * ld + col) = r.v[p];
    }
  }
  // tile[row][col] = x * rs[row]
  static __device__ __forceinline__ void store_lds_scaled(const Regs& r, T* tile, int ld, const float* rs, int tid = threadIdx.x & (NTHR - 1)) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      if (row < ROWS) {
        const float s = rs[row];
        vec o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(ET<T>::to_f(r.v[p][i]) * s);
        *(vec*)(tile + row * ld + col) = o;
      }
    }
  }
  // tileT[col][row] = x * (rs ? rs[row] : 1)
  static __device__ __forceinline__ void store_lds_t(const Regs& r, T* tileT, int ldT, const float* rs) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col);
      if (row < ROWS) {
        const float s = rs ? rs[row] : 1.0f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) tileT[(col + i) * ldT + row] = ET<T>::from_f(ET<T>::to_f(r.v[p][i]) * s);
      }
    }
  }
  // fp32 tile[row][col] = (float) x
  static __device__ __forceinline__ void store_lds_f32(const Regs& r, float* tile, int ld) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col);
      if (row < ROWS) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) tile[row * ld + col + i] = ET<T>::to_f(r.v[p][i]);
      }
    }
  }
  // tile[row][col] = x * f(row, col)           (f: fp32 factor per element)
  template <typename F>
  static __device__ __forceinline__ void store_lds_elem(const Regs& r, T* tile, int ld, F f) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col);
      if (row < ROWS) {
        vec o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) o[i] = ET<T>::from_f(ET<T>::to_f(r.v[p][i]) * f(row, col + i));
        *(vec*)(tile + row * ld + col) = o;
      }
    }
  }
  // tileT[col][row] = x * f(row, col)
  template <typename F>
  static __device__ __forceinline__ void store_lds_t_elem(const Regs& r, T* tileT, int ldT, F f) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col);
      if (row < ROWS) {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          tileT[(col + i) * ldT + row] = ET<T>::from_f(ET<T>::to_f(r.v[p][i]) * f(row, col + i));
      }
    }
  }
  // registers <- tile[row][col]  /  global[row][col] <- registers (rows < nvalid): the two halves of
  // lds_to_global for callers that must leave the tile before the stores are issued
  static __device__ __forceinline__ void load_lds(Regs& r, const T* tile, int ld, int tid = threadIdx.x & (NTHR - 1)) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      row = row < ROWS ? row : ROWS - 1;
      r.v[p] = *(const vec*)(tile + row * ld + col);
    }
  }
  // STREAM: the tile is written once and read much later by another kernel (an intermediate or a result of a
  // large call): stored with the non-temporal hint, so that it does not displace what the work-groups of
  // this kernel share through the L2 (measured on the gated delta rule at 32 K tokens x 16 heads: the
  // two sequential passes 2 to 3 % faster)
  template <bool STREAM> static __device__ __forceinline__ void put(const vec& x, vec* p) {
    if constexpr (STREAM) __builtin_nontemporal_store(x, p);
    else *p = x;
  }
  template <bool STREAM = false>
  static __device__ __forceinline__ void store_global(const Regs& r, T* __restrict__ dst, int64_t row_stride, int nvalid, int tid = threadIdx.x & (NTHR - 1)) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      if (row < ROWS && row < nvalid) put<STREAM>(r.v[p], (vec*)(dst + (int64_t)row * row_stride + col));
    }
  }
  // Branch-free form of load_lds + store_global (nvalid >= 1): a thread whose row is >= nvalid reads
  // and rewrites row nvalid - 1, i.e. stores the same bytes to the same address as the thread that
  // owns that row.  No store sits behind a branch, so the compiler can count outstanding memory
  // operations exactly and the caller's prefetches stay in flight across the stores.
  static __device__ __forceinline__ void load_lds_clamped(Regs& r, const T* tile, int ld, int nvalid, int tid = threadIdx.x & (NTHR - 1)) {
    const int last = (nvalid < ROWS ? nvalid : ROWS) - 1;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      row = row < last ? row : last;
      r.v[p] = *(const vec*)(tile + row * ld + col);
    }
  }
  template <bool STREAM = false>
  static __device__ __forceinline__ void store_global_clamped(const Regs& r, T* __restrict__ dst, int64_t row_stride, int nvalid, int tid = threadIdx.x & (NTHR - 1)) {
    const int last = (nvalid < ROWS ? nvalid : ROWS) - 1;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      row = row < last ? row : last;
      put<STREAM>(r.v[p], (vec*)(dst + (int64_t)row * row_stride + col));
    }
  }
  // global[row][col] = tile[row][col]
  template <bool STREAM = false>
  static __device__ __forceinline__ void lds_to_global(const T* tile, int ld, T* __restrict__ dst, int64_t row_stride, int nvalid, int tid = threadIdx.x & (NTHR - 1)) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      int row, col; coords(p, row, col, tid);
      if (row < ROWS && row < nvalid) put<STREAM>(*(const vec*)(tile + row * ld + col), (vec*)(dst + (int64_t)row * row_stride + col));
    }
  }
};

// ------------------------------------------------------------------------- //
// gates
// ------------------------------------------------------------------------- //
// scalar gate / beta value for one token; dtype: 0 = bf16, 1 = fp32; null pointer = 0
__device__ __forceinline__ float load_scalar(const void* p, int dtype, int64_t idx) {
  if (p == nullptr) return 0.f;
  return dtype == 1 ? ((const float*)p)[idx] : (float)((const bf16*)p)[idx];
}

// Two-step variant for prefetching: fetch the raw bits now, convert when the value is used, so
// that no wait on the load is placed right behind the issue of a batch of prefetches.
__device__ __forceinline__ uint32_t load_scalar_raw(const void* p, int dtype, int64_t idx) {
  return dtype == 1 ? ((const uint32_t*)p)[idx] : (uint32_t)((const uint16_t*)p)[idx];
}
__device__ __forceinline__ float scalar_from_raw(uint32_t raw, int dtype) {
  return __uint_as_float(dtype == 1 ? raw : raw << 16);
}

// inclusive prefix sum across the 64 lanes of a wavefront
// (data-parallel-primitive moves on the vector ALU: shifts by 1, 2, 4, 8 inside each row of 16 lanes, then
// the last lane of rows 0 and 2 into rows 1 and 3, then lane 31 into rows 2 and 3; six exchanges through the
// LDS crossbar cost about 0.2 us on a chain that has nothing else to do)
template <int CTRL, int ROWS> __device__ __forceinline__ float dpp_or_zero(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROWS, 0xf, false));
}
__device__ __forceinline__ float wave_incl_scan(float x) {
  x += dpp_or_zero<0x111, 0xf>(x);      // row_shr:1
  x += dpp_or_zero<0x112, 0xf>(x);      // row_shr:2
  x += dpp_or_zero<0x114, 0xf>(x);      // row_shr:4
  x += dpp_or_zero<0x118, 0xf>(x);      // row_shr:8
  x += dpp_or_zero<0x142, 0xa>(x);      // row_bcast:15 into rows 1 and 3
  x += dpp_or_zero<0x143, 0xc>(x);      // row_bcast:31 into rows 2 and 3
  return x;
}
// sum over aligned groups of N consecutive lanes (N = 2, 4, 8, 16: inside a row of 16 lanes), every lane of a group
// receives the total: lane exchanges on the vector ALU (pairs, quads, the mirrored half-row, the mirrored row)
// instead of trips through the LDS crossbar
template <int N> __device__ __forceinline__ float group_sum(float x) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8 || N == 16, "a power of two inside a row of 16 lanes");
  if constexpr (N >= 2) x += dpp_or_zero<0xB1, 0xf>(x);     // quad_perm [1, 0, 3, 2]
  if constexpr (N >= 4) x += dpp_or_zero<0x4E, 0xf>(x);     // quad_perm [2, 3, 0, 1]
  if constexpr (N >= 8) x += dpp_or_zero<0x141, 0xf>(x);    // row_half_mirror
  if constexpr (N >= 16) x += dpp_or_zero<0x140, 0xf>(x);   // row_mirror
  return x;
}
// inclusive suffix sum (reverse cumulative sum) across the 64 lanes: total - (prefix sum before the lane), with the
// prefix sums from the exchanges on the vector ALU above (six dependent exchanges through the LDS crossbar sat on the
// path of the one wave every other wave of the work-group waits for).  The difference is exact to an ulp of the
// largest prefix sum, which is at most twice the largest suffix sum.
__device__ __forceinline__ float wave_rev_scan(float x) {
  const float incl = wave_incl_scan(x);
  const float total = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, incl), 63));
  return total - (incl - x);
}
// sum over the 64 lanes, in every lane: the row totals, then the four of them through scalar registers
// (to be called with all 64 lanes active, like group_sum: a lane that is switched off contributes whatever its
// register held, and reading lane 0, 16, 32 or 48 while it is off returns that stale value)
__device__ __forceinline__ float wave_sum(float x) {
  x = group_sum<16>(x);
  const int xi = __builtin_bit_cast(int, x);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 16)) +
         (__builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(xi, 48)));
}

}  // namespace lmoe
