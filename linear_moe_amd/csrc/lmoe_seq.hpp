// Sequence / chunk addressing shared by all kernels: maps a sequence index or a global
// chunk index to token ranges, for dense [B,T,...] input and for packed variable-length
// input (cu_seqlens).  Chunks never straddle a sequence boundary; the last chunk of a
// sequence may be partial.
#pragma once
#include "../../include/lmoe.h"
#include "lmoe_common.hpp"

namespace lmoe {

// The index arrays of packed input (cu_seqlens, seq_chunk0, chunk_map) are read-only for every
// kernel: reading them through the constant address space lets a uniform index become a scalar
// load, which does not wait for (or drain) the vector loads a kernel keeps in flight.
typedef const __attribute__((address_space(4))) int32_t* const_i32;
__device__ __forceinline__ const_i32 as_const(const int32_t* p) { return (const_i32)(uintptr_t)p; }

struct SeqInfo {
  int b;        // batch row holding the sequence
  int tok0;     // first token of the sequence inside that batch row
  int len;      // number of tokens
  int chunk0;   // global index of the sequence's first chunk
  int nchunks;  // ceil(len / 64)
};

__device__ __forceinline__ SeqInfo seq_info(const lmoe_args& a, int n) {
  SeqInfo s;
  if (a.cu_seqlens) {
    const const_i32 cu = as_const(a.cu_seqlens);
    s.b = 0; s.tok0 = cu[n]; s.len = cu[n + 1] - s.tok0;
    s.chunk0 = as_const(a.seq_chunk0)[n];
  } else {
    s.b = n; s.tok0 = 0; s.len = a.T;
    s.chunk0 = n * ((a.T + CH - 1) / CH);
  }
  s.nchunks = (s.len + CH - 1) / CH;
  return s;
}

// The i-th sequence a sequential pass takes: work-groups are dispatched in the order of their index, so a packed
// batch of unequal lengths runs its longest sequences first when the caller passes such an order (seq_order; NULL =
// as given).  Which work-group computes a (sequence, head, slice) does not change what it computes.
__device__ __forceinline__ int seq_at(const lmoe_args& a, int i) {
  return a.seq_order ? as_const(a.seq_order)[i] : i;
}

// Number of chunks of the call.  Packed input whose offsets never left the device comes with tables sized for an upper
// bound (a.NT >= the true count, which a.nt_dev holds): launches are sized by the bound, and no kernel touches a
// chunk index at or beyond the true count.
__device__ __forceinline__ int num_chunks(const lmoe_args& a) {
  return a.nt_dev ? as_const(a.nt_dev)[0] : a.NT;
}

struct ChunkInfo {
  int n;       // sequence
  int b;       // batch row
  int tok;     // first token of the chunk inside the batch row
  int len;     // valid tokens in this chunk (1..64)
  int last;    // 1 if this is the last chunk of its sequence
};

__device__ __forceinline__ ChunkInfo chunk_info(const lmoe_args& a, int cid) {
  ChunkInfo c;
  int lc, slen;
  if (a.cu_seqlens) {
    const const_i32 cm = as_const(a.chunk_map), cu = as_const(a.cu_seqlens);
    c.n = cm[2 * cid]; lc = cm[2 * cid + 1];
    c.b = 0;
    const int t0 = cu[c.n];
    slen = cu[c.n + 1] - t0;
    c.tok = t0 + lc * CH;
  } else {
    const int nts = (a.T + CH - 1) / CH;
    c.n = cid / nts; lc = cid % nts;
    c.b = c.n; slen = a.T;
    c.tok = lc * CH;
  }
  const int rem = slen - lc * CH;
  c.len = rem < CH ? rem : CH;
  c.last = rem <= CH;
  return c;
}

// pointer to row (b, tok, h) of a strided tensor with element type T
template <typename T>
__device__ __forceinline__ T* row_ptr(const lmoe_tensor& x, int b, int tok, int h) {
  return (T*)x.ptr + (int64_t)b * x.sb + (int64_t)tok * x.st + (int64_t)h * x.sh;
}
// The pseudo values of the gated delta rule and their gradient (vnew, dvnew) are library-side buffers laid out for the
// kernels that pass them on, not token-major: [chunk][head][V / 32][64 tokens][32 columns].  A 32-column slice of a
// chunk is one contiguous 4 KB (2-byte elements) block: the sequential passes write it as whole 128-byte lines
// (token-major, a slice's rows are 64-byte pieces 4 KB apart) and the chunk-parallel backward reads it in one piece.
// Pointer to (chunk cid, head h, column v0, token 0); the token stride is SLICE_COLS elements.
constexpr int SLICE_COLS = 32;
template <typename T>
__device__ __forceinline__ T* slice_ptr(const lmoe_tensor& x, int cid, int h, int H, int V, int v0) {
  return (T*)x.ptr + (((int64_t)cid * H + h) * (V / SLICE_COLS) + v0 / SLICE_COLS) * (CH * SLICE_COLS) + v0 % SLICE_COLS;
}
__device__ __forceinline__ int64_t row_off(const lmoe_tensor& x, int b, int tok, int h) {
  return (int64_t)b * x.sb + (int64_t)tok * x.st + (int64_t)h * x.sh;
}

// Load the chunk's 64 scalar log-decays, form the inclusive cumulative sum b_j in fp32 and
// leave in LDS: sb[j] = b_j, seb[j] = e^{b_j}, sed[j] = e^{b_63 - b_j} (seb / sed may be null).
// Tokens past the end of the chunk contribute 0.  All exponents are <= 0 for g <= 0.
// Must be called by all threads of the work-group; ends with a barrier.
__device__ __forceinline__ void chunk_gate_cumsum(const lmoe_args& a, int b, int tok, int len, int h,
                                                  float* sb, float* seb, float* sed) {
  if (threadIdx.x < 64) {
    const int j = threadIdx.x;
    float g = 0.f;
    if (a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr && j < len)
      g = load_scalar(a.g.ptr, a.g_dtype, row_off(a.g, b, tok + j, h));
    const float x = wave_incl_scan(g);
    const float xl = __shfl(x, 63, 64);
    sb[j] = x;
    if (seb) seb[j] = expf(x);
    if (sed) sed[j] = expf(xl - x);
  }
  __syncthreads();
}

// Split form of chunk_gate_cumsum for software-pipelined kernels: gate_prefetch issues the loads
// of a chunk's log-decays (lanes 0..63 of wave 0 hold one token each, raw bits), gate_finish
// turns them into the LDS arrays later.  Neither contains a barrier.
__device__ __forceinline__ uint32_t gate_prefetch(const lmoe_args& a, int b, int tok, int len, int h) {
  // branch-free: an ungated call reads a dummy word of k, tokens past the end re-read the last one
  const bool gated = a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr;
  const int j = min((int)(threadIdx.x & 63), len - 1);
  return load_scalar_raw(gated ? a.g.ptr : a.k.ptr, a.g_dtype, gated ? row_off(a.g, b, tok + j, h) : 0);
}
__device__ __forceinline__ void gate_finish(const lmoe_args& a, uint32_t raw, int len, float* sb, float* seb, float* sed) {
  if (threadIdx.x < 64) {
    const int j = threadIdx.x;
    const bool gated = a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr;
    const float x = wave_incl_scan((gated && j < len) ? scalar_from_raw(raw, a.g_dtype) : 0.f);
    const float xl = __shfl(x, 63, 64);
    if (sb) sb[j] = x;
    if (seb) seb[j] = expf(x);
    if (sed) sed[j] = expf(xl - x);
  }
}

// gate_finish for a caller that holds the raw bits in the lanes of one wave of its choice:
// `active` selects that wave (wave-uniform), `l` is the lane
__device__ __forceinline__ void gate_finish_wave(const lmoe_args& a, uint32_t raw, int len, int l, bool active,
                                                 float* sb, float* seb, float* sed) {
  if (active) {
    const bool gated = a.gate != LMOE_GATE_NONE && a.g.ptr != nullptr;
    const float x = wave_incl_scan((gated && l < len) ? scalar_from_raw(raw, a.g_dtype) : 0.f);
    const float xl = __shfl(x, 63, 64);
    sb[l] = x;
    seb[l] = expf(x);
    sed[l] = expf(xl - x);
  }
}

// number of work-groups of a persistent chunk-parallel kernel: `per_cu` per compute unit
inline int cu_count() {
  static int ncu = 0;
  if (ncu == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    ncu = n;
  }
  return ncu;
}
inline int persistent_grid(int nitems, int per_cu) {
  const int g = cu_count() * per_cu;
  return nitems < g ? nitems : g;
}

}  // namespace lmoe
