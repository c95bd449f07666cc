// Host-side launch functions, one translation unit per kernel family, and the
// (dtype, K, V) dispatcher they share.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/lmoe.h"

namespace lmoe {

// Stages of the three ops (argument of lmoe_launch_stage; declared in include/lmoe.h)
enum Stage {
  ST_GDN_WY_FWD = 0,   // gated delta rule: w, u, Tinv, P                (chunk-parallel)
  ST_STATE_FWD = 1,    // sequential state pass: hs (, vnew), ht; scalar gates and 2-byte chunk_gla: also the output o
  ST_OUT_FWD = 2,      // chunk_gla: output o (the forward runs it for fp32 only)   (chunk-parallel)
  ST_DV = 3,           // dv (simple_gla / gla; the backward entry points run it for fp32 only: ST_DQK forms dv for 2-byte elements)
  ST_STATE_BWD = 4,    // reverse sequential state pass: dhs (, dv_new), dh0
  ST_DQK = 5,          // dq, dk, gate gradient; gated delta rule: every gradient that follows the
                       // reverse state pass (dq, dk, dv, dbeta, dg)     (chunk-parallel)
  ST_GLA_INTRA_FWD = 7 // chunk_gla: intra-chunk attention matrix        (chunk-parallel)
};

// F<T, K, V>::run(a, st) for the runtime (dtype, K, V) of the problem
template <template <typename, int, int> class F>
inline void dispatch(const lmoe_args& a, hipStream_t st) {
  typedef __bf16 bf16_t;
#define LMOE_KV(T)                                                   \
  if (a.K == 64 && a.V == 64) F<T, 64, 64>::run(a, st);              \
  else if (a.K == 64 && a.V == 128) F<T, 64, 128>::run(a, st);       \
  else if (a.K == 128 && a.V == 64) F<T, 128, 64>::run(a, st);       \
  else F<T, 128, 128>::run(a, st);
  if (a.dtype == LMOE_BF16) { LMOE_KV(bf16_t) } else { LMOE_KV(float) }
#undef LMOE_KV
}

// the kernels of the gated delta rule also exist for K = 128, V = 256 (a value head twice as wide as the key head:
// expand_v = 2 at a head dimension of 128); the state passes cut V into slices anyway and the chunk-parallel
// backward loops over them, so one WY preparation and one read of q, k per kernel serve all 256 columns
template <template <typename, int, int> class F>
inline void dispatch_gdn(const lmoe_args& a, hipStream_t st) {
  typedef __bf16 bf16_t;
  if (a.K == 128 && a.V == 256) {
    if (a.dtype == LMOE_BF16) F<bf16_t, 128, 256>::run(a, st);
    else F<float, 128, 256>::run(a, st);
    return;
  }
  dispatch<F>(a, st);
}

void launch_state_fwd(const lmoe_args& a, hipStream_t st);        // chunk_simple_gla
// traced forward pass of chunk_simple_gla (bf16, K = V = 128, forward-only): false when the problem is not of that shape
bool launch_state_fwd_trace(const lmoe_args& a, long long* tr, int work_group, hipStream_t st);
void launch_gdn_state_fwd(const lmoe_args& a, hipStream_t st);    // gated delta rule
void launch_gdn_state_bwd(const lmoe_args& a, hipStream_t st);
// traced forward pass (bf16, K = V = 128, Tinv and hs given): false when the problem is not of that shape
bool launch_gdn_state_fwd_trace(const lmoe_args& a, long long* tr, int work_group, hipStream_t st);
void launch_gdn_wy_fwd(const lmoe_args& a, hipStream_t st);
void launch_bwd_dv(const lmoe_args& a, bool local, hipStream_t st);
void launch_state_bwd(const lmoe_args& a, hipStream_t st);        // chunk_simple_gla
void launch_bwd_dqk(const lmoe_args& a, hipStream_t st);          // chunk_simple_gla
void launch_gdn_bwd_chunk(const lmoe_args& a, hipStream_t st);    // gated delta rule: all chunk-parallel gradients
// chunk_gla: one kernel of the pipeline (stage = ST_GLA_INTRA_FWD, ST_STATE_FWD, ST_OUT_FWD,
// ST_STATE_BWD, ST_DV, ST_DQK)
void launch_gla(const lmoe_args& a, int stage, hipStream_t st);
// whether ST_STATE_FWD of this problem also forms the output o (then the forward does not run ST_OUT_FWD)
bool gla_fwd_fused(const lmoe_args& a);
// row-wise L2 normalisation of `rows` contiguous rows of D in {64, 128, 256} elements (bwd: out = dx)
void launch_l2norm(int dtype, int D, const void* x, const void* dy, void* out, int64_t rows, float eps, bool bwd,
                   hipStream_t st);
// RMS norm of `rows` contiguous rows (w, gate may be null); bwd: out = dx, dw_part = [rmsnorm_partials()][D]
void launch_rmsnorm(int dtype, int D, const void* x, const void* w, const void* gate, const void* dy, void* out,
                    void* dgate, float* rstd, float* dw_part, float* dw, int64_t rows, float eps, bool bwd, hipStream_t st);
int rmsnorm_partials(int dtype, int D, int64_t rows);
// the library-owned partial-row scratch of the current device (set up on its first use there); 0 or a hipError_t
int rmsnorm_scratch(float** ptr, int64_t* capacity_floats);
// y = l2norm(silu(x)) (bwd: out = dx)
void launch_silu_l2norm(int dtype, int D, const void* x, const void* dy, void* out, int64_t rows, float eps, bool bwd,
                        hipStream_t st);
// the gated-delta-rule mixer's prologue on the fused projection [T, B, H, 3 D] (fwd: o0, o1, o2 = q^, k^, silu(v) in
// [B, T, H, D]; bwd: o0 = d(projection)) and its epilogue o * swish(o_gate) with the change of layout (W = H D)
void launch_gdn_qkv_prologue(int dtype, int D, const void* qkv, const void* dq, const void* dk, const void* dv, void* o0,
                             void* o1, void* o2, int Tn, int Bn, int H, float eps, bool bwd, hipStream_t st);
void launch_swish_gate_relayout(int dtype, const void* o, const void* gate, const void* dy, void* out, void* dgate, int Tn,
                                int Bn, int W, bool bwd, hipStream_t st);
// gate construction of the gated delta rule (rows x H elements; bwd also fills dparams = [dA_log | ddt_bias])
void launch_gdn_gates(int dtype, const void* a, const void* b, const float* A_log, const float* dt_bias, float* g,
                      void* beta, const float* dg, const void* dbeta, void* da, void* db, float* part, float* dparams,
                      int64_t rows, int H, bool bwd, hipStream_t st);
int gdn_gates_partials(int64_t rows, int H);
// chunk_gla gate: logsigmoid(x) / normalizer, clamped from below (n elements, a multiple of 8)
void launch_gla_gate(int dtype, const void* x, const void* dy, void* out, int64_t n, float normalizer, float clamp_min,
                     bool bwd, hipStream_t st);
// HGRN2 gates: k = 1 - G, g = log G, G = lb + (1 - lb) sigmoid(f) (n elements, last dimension D, lb [D] or null)
void launch_hgrn2_gate(int dtype, const void* f, const float* lb, void* k, float* g, const void* dk, const float* dg,
                       void* df, int64_t n, int D, bool bwd, hipStream_t st);
// quadratic feature maps (Taylor / ReBased) into key blocks of 128 columns
int quad_featmap_features(int D, float c0, float c1);
void launch_quad_featmap(int dtype, const void* x, void* y, const void* dy, void* dx, int64_t rows, int D, int Kp,
                         float c0, float c1, float cd, float co, bool bwd, hipStream_t st);
// row routing of mixture-of-memories layers (rows of D elements, D a multiple of 8)
void launch_mom_gather(int dtype, const void* src, const int32_t* idx, const void* scale, void* out, int64_t nout, int D,
                       hipStream_t st);
void launch_mom_combine(int dtype, const void* src, const int32_t* idx, const void* w, void* out, int64_t ntok, int topk,
                        int D, hipStream_t st);
void launch_mom_rowdot(int dtype, const void* src, const int32_t* idx, const void* g, void* dw, int64_t ntok, int topk,
                       int D, hipStream_t st);
// token-by-token forward (decoding); delta = the (gated) delta rule
void launch_recurrent(const lmoe_args& a, bool delta, hipStream_t st);
void launch_selftest(int dtype, int kd, const void* A, const void* B, float* C, float* G, hipStream_t st);
}  // namespace lmoe
