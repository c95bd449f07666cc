/*
 * lmoe.h -- C ABI of liblmoe_hip.so: MI355X (gfx950) chunked linear-attention kernels.
 *
 * This is the drop-in boundary for the one hot path the reference
 * (OpenSparseLLMs/Linear-MoE) delegates to flash-linear-attention ("fla"):
 * the reference's token mixers bind python callables at import time and call them in
 * forward(); a maintainer binds this library with ctypes instead.
 * Every entry point below names the reference call site it serves.
 *
 * Conventions
 *  - plain C types only; the caller owns all memory (device pointers unless stated);
 *    the library never allocates or frees device memory and keeps no pointer after return;
 *  - every function returns 0 on success, a negative value for an invalid argument
 *    (nothing was launched) or a positive hipError_t; lmoe_last_error() gives the text
 *    (thread-local);
 *  - all work is enqueued asynchronously on the `stream` argument (a hipStream_t passed
 *    as void*); no host synchronisation, no use of the default stream;
 *  - results are deterministic (no atomics): re-execution by activation recompute gives
 *    bit-identical outputs.
 */
#ifndef LMOE_H_
#define LMOE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LMOE_BF16 0
#define LMOE_F32 1

#define LMOE_GATE_NONE 0   /* no decay (basic linear attention)                  */
#define LMOE_GATE_SCALAR 1 /* one log-decay per token and head   g: [B,T,H]      */
#define LMOE_GATE_VECTOR 2 /* one log-decay per token, head, key channel [B,T,H,K] */

#define LMOE_CHUNK 64

/* A tensor addressed as x[b][t][h][d]: element offset b*sb + t*st + h*sh + d.
 * Both fla layouts ([B,H,T,D] "head first" and [B,T,H,D]) and transposed views are
 * described without a copy.  The last dimension is contiguous; ptr and all strides must
 * keep 16-byte alignment for tensors with a last dimension (q,k,v,o,w,...). */
typedef struct lmoe_tensor {
  void* ptr;
  int64_t sb, st, sh;
} lmoe_tensor;

/* One problem instance.  Fields an entry point does not use may be zero / NULL. */
typedef struct lmoe_args {
  int32_t dtype;      /* LMOE_BF16 | LMOE_F32: q,k,v,o,do,dq,dk,dv and the saved intermediates */
  int32_t g_dtype;    /* element type of g    */
  int32_t beta_dtype; /* element type of beta */
  int32_t gate;       /* LMOE_GATE_*          */
  int32_t B, T, H, K, V;
  int32_t N;          /* number of sequences: B, or len(cu_seqlens)-1 when packed (then B == 1) */
  int32_t NT;         /* total number of 64-token chunks over all sequences: B * ceil(T / 64) for dense
                       * input (checked), at most ceil(T / 64) + N for packed input (checked)     */
  float scale;
  /* packed variable-length input (all NULL for dense input) -- device int32 arrays */
  const int32_t* cu_seqlens; /* [N+1] token offsets                                   */
  const int32_t* chunk_map;  /* [NT][2] (sequence index, chunk index inside sequence) */
  const int32_t* seq_chunk0; /* [N+1] index of the first chunk of each sequence       */
  /* inputs */
  lmoe_tensor q, k, v; /* [B,T,H,K], [B,T,H,K], [B,T,H,V]                              */
  lmoe_tensor g;       /* [B,T,H] or [B,T,H,K]; log-space decay; ptr NULL = no decay   */
  lmoe_tensor beta;    /* [B,T,H] (gated delta rule only)                              */
  const float* h0;     /* [N,H,K,V] fp32 initial state or NULL                         */
  /* outputs */
  lmoe_tensor o;       /* [B,T,H,V]                                                    */
  float* ht;           /* [N,H,K,V] fp32 final state or NULL                           */
  /* intermediates written by *_fwd and read by *_bwd (caller-allocated, element type = dtype) */
  void* hs;            /* state at the start of every chunk: [NT,H,V,K] (transposed) for
                          simple_gla and the gated delta rule, [NT,H,K,V] for chunk_gla    */
  lmoe_tensor vnew;    /* delta-rule pseudo values (gated delta rule): only .ptr is used, the layout is the
                          library's: [NT,H,V/32,64,32] (chunk, head, 32-column slice, token in chunk, column),
                          NT*H*64*V elements                                                          */
  lmoe_tensor w;       /* [B,T,H,K]   WY factor w (gated delta rule)                   */
  lmoe_tensor u;       /* [B,T,H,V]   WY factor u (gated delta rule; forward only)     */
  void* tinv;          /* [NT,H,64,64] (I + L)^-1 per chunk (gated delta rule)         */
  void* amat;          /* [NT,H,64,64] intra-chunk attention matrix (chunk_gla)        */
  void* pmat;          /* [NT,H,64,64] P = (q k^T) . Gamma per chunk (gated delta rule; written by the
                          WY preparation, or, for bf16 calls with tinv, by the forward state pass and
                          only when hs is given: a forward-only bf16 call leaves it untouched)      */
  float* gcum;         /* gated delta rule: [NT,H,5,64] fp32 gate table per chunk, written by the WY preparation:
                          e^{b_j}, e^{b_C - b_j}, beta_j, beta_j e^{b_j}, b_j (b = cumulative log-decay inside the
                          chunk; beta rows zero past the end of a partial chunk);
                          chunk_gla: [NT,H,K] fp32 e^{b_C} per channel, the decay of a whole chunk */
  void* qe;            /* [NT,H,64,K] q e^{b}       per chunk, rows past its end zero (chunk_gla) */
  void* ke;            /* [NT,H,64,K] k e^{b_C - b} per chunk, rows past its end zero (chunk_gla) */
  /* backward inputs */
  lmoe_tensor d_o;     /* [B,T,H,V] gradient of o                                      */
  const float* dht;    /* [N,H,K,V] fp32 gradient of the final state or NULL           */
  /* backward outputs */
  lmoe_tensor dq, dk, dv; /* same shapes as q,k,v, element type = dtype                */
  lmoe_tensor dg;      /* shape of g; fp32, except chunk_gla: element type of g (g_dtype) */
  lmoe_tensor dbeta;   /* fp32, shape of beta                                          */
  float* dh0;          /* [N,H,K,V] fp32 or NULL                                       */
  /* backward workspace (caller-allocated, element type = dtype) */
  void* dhs;           /* gradient w.r.t. the state at the END of every chunk, laid out as hs */
  lmoe_tensor dvnew;   /* gradient of vnew (gated delta rule): .ptr only, laid out as vnew */
  /* packed input, optional: device int32 [N], a permutation of 0..N-1 = the order in which the sequential state passes
   * take the sequences (their work-groups are dispatched in that order).  Longest first keeps a batch of unequal
   * lengths from ending on one long sequence that started late; NULL = as given.  Results do not depend on it.
   * No counterpart in fla, whose state kernels take the sequences in the order of cu_seqlens. */
  const int32_t* seq_order;
  /* packed input, optional: device int32 [1], the number of chunks of the call when NT above is only an upper bound of
   * it (tables built on the device from offsets that were never read on the host: chunk_map has NT rows, the first
   * *nt_dev of them valid; every per-chunk buffer is sized for NT).  NULL = NT is exact.  No counterpart in fla. */
  const int32_t* nt_dev;
  /* chunk_simple_gla with the output normalised inside the kernels (2-byte elements, gate = NONE):
   *   o_t = scale q_t S_t / (den_t + norm_eps),   den_t = scale q_t . sum_{s <= t} k_s   (the sum starts inside the call)
   * what fla.ops.linear_attn.chunk_linear_attn(normalize=True) forms behind its kernel with a cumulative sum over k in
   * memory (linear_moe/sequence_modeling/basic_linear_attention/basic_linear_attention.py:133).  normalize = 0: the
   * fields below are ignored.
   * fwd writes den (the divisor den_t + norm_eps, fp32, laid out like g) and, when hs is given, zs (fp32 [NT,H,K]:
   * the sum of the keys before each chunk).  bwd reads them and o (the normalised output the forward wrote) beside
   * d_o (the gradient of that output), and uses norm_ws, fp32 [NT,H,V/32,64+K], as workspace.  (These three
   * buffers are not part of what lmoe_workspace_bytes counts, which has no argument for the flag.)
   * normalize = 2: for a caller that adds the den of several key blocks before it divides (the op is a sum over key
   * blocks).  fwd writes o undivided and den (norm_eps is added as given: pass 0) beside it, and zs; bwd takes d_o,
   * the gradient of that o, and dden (fp32, laid out like den), the gradient of den, and uses zs and norm_ws; o and
   * den are not read. */
  int32_t normalize;
  float norm_eps;
  lmoe_tensor den;
  float* zs;
  float* norm_ws;
  /* gated delta rule, 2-byte elements with tinv: v_act = 1 makes the kernels take silu(v) where they read v (the
   * activation the reference applies in front of the op, gated_deltanet/gated_deltanet.py:101) and return in dv the
   * gradient with respect to v as given (dv = silu'(v) times the gradient of silu(v)).  0 = v as given.  No
   * counterpart in fla's signature: a caller that holds the fused projection saves the pass that would write silu(v)
   * and the one that would apply silu' (see lmoe_gdn_qkv_prologue_*). */
  int32_t v_act;
  lmoe_tensor dden;    /* normalize = 2, bwd: gradient of den (fp32, laid out like den) */
  /* gated delta rule, bwd, 2-byte elements: q_raw, k_raw given (both or neither; shaped and typed like q, k, any
   * strides the kernels take) say that q = l2norm(silu(q_raw)) and k = l2norm(silu(k_raw)) row by row, with qk_eps
   * inside the root (what gated_deltanet/gated_deltanet.py:101, :105-106 apply in front of the op and
   * lmoe_gdn_qkv_prologue_fwd forms): dq and dk then leave as the gradients with respect to q_raw and k_raw, so that
   * a caller who holds the fused projection needs no pass of its own for the backward of the two activations.  No
   * counterpart in fla's signature. */
  lmoe_tensor q_raw, k_raw;
  float qk_eps;
} lmoe_args;

/* Library version (major*10000 + minor*100 + patch). */
int lmoe_version(void);
/* Text of the last error on the calling thread ("" if none). */
const char* lmoe_last_error(void);

/* Bytes of caller-allocated intermediates of one call: part 0 = what *_fwd writes for *_bwd
 * (hs, and per op amat, qe, ke, gcum / vnew, w, u, tinv, pmat, gcum), part 1 = the backward workspace (dhs, and dvnew
 * for the gated delta rule).  Each buffer is still passed through its own lmoe_args field; this
 * is the sum a caller that carves them out of one arena must reserve (every buffer's size is a
 * multiple of 256 bytes for the supported K, V).  Negative for an invalid op / dtype / part.
 * Stands where fla sizes its saved tensors inside its autograd functions (no single call site
 * in the reference; the ops are reached from the files named below). */
int64_t lmoe_workspace_bytes(int32_t op, int32_t dtype, int32_t part, int32_t B, int32_t T, int32_t H, int32_t K,
                             int32_t V, int32_t NT);

/* chunk_simple_gla: S_t = e^{g_t} S_{t-1} + k_t^T v_t, o_t = scale q_t S_t, g scalar per
 * token-head (gate = SCALAR) or absent (gate = NONE).
 * Replaces fla.ops.simple_gla.chunk_simple_gla reached from the reference through
 *   linear_moe/sequence_modeling/retention/retention.py:91                (chunk_retention)
 *   linear_moe/sequence_modeling/basic_linear_attention/basic_linear_attention.py:133 (chunk_linear_attn)
 *   linear_moe/sequence_modeling/lightning_attention/lightning_attention.py:121-123 (lightning_attn2)
 * fwd uses q,k,v,g,h0 -> o,ht,hs (hs may be NULL: a forward-only call, which then saves nothing for a backward).
 * bwd uses q,k,v,g,hs,d_o,dht -> dq,dk,dv,dg,dh0 (+ dhs).
 * With normalize = 1 (see lmoe_args): fwd also -> den (, zs); bwd also uses o, den, zs (+ norm_ws). */
int lmoe_chunk_simple_gla_fwd(const lmoe_args* a, void* stream);
int lmoe_chunk_simple_gla_bwd(const lmoe_args* a, void* stream);

/* chunk_gla: S_t = diag(e^{g_t}) S_{t-1} + k_t^T v_t, g_t in R^K (gate = VECTOR).
 * Replaces fla.ops.gla.chunk_gla called at
 *   linear_moe/sequence_modeling/gla/gla.py:94 and linear_moe/sequence_modeling/hgrn2/hgrn2.py:76.
 * fwd uses q,k,v,g,h0 -> o,ht,hs,amat,qe,ke,gcum (the gated operands of the state passes, formed once by
 * the chunk-parallel kernel).  bwd uses those + d_o,dht -> dq,dk,dv,dg,dh0 (+ dhs).  hs, which only the backward
 * reads where the forward state pass forms the output itself (2-byte elements), may be NULL there (a forward-only
 * call: nothing saved); the 4-byte instances hand the states to their output kernel through it. */
int lmoe_chunk_gla_fwd(const lmoe_args* a, void* stream);
int lmoe_chunk_gla_bwd(const lmoe_args* a, void* stream);

/* chunk_gated_delta_rule: S~_t = e^{g_t} S_{t-1}; S_t = S~_t + k_t^T beta_t (v_t - k_t S~_t);
 * o_t = scale q_t S_t.
 * Replaces fla.ops.gated_delta_rule.chunk_gated_delta_rule called at
 *   linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:112.
 * fwd uses q,k,v,g,beta,h0 -> o,ht,hs,vnew,tinv,pmat,gcum (+ w,u).  hs and vnew, which only the backward reads,
 * may both be NULL (a forward-only call); tinv may then be NULL too, but should be given: with it the 2-byte
 * state pass forms w and u on the chip from tinv, k, v, beta instead of reading them, and w, u are neither
 * written nor needed (they may be NULL; less memory traffic; the results of a call with and without tinv differ
 * in the last bit of w, u).  4-byte elements, or no tinv: w and u are required.  pmat: required for 4-byte elements,
 * without tinv, or when hs is given; a forward-only 2-byte call with tinv forms P on the chip and may pass NULL.
 * bwd uses q,k,v,g,beta,hs,vnew,tinv,pmat,gcum,d_o,dht -> dq,dk,dv,dg,dbeta,dh0 (+ dhs, dvnew).
 * Head dimensions: K, V in {64, 128}, and K = 128 with V = 256 (the value head of expand_v = 2 at a head dimension
 * of 128, linear_moe/arguments.py:595-598): one pass over q and k and one WY preparation serve all 256 columns. */
int lmoe_chunk_gated_delta_rule_fwd(const lmoe_args* a, void* stream);
int lmoe_chunk_gated_delta_rule_bwd(const lmoe_args* a, void* stream);

/* Row-wise L2 normalisation over the last dimension, y = x / sqrt(sum x^2 + eps), and its
 * backward dx = dy rstd - (sum dy x) rstd^3 x, for `rows` contiguous rows of D elements
 * (D in {64, 128, 256}; dtype LMOE_BF16 | LMOE_F32; fp32 arithmetic; pointers 16-byte aligned).
 * Replaces l2_norm_fn of the reference, which normalises q and k in front of the delta-rule ops:
 *   linear_moe/model/common_modules/l2norm.py:22-45 (forward kernel), :64-95 (backward kernel),
 *   :172-201 (autograd wrapper), called at linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:105-106. */
int lmoe_l2norm_fwd(const void* x, void* y, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream);
int lmoe_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t D, int32_t dtype, float eps,
                    void* stream);

/* y = l2norm(silu(x)) row-wise, and its backward dx: the two steps the reference applies to q and k of
 * the gated delta rule in sequence, linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:101
 * (SiLU) and :105-106 (l2_norm_fn), as one pass over the rows.  Arguments as lmoe_l2norm_*. */
int lmoe_silu_l2norm_fwd(const void* x, void* y, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream);
int lmoe_silu_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t D, int32_t dtype, float eps,
                         void* stream);

/* The gated-delta-rule mixer's prologue on its fused projection, in one pass: qkv is [T][B][H][3 D] (q | k | v per
 * head, contiguous, as linear_moe/sequence_modeling/linear_attention.py:146 produces and :159-163 splits it);
 *   q = l2norm(silu(q_in)),  k = l2norm(silu(k_in)),  v = silu(v_in)      each [B][T][H][D] contiguous,
 * i.e. 'n b h d -> b n h d', SiLU and l2_norm_fn of gated_deltanet/gated_deltanet.py:99, :101, :105-106 (eps inside
 * the root, as lmoe_silu_l2norm_*).  bwd: dqkv [T][B][H][3 D] from dq, dk, dv [B][T][H][D] and qkv.
 * v == NULL (fwd) / dv == NULL (bwd): v is left to the op, which is then called with lmoe_args.v_act = 1 on the v
 * block of qkv itself (a strided view) and writes its gradient into the v block of dqkv; bwd then fills only the q
 * and k blocks of dqkv.
 * D in {64, 128}; pointers 16-byte aligned; fp32 arithmetic. */
int lmoe_gdn_qkv_prologue_fwd(const void* qkv, void* q, void* k, void* v, int32_t T, int32_t B, int32_t H, int32_t D,
                              int32_t dtype, float eps, void* stream);
int lmoe_gdn_qkv_prologue_bwd(const void* qkv, const void* dq, const void* dk, const void* dv, void* dqkv, int32_t T,
                              int32_t B, int32_t H, int32_t D, int32_t dtype, float eps, void* stream);

/* The same mixer's epilogue in one pass: y[t][b][:] = o[b][t][:] * swish(gate[t][b][:]) for rows of W = H D
 * elements, i.e. 'b n h d -> n b (h d)' of gated_deltanet.py:114 and `o * self.la_gate_fn(o_gate)` of
 * linear_moe/sequence_modeling/linear_attention.py:255 (la_gate_fn = swish).  bwd: d_o [B][T][W] and
 * dgate [T][B][W] from dy [T][B][W], o and gate.  W a multiple of 8; pointers 16-byte aligned. */
int lmoe_swish_gate_relayout_fwd(const void* o, const void* gate, void* y, int32_t T, int32_t B, int32_t W, int32_t dtype,
                                 void* stream);
int lmoe_swish_gate_relayout_bwd(const void* o, const void* gate, const void* dy, void* d_o, void* dgate, int32_t T,
                                 int32_t B, int32_t W, int32_t dtype, void* stream);

/* RMS norm over the last dimension of `rows` contiguous rows of D elements (D in {64, 128, 256}),
 *   y = x rstd w [* gate sigmoid(gate)],  rstd = 1 / sqrt(mean(x^2) + eps),
 * w ([D], element type of x) and gate ([rows][D]) may be null; rstd ([rows] fp32) is written when not null.
 * Replaces rms_norm_fn of the reference (linear_moe/model/common_modules/layernorm.py:515-537 ->
 * LayerNormFn :383-466 with is_rms_norm; kernels :69-132 forward, :212-300 backward; no bias, no residual),
 * the output norm of gla.py:95 and retention.py:92; the gate product is the reference's
 * `o * swish(o_gate)` (linear_moe/sequence_modeling/linear_attention.py:255) folded into the same pass.
 * Backward: dx, dgate (with gate), and dw ([D] fp32) through dw_part, a caller-allocated fp32
 * [lmoe_rmsnorm_partials(rows, D, dtype)][D] workspace that is summed in a fixed order
 * (the reference sums per-SM partial rows the same way, layernorm.py:349-377). dw_part and dw may both be null. */
int lmoe_rmsnorm_partials(int64_t rows, int32_t D, int32_t dtype);
int lmoe_rmsnorm_fwd(const void* x, const void* w, const void* gate, void* y, float* rstd, int64_t rows, int32_t D,
                     int32_t dtype, float eps, void* stream);
int lmoe_rmsnorm_bwd(const void* x, const void* w, const void* gate, const void* dy, void* dx, void* dgate,
                     float* dw_part, float* dw, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream);

/* lmoe_rmsnorm_bwd for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc): the same kernels, the same results bit for bit, with the partial rows of dw in a scratch
 * array the library holds itself (static device memory, 2 MiB per GPU until the process ends) instead of a
 * caller-allocated dw_part.  No counterpart in the reference.  Calls no hipMalloc / hipFree.  dw ([D] fp32) is
 * required (a caller that wants no dw needs no workspace either: lmoe_rmsnorm_bwd with dw_part = dw = NULL).
 * Returns -23 when rows x D needs more partial rows than the scratch holds (2048 rows of 256 floats: never on a GPU
 * of up to 256 compute units).  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU
 * (two streams, two threads) race; every call overwrites the rows it later reads, so nothing has to be cleared
 * between calls. */
int lmoe_rmsnorm_bwd_noalloc(const void* x, const void* w, const void* gate, const void* dy, void* dx, void* dgate,
                             float* dw, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream);

/* Gate construction of the gated delta rule for a, b of shape [rows][H] (element type by dtype):
 *   beta = sigmoid(b)  (element type of b),   g = -exp(A_log[h]) softplus(a + dt_bias[h])  (fp32)
 * as linear_moe/sequence_modeling/linear_attention.py:153-154 forms them in front of the op (parameters
 * :92-113).  Backward: da, db in the element type, dparams = [dA_log | ddt_bias] ([2][H] fp32) through
 * `part`, a caller-allocated fp32 [lmoe_gdn_gates_partials(rows, H)][2][H] workspace summed in a fixed order. */
int lmoe_gdn_gates_partials(int64_t rows, int32_t H);
int lmoe_gdn_gates_fwd(const void* a, const void* b, const float* A_log, const float* dt_bias, float* g, void* beta,
                       int64_t rows, int32_t H, int32_t dtype, void* stream);
int lmoe_gdn_gates_bwd(const void* a, const void* b, const float* A_log, const float* dt_bias, const float* dg,
                       const void* dbeta, void* da, void* db, float* part, float* dparams, int64_t rows, int32_t H,
                       int32_t dtype, void* stream);

/* Gate of chunk_gla over n contiguous elements (n a multiple of 8, 16-byte aligned):
 *   gk = max(logsigmoid(x) / normalizer, clamp_min)      (clamp_min = -INFINITY: no clamp)
 * as linear_moe/sequence_modeling/gla/gla.py:85 (normalizer) and :90-91 (clamp_min); backward
 *   dx = dy (1 - sigmoid(x)) / normalizer where gk > clamp_min, else 0. */
int lmoe_gla_gate_fwd(const void* x, void* y, int64_t n, int32_t dtype, float normalizer, float clamp_min, void* stream);
int lmoe_gla_gate_bwd(const void* x, const void* dy, void* dx, int64_t n, int32_t dtype, float normalizer,
                      float clamp_min, void* stream);

/* Gates of HGRN2 over n contiguous elements whose last dimension is D (n a multiple of D, D a multiple of 8):
 *   k = 1 - G (element type),  g = log G (fp32),  G = lb + (1 - lb) sigmoid(f),
 * lower_bound ([D] fp32) null: lb = 0, i.e. k = 1 - sigmoid(f), g = logsigmoid(f)
 * (linear_moe/sequence_modeling/linear_rnn.py:327-335; the op is then called as chunk_gla(q, k, i, g),
 * linear_moe/sequence_modeling/hgrn2/hgrn2.py:76).  Backward: df from dk (element type) and dg (fp32). */
int lmoe_hgrn2_gate_fwd(const void* f, const float* lower_bound, void* k, float* g, int64_t n, int32_t D, int32_t dtype,
                        void* stream);
int lmoe_hgrn2_gate_bwd(const void* f, const float* lower_bound, const void* dk, const float* dg, void* df, int64_t n,
                        int32_t D, int32_t dtype, void* stream);

/* Quadratic feature maps in front of chunk_linear_attn, rows of D in {8, 16, 32} numbers:
 *   phi(x) = [ c0 (if c0 != 0) | c1 x_i (if c1 != 0) | cd x_i^2 | co x_i x_j (i < j, row-major) ]
 * TaylorFeatureMap of Based (linear_moe/model/common_modules/feature_map.py:190-203; call
 * linear_moe/sequence_modeling/based/based.py:68): c0 = 1, c1 = D^-1/4, cd = (2D)^-1/2, co = D^-1/2;
 * RebasedFeatureMap flattened (feature_map.py:243-246; call .../rebased/rebased.py:72): c0 = c1 = 0,
 * cd = D^-1/2, co = (2/D)^1/2.  lmoe_quad_featmap_features gives the feature count F; the output is zero-padded to
 * Kp >= F (a multiple of 64) and laid out as key blocks of 128 columns (the last may have 64): block b is a
 * contiguous [rows][width_b] matrix at element offset rows * 128 * b.  Backward: dx from dy in that layout. */
int lmoe_quad_featmap_features(int32_t D, float c0, float c1);
int lmoe_quad_featmap_fwd(const void* x, void* y, int64_t rows, int32_t D, int32_t Kp, float c0, float c1, float cd,
                          float co, int32_t dtype, void* stream);
int lmoe_quad_featmap_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t D, int32_t Kp, float c0,
                          float c1, float cd, float co, int32_t dtype, void* stream);

/* Row routing for mixture-of-memories layers.  The reference pads the tokens routed to each (memory, batch
 * row) to a common capacity (`transform`, linear_moe/sequence_modeling/mom_linear_attention.py:15-77), calls
 * the op once per memory (:369-409) and scatters the results back (`reconstruct`, :79-120).  Here the routed
 * tokens are packed into one variable-length batch (one cu_seqlens call of the op for all memories):
 *   lmoe_mom_gather : out[i] = scale[i] * src[idx[i]]            rows of D elements; idx[i] < 0 -> zeros;
 *                                                                scale ([nout], element type) may be null
 *   lmoe_mom_combine: out[t] = sum_k w[t][k] * src[idx[t][k]]    idx < 0 skipped; w ([ntok][topk]) null -> 1
 *   lmoe_mom_rowdot : dw[t][k] = <g[t], src[idx[t][k]]>          the gradient of combine w.r.t. w
 * (pack = gather, its backward = combine with w = null; unpack = combine, its backward = gather with scale
 * and rowdot).  D a multiple of 8; idx int32 on the device; no atomics. */
int lmoe_mom_gather(const void* src, const int32_t* idx, const void* scale, void* out, int64_t nout, int32_t D,
                    int32_t dtype, void* stream);
int lmoe_mom_combine(const void* src, const int32_t* idx, const void* w, void* out, int64_t ntok, int32_t topk, int32_t D,
                     int32_t dtype, void* stream);
int lmoe_mom_rowdot(const void* src, const int32_t* idx, const void* g, void* dw, int64_t ntok, int32_t topk, int32_t D,
                    int32_t dtype, void* stream);

/* Launch ONE kernel of an op's pipeline (profiling support: lets a harness time each kernel
 * with events on its own stream).  `a` must be the fully populated argument block of the
 * op's fwd (stages 0-2, 7) or bwd (stages 3-5) entry point, with the intermediates of the
 * earlier stages already in place.  Stages: 0 gated-delta-rule WY preparation, 1 forward state
 * pass (scalar gates, and chunk_gla with 2-byte elements: the output o as well, so that the forward entry point
 * does not run stage 2, which stays available and gives the same o from the saved states), 2 output (chunk_gla),
 * 3 dv, 4 reverse state pass, 5 dq dk and gate gradient (gated delta rule: every
 * gradient that follows the reverse state pass; chunk_simple_gla and chunk_gla with 2-byte elements: dv as well, so
 * that their backward entry points do not run stage 3, which stays available and gives the same dv), 7 chunk_gla
 * intra-chunk matrix.
 * No counterpart in the reference (measurement support). */
#define LMOE_OP_SIMPLE_GLA 0
#define LMOE_OP_GLA 1
#define LMOE_OP_GATED_DELTA_RULE 2
int lmoe_launch_stage(const lmoe_args* a, int32_t op, int32_t stage, void* stream);

/* Per-phase timing of the forward sequential pass of the gated delta rule (profiling support; no counterpart in the
 * reference).  Runs the pass once for the problem `a` (the fully populated argument block of
 * lmoe_chunk_gated_delta_rule_fwd, after its WY preparation has run: lmoe_launch_stage stage 0) with the instance
 * that records the shader clock in work-group `work_group`, and leaves in `trace` (device memory,
 * int64 [4 slots][128 chunks][8 marks], zero where nothing was recorded; sequences longer than 128 chunks are traced
 * for their first 128) the cycle counter at these points of every chunk:
 *   slot 0, the consumer wave (carries the state):  0 arrives at barrier 1, 1 leaves it, 5 k S formed, 2 arrives at
 *           barrier 2 (v_new written), 3 leaves it, 6 state updated, 4 state written for the next chunk
 *   slot 1, the helper wave (forms the output):     0, 1, 2 (q S formed), 3 as above, 4 o written
 *   slot 2, loader team 1 (k, P; all stores):       0, 1, 2 (tiles staged, results lifted), 3, 4 stores issued,
 *           5 loads issued
 *   slot 3, loader team 2 (q, Tinv, v, gates):      0, 1, 2 loads issued, 3, 4 tiles staged
 * Instance available for LMOE_BF16, K = V = 128, with tinv and hs given (-24 otherwise). */
int lmoe_trace_gdn_state_fwd(const lmoe_args* a, int64_t* trace, int32_t work_group, void* stream);

/* The same for the forward pass of chunk_simple_gla on 2-byte elements (k_state_fwd_b, one barrier per chunk):
 * trace = 3 x 24 x 8 int64 device words, trace[slot][chunk][mark] (chunks beyond 24 are not recorded), stamps of one
 * wave per team of work-group `work_group`.  Marks: 0 arrives at the barrier of the chunk, 1 leaves it, and
 *   slot 0, consumers: 5 state updated, 6 state copied to LDS, 2 their blocks of P of the next chunk formed, 3 the
 *     operands of the next state update read
 *   slot 1, loaders: 5 loads of chunk c + 4 issued, 2 chunk c + 2 staged, 4 per-chunk state stored (saving calls)
 *   slot 2, output team: 5 products of q S issued, 2 (P v)^T done, 4 rows stored, 6 its block of P of the next chunk
 *     formed and the next chunk's q rows and v^T fragments read
 * Instance available for LMOE_BF16, K = V = 128, forward-only calls (hs NULL; -24 otherwise).  No counterpart in
 * the reference (profiling support). */
int lmoe_trace_simple_gla_fwd(const lmoe_args* a, int64_t* trace, int32_t work_group, void* stream);

/* Token-by-token forward of an op (op = LMOE_OP_*; the delta rule without a gate: gate = LMOE_GATE_NONE):
 * the state stays in registers, nothing is saved for a backward.  For decoding (T = 1 with h0 / ht) and
 * short sequences.  Uses q, k, v, g, beta, h0, scale, cu_seqlens (+ seq_chunk0, chunk_map as for the chunk
 * entry points) -> o, ht.  Stands where the reference selects fla's fused_recurrent_* callables
 * (la_mode = 'fused_recurrent': linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:72-73,
 * gla/gla.py:58-59, deltanet/deltanet.py:81-82, basic_linear_attention/basic_linear_attention.py:99-100). */
int lmoe_fused_recurrent_fwd(const lmoe_args* a, int32_t op, void* stream);

/* Toolkit self-test over one pair of 64 x kd tiles A, B (element type by dtype, kd in {64,128}),
 * through the same tile loaders, MFMA fragments and accumulator stores the kernels use:
 * C[64][64] (fp32) = A B^T (contraction along tile columns), G[kd][kd] (fp32) = A^T B
 * (contraction along tile rows: the transposed-fragment path).
 * No counterpart in the reference (test support). */
int lmoe_selftest_gemm(int32_t dtype, int32_t kd, const void* A, const void* B, float* C, float* G, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LMOE_H_ */
