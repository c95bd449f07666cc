// C ABI of liblmoe_hip.so (declared in include/lmoe.h): argument validation and kernel dispatch.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/lmoe.h"
#include "lmoe_launch.hpp"

namespace {
thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// wide_v: the op has instances for K = 128, V = 256 (the gated delta rule)
int check_common(const lmoe_args* a, const char* op, bool wide_v = false) {
  if (!a) return fail(-1, "%s: null argument block", op);
  if (a->dtype != LMOE_BF16 && a->dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", op);
  if (!((a->K == 64 || a->K == 128) && (a->V == 64 || a->V == 128)) && !(wide_v && a->K == 128 && a->V == 256))
    return fail(-3, "%s: head dims K=%d V=%d unsupported (K, V must be 64 or 128%s)", op, a->K, a->V,
                wide_v ? "; or K = 128 with V = 256" : "");
  if (a->B < 0 || a->T < 0 || a->H <= 0 || a->N < 0 || a->NT < 0) return fail(-4, "%s: negative dimension", op);
  if (a->cu_seqlens && (a->B != 1 || !a->chunk_map || !a->seq_chunk0))
    return fail(-5, "%s: packed input needs B == 1, chunk_map and seq_chunk0", op);
  if (!a->cu_seqlens && a->N != a->B) return fail(-6, "%s: dense input needs N == B", op);
  if (!a->q.ptr || !a->k.ptr || !a->v.ptr) return fail(-7, "%s: q, k, v must not be null", op);
  if (a->H > 65535 || a->N > 65535) return fail(-8, "%s: H and N must be <= 65535", op);
  // The kernels derive every address from these numbers: a chunk count that does not belong to B and T would send
  // them past the end of the inputs, rows that are not 16-byte aligned break their 16-byte accesses.
  const int64_t per_row = ((int64_t)a->T + LMOE_CHUNK - 1) / LMOE_CHUNK;
  if (!a->cu_seqlens && (int64_t)a->NT != (int64_t)a->B * per_row)
    return fail(-4, "%s: dense input of B=%d, T=%d has %lld chunks, NT=%d given", op, a->B, a->T,
                (long long)(a->B * per_row), a->NT);
  if (a->cu_seqlens && (int64_t)a->NT > per_row + a->N)
    return fail(-4, "%s: packed input of T=%d, N=%d has at most %lld chunks, NT=%d given", op, a->T, a->N,
                (long long)(per_row + a->N), a->NT);
  const int64_t vec = a->dtype == LMOE_BF16 ? 8 : 4;            // elements per 16 bytes
  const lmoe_tensor* rows[] = {&a->q, &a->k, &a->v, &a->o, &a->d_o, &a->dq, &a->dk, &a->dv, &a->q_raw, &a->k_raw};
  for (const lmoe_tensor* t : rows)
    if (t->ptr && (((uintptr_t)t->ptr & 15) || t->sb % vec || t->st % vec || t->sh % vec))
      return fail(-9, "%s: q, k, v, o and their gradients need 16-byte aligned rows (pointer and strides)", op);
  return 0;
}

// chunk_simple_gla with the output normalised inside the kernels (lmoe_args.normalize)
int check_normalize(const lmoe_args* a, const char* op, bool bwd) {
  if (!a->normalize) return 0;
  if (a->normalize != 1 && a->normalize != 2) return fail(-15, "%s: normalize must be 0, 1 or 2", op);
  if (a->dtype != LMOE_BF16) return fail(-15, "%s: normalize needs 2-byte elements", op);
  if (a->gate != LMOE_GATE_NONE) return fail(-15, "%s: normalize needs gate = LMOE_GATE_NONE", op);
  if (!bwd && !a->den.ptr) return fail(-11, "%s: normalize needs den", op);
  if (!bwd && a->hs && !a->zs) return fail(-11, "%s: normalize with hs given needs zs", op);
  if (bwd && a->normalize == 1 && (!a->den.ptr || !a->zs || !a->norm_ws || !a->o.ptr))
    return fail(-11, "%s: normalize = 1 needs o, den, zs and norm_ws", op);
  if (bwd && a->normalize == 2 && (!a->dden.ptr || !a->zs || !a->norm_ws))
    return fail(-11, "%s: normalize = 2 needs dden, zs and norm_ws", op);
  return 0;
}

int launched(const char* op) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "%s: launch failed: %s", op, hipGetErrorString(e));
  return 0;
}
}  // namespace

extern "C" {

int lmoe_version(void) { return 102; }
const char* lmoe_last_error(void) { return g_err; }

int64_t lmoe_workspace_bytes(int32_t op, int32_t dtype, int32_t part, int32_t B, int32_t T, int32_t H, int32_t K,
                             int32_t V, int32_t NT) {
  const char* nm = "lmoe_workspace_bytes";
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (op != LMOE_OP_SIMPLE_GLA && op != LMOE_OP_GLA && op != LMOE_OP_GATED_DELTA_RULE)
    return fail(-21, "%s: unknown op %d", nm, op);
  if (part != 0 && part != 1) return fail(-22, "%s: part must be 0 (saved by fwd) or 1 (bwd workspace)", nm);
  if (B < 0 || T < 0 || H <= 0 || K <= 0 || V <= 0 || NT < 0) return fail(-4, "%s: negative dimension", nm);
  const int64_t s = dtype == LMOE_BF16 ? 2 : 4;
  const int64_t states = (int64_t)NT * H * K * V, tiles = (int64_t)NT * H * LMOE_CHUNK * LMOE_CHUNK;
  const int64_t rows_k = (int64_t)B * T * H * K, rows_v = (int64_t)B * T * H * V;
  int64_t n = states;                                                    // hs | dhs
  if (op == LMOE_OP_GLA && part == 0) n += tiles + 2 * (int64_t)NT * H * LMOE_CHUNK * K;   // amat, qe, ke
  // vnew, tinv, pmat, and for 4-byte elements u, w (the 2-byte state passes form them on the chip) | dvnew
  const int64_t blocks_v = (int64_t)NT * H * LMOE_CHUNK * V;             // vnew | dvnew: whole chunks, [NT,H,V/32,64,32]
  if (op == LMOE_OP_GATED_DELTA_RULE) n += part == 0 ? blocks_v + 2 * tiles + (s == 4 ? rows_v + rows_k : 0) : blocks_v;
  int64_t bytes = n * s;
  if (op == LMOE_OP_GATED_DELTA_RULE && part == 0) bytes += (int64_t)NT * H * 5 * LMOE_CHUNK * 4;   // gcum (fp32)
  if (op == LMOE_OP_GLA && part == 0) bytes += (int64_t)NT * H * K * 4;                              // gcum (fp32)
  return bytes;
}

int lmoe_chunk_simple_gla_fwd(const lmoe_args* a, void* stream) {
  const char* op = "lmoe_chunk_simple_gla_fwd";
  if (int r = check_common(a, op)) return r;
  if (a->gate == LMOE_GATE_VECTOR) return fail(-10, "%s: vector gates belong to lmoe_chunk_gla_fwd", op);
  if (!a->o.ptr) return fail(-11, "%s: o must not be null", op);      // hs == NULL: forward only, nothing saved
  if (int r = check_normalize(a, op, false)) return r;
  if (a->NT == 0 || a->N == 0) return 0;
  lmoe::launch_state_fwd(*a, (hipStream_t)stream);
  return launched(op);
}

int lmoe_chunk_simple_gla_bwd(const lmoe_args* a, void* stream) {
  const char* op = "lmoe_chunk_simple_gla_bwd";
  if (int r = check_common(a, op)) return r;
  if (a->gate == LMOE_GATE_VECTOR) return fail(-10, "%s: vector gates belong to lmoe_chunk_gla_bwd", op);
  if (!a->hs || !a->dhs || !a->d_o.ptr || !a->dq.ptr || !a->dk.ptr || !a->dv.ptr)
    return fail(-11, "%s: hs, dhs, d_o, dq, dk and dv must not be null", op);
  if (a->gate == LMOE_GATE_SCALAR && !a->dg.ptr) return fail(-13, "%s: dg must not be null for a gated call", op);
  if (int r = check_normalize(a, op, true)) return r;
  if (a->NT == 0 || a->N == 0) return 0;
  lmoe::launch_state_bwd(*a, (hipStream_t)stream);
  // 2-byte elements: dv is formed by the kernel that forms dq and dk, from the tiles it holds anyway
  if (a->dtype == LMOE_F32) lmoe::launch_bwd_dv(*a, false, (hipStream_t)stream);
  lmoe::launch_bwd_dqk(*a, (hipStream_t)stream);
  return launched(op);
}
static int check_gla(const lmoe_args* a, const char* op, bool need_hs = true) {
  if (int r = check_common(a, op)) return r;
  if (a->gate != LMOE_GATE_VECTOR || !a->g.ptr) return fail(-10, "%s: needs a vector gate g [B,T,H,K]", op);
  if (a->dtype == LMOE_F32 && a->g_dtype != LMOE_F32) return fail(-14, "%s: fp32 q/k/v need an fp32 gate", op);
  if ((need_hs && !a->hs) || !a->amat || !a->qe || !a->ke || !a->gcum)
    return fail(-11, "%s: hs, amat, qe, ke and gcum must not be null", op);
  return 0;
}

int lmoe_chunk_gla_fwd(const lmoe_args* a, void* stream) {
  const char* op = "lmoe_chunk_gla_fwd";
  // hs == NULL: a forward-only call, nothing saved -- where the state pass forms the output itself (2-byte
  // elements); the 4-byte instances hand the states to their output kernel through hs
  if (int r = check_gla(a, op, false)) return r;
  if (!a->hs && !lmoe::gla_fwd_fused(*a)) return fail(-11, "%s: hs must not be null for 4-byte elements", op);
  if (!a->o.ptr) return fail(-11, "%s: o must not be null", op);
  if (a->NT == 0 || a->N == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  lmoe::launch_gla(*a, lmoe::ST_GLA_INTRA_FWD, st);
  lmoe::launch_gla(*a, lmoe::ST_STATE_FWD, st);
  if (!lmoe::gla_fwd_fused(*a)) lmoe::launch_gla(*a, lmoe::ST_OUT_FWD, st);      // else the state pass formed o
  return launched(op);
}

int lmoe_chunk_gla_bwd(const lmoe_args* a, void* stream) {
  const char* op = "lmoe_chunk_gla_bwd";
  if (int r = check_gla(a, op)) return r;
  if (!a->dhs || !a->d_o.ptr || !a->dq.ptr || !a->dk.ptr || !a->dv.ptr || !a->dg.ptr)
    return fail(-11, "%s: dhs, d_o, dq, dk, dv and dg must not be null", op);
  if (a->NT == 0 || a->N == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  lmoe::launch_gla(*a, lmoe::ST_STATE_BWD, st);
  // 2-byte elements: dv is formed by the kernel that forms dq, dk and dg, from the slices it stages anyway
  if (a->dtype == LMOE_F32) lmoe::launch_gla(*a, lmoe::ST_DV, st);
  lmoe::launch_gla(*a, lmoe::ST_DQK, st);
  return launched(op);
}
int lmoe_chunk_gated_delta_rule_fwd(const lmoe_args* a, void* stream) {
  const char* op = "lmoe_chunk_gated_delta_rule_fwd";
  if (int r = check_common(a, op, true)) return r;
  if (a->gate == LMOE_GATE_VECTOR) return fail(-10, "%s: the gate is one scalar per token and head", op);
  if (!a->beta.ptr) return fail(-12, "%s: beta must not be null", op);
  if (!a->o.ptr || !a->gcum) return fail(-11, "%s: o and gcum must not be null", op);
  if (a->V == 256 && a->dtype == LMOE_BF16 && !a->tinv) return fail(-11, "%s: V = 256 with 2-byte elements needs tinv", op);
  if (a->v_act && (a->dtype != LMOE_BF16 || !a->tinv)) return fail(-15, "%s: v_act needs 2-byte elements and tinv", op);
  // P reaches memory where the WY preparation forms it (4-byte elements, or no tinv) or where the backward will
  // read it (hs given); a forward-only 2-byte call with tinv forms it inside the state pass and never stores it
  if ((a->dtype != LMOE_BF16 || !a->tinv || a->hs) && !a->pmat)
    return fail(-11, "%s: pmat must not be null (4-byte elements, no tinv given, or hs given)", op);
  // w, u are written and read only where the state pass does not form them itself from tinv
  if ((a->dtype != LMOE_BF16 || !a->tinv) && (!a->w.ptr || !a->u.ptr))
    return fail(-11, "%s: w and u must not be null (4-byte elements, or no tinv given)", op);
  // what only the backward reads: hs and vnew together or not at all (a forward-only call); tinv goes with
  // them, and may also be given alone (the state pass then forms w from it instead of reading w)
  if ((a->hs != nullptr) != (a->vnew.ptr != nullptr) || (a->hs != nullptr && a->tinv == nullptr))
    return fail(-11, "%s: hs and vnew must be given together, and tinv with them (all null: forward only)", op);
  if (a->NT == 0 || a->N == 0) return 0;
  lmoe::launch_gdn_wy_fwd(*a, (hipStream_t)stream);
  lmoe::launch_gdn_state_fwd(*a, (hipStream_t)stream);
  return launched(op);
}
int lmoe_chunk_gated_delta_rule_bwd(const lmoe_args* a, void* stream) {
  const char* op = "lmoe_chunk_gated_delta_rule_bwd";
  if (int r = check_common(a, op, true)) return r;
  if (a->gate == LMOE_GATE_VECTOR) return fail(-10, "%s: the gate is one scalar per token and head", op);
  if (!a->beta.ptr) return fail(-12, "%s: beta must not be null", op);
  if (!a->hs || !a->dhs || !a->vnew.ptr || !a->tinv || !a->pmat || !a->gcum || !a->dvnew.ptr)
    return fail(-11, "%s: hs, dhs, vnew, tinv, pmat, gcum and dvnew must not be null", op);
  if (!a->d_o.ptr || !a->dq.ptr || !a->dk.ptr || !a->dv.ptr || !a->dg.ptr || !a->dbeta.ptr)
    return fail(-13, "%s: d_o, dq, dk, dv, dg and dbeta must not be null", op);
  if (a->v_act && a->dtype != LMOE_BF16) return fail(-15, "%s: v_act needs 2-byte elements", op);
  if ((a->q_raw.ptr != nullptr) != (a->k_raw.ptr != nullptr)) return fail(-11, "%s: q_raw and k_raw go together", op);
  if (a->q_raw.ptr && (a->dtype != LMOE_BF16 || a->V > 128))
    return fail(-15, "%s: q_raw, k_raw need 2-byte elements and V <= 128", op);
  if (a->NT == 0 || a->N == 0) return 0;
  lmoe::launch_gdn_state_bwd(*a, (hipStream_t)stream);
  lmoe::launch_gdn_bwd_chunk(*a, (hipStream_t)stream);
  return launched(op);
}

static int check_l2norm(const char* nm, const void* x, const void* out, int64_t rows, int32_t D, int32_t dtype) {
  if (!x || !out) return fail(-1, "%s: null pointer", nm);
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (D != 64 && D != 128 && D != 256) return fail(-3, "%s: row length %d unsupported (64, 128 or 256)", nm, D);
  if (rows < 0) return fail(-4, "%s: negative row count", nm);
  if (((uintptr_t)x | (uintptr_t)out) & 15) return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  return 0;
}
int lmoe_l2norm_fwd(const void* x, void* y, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream) {
  const char* nm = "lmoe_l2norm_fwd";
  if (int r = check_l2norm(nm, x, y, rows, D, dtype)) return r;
  if (rows == 0) return 0;
  lmoe::launch_l2norm(dtype, D, x, nullptr, y, rows, eps, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t D, int32_t dtype, float eps,
                    void* stream) {
  const char* nm = "lmoe_l2norm_bwd";
  if (int r = check_l2norm(nm, x, dx, rows, D, dtype)) return r;
  if (!dy || ((uintptr_t)dy & 15)) return fail(-1, "%s: dy must be a 16-byte aligned pointer", nm);
  if (rows == 0) return 0;
  lmoe::launch_l2norm(dtype, D, x, dy, dx, rows, eps, true, (hipStream_t)stream);
  return launched(nm);
}

int lmoe_silu_l2norm_fwd(const void* x, void* y, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream) {
  const char* nm = "lmoe_silu_l2norm_fwd";
  if (int r = check_l2norm(nm, x, y, rows, D, dtype)) return r;
  if (rows == 0) return 0;
  lmoe::launch_silu_l2norm(dtype, D, x, nullptr, y, rows, eps, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_silu_l2norm_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t D, int32_t dtype, float eps,
                         void* stream) {
  const char* nm = "lmoe_silu_l2norm_bwd";
  if (int r = check_l2norm(nm, x, dx, rows, D, dtype)) return r;
  if (!dy || ((uintptr_t)dy & 15)) return fail(-1, "%s: dy must be a 16-byte aligned pointer", nm);
  if (rows == 0) return 0;
  lmoe::launch_silu_l2norm(dtype, D, x, dy, dx, rows, eps, true, (hipStream_t)stream);
  return launched(nm);
}

static int check_layerio(const char* nm, int32_t T, int32_t B, int32_t dtype) {
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (T < 0 || B < 0) return fail(-4, "%s: negative dimension", nm);
  return 0;
}
int lmoe_gdn_qkv_prologue_fwd(const void* qkv, void* q, void* k, void* v, int32_t T, int32_t B, int32_t H, int32_t D,
                              int32_t dtype, float eps, void* stream) {
  const char* nm = "lmoe_gdn_qkv_prologue_fwd";
  if (int r = check_layerio(nm, T, B, dtype)) return r;
  if (!qkv || !q || !k) return fail(-1, "%s: null pointer", nm);           // v == NULL: v is left to the op
  if (D != 64 && D != 128) return fail(-3, "%s: head dimension %d unsupported (64 or 128)", nm, D);
  if (H <= 0) return fail(-4, "%s: H must be positive", nm);
  if (((uintptr_t)qkv | (uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  if ((int64_t)T * B == 0) return 0;
  lmoe::launch_gdn_qkv_prologue(dtype, D, qkv, nullptr, nullptr, nullptr, q, k, v, T, B, H, eps, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_gdn_qkv_prologue_bwd(const void* qkv, const void* dq, const void* dk, const void* dv, void* dqkv, int32_t T,
                              int32_t B, int32_t H, int32_t D, int32_t dtype, float eps, void* stream) {
  const char* nm = "lmoe_gdn_qkv_prologue_bwd";
  if (int r = check_layerio(nm, T, B, dtype)) return r;
  if (!qkv || !dq || !dk || !dqkv) return fail(-1, "%s: null pointer", nm);  // dv == NULL: the op wrote that block
  if (D != 64 && D != 128) return fail(-3, "%s: head dimension %d unsupported (64 or 128)", nm, D);
  if (H <= 0) return fail(-4, "%s: H must be positive", nm);
  if (((uintptr_t)qkv | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv | (uintptr_t)dqkv) & 15)
    return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  if ((int64_t)T * B == 0) return 0;
  lmoe::launch_gdn_qkv_prologue(dtype, D, qkv, dq, dk, dv, dqkv, nullptr, nullptr, T, B, H, eps, true, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_swish_gate_relayout_fwd(const void* o, const void* gate, void* y, int32_t T, int32_t B, int32_t W, int32_t dtype,
                                 void* stream) {
  const char* nm = "lmoe_swish_gate_relayout_fwd";
  if (int r = check_layerio(nm, T, B, dtype)) return r;
  if (!o || !gate || !y) return fail(-1, "%s: null pointer", nm);
  if (W <= 0 || W % 8) return fail(-3, "%s: row length %d must be a positive multiple of 8", nm, W);
  if (((uintptr_t)o | (uintptr_t)gate | (uintptr_t)y) & 15) return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  if ((int64_t)T * B == 0) return 0;
  lmoe::launch_swish_gate_relayout(dtype, o, gate, nullptr, y, nullptr, T, B, W, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_swish_gate_relayout_bwd(const void* o, const void* gate, const void* dy, void* d_o, void* dgate, int32_t T,
                                 int32_t B, int32_t W, int32_t dtype, void* stream) {
  const char* nm = "lmoe_swish_gate_relayout_bwd";
  if (int r = check_layerio(nm, T, B, dtype)) return r;
  if (!o || !gate || !dy || !d_o || !dgate) return fail(-1, "%s: null pointer", nm);
  if (W <= 0 || W % 8) return fail(-3, "%s: row length %d must be a positive multiple of 8", nm, W);
  if (((uintptr_t)o | (uintptr_t)gate | (uintptr_t)dy | (uintptr_t)d_o | (uintptr_t)dgate) & 15)
    return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  if ((int64_t)T * B == 0) return 0;
  lmoe::launch_swish_gate_relayout(dtype, o, gate, dy, d_o, dgate, T, B, W, true, (hipStream_t)stream);
  return launched(nm);
}

int lmoe_rmsnorm_partials(int64_t rows, int32_t D, int32_t dtype) {
  const char* nm = "lmoe_rmsnorm_partials";
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (D != 64 && D != 128 && D != 256) return fail(-3, "%s: row length %d unsupported (64, 128 or 256)", nm, D);
  if (rows < 0) return fail(-4, "%s: negative row count", nm);
  return lmoe::rmsnorm_partials(dtype, D, rows);
}
int lmoe_rmsnorm_fwd(const void* x, const void* w, const void* gate, void* y, float* rstd, int64_t rows, int32_t D,
                     int32_t dtype, float eps, void* stream) {
  const char* nm = "lmoe_rmsnorm_fwd";
  if (int r = check_l2norm(nm, x, y, rows, D, dtype)) return r;
  if (((uintptr_t)w | (uintptr_t)gate) & 15) return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  if (rows == 0) return 0;
  lmoe::launch_rmsnorm(dtype, D, x, w, gate, nullptr, y, nullptr, rstd, nullptr, nullptr, rows, eps, false,
                       (hipStream_t)stream);
  return launched(nm);
}
int lmoe_rmsnorm_bwd(const void* x, const void* w, const void* gate, const void* dy, void* dx, void* dgate,
                     float* dw_part, float* dw, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream) {
  const char* nm = "lmoe_rmsnorm_bwd";
  if (int r = check_l2norm(nm, x, dx, rows, D, dtype)) return r;
  if (!dy) return fail(-1, "%s: dy must not be null", nm);
  if (((uintptr_t)w | (uintptr_t)gate | (uintptr_t)dy | (uintptr_t)dgate) & 15)
    return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  if ((gate != nullptr) != (dgate != nullptr)) return fail(-1, "%s: gate and dgate go together", nm);
  if ((dw_part != nullptr) != (dw != nullptr)) return fail(-1, "%s: dw_part and dw go together", nm);
  if (rows == 0) return 0;              // nothing to do (dw is not written)
  lmoe::launch_rmsnorm(dtype, D, x, w, gate, dy, dx, dgate, nullptr, dw_part, dw, rows, eps, true, (hipStream_t)stream);
  return launched(nm);
}

int lmoe_rmsnorm_bwd_noalloc(const void* x, const void* w, const void* gate, const void* dy, void* dx, void* dgate,
                             float* dw, int64_t rows, int32_t D, int32_t dtype, float eps, void* stream) {
  const char* nm = "lmoe_rmsnorm_bwd_noalloc";
  if (int r = check_l2norm(nm, x, dx, rows, D, dtype)) return r;
  if (!dy || !dw) return fail(-1, "%s: dy and dw must not be null", nm);
  if (((uintptr_t)w | (uintptr_t)gate | (uintptr_t)dy | (uintptr_t)dgate) & 15)
    return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  if ((gate != nullptr) != (dgate != nullptr)) return fail(-1, "%s: gate and dgate go together", nm);
  if (rows == 0) return 0;              // nothing to do (dw is not written)
  float* part = nullptr;
  int64_t cap = 0;
  if (int e = lmoe::rmsnorm_scratch(&part, &cap)) return fail(e, "%s: no address for the library's scratch array: %s", nm, hipGetErrorString((hipError_t)e));
  const int64_t need = (int64_t)lmoe::rmsnorm_partials(dtype, D, rows) * D;
  if (need > cap)
    return fail(-23, "%s: %lld partial rows of %d floats exceed the library's scratch (%lld floats); use lmoe_rmsnorm_bwd "
                     "with a caller-allocated dw_part", nm, (long long)(need / D), D, (long long)cap);
  lmoe::launch_rmsnorm(dtype, D, x, w, gate, dy, dx, dgate, nullptr, part, dw, rows, eps, true, (hipStream_t)stream);
  return launched(nm);
}

int lmoe_trace_simple_gla_fwd(const lmoe_args* a, int64_t* trace, int32_t work_group, void* stream) {
  const char* nm = "lmoe_trace_simple_gla_fwd";
  if (int r = check_common(a, nm)) return r;
  if (!trace) return fail(-1, "%s: trace must not be null", nm);
  if (a->gate == LMOE_GATE_VECTOR || !a->o.ptr)
    return fail(-11, "%s: needs the populated argument block of lmoe_chunk_simple_gla_fwd", nm);
  if (a->NT == 0 || a->N == 0) return fail(-4, "%s: nothing to trace in an empty problem", nm);
  if (!lmoe::launch_state_fwd_trace(*a, (long long*)trace, work_group, (hipStream_t)stream))
    return fail(-24, "%s: traced instance exists for bf16, K = V = 128, forward-only (hs NULL), work_group inside the grid", nm);
  return launched(nm);
}

int lmoe_trace_gdn_state_fwd(const lmoe_args* a, int64_t* trace, int32_t work_group, void* stream) {
  const char* nm = "lmoe_trace_gdn_state_fwd";
  if (int r = check_common(a, nm)) return r;
  if (!trace) return fail(-1, "%s: trace must not be null", nm);
  if (a->gate == LMOE_GATE_VECTOR || !a->beta.ptr || !a->o.ptr || !a->pmat || !a->gcum || !a->vnew.ptr)
    return fail(-11, "%s: needs the populated argument block of lmoe_chunk_gated_delta_rule_fwd", nm);
  if (a->NT == 0 || a->N == 0) return fail(-4, "%s: nothing to trace in an empty problem", nm);
  if (!lmoe::launch_gdn_state_fwd_trace(*a, (long long*)trace, work_group, (hipStream_t)stream))
    return fail(-24, "%s: traced instance exists for bf16, K = V = 128 with tinv and hs given, work_group inside the grid", nm);
  return launched(nm);
}

int lmoe_fused_recurrent_fwd(const lmoe_args* a, int32_t op, void* stream) {
  const char* nm = "lmoe_fused_recurrent_fwd";
  if (int r = check_common(a, nm)) return r;
  if (op != LMOE_OP_SIMPLE_GLA && op != LMOE_OP_GLA && op != LMOE_OP_GATED_DELTA_RULE)
    return fail(-21, "%s: unknown op %d", nm, op);
  if (!a->o.ptr) return fail(-11, "%s: o must not be null", nm);
  if (op == LMOE_OP_GLA && (a->gate != LMOE_GATE_VECTOR || !a->g.ptr)) return fail(-10, "%s: chunk_gla needs a vector gate", nm);
  if (op != LMOE_OP_GLA && a->gate == LMOE_GATE_VECTOR) return fail(-10, "%s: vector gates belong to LMOE_OP_GLA", nm);
  if (op == LMOE_OP_GATED_DELTA_RULE && !a->beta.ptr) return fail(-12, "%s: beta must not be null", nm);
  if (a->N == 0 || a->T == 0) return 0;
  lmoe::launch_recurrent(*a, op == LMOE_OP_GATED_DELTA_RULE, (hipStream_t)stream);
  return launched(nm);
}

static int check_mom(const char* nm, const void* src, const void* idx, const void* out, int64_t n, int32_t D, int32_t dtype) {
  if (!src || !idx || !out) return fail(-1, "%s: null pointer", nm);
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (D <= 0 || D % 8) return fail(-3, "%s: row length %d must be a positive multiple of 8", nm, D);
  if (n < 0) return fail(-4, "%s: negative row count", nm);
  if (((uintptr_t)src | (uintptr_t)out) & 15) return fail(-9, "%s: row pointers must be 16-byte aligned", nm);
  return 0;
}
int lmoe_mom_gather(const void* src, const int32_t* idx, const void* scale, void* out, int64_t nout, int32_t D,
                    int32_t dtype, void* stream) {
  const char* nm = "lmoe_mom_gather";
  if (int r = check_mom(nm, src, idx, out, nout, D, dtype)) return r;
  if (nout == 0) return 0;
  lmoe::launch_mom_gather(dtype, src, idx, scale, out, nout, D, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_mom_combine(const void* src, const int32_t* idx, const void* w, void* out, int64_t ntok, int32_t topk, int32_t D,
                     int32_t dtype, void* stream) {
  const char* nm = "lmoe_mom_combine";
  if (int r = check_mom(nm, src, idx, out, ntok, D, dtype)) return r;
  if (topk <= 0) return fail(-4, "%s: topk must be positive", nm);
  if (ntok == 0) return 0;
  lmoe::launch_mom_combine(dtype, src, idx, w, out, ntok, topk, D, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_mom_rowdot(const void* src, const int32_t* idx, const void* g, void* dw, int64_t ntok, int32_t topk, int32_t D,
                    int32_t dtype, void* stream) {
  const char* nm = "lmoe_mom_rowdot";
  if (int r = check_mom(nm, src, idx, dw, ntok, D, dtype)) return r;
  if (!g || ((uintptr_t)g & 15)) return fail(-1, "%s: g must be a 16-byte aligned pointer", nm);
  if (topk <= 0) return fail(-4, "%s: topk must be positive", nm);
  if (ntok == 0) return 0;
  lmoe::launch_mom_rowdot(dtype, src, idx, g, dw, ntok, topk, D, (hipStream_t)stream);
  return launched(nm);
}

static int check_gates(const char* nm, int64_t rows, int32_t H, int32_t dtype) {
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (H <= 0 || H > 256) return fail(-3, "%s: H = %d outside 1..256", nm, H);
  if (rows < 0) return fail(-4, "%s: negative row count", nm);
  return 0;
}
int lmoe_gdn_gates_partials(int64_t rows, int32_t H) {
  if (int r = check_gates("lmoe_gdn_gates_partials", rows, H, LMOE_F32)) return r;
  return lmoe::gdn_gates_partials(rows, H);
}
int lmoe_gdn_gates_fwd(const void* a, const void* b, const float* A_log, const float* dt_bias, float* g, void* beta,
                       int64_t rows, int32_t H, int32_t dtype, void* stream) {
  const char* nm = "lmoe_gdn_gates_fwd";
  if (int r = check_gates(nm, rows, H, dtype)) return r;
  if (!a || !b || !A_log || !dt_bias || !g || !beta) return fail(-1, "%s: null pointer", nm);
  if (rows == 0) return 0;
  lmoe::launch_gdn_gates(dtype, a, b, A_log, dt_bias, g, beta, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, rows,
                         H, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_gdn_gates_bwd(const void* a, const void* b, const float* A_log, const float* dt_bias, const float* dg,
                       const void* dbeta, void* da, void* db, float* part, float* dparams, int64_t rows, int32_t H,
                       int32_t dtype, void* stream) {
  const char* nm = "lmoe_gdn_gates_bwd";
  if (int r = check_gates(nm, rows, H, dtype)) return r;
  if (!a || !b || !A_log || !dt_bias || !dg || !dbeta || !da || !db || !dparams) return fail(-1, "%s: null pointer", nm);
  if (rows == 0) return 0;
  if (!part) return fail(-1, "%s: part must not be null", nm);
  lmoe::launch_gdn_gates(dtype, a, b, A_log, dt_bias, nullptr, nullptr, dg, dbeta, da, db, part, dparams, rows, H, true,
                         (hipStream_t)stream);
  return launched(nm);
}
static int check_gla_gate(const char* nm, const void* x, const void* out, int64_t n, int32_t dtype, float normalizer) {
  if (!x || !out) return fail(-1, "%s: null pointer", nm);
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (n < 0 || n % 8) return fail(-4, "%s: element count must be a non-negative multiple of 8", nm);
  if (!(normalizer > 0.f)) return fail(-5, "%s: normalizer must be positive", nm);
  if (((uintptr_t)x | (uintptr_t)out) & 15) return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  return 0;
}
int lmoe_gla_gate_fwd(const void* x, void* y, int64_t n, int32_t dtype, float normalizer, float clamp_min, void* stream) {
  const char* nm = "lmoe_gla_gate_fwd";
  if (int r = check_gla_gate(nm, x, y, n, dtype, normalizer)) return r;
  if (n == 0) return 0;
  lmoe::launch_gla_gate(dtype, x, nullptr, y, n, normalizer, clamp_min, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_gla_gate_bwd(const void* x, const void* dy, void* dx, int64_t n, int32_t dtype, float normalizer,
                      float clamp_min, void* stream) {
  const char* nm = "lmoe_gla_gate_bwd";
  if (int r = check_gla_gate(nm, x, dx, n, dtype, normalizer)) return r;
  if (!dy || ((uintptr_t)dy & 15)) return fail(-1, "%s: dy must be a 16-byte aligned pointer", nm);
  if (n == 0) return 0;
  lmoe::launch_gla_gate(dtype, x, dy, dx, n, normalizer, clamp_min, true, (hipStream_t)stream);
  return launched(nm);
}

static int check_hgrn2(const char* nm, const void* f, const void* lb, int64_t n, int32_t D, int32_t dtype) {
  if (!f) return fail(-1, "%s: null pointer", nm);
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (D <= 0 || D % 8) return fail(-4, "%s: D must be a positive multiple of 8", nm);
  if (n < 0 || n % D) return fail(-4, "%s: element count must be a non-negative multiple of D", nm);
  if (((uintptr_t)f & 15) || ((uintptr_t)lb & 3)) return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  return 0;
}
int lmoe_hgrn2_gate_fwd(const void* f, const float* lower_bound, void* k, float* g, int64_t n, int32_t D, int32_t dtype,
                        void* stream) {
  const char* nm = "lmoe_hgrn2_gate_fwd";
  if (int r = check_hgrn2(nm, f, lower_bound, n, D, dtype)) return r;
  if (!k || !g || (((uintptr_t)k | (uintptr_t)g) & 15)) return fail(-1, "%s: k and g must be 16-byte aligned pointers", nm);
  if (n == 0) return 0;
  lmoe::launch_hgrn2_gate(dtype, f, lower_bound, k, g, nullptr, nullptr, nullptr, n, D, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_hgrn2_gate_bwd(const void* f, const float* lower_bound, const void* dk, const float* dg, void* df, int64_t n,
                        int32_t D, int32_t dtype, void* stream) {
  const char* nm = "lmoe_hgrn2_gate_bwd";
  if (int r = check_hgrn2(nm, f, lower_bound, n, D, dtype)) return r;
  if (!dk || !dg || !df || (((uintptr_t)dk | (uintptr_t)dg | (uintptr_t)df) & 15))
    return fail(-1, "%s: dk, dg and df must be 16-byte aligned pointers", nm);
  if (n == 0) return 0;
  lmoe::launch_hgrn2_gate(dtype, f, lower_bound, nullptr, nullptr, dk, dg, df, n, D, true, (hipStream_t)stream);
  return launched(nm);
}

int lmoe_quad_featmap_features(int32_t D, float c0, float c1) { return lmoe::quad_featmap_features(D, c0, c1); }
static int check_featmap(const char* nm, const void* x, const void* y, int64_t rows, int32_t D, int32_t Kp, float c0,
                         float c1, int32_t dtype) {
  if (!x || !y) return fail(-1, "%s: null pointer", nm);
  if (dtype != LMOE_BF16 && dtype != LMOE_F32) return fail(-2, "%s: dtype must be LMOE_BF16 or LMOE_F32", nm);
  if (D != 8 && D != 16 && D != 32) return fail(-4, "%s: D must be 8, 16 or 32", nm);
  if (rows < 0) return fail(-4, "%s: negative row count", nm);
  if (Kp <= 0 || Kp % 64 || Kp < lmoe::quad_featmap_features(D, c0, c1))
    return fail(-4, "%s: Kp must be a multiple of 64 not below the feature count %d", nm, lmoe::quad_featmap_features(D, c0, c1));
  if (((uintptr_t)x | (uintptr_t)y) & 15) return fail(-9, "%s: pointers must be 16-byte aligned", nm);
  return 0;
}
int lmoe_quad_featmap_fwd(const void* x, void* y, int64_t rows, int32_t D, int32_t Kp, float c0, float c1, float cd,
                          float co, int32_t dtype, void* stream) {
  const char* nm = "lmoe_quad_featmap_fwd";
  if (int r = check_featmap(nm, x, y, rows, D, Kp, c0, c1, dtype)) return r;
  if (rows == 0) return 0;
  lmoe::launch_quad_featmap(dtype, x, y, nullptr, nullptr, rows, D, Kp, c0, c1, cd, co, false, (hipStream_t)stream);
  return launched(nm);
}
int lmoe_quad_featmap_bwd(const void* x, const void* dy, void* dx, int64_t rows, int32_t D, int32_t Kp, float c0,
                          float c1, float cd, float co, int32_t dtype, void* stream) {
  const char* nm = "lmoe_quad_featmap_bwd";
  if (int r = check_featmap(nm, x, dx, rows, D, Kp, c0, c1, dtype)) return r;
  if (!dy || ((uintptr_t)dy & 15)) return fail(-1, "%s: dy must be a 16-byte aligned pointer", nm);
  if (rows == 0) return 0;
  lmoe::launch_quad_featmap(dtype, x, nullptr, dy, dx, rows, D, Kp, c0, c1, cd, co, true, (hipStream_t)stream);
  return launched(nm);
}

int lmoe_launch_stage(const lmoe_args* a, int32_t op, int32_t stage, void* stream) {
  const char* nm = "lmoe_launch_stage";
  if (int r = check_common(a, nm, op == LMOE_OP_GATED_DELTA_RULE)) return r;
  if (op == LMOE_OP_SIMPLE_GLA)
    if (int r = check_normalize(a, nm, stage != lmoe::ST_STATE_FWD)) return r;
  if (a->NT == 0 || a->N == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const bool gdn = op == LMOE_OP_GATED_DELTA_RULE;
  if (op == LMOE_OP_SIMPLE_GLA || gdn) {
    switch (stage) {
      case lmoe::ST_GDN_WY_FWD: if (!gdn) return fail(-20, "%s: stage not part of this op", nm);
        if (!a->gcum || ((a->dtype != LMOE_BF16 || !a->tinv) && !a->pmat))
          return fail(-11, "%s: gcum (and pmat: 4-byte elements or no tinv) must not be null", nm);
        if (a->V == 256 && a->dtype == LMOE_BF16 && !a->tinv) return fail(-11, "%s: V = 256 with 2-byte elements needs tinv", nm);
        lmoe::launch_gdn_wy_fwd(*a, st); break;
      case lmoe::ST_STATE_FWD:
        if (gdn) {
          if (!a->gcum || ((a->dtype != LMOE_BF16 || !a->tinv || a->hs) && !a->pmat))
            return fail(-11, "%s: gcum (and pmat: 4-byte elements, no tinv, or hs given) must not be null", nm);
          if (a->V == 256 && a->dtype == LMOE_BF16 && !a->tinv) return fail(-11, "%s: V = 256 with 2-byte elements needs tinv", nm);
          lmoe::launch_gdn_state_fwd(*a, st);
        } else {
          lmoe::launch_state_fwd(*a, st);
        }
        break;
      case lmoe::ST_DV: if (gdn) return fail(-20, "%s: the delta rule forms dv inside its state pass", nm);
        lmoe::launch_bwd_dv(*a, false, st); break;
      case lmoe::ST_STATE_BWD:
        if (gdn) {
          if (!a->pmat || !a->gcum || !a->tinv || !a->beta.ptr)
            return fail(-11, "%s: pmat, gcum, tinv and beta must not be null", nm);
          lmoe::launch_gdn_state_bwd(*a, st);
        } else {
          lmoe::launch_state_bwd(*a, st);
        }
        break;
      case lmoe::ST_DQK:
        if (gdn) {
          if (!a->dvnew.ptr || !a->beta.ptr) return fail(-11, "%s: dvnew and beta must not be null", nm);
          lmoe::launch_gdn_bwd_chunk(*a, st);
        } else {
          if (!a->hs || !a->dhs || !a->d_o.ptr || !a->dq.ptr || !a->dk.ptr || (a->dtype != LMOE_F32 && !a->dv.ptr))
            return fail(-11, "%s: hs, dhs, d_o, dq, dk (and dv: 2-byte elements) must not be null", nm);
          lmoe::launch_bwd_dqk(*a, st);
        }
        break;
      default: return fail(-20, "%s: stage %d not part of this op", nm, stage);
    }
  } else if (op == LMOE_OP_GLA) {
    if (int r = check_gla(a, nm)) return r;
    if (stage != lmoe::ST_GLA_INTRA_FWD && stage != lmoe::ST_STATE_FWD && stage != lmoe::ST_OUT_FWD &&
        stage != lmoe::ST_STATE_BWD && stage != lmoe::ST_DV && stage != lmoe::ST_DQK)
      return fail(-20, "%s: stage %d not part of this op", nm, stage);
    lmoe::launch_gla(*a, stage, st);
  } else {
    return fail(-21, "%s: unknown op %d", nm, op);
  }
  return launched(nm);
}

int lmoe_selftest_gemm(int32_t dtype, int32_t kd, const void* A, const void* B, float* C, float* G, void* stream) {
  if (!A || !B || !C || !G) return fail(-1, "lmoe_selftest_gemm: null pointer");
  if ((dtype != LMOE_BF16 && dtype != LMOE_F32) || (kd != 64 && kd != 128))
    return fail(-2, "lmoe_selftest_gemm: dtype/kd unsupported");
  lmoe::launch_selftest(dtype, kd, A, B, C, G, (hipStream_t)stream);
  return launched("lmoe_selftest_gemm");
}

}  // extern "C"
