// Host-side launch functions, one translation unit per kernel family.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/lmoe.h"

namespace lmoe {
// simple_gla / gated delta rule forward: state pass + output (gdn = false: plain values)
void launch_scalar_fwd(const lmoe_args& a, bool gdn, hipStream_t st);
// gated delta rule: chunk-parallel WY preparation (w, u, Tinv)
void launch_gdn_wy_fwd(const lmoe_args& a, hipStream_t st);
// simple_gla / gated delta rule backward: dv (local), reverse state pass, dq/dk/gate gradient
void launch_scalar_bwd(const lmoe_args& a, bool gdn, hipStream_t st);
// gated delta rule: backward through the WY factors (finishes dk, dv, dbeta, dg)
void launch_gdn_wy_bwd(const lmoe_args& a, hipStream_t st);
void launch_selftest(int dtype, int kd, const void* A, const void* B, float* C, float* Ct, hipStream_t st);
}  // namespace lmoe
