// extern "C" entry points: argument validation, dispatch between the MFMA and the layout-agnostic
// kernels.  Nothing here allocates; every launch goes to the caller's stream.
#include "common.hpp"
#include <cstdarg>
#include <cstdio>

namespace smoe {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  set_error("%s: launch failed: %s", what, hipGetErrorString(e));
  return (int)e;
}

static bool dtype_ok(int d) { return d == SMOE_F32 || d == SMOE_BF16 || d == SMOE_F16; }

}  // namespace smoe

using namespace smoe;

extern "C" {

int smoe_version(void) { return SMOE_ABI_VERSION; }

const char* smoe_last_error(void) { return g_err; }

#ifndef SMOE_SOURCE_HASH
#define SMOE_SOURCE_HASH "unknown"
#endif
const char* smoe_source_hash(void) { return SMOE_SOURCE_HASH; }

size_t smoe_route_workspace_bytes(int64_t L, int E) {
  if (L < 0 || E <= 0) return 0;
  return route_workspace_bytes(L, E);
}

int smoe_route(const void* expert_idxs, int idx_dtype, int64_t L, int E, int64_t* eid_out,
               int64_t* idx_out, int64_t* off_out, void* workspace, size_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  if (L < 0 || E <= 0) { set_error("smoe_route: bad sizes L=%lld E=%d", (long long)L, E); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL) { set_error("smoe_route: L=%lld does not fit int32 row indexing", (long long)L); return SMOE_ERR_RANGE; }
  if (!off_out || (L > 0 && (!expert_idxs || !eid_out || !idx_out))) { set_error("smoe_route: NULL pointer"); return SMOE_ERR_NULL; }
  const size_t need = route_workspace_bytes(L, E);
  if (need > 0 && (!workspace || workspace_bytes < need)) {
    set_error("smoe_route: workspace of %zu bytes needed, %zu given", need, workspace ? workspace_bytes : (size_t)0);
    return SMOE_ERR_WORKSPACE;
  }
  return launch_route(expert_idxs, idx_dtype, L, E, eid_out, idx_out, off_out, workspace, (hipStream_t)stream);
}

int smoe_route_static_init(void) {
  g_err[0] = 0;
  return route_static_init();
}

int smoe_route_static(const void* expert_idxs, int idx_dtype, int64_t L, int E, int64_t* eid_out,
                      int64_t* idx_out, int64_t* off_out, void* stream) {
  g_err[0] = 0;
  if (L < 0 || E <= 0) { set_error("smoe_route_static: bad sizes L=%lld E=%d", (long long)L, E); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL) { set_error("smoe_route_static: L=%lld does not fit int32 row indexing", (long long)L); return SMOE_ERR_RANGE; }
  if (!off_out || (L > 0 && (!expert_idxs || !eid_out || !idx_out))) { set_error("smoe_route_static: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_route_static(expert_idxs, idx_dtype, L, E, eid_out, idx_out, off_out, (hipStream_t)stream);
}

int smoe_offsets_from_sorted(const int64_t* eid, int64_t L, int E, int64_t* off_out, void* stream) {
  g_err[0] = 0;
  if (L < 0 || E <= 0) { set_error("smoe_offsets_from_sorted: bad sizes"); return SMOE_ERR_SHAPE; }
  if (!off_out || (L > 0 && !eid)) { set_error("smoe_offsets_from_sorted: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_offsets_from_sorted(eid, L, E, off_out, (hipStream_t)stream);
}

size_t smoe_scatter2scatter_workspace_bytes(int64_t L, int64_t K, int64_t N, int E, int dtype) {
  if (L <= 0 || K <= 0 || N <= 0 || E <= 0) return 0;
  return (size_t)s2s_workspace_floats(L, K, N, E, dtype) * sizeof(float);
}

int smoe_scatter2scatter(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk,
                         int64_t swn, const void* b, int64_t sbe, int64_t sbn, void* Y, int64_t sym,
                         int64_t syn, const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L,
                         int64_t K, int64_t N, int E, int fan_out, int x_grouped, int y_grouped, int dtype,
                         void* stream) {
  return smoe_scatter2scatter_ws(X, sxm, sxk, W, swe, swk, swn, b, sbe, sbn, Y, sym, syn, eid, idx, off, L, K, N, E,
                                 fan_out, x_grouped, y_grouped, dtype, nullptr, 0, stream);
}

int smoe_scatter2scatter_ws(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk,
                            int64_t swn, const void* b, int64_t sbe, int64_t sbn, void* Y, int64_t sym,
                            int64_t syn, const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L,
                            int64_t K, int64_t N, int E, int fan_out, int x_grouped, int y_grouped, int dtype,
                            void* workspace, size_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_scatter2scatter: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (L < 0 || K < 0 || N < 0 || E <= 0 || fan_out <= 0) { set_error("smoe_scatter2scatter: bad sizes"); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL || K > 0x7fffffffLL || N > 0x7fffffffLL) { set_error("smoe_scatter2scatter: size beyond int32"); return SMOE_ERR_RANGE; }
  if (L == 0 || N == 0) return 0;
  if (!X || !W || !Y || !idx || !off) { set_error("smoe_scatter2scatter: NULL pointer"); return SMOE_ERR_NULL; }
  (void)eid;  // expert boundaries come from `off`; kept in the signature for parity with the reference call
  S2SArgs a{X, sxm, sxk, W, swe, swk, swn, b, sbe, sbn, Y, sym, syn, eid, idx, off,
            (int)L, (int)K, (int)N, E, fan_out, x_grouped, y_grouped};
  if (workspace != nullptr && ((uintptr_t)workspace & 15) == 0) {       // optional: without it nothing is split
    a.partial = (float*)workspace;
    a.partial_floats = (int64_t)(workspace_bytes / sizeof(float));
  }
  int rc = 0;
  if (try_s2s_mfma(a, dtype, (hipStream_t)stream, rc)) return rc;
  return launch_s2s_generic(a, dtype, (hipStream_t)stream);
}

static int glu_common_checks(const char* who, int64_t L, int64_t K, int64_t F, int E, int act, int dtype) {
  if (!dtype_ok(dtype)) { set_error("%s: unknown dtype %d", who, dtype); return SMOE_ERR_DTYPE; }
  if (L < 0 || K < 0 || F < 0 || E <= 0) { set_error("%s: bad sizes", who); return SMOE_ERR_SHAPE; }
  if (act != SMOE_ACT_SILU && act != SMOE_ACT_SILU_GATE_FIRST) { set_error("%s: unknown activation %d", who, act); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL || K > 0x7fffffffLL || F > 0x3fffffffLL) { set_error("%s: size beyond int32", who); return SMOE_ERR_RANGE; }
  return 0;
}

int smoe_scatter2scatter_glu(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk,
                             int64_t swn, const void* b, int64_t sbe, int64_t sbn, void* PRE, int64_t spm, void* H,
                             int64_t shm, const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L,
                             int64_t K, int64_t F, int E, int fan_out, int x_grouped, int act, int dtype,
                             void* stream) {
  g_err[0] = 0;
  if (int rc = glu_common_checks("smoe_scatter2scatter_glu", L, K, F, E, act, dtype)) return rc;
  if (fan_out <= 0) { set_error("smoe_scatter2scatter_glu: bad fan_out"); return SMOE_ERR_SHAPE; }
  if (L == 0 || F == 0) return 0;
  if (!X || !W || !H || !idx || !off) { set_error("smoe_scatter2scatter_glu: NULL pointer"); return SMOE_ERR_NULL; }
  S2SArgs a{X, sxm, sxk, W, swe, swk, swn, b, sbe, sbn, PRE, spm, 1, eid, idx, off,
            (int)L, (int)K, (int)F, E, fan_out, x_grouped, 1};
  a.glu = 1; a.act = act; a.H = H; a.shm = shm;
  int rc = 0;
  if (try_s2s_mfma(a, dtype, (hipStream_t)stream, rc)) return rc;
  return SMOE_ERR_UNSUPPORTED;
}

int smoe_scatter2scatter_glu_bwd(const void* DY, int64_t sdm, int64_t sdk, const void* W, int64_t swe, int64_t swk,
                                 int64_t swn, const void* PRE, int64_t spm, void* DPRE, int64_t sdpm,
                                 const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L, int64_t K,
                                 int64_t F, int E, int act, int dtype, void* stream) {
  g_err[0] = 0;
  if (int rc = glu_common_checks("smoe_scatter2scatter_glu_bwd", L, K, F, E, act, dtype)) return rc;
  if (L == 0 || F == 0) return 0;
  if (!DY || !W || !PRE || !DPRE || !idx || !off) { set_error("smoe_scatter2scatter_glu_bwd: NULL pointer"); return SMOE_ERR_NULL; }
  S2SArgs a{DY, sdm, sdk, W, swe, swk, swn, nullptr, 0, 0, DPRE, sdpm, 1, eid, idx, off,
            (int)L, (int)K, (int)F, E, 1, 1, 1};
  a.glu = 2; a.act = act; a.aux = PRE; a.saux = spm;
  int rc = 0;
  if (try_s2s_mfma(a, dtype, (hipStream_t)stream, rc)) return rc;
  return SMOE_ERR_UNSUPPORTED;
}

int smoe_scatter2scatter_oss_glu(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk,
                                 int64_t swn, const void* b, int64_t sbe, int64_t sbn, void* PRE, int64_t spm, void* H,
                                 int64_t shm, const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L,
                                 int64_t K, int64_t F, int E, int fan_out, int x_grouped, float alpha, float limit,
                                 int dtype, void* stream) {
  g_err[0] = 0;
  if (int rc = glu_common_checks("smoe_scatter2scatter_oss_glu", L, K, F, E, SMOE_ACT_SILU, dtype)) return rc;
  if (fan_out <= 0) { set_error("smoe_scatter2scatter_oss_glu: bad fan_out"); return SMOE_ERR_SHAPE; }
  if (L == 0 || F == 0) return 0;
  if (!X || !W || !H || !idx || !off) { set_error("smoe_scatter2scatter_oss_glu: NULL pointer"); return SMOE_ERR_NULL; }
  if (dtype == SMOE_F32) return SMOE_ERR_UNSUPPORTED;
  S2SArgs a{X, sxm, sxk, W, swe, swk, swn, b, sbe, sbn, PRE, spm, 1, eid, idx, off,
            (int)L, (int)K, (int)(2 * F), E, fan_out, x_grouped, 1};
  a.glu = 3; a.H = H; a.shm = shm; a.alpha = alpha; a.limit = limit;
  int rc = 0;
  if (try_s2s_mfma(a, dtype, (hipStream_t)stream, rc)) return rc;
  return SMOE_ERR_UNSUPPORTED;
}

int smoe_scatter2scatter_oss_glu_bwd(const void* DY, int64_t sdm, int64_t sdk, const void* W, int64_t swe, int64_t swk,
                                     int64_t swn, const void* PRE, int64_t spm, void* DPRE, int64_t sdpm,
                                     const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L, int64_t K,
                                     int64_t F, int E, float alpha, float limit, int dtype, void* stream) {
  g_err[0] = 0;
  if (int rc = glu_common_checks("smoe_scatter2scatter_oss_glu_bwd", L, K, F, E, SMOE_ACT_SILU, dtype)) return rc;
  if (L == 0 || F == 0) return 0;
  if (!DY || !W || !PRE || !DPRE || !idx || !off) { set_error("smoe_scatter2scatter_oss_glu_bwd: NULL pointer"); return SMOE_ERR_NULL; }
  if (dtype == SMOE_F32) return SMOE_ERR_UNSUPPORTED;
  S2SArgs a{DY, sdm, sdk, W, swe, swk, swn, nullptr, 0, 0, DPRE, sdpm, 1, eid, idx, off,
            (int)L, (int)K, (int)F, E, 1, 1, 1};
  a.glu = 4; a.aux = PRE; a.saux = spm; a.alpha = alpha; a.limit = limit;
  int rc = 0;
  if (try_s2s_mfma(a, dtype, (hipStream_t)stream, rc)) return rc;
  return SMOE_ERR_UNSUPPORTED;
}

int smoe_group(const void* A, int64_t sam, int64_t sak, const void* coeff, void* Y, int64_t sym, int64_t syk,
               const int64_t* idx, int64_t L, int64_t K, int fan_out, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_group: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (L < 0 || K < 0 || fan_out <= 0) { set_error("smoe_group: bad sizes"); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL || K > 0x7fffffffLL) { set_error("smoe_group: size beyond int32"); return SMOE_ERR_RANGE; }
  if (L == 0 || K == 0) return 0;
  if (!A || !Y || !idx) { set_error("smoe_group: NULL pointer"); return SMOE_ERR_NULL; }
  GroupArgs a{A, sam, sak, coeff, Y, sym, syk, idx, (int)L, (int)K, fan_out};
  return launch_group(a, dtype, (hipStream_t)stream);
}

int smoe_group_by_source(const void* A, int64_t sam, int64_t sak, const void* coeff, void* Y, int64_t sym,
                         int64_t syk, const int64_t* idx, int32_t* inverse_workspace, int64_t L, int64_t K,
                         int fan_out, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_group_by_source: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (L < 0 || K < 0 || fan_out <= 0) { set_error("smoe_group_by_source: bad sizes"); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL || K > 0x7fffffffLL) { set_error("smoe_group_by_source: size beyond int32"); return SMOE_ERR_RANGE; }
  if (L == 0 || K == 0) return 0;
  if (!A || !Y || !idx || !inverse_workspace) { set_error("smoe_group_by_source: NULL pointer"); return SMOE_ERR_NULL; }
  GroupArgs a{A, sam, sak, coeff, Y, sym, syk, idx, (int)L, (int)K, fan_out};
  return launch_group_by_source(a, (int*)inverse_workspace, dtype, (hipStream_t)stream);
}

int smoe_groupXtY(const void* DY, int64_t sdym, int64_t sdyn, const void* X, int64_t sxm, int64_t sxk,
                  void* DW, int64_t sdwe, int64_t sdwk, int64_t sdwn, void* Db, int64_t sdbe, int64_t sdbn,
                  const int64_t* off, int64_t L, int64_t K, int64_t N, int E, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_groupXtY: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (L < 0 || K < 0 || N < 0 || E <= 0) { set_error("smoe_groupXtY: bad sizes"); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL || K > 0x7fffffffLL || N > 0x7fffffffLL) { set_error("smoe_groupXtY: size beyond int32"); return SMOE_ERR_RANGE; }
  if (K == 0 || N == 0) return 0;
  if (!DW || !off || (L > 0 && (!DY || !X))) { set_error("smoe_groupXtY: NULL pointer"); return SMOE_ERR_NULL; }
  XtYArgs a{DY, sdym, sdyn, X, sxm, sxk, DW, sdwe, sdwk, sdwn, Db, sdbe, sdbn, off, (int)L, (int)K, (int)N, E};
  int rc = 0;
  if (try_xty_mfma(a, dtype, (hipStream_t)stream, rc)) return rc;
  return launch_xty_generic(a, dtype, (hipStream_t)stream);
}

int smoe_groupXtY_gathered(const void* DY, int64_t sdym, int64_t sdyn, const void* X, int64_t sxm, int64_t sxk,
                           const int64_t* idx, int fan_out, void* DW, int64_t sdwe, int64_t sdwk, int64_t sdwn,
                           void* Db, int64_t sdbe, int64_t sdbn, const int64_t* off, int64_t L, int64_t K, int64_t N,
                           int E, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_groupXtY_gathered: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (L < 0 || K < 0 || N < 0 || E <= 0 || fan_out <= 0) { set_error("smoe_groupXtY_gathered: bad sizes"); return SMOE_ERR_SHAPE; }
  if (L > 0x7fffffffLL || K > 0x7fffffffLL || N > 0x7fffffffLL) { set_error("smoe_groupXtY_gathered: size beyond int32"); return SMOE_ERR_RANGE; }
  if (L % fan_out != 0) { set_error("smoe_groupXtY_gathered: L=%lld is not a multiple of fan_out=%d", (long long)L, fan_out); return SMOE_ERR_SHAPE; }
  // Only the bf16 / fp16 MFMA kernel reads X through the index vector; the float32 kernels would take X for the
  // grouped (L, K) matrix and read past the end of the (L / fan_out, K) one.  Nothing is launched.
  if (dtype == SMOE_F32) { set_error("smoe_groupXtY_gathered: float32 is not gathered; group X and call smoe_groupXtY"); return SMOE_ERR_UNSUPPORTED; }
  if (K == 0 || N == 0) return 0;
  if (!DW || !off || (L > 0 && (!DY || !X || !idx))) { set_error("smoe_groupXtY_gathered: NULL pointer"); return SMOE_ERR_NULL; }
  XtYArgs a{DY, sdym, sdyn, X, sxm, sxk, DW, sdwe, sdwk, sdwn, Db, sdbe, sdbn, off, (int)L, (int)K, (int)N, E};
  a.idx = idx;
  a.fan_out = fan_out;
  int rc = 0;
  if (try_xty_mfma(a, dtype, (hipStream_t)stream, rc)) return rc;
  return SMOE_ERR_UNSUPPORTED;       // only the MFMA kernels gather; the caller groups X itself and calls smoe_groupXtY
}

int smoe_combine(const void* Y, int64_t sym, const void* gates, int64_t sgt, int64_t sgk, void* out, int64_t som,
                 int64_t T, int k, int64_t N, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_combine: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (T < 0 || k <= 0 || N < 0) { set_error("smoe_combine: bad sizes"); return SMOE_ERR_SHAPE; }
  if (T > 0x7fffffffLL || N > 0x7fffffffLL) { set_error("smoe_combine: size beyond int32"); return SMOE_ERR_RANGE; }
  if (T == 0 || N == 0) return 0;
  if (!Y || !out) { set_error("smoe_combine: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_combine(Y, sym, gates, sgt, sgk, out, som, T, k, (int)N, dtype, (hipStream_t)stream);
}

int smoe_gate_grad(const void* Y, int64_t sym, const void* dOut, int64_t sdm, void* dgates, int64_t sgt, int64_t sgk,
                   int64_t T, int k, int64_t N, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_gate_grad: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (T < 0 || k <= 0 || N < 0) { set_error("smoe_gate_grad: bad sizes"); return SMOE_ERR_SHAPE; }
  if (T > 0x7fffffffLL || N > 0x7fffffffLL) { set_error("smoe_gate_grad: size beyond int32"); return SMOE_ERR_RANGE; }
  if (T == 0) return 0;
  if (!dgates || (N > 0 && (!Y || !dOut))) { set_error("smoe_gate_grad: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_gate_grad(Y, sym, dOut, sdm, dgates, sgt, sgk, T, k, (int)N, dtype, (hipStream_t)stream);
}

int smoe_gate_grad_group(const void* Y, int64_t sym, const void* dOut, int64_t sdm, const void* gates, int64_t sgt,
                         int64_t sgk, const int64_t* idx, int32_t* inverse_workspace, void* dY, int64_t sdym,
                         void* dgates, int64_t sdgt, int64_t sdgk, int64_t T, int k, int64_t N, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_gate_grad_group: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (T < 0 || k <= 0 || N < 0) { set_error("smoe_gate_grad_group: bad sizes"); return SMOE_ERR_SHAPE; }
  if (T > 0x7fffffffLL || N > 0x7fffffffLL || T * k > 0x7fffffffLL) { set_error("smoe_gate_grad_group: size beyond int32"); return SMOE_ERR_RANGE; }
  if (T == 0) return 0;
  if (!Y || !dOut || !gates || !idx || !inverse_workspace || !dY || !dgates) { set_error("smoe_gate_grad_group: NULL pointer"); return SMOE_ERR_NULL; }
  if (N == 0) return SMOE_ERR_UNSUPPORTED;
  return launch_gate_grad_group(Y, sym, dOut, sdm, gates, sgt, sgk, idx, (int*)inverse_workspace, dY, sdym, dgates, sdgt,
                                sdgk, T, k, (int)N, dtype, (hipStream_t)stream);
}

int smoe_glu_fwd(const void* pre, int64_t spm, void* h, int64_t shm, int64_t rows, int64_t f, int act, int dtype,
                 void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_glu_fwd: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (rows < 0 || f < 0) { set_error("smoe_glu_fwd: bad sizes"); return SMOE_ERR_SHAPE; }
  if (act != SMOE_ACT_SILU && act != SMOE_ACT_SILU_GATE_FIRST) { set_error("smoe_glu_fwd: unknown activation %d", act); return SMOE_ERR_SHAPE; }
  if (f > 0x3fffffffLL) { set_error("smoe_glu_fwd: size beyond int32"); return SMOE_ERR_RANGE; }
  if (rows == 0 || f == 0) return 0;
  if (!pre || !h) { set_error("smoe_glu_fwd: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_glu_fwd(pre, spm, h, shm, rows, (int)f, act, dtype, (hipStream_t)stream);
}

int smoe_glu_bwd(const void* pre, int64_t spm, const void* dh, int64_t sdhm, void* dpre, int64_t sdpm, int64_t rows,
                 int64_t f, int act, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_glu_bwd: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (rows < 0 || f < 0) { set_error("smoe_glu_bwd: bad sizes"); return SMOE_ERR_SHAPE; }
  if (act != SMOE_ACT_SILU && act != SMOE_ACT_SILU_GATE_FIRST) { set_error("smoe_glu_bwd: unknown activation %d", act); return SMOE_ERR_SHAPE; }
  if (f > 0x3fffffffLL) { set_error("smoe_glu_bwd: size beyond int32"); return SMOE_ERR_RANGE; }
  if (rows == 0 || f == 0) return 0;
  if (!pre || !dh || !dpre) { set_error("smoe_glu_bwd: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_glu_bwd(pre, spm, dh, sdhm, dpre, sdpm, rows, (int)f, act, dtype, (hipStream_t)stream);
}

int smoe_gpt_oss_glu_fwd(const void* pre, int64_t spm, void* h, int64_t shm, int64_t rows, int64_t f, float alpha,
                         float limit, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_gpt_oss_glu_fwd: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (rows < 0 || f < 0) { set_error("smoe_gpt_oss_glu_fwd: bad sizes"); return SMOE_ERR_SHAPE; }
  if (f > 0x3fffffffLL) { set_error("smoe_gpt_oss_glu_fwd: size beyond int32"); return SMOE_ERR_RANGE; }
  if (rows == 0 || f == 0) return 0;
  if (!pre || !h) { set_error("smoe_gpt_oss_glu_fwd: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_oss_glu_fwd(pre, spm, h, shm, rows, (int)f, alpha, limit, dtype, (hipStream_t)stream);
}

int smoe_gpt_oss_glu_bwd(const void* pre, int64_t spm, const void* dh, int64_t sdhm, void* dpre, int64_t sdpm,
                         int64_t rows, int64_t f, float alpha, float limit, int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_gpt_oss_glu_bwd: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (rows < 0 || f < 0) { set_error("smoe_gpt_oss_glu_bwd: bad sizes"); return SMOE_ERR_SHAPE; }
  if (f > 0x3fffffffLL) { set_error("smoe_gpt_oss_glu_bwd: size beyond int32"); return SMOE_ERR_RANGE; }
  if (rows == 0 || f == 0) return 0;
  if (!pre || !dh || !dpre) { set_error("smoe_gpt_oss_glu_bwd: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_oss_glu_bwd(pre, spm, dh, sdhm, dpre, sdpm, rows, (int)f, alpha, limit, dtype, (hipStream_t)stream);
}

int smoe_decode_glu_mlp(const void* X, int64_t sxm, const int64_t* experts, int64_t set, int64_t sek, const void* gates,
                        int64_t sgt, int64_t sgk, const void* W1, int64_t sw1e, int64_t sw1n, const void* b1,
                        int64_t sb1e, int64_t sb1n, const void* W2, int64_t sw2e, int64_t sw2n, const void* b2,
                        int64_t sb2e, int64_t sb2n, void* H, int64_t shm, void* OUT, int64_t som, int64_t T, int k,
                        int64_t d, int64_t F, int E, int act, int dtype, void* stream) {
  g_err[0] = 0;
  if (int rc = glu_common_checks("smoe_decode_glu_mlp", T, d, F, E, act, dtype)) return rc;
  if (k <= 0) { set_error("smoe_decode_glu_mlp: bad top-k"); return SMOE_ERR_SHAPE; }
  if (T == 0 || d == 0) return 0;
  if (!X || !experts || !gates || !W1 || !W2 || !H || !OUT) { set_error("smoe_decode_glu_mlp: NULL pointer"); return SMOE_ERR_NULL; }
  // Not an error: the caller then takes the general path (routing, two scatter2scatter launches, combine)
  auto al16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  if (dtype == SMOE_F32 || T * k > DECODE_MAX_ROWS || F == 0 || d % 8 || F % 8 || sxm % 8 || shm % 8 ||
      sw1e % 8 || sw1n % 8 || sw2e % 8 || sw2n % 8 || !al16(X) || !al16(W1) || !al16(W2) || !al16(H))
    return SMOE_ERR_UNSUPPORTED;
  DecodeArgs a{X, sxm, experts, set, sek, gates, sgt, sgk, W1, sw1e, sw1n, b1, sb1e, sb1n, W2, sw2e, sw2n,
               b2, sb2e, sb2n, H, shm, OUT, som, (int)T, k, (int)d, (int)F, E, act};
  return launch_decode_glu_mlp(a, dtype, (hipStream_t)stream);
}

int smoe_topk_softmax(const void* logits, int64_t slt, int64_t sle, int64_t T, int E, int k, int renormalize,
                      float* weights_out, int64_t swt, int64_t swk, int64_t* idx_out, int64_t sit, int64_t sik,
                      int dtype, void* stream) {
  g_err[0] = 0;
  if (!dtype_ok(dtype)) { set_error("smoe_topk_softmax: unknown dtype %d", dtype); return SMOE_ERR_DTYPE; }
  if (T < 0 || E <= 0 || k <= 0 || k > E) { set_error("smoe_topk_softmax: bad sizes"); return SMOE_ERR_SHAPE; }
  if (E > 512 || k > 64) { set_error("smoe_topk_softmax: at most 512 experts and top-64"); return SMOE_ERR_RANGE; }
  if (T == 0) return 0;
  if (!logits || !weights_out || !idx_out) { set_error("smoe_topk_softmax: NULL pointer"); return SMOE_ERR_NULL; }
  return launch_topk_softmax(logits, slt, sle, weights_out, swt, swk, idx_out, sit, sik, T, E, k, renormalize, dtype,
                             (hipStream_t)stream);
}

}  // extern "C"
