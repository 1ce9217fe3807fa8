// Shared device/host helpers for the gfx950 ScatterMoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/scattermoe_amd.h"

namespace smoe {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

// ---- error text, one slot per host thread -------------------------------------------------------
void set_error(const char* fmt, ...);
int launch_status(const char* what);  // hipGetLastError() -> return code (+ error text)

// ---- element conversion --------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return (T)v; }

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

// ---- gated linear unit math (shared by the stand-alone passes and the fused GEMM epilogues) ----------------
// Every multiplication / addition below is kept as written (no contraction into FMAs, no reassociation), so
// that the fused epilogues and the stand-alone passes give the same bits whatever code surrounds them.
// The reciprocal is the hardware's (v_rcp_f32, 1 ulp) rather than a correctly rounded division: the epilogues of
// the fused launches spend their time in this function (a division is about ten instructions), and every result
// is rounded to a 16-bit type or compared at 1e-4 afterwards.
__device__ __forceinline__ float sigmoidf_(float x) {
#pragma clang fp contract(off) reassociate(off)
  const float e = __expf(-x);
  const float d = 1.0f + e;
  return __builtin_amdgcn_rcpf(d);
}
// act & 1 selects which half of `pre` is the activated (gate) half: 0 = second half (GLUMLP of the reference),
// 1 = first half (the Hugging Face `act(gate) * up` convention).  The activation itself is SiLU.
__device__ __forceinline__ float act_f(int act, float g) {
#pragma clang fp contract(off) reassociate(off)
  (void)act;
  const float s = sigmoidf_(g);
  return g * s;
}
__device__ __forceinline__ float act_df(int act, float g) {
#pragma clang fp contract(off) reassociate(off)
  (void)act;
  const float s = sigmoidf_(g);
  const float a = 1.0f - s;
  const float b = g * a;
  const float c = 1.0f + b;
  return s * c;
}
// hidden value and the two gradients of h = act(gate) * lin
__device__ __forceinline__ float glu_h(int act, float gat, float lin) {
#pragma clang fp contract(off) reassociate(off)
  const float a = act_f(act, gat);
  return a * lin;
}
__device__ __forceinline__ float glu_dlin(int act, float dh, float gat) {
#pragma clang fp contract(off) reassociate(off)
  const float a = act_f(act, gat);
  return dh * a;
}
__device__ __forceinline__ float glu_dgat(int act, float dh, float gat, float lin) {
#pragma clang fp contract(off) reassociate(off)
  const float t = dh * lin;
  const float d = act_df(act, gat);
  return t * d;
}

// both gradients at once (one sigmoid); same operations in the same order as glu_dlin and glu_dgat
__device__ __forceinline__ void glu_grad(int act, float dh, float gat, float lin, float& d_lin, float& d_gat) {
#pragma clang fp contract(off) reassociate(off)
  (void)act;
  const float s = sigmoidf_(gat);
  const float a0 = gat * s;
  d_lin = dh * a0;
  const float t = dh * lin;
  const float a = 1.0f - s;
  const float b = gat * a;
  const float c = 1.0f + b;
  const float d = s * c;
  d_gat = t * d;
}

// gated unit of the gpt-oss experts over one (gate, up) pair and its gradient (clamped inputs pass no gradient)
__device__ __forceinline__ float oss_h(float gate, float up, float alpha, float limit) {
  const float g = fminf(gate, limit), u = fminf(fmaxf(up, -limit), limit);
  return (u + 1.0f) * (g * sigmoidf_(alpha * g));
}
__device__ __forceinline__ void oss_grad(float gate, float up, float dh, float alpha, float limit, float& dgate,
                                         float& dup) {
  const float g = fminf(gate, limit), u = fminf(fmaxf(up, -limit), limit);
  const float s = sigmoidf_(alpha * g);
  const float glu = g * s;
  dup = (up >= -limit && up <= limit) ? dh * glu : 0.0f;
  const float dglu = dh * (u + 1.0f);
  dgate = gate <= limit ? dglu * (s + alpha * g * s * (1.0f - s)) : 0.0f;
}

// ---- expert-aligned tile lookup -------------------------------------------------------------------
// Rows are expert-sorted; expert e owns rows [off[e-1], off[e]).  Tiles of height BM never straddle
// two experts: expert e contributes ceil(count_e / BM) tiles and tiles are numbered expert-major.
// Every wave of the block runs this redundantly and gets the same (uniform) answer.
// Returns false when `t` is past the last tile (the grid is sized by the host-known upper bound
// floor(L/BM) + E, so surplus blocks simply exit).
// `skip_small` > 0: an expert's last, partly filled tile is left out when it holds at most `skip_small` rows (another
// launch with lower tiles takes those rows, see find_remainder).
template <int BM>
__device__ __forceinline__ bool find_tile(const int64_t* __restrict__ off, int E, int t,
                                          int& expert, int& row_start, int& rows, int skip_small = 0) {
  const int lane = lane_id();
  int tiles_before = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int e = e0 + lane;
    int lo = 0, hi = 0;
    if (e < E) {
      hi = (int)off[e];
      lo = e ? (int)off[e - 1] : 0;
    }
    int nt = (hi - lo + BM - 1) / BM;
    const int rem = (hi - lo) % BM;
    if (rem != 0 && rem <= skip_small) nt -= 1;
    int incl = nt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      int v = __shfl_up(incl, d, 64);
      if (lane >= d) incl += v;
    }
    const int cum = tiles_before + incl;
    const unsigned long long hit = __ballot(cum > t);
    if (hit) {
      const int src = __ffsll((long long)hit) - 1;
      const int lo_s = __shfl(lo, src, 64), hi_s = __shfl(hi, src, 64);
      const int first = __shfl(cum - nt, src, 64);
      expert = e0 + src;
      row_start = lo_s + (t - first) * BM;
      rows = min(BM, hi_s - row_start);
      return true;
    }
    tiles_before += __shfl(incl, 63, 64);
  }
  return false;
}

// The rows that find_tile<BM>(..., skip_small) leaves out, as one tile per expert: the last n % BM rows of expert e
// when there are between 1 and `small` of them.
template <int BM>
__device__ __forceinline__ bool find_remainder(const int64_t* __restrict__ off, int E, int e, int small,
                                               int& row_start, int& rows) {
  if (e >= E) return false;
  const int hi = (int)off[e], lo = e ? (int)off[e - 1] : 0;
  const int rem = (hi - lo) % BM;
  if (rem == 0 || rem > small) return false;
  row_start = hi - rem;
  rows = rem;
  return true;
}

static inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Upper bound on the number of expert-aligned tiles of height bm over L rows and E experts.
static inline int64_t max_tiles(int64_t L, int E, int bm) {
  int64_t a = L / bm + E;        // sum ceil(c_e/bm) <= floor(L/bm) + E
  int64_t b = L;                 // and never more than one tile per row
  int64_t r = a < b ? a : b;
  return r < 1 ? 1 : r;
}

// ---- kernel launchers implemented in the individual .hip files ---------------------------------------
struct S2SArgs {
  const void* X; int64_t sxm, sxk;
  const void* W; int64_t swe, swk, swn;
  const void* b; int64_t sbe, sbn;
  void* Y; int64_t sym, syn;
  const int64_t* eid; const int64_t* idx; const int64_t* off;
  int L, K, N, E, fan_out;
  int x_grouped, y_grouped;
  // fused gated-linear-unit epilogues (MFMA path only, rows in grouped order):
  //   glu == 1: W has 2N columns; Y (may be NULL) receives the pre-activation (L, 2N), H the hidden (L, N)
  //   glu == 2: Y receives d(pre) (L, 2N) computed from the product (= d hidden) and the saved pre-activation AUX
  //   glu == 3: gpt-oss form, N = 2F columns holding (gate, up) pairs: Y (may be NULL) receives the pre-activation
  //             (L, 2F), H the hidden (L, F)
  //   glu == 4: gpt-oss form, N = F: Y receives d(pre) (L, 2F) from the product (= d hidden) and the saved AUX
  int glu = 0, act = 0;
  const void* aux = nullptr; int64_t saux = 0;
  void* H = nullptr; int64_t shm = 0;
  float alpha = 0.0f, limit = 0.0f;
  // Part of a product split by tile rows (MFMA path only): the launch covers the tile rows
  // [m_begin, m_begin + m_count) of its tile height.
  int m_begin = 0, m_count = 0x7fffffff;
  // Products whose experts end in a partly filled tile (MFMA path only).  1: this launch leaves out every expert's
  // last tile when it holds at most 128 rows; 2: this launch takes exactly those rows, one tile row per expert.
  int tail_mode = 0;
  // tail_mode 2 only: the contraction of every tile is cut into `ksplit` equal parts, one workgroup each, which
  // leave their float32 accumulators in `partial` (see splitk_floats); a second launch adds the parts up in a
  // fixed order and writes the output rows.  `partial` / `partial_floats`: the caller's workspace, may be NULL / 0.
  int ksplit = 1, k_part = 0;           // k_part = K / ksplit
  float* partial = nullptr;
  int64_t partial_floats = 0;
};

struct XtYArgs {
  const void* DY; int64_t sdym, sdyn;
  const void* X; int64_t sxm, sxk;
  void* DW; int64_t sdwe, sdwk, sdwn;
  void* Db; int64_t sdbe, sdbn;
  const int64_t* off;
  int L, K, N, E;
  // X is the (L / fan_out, K) matrix the grouped rows would be gathered from: grouped row r = X[idx[r] / fan_out]
  // (MFMA path only); NULL: X holds the L grouped rows themselves
  const int64_t* idx = nullptr;
  int fan_out = 1;
};

struct GroupArgs {
  const void* A; int64_t sam, sak;
  const void* coeff;
  void* Y; int64_t sym, syk;
  const int64_t* idx;
  int L, K, fan_out;
};

// Whole gated MLP for at most DECODE_MAX_ROWS (token, slot) rows, forward only (csrc/s2s_rowdot.hip)
static constexpr int DECODE_MAX_ROWS = 8;
struct DecodeArgs {
  const void* X; int64_t sxm;                        // (T, d) tokens, columns contiguous
  const int64_t* experts; int64_t set, sek;          // (T, k) expert ids
  const void* gates; int64_t sgt, sgk;               // (T, k) routing weights
  const void* W1; int64_t sw1e, sw1n;                // (E, 2F, d), d contiguous
  const void* b1; int64_t sb1e, sb1n;                // (E, 2F) or NULL
  const void* W2; int64_t sw2e, sw2n;                // (E, d, F), F contiguous
  const void* b2; int64_t sb2e, sb2n;                // (E, d) or NULL
  void* H; int64_t shm;                              // (T*k, F) workspace: hidden rows in slot order
  void* OUT; int64_t som;                            // (T, d)
  int T, k, d, F, E, act;
};
int launch_decode_glu_mlp(const DecodeArgs& a, int dtype, hipStream_t st);

int launch_s2s_generic(const S2SArgs& a, int dtype, hipStream_t st);
int launch_xty_generic(const XtYArgs& a, int dtype, hipStream_t st);
int launch_group(const GroupArgs& a, int dtype, hipStream_t st);
// MFMA paths return 1 if they took the call, 0 if the shape/layout is not theirs, <0 / >1 never.
bool try_s2s_mfma(const S2SArgs& a, int dtype, hipStream_t st, int& rc);
// float32 values of workspace with which a plain bf16 / fp16 product of these sizes can split the contraction of
// its experts' last, sparsely filled tiles (0: the product would not use one)
int64_t s2s_workspace_floats(int64_t L, int64_t K, int64_t N, int E, int dtype);
bool try_s2s_f32(const S2SArgs& a, hipStream_t st, int& rc);     // float32 MFMA paths (csrc/gemm_f32.hip)
bool try_xty_f32(const XtYArgs& a, hipStream_t st, int& rc);
bool try_s2s_rowdot(const S2SArgs& a, int dtype, hipStream_t st, int& rc);   // few-row launches; after try_s2s_mfma's checks
bool try_xty_mfma(const XtYArgs& a, int dtype, hipStream_t st, int& rc);

int launch_combine(const void* Y, int64_t sy, const void* G, int64_t sgt, int64_t sgk, void* O, int64_t so,
                   int64_t Tn, int k, int N, int dtype, hipStream_t st);
int launch_gate_grad(const void* Y, int64_t sy, const void* D, int64_t sd, void* DG, int64_t sgt, int64_t sgk,
                     int64_t Tn, int k, int N, int dtype, hipStream_t st);
int launch_glu_fwd(const void* pre, int64_t sp, void* h, int64_t sh, int64_t rows, int f, int act, int dtype,
                   hipStream_t st);
int launch_glu_bwd(const void* pre, int64_t sp, const void* dh, int64_t sdh, void* dpre, int64_t sdp, int64_t rows,
                   int f, int act, int dtype, hipStream_t st);

int launch_oss_glu_fwd(const void* pre, int64_t sp, void* h, int64_t sh, int64_t rows, int f, float alpha, float limit,
                       int dtype, hipStream_t st);
int launch_oss_glu_bwd(const void* pre, int64_t sp, const void* dh, int64_t sdh, void* dpre, int64_t sdp, int64_t rows,
                       int f, float alpha, float limit, int dtype, hipStream_t st);
int launch_topk_softmax(const void* logits, int64_t slt, int64_t sle, float* w, int64_t swt, int64_t swk,
                        int64_t* idx, int64_t sit, int64_t sik, int64_t Tn, int E, int k, int renorm, int dtype,
                        hipStream_t st);
int launch_route(const void* expert_idxs, int idx_dtype, int64_t L, int E, int64_t* eid_out,
                 int64_t* idx_out, int64_t* off_out, void* ws, hipStream_t st);
size_t route_workspace_bytes(int64_t L, int E);
int launch_route_static(const void* expert_idxs, int idx_dtype, int64_t L, int E, int64_t* eid_out,
                        int64_t* idx_out, int64_t* off_out, hipStream_t st);
int route_static_init();
int launch_offsets_from_sorted(const int64_t* eid, int64_t L, int E, int64_t* off, hipStream_t st);
int launch_group_by_source(const GroupArgs& a, int* inv, int dtype, hipStream_t st);
int launch_invert_index(const int64_t* idx, int64_t L, int* inv, hipStream_t st);   // inv[idx[r]] = r
// gate gradient and the scaled, expert-sorted copy of the output gradient in one pass (csrc/fused.hip);
// SMOE_ERR_UNSUPPORTED when rows are not 16-byte pieces
int launch_gate_grad_group(const void* Y, int64_t sy, const void* D, int64_t sd, const void* G, int64_t sgt, int64_t sgk,
                           const int64_t* idx, int* inv, void* DY, int64_t sdy, void* DG, int64_t sdgt, int64_t sdgk,
                           int64_t Tn, int k, int N, int dtype, hipStream_t st);

}  // namespace smoe
