/*
 * scattermoe_amd — C ABI of the MI355X (gfx950) ScatterMoE hot path.
 *
 * Every entry point is `extern "C"`, takes plain pointers / sizes / element strides, launches
 * asynchronously on the HIP stream it is given, allocates nothing, frees nothing and keeps no
 * pointer after it returns.  Device pointers are passed as `void*`; strides are in ELEMENTS of the
 * tensor's dtype.  Return value: 0 = launched, >0 = the hipError_t of a failed launch,
 * <0 = argument error (SMOE_ERR_*); `smoe_last_error()` gives the text for the calling thread.
 *
 * The reference (shawntan/scattermoe) has no FFI: its Python wrappers launch Triton kernels.  Each
 * function below names the reference wrapper + kernel it replaces.
 *
 * Notation: T tokens, k = top-k, L = T*k rows in expert-sorted order, E experts.
 *   eid[L]  sorted_expert_idxs      (int64, ascending)
 *   idx[L]  sorted_scattered_idxs   (int64, permutation of 0..L-1; token = idx / k)
 *   off[E]  expert_offsets          (int64, inclusive prefix sum of per-expert row counts)
 */
#ifndef SCATTERMOE_AMD_H
#define SCATTERMOE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SMOE_ABI_VERSION 1

/* element types of floating-point tensors */
enum { SMOE_F32 = 0, SMOE_BF16 = 1, SMOE_F16 = 2 };
/* element types of the unsorted expert-index tensor handed to smoe_route */
enum { SMOE_I64 = 0, SMOE_I32 = 1, SMOE_I16 = 2, SMOE_U8 = 3 };

/* activations of the gated linear unit kernels */
/* SILU: h = silu(pre[:, f:2f]) * pre[:, 0:f];  SILU_GATE_FIRST: h = silu(pre[:, 0:f]) * pre[:, f:2f] */
enum { SMOE_ACT_SILU = 0, SMOE_ACT_SILU_GATE_FIRST = 1 };

/* argument errors */
enum {
  SMOE_ERR_NULL = -1,      /* a required pointer is NULL */
  SMOE_ERR_SHAPE = -2,     /* negative / inconsistent sizes */
  SMOE_ERR_DTYPE = -3,     /* unknown dtype enum */
  SMOE_ERR_WORKSPACE = -4, /* workspace too small */
  SMOE_ERR_RANGE = -5,     /* size beyond what the kernels index with (int32 rows, E limit) */
  SMOE_ERR_UNSUPPORTED = -6 /* the fused entry point has no kernel for this dtype / layout / shape; nothing was
                              launched and the caller runs the unfused sequence instead */
};

/* ABI version of the loaded library (== SMOE_ABI_VERSION it was built with). */
int smoe_version(void);

/* Hex digest of the sources (csrc/ and include/) the library was compiled from, or "unknown".  The Python loader
 * compares it with the sources beside it and refuses a library that was built from different ones.  No counterpart
 * in the reference (its kernels are compiled by Triton at run time). */
const char* smoe_source_hash(void);

/* Text of the last error raised on the calling thread ("" if none). Never NULL. */
const char* smoe_last_error(void);

/*
 * Routing prep: stable counting sort of the flattened expert ids + inclusive per-expert offsets.
 * Replaces scattermoe/parallel_experts.py:14-21 (flatten_sort_count: torch.sort + bincount + cumsum,
 * with the custom op scattermoe::bincount :6-12).  Tie order is the stable one (ascending flat slot
 * inside an expert segment), i.e. torch.sort(flat, stable=True).
 *   expert_idxs  L unsorted ids in [0,E), contiguous, dtype `idx_dtype` (SMOE_I64 ...)
 *   eid_out/idx_out  L int64 each;  off_out  E int64
 *   workspace    device scratch of at least smoe_route_workspace_bytes(L,E) bytes (may be NULL iff that is 0)
 * Ids outside [0,E) are undefined behaviour in the reference; here such rows are dropped from the
 * histogram and the outputs are unspecified (no out-of-bounds access happens).
 */
size_t smoe_route_workspace_bytes(int64_t L, int E);
int smoe_route(const void* expert_idxs, int idx_dtype, int64_t L, int E,
               int64_t* eid_out, int64_t* idx_out, int64_t* off_out,
               void* workspace, size_t workspace_bytes, void* stream);

/*
 * smoe_route for callers that cannot allocate: the same routing prep, same arguments and same results, but with
 * no workspace argument.  NO COUNTERPART IN THE REFERENCE; it exists for callers that can neither call hipMalloc
 * nor bring a workspace: code under HIP stream / graph capture, tight serving loops, harnesses that forbid
 * allocation.  The per-chunk histograms that smoe_route keeps in the caller's workspace live in a fixed
 * SMOE_ROUTE_STATIC_BYTES device array inside the library (one copy per GPU, held until the process ends), so the
 * call allocates and frees nothing.  Inputs needing more than that (smoe_route_workspace_bytes(L, E) >
 * SMOE_ROUTE_STATIC_BYTES, i.e. about ceil(L / 4096) * E > 262144) are rejected with SMOE_ERR_WORKSPACE and nothing
 * is launched.  All calls on one GPU share the array: calls that overlap on one GPU (different streams or
 * threads) race; calls on one stream, or otherwise ordered, are safe, and nothing has to be cleared between them.
 * smoe_route_static_init() resolves the array's address for the CURRENT device (once per device; also done lazily
 * by the first smoe_route_static call on a device, which therefore should not happen under stream capture).
 */
#define SMOE_ROUTE_STATIC_BYTES (1 << 20)
int smoe_route_static_init(void);
int smoe_route_static(const void* expert_idxs, int idx_dtype, int64_t L, int E,
                      int64_t* eid_out, int64_t* idx_out, int64_t* off_out, void* stream);

/*
 * Inclusive expert offsets from an already sorted id vector (off[e] = #{n : eid[n] <= e}).
 * The reference's scatter2scatter (scattermoe/kernels/ops.py:120-137) receives only eid/idx and
 * re-derives expert boundaries per 128-row block (ops.py:85-91); this library schedules
 * expert-aligned tiles from `off`, so callers that hold no offsets build them with this call.
 */
int smoe_offsets_from_sorted(const int64_t* eid, int64_t L, int E, int64_t* off_out, void* stream);

/*
 * Fused gather -> grouped GEMM (+bias) -> scatter.
 * Replaces scattermoe/kernels/ops.py:120-183 (scatter2scatter / op scattermoe::scatter2scatter)
 * and its Triton kernel ops.py:11-42, 50-118.
 *   for n in [0,L): e = eid[n]; src = x_grouped ? n : idx[n] / fan_out; dst = y_grouped ? n : idx[n]
 *                   Y[dst, :] = X[src, :] @ W[e] (+ b[e]);  fp32 accumulation, stored in `dtype`
 *   X (L/fan_out or L rows, K)  strides sxm,sxk     W (E,K,N) strides swe,swk,swn (any layout)
 *   b (E,N) or NULL  strides sbe,sbn                Y (L,N) strides sym,syn
 * `off` (E int64) is required.  X, W, b, Y share `dtype`.
 */
int smoe_scatter2scatter(const void* X, int64_t sxm, int64_t sxk,
                         const void* W, int64_t swe, int64_t swk, int64_t swn,
                         const void* b, int64_t sbe, int64_t sbn,
                         void* Y, int64_t sym, int64_t syn,
                         const int64_t* eid, const int64_t* idx, const int64_t* off,
                         int64_t L, int64_t K, int64_t N, int E, int fan_out,
                         int x_grouped, int y_grouped, int dtype, void* stream);

/*
 * smoe_scatter2scatter with a caller workspace (same reference function, scattermoe/kernels/ops.py:120-183; the
 * reference has no such argument).  Every expert ends in a partly filled tile of rows; in a product with many rows
 * per expert, few output columns and a long contraction (Mixtral layer-2 forward and layer-1 input gradient:
 * 8 experts x 16 tile columns) those tiles are too few to fill the chip and each walks the whole contraction.
 * With `workspace` of at least smoe_scatter2scatter_workspace_bytes(L, K, N, E, dtype) bytes (16-byte aligned)
 * their contraction is cut into parts that run side by side; a second small launch adds the float32 partial
 * sums in a fixed order and writes the rows.  Results are the same on every run, and within float32 rounding
 * of - not bit-identical to - the product without workspace (the additions are grouped differently).
 * workspace == NULL, too small or not 16-byte aligned: exactly smoe_scatter2scatter (the workspace is then not
 * touched; no error).  The workspace is free again when the launches
 * of the call have run.  smoe_scatter2scatter_workspace_bytes returns 0 for products that would not use one.
 */
size_t smoe_scatter2scatter_workspace_bytes(int64_t L, int64_t K, int64_t N, int E, int dtype);
int smoe_scatter2scatter_ws(const void* X, int64_t sxm, int64_t sxk,
                            const void* W, int64_t swe, int64_t swk, int64_t swn,
                            const void* b, int64_t sbe, int64_t sbn,
                            void* Y, int64_t sym, int64_t syn,
                            const int64_t* eid, const int64_t* idx, const int64_t* off,
                            int64_t L, int64_t K, int64_t N, int E, int fan_out,
                            int x_grouped, int y_grouped, int dtype,
                            void* workspace, size_t workspace_bytes, void* stream);

/*
 * Row gather into expert-sorted order with optional per-row coefficient.
 * Replaces scattermoe/kernels/ops.py:377-410 (group / op scattermoe::group), kernel ops.py:413-457.
 *   Y[n, :] = A[idx[n] / fan_out, :] * (coeff ? coeff[idx[n]] : 1)      n in [0,L)
 *   A (L/fan_out, K) strides sam,sak;  coeff (L) contiguous or NULL;  Y (L,K) strides sym,syk
 */
int smoe_group(const void* A, int64_t sam, int64_t sak, const void* coeff,
               void* Y, int64_t sym, int64_t syk, const int64_t* idx,
               int64_t L, int64_t K, int fan_out, int dtype, void* stream);

/*
 * smoe_group for an index vector that is a permutation of [0, L), which is what smoe_route produces: the same Y, the
 * same bits, but every row of A is read once instead of fan_out times (the walk goes by source row and writes its
 * fan_out scaled copies through the inverse permutation, which a first launch builds in `inverse_workspace`, L
 * int32 of device memory).  For the `group(grad_out, sorted_scattered_idxs, coeff=gates, fan_out=k)` of
 * ParallelLinear.backward (scattermoe/parallel_experts.py:88-93).  Rows of Y whose index entry is shared with
 * another row or lies outside [0, L) are left unwritten - use smoe_group for such vectors.  Returns
 * SMOE_ERR_UNSUPPORTED (nothing launched) unless rows are contiguous and 16-byte aligned and fan_out <= 64.
 */
int smoe_group_by_source(const void* A, int64_t sam, int64_t sak, const void* coeff, void* Y, int64_t sym,
                         int64_t syk, const int64_t* idx, int32_t* inverse_workspace, int64_t L, int64_t K,
                         int fan_out, int dtype, void* stream);

/*
 * Per-expert weight / bias gradient over contiguous expert-sorted row ranges.
 * Replaces scattermoe/kernels/ops.py:191-239 (group_bwd_W / op scattermoe::groupXtY), kernels
 * ops.py:242-318, 321-366.
 *   rows(e) = [e ? off[e-1] : 0, off[e])
 *   DW[e] (K x N) = sum_{r in rows(e)} X[r,:]^T DY[r,:]       Db[e] (N) = sum_{r in rows(e)} DY[r,:]
 * Unlike the reference, which relies on a torch.zeros pre-fill (ops.py:192-195) for experts without
 * rows (guard at ops.py:279), every element of DW / Db is written here (zeros for empty experts),
 * so the caller may pass uninitialised memory.  fp32 accumulation, fixed summation order.
 *   DY (L,N) strides sdym,sdyn;  X (L,K) strides sxm,sxk;  DW (E,K,N) strides sdwe,sdwk,sdwn;
 *   Db (E,N) strides sdbe,sdbn or NULL.
 */
int smoe_groupXtY(const void* DY, int64_t sdym, int64_t sdyn,
                  const void* X, int64_t sxm, int64_t sxk,
                  void* DW, int64_t sdwe, int64_t sdwk, int64_t sdwn,
                  void* Db, int64_t sdbe, int64_t sdbn,
                  const int64_t* off, int64_t L, int64_t K, int64_t N, int E,
                  int dtype, void* stream);

/*
 * smoe_groupXtY with X given as the (L / fan_out, K) matrix its grouped rows come from: grouped row r of X is
 * X[idx[r] / fan_out].  Replaces the pair `group(x, sorted_scattered_idxs, fan_out=k)` + `group_bwd_W(...)` of
 * ParallelLinear.backward (scattermoe/parallel_experts.py:95-107: the gathered copy of x exists only to feed the
 * weight gradient), saving one write and one read of an (L, K) matrix.  Same results as grouping first.
 * Returns SMOE_ERR_UNSUPPORTED (nothing launched) for float32 or operands the MFMA kernels do not take; the caller
 * then groups X and calls smoe_groupXtY.
 */
int smoe_groupXtY_gathered(const void* DY, int64_t sdym, int64_t sdyn,
                           const void* X, int64_t sxm, int64_t sxk, const int64_t* idx, int fan_out,
                           void* DW, int64_t sdwe, int64_t sdwk, int64_t sdwn,
                           void* Db, int64_t sdbe, int64_t sdbn,
                           const int64_t* off, int64_t L, int64_t K, int64_t N, int E,
                           int dtype, void* stream);

/*
 * Gate-weighted sum of the k expert outputs of each token:  out[t,:] = sum_j gates[t,j] * Y[t*k+j,:].
 * Replaces the batched matmul `gates.unsqueeze(1) @ output_expanded` of ParallelLinear.forward
 * (scattermoe/parallel_experts.py:44-46).  Y (T*k, N) row stride sym (columns contiguous), gates (T,k)
 * strides sgt,sgk, out (T,N) row stride som.  fp32 accumulation in slot order, one rounding.
 * gates == NULL: unit weights, i.e. the plain sum over the k slots of a token, which replaces
 * `d_expanded_input.view(T, k, d).sum(-2)` of ParallelLinear.backward (scattermoe/parallel_experts.py:120-123).
 */
int smoe_combine(const void* Y, int64_t sym, const void* gates, int64_t sgt, int64_t sgk, void* out, int64_t som,
                 int64_t T, int k, int64_t N, int dtype, void* stream);

/*
 * Gradient of the gates:  dgates[t,j] = < Y[t*k+j,:], dOut[t,:] >.
 * Replaces `output_expanded @ grad_out.unsqueeze(-1)` of ParallelLinear.backward
 * (scattermoe/parallel_experts.py:76-82).  Y (T*k, N) row stride sym, dOut (T,N) row stride sdm,
 * dgates (T,k) strides sgt,sgk.
 */
int smoe_gate_grad(const void* Y, int64_t sym, const void* dOut, int64_t sdm, void* dgates, int64_t sgt, int64_t sgk,
                   int64_t T, int k, int64_t N, int dtype, void* stream);

/*
 * smoe_gate_grad and the scaled gather of the output gradient in ONE pass over the expert outputs: the two steps with
 * which the backward of a gate-weighted expert layer begins (scattermoe/parallel_experts.py:76-93:
 * `d_gates = output_expanded @ grad_out` as a bmm, then `group(grad_out, sorted_scattered_idxs, fan_out=k,
 * coeff=gates.flatten(), out=output_expanded)`).
 *   dgates[t, j] = <Y[t*k + j, :], dOut[t, :]>            dY[inv[t*k + j], :] = dOut[t, :] * gates[t, j]
 * with inv the inverse of the permutation idx (built by a first small launch in `inverse_workspace`, L = T*k int32).
 * dOut is read from memory once instead of twice.  Unlike the reference's in-place reuse, dY must NOT overlap Y
 * (row s of Y may still be unread when another row of dY is written).  Y (L,N) rows in slot order, dOut (T,N),
 * gates (T,k) strides sgt,sgk, dY (L,N) in expert-sorted order, dgates (T,k) strides sdgt,sdgk; columns contiguous.
 * A row whose index entry is shared or out of range is left unwritten (use smoe_gate_grad + smoe_group then).
 * Returns SMOE_ERR_UNSUPPORTED (nothing launched) unless rows are whole 16-byte pieces and 16-byte aligned.
 */
int smoe_gate_grad_group(const void* Y, int64_t sym, const void* dOut, int64_t sdm,
                         const void* gates, int64_t sgt, int64_t sgk,
                         const int64_t* idx, int32_t* inverse_workspace,
                         void* dY, int64_t sdym, void* dgates, int64_t sdgt, int64_t sdgk,
                         int64_t T, int k, int64_t N, int dtype, void* stream);

/*
 * Gated linear unit of GLUMLP in one pass:  h = act(pre[:, f:2f]) * pre[:, 0:f]   (first half linear,
 * second half activated), replacing chunk + activation + multiply of scattermoe/mlp.py:81-87, and its
 * gradient  dpre[:, 0:f] = dh * act(g),  dpre[:, f:2f] = dh * lin * act'(g)  that autograd derives from it.
 * SMOE_ACT_SILU_GATE_FIRST swaps the roles of the halves (the `act(gate) * up` convention of Hugging Face experts).
 * pre / dpre (rows, 2f) row strides spm / sdpm, h / dh (rows, f) row strides shm / sdhm; `act` = SMOE_ACT_*.
 */
int smoe_glu_fwd(const void* pre, int64_t spm, void* h, int64_t shm, int64_t rows, int64_t f, int act, int dtype,
                 void* stream);
int smoe_glu_bwd(const void* pre, int64_t spm, const void* dh, int64_t sdhm, void* dpre, int64_t sdpm, int64_t rows,
                 int64_t f, int act, int dtype, void* stream);

/*
 * Layer 1 of GLUMLP and its gated linear unit in one launch (scattermoe/mlp.py:74-87: the
 * `self.experts(..., grouped_out=True)` scatter2scatter followed by chunk / activation / multiply):
 *   pre[n, :] = X[src(n), :] @ W[e(n)] (+ b[e(n)])     (L, 2F), rows in expert-sorted order
 *   H[n, :]   = act(pre[n, F:2F]) * pre[n, 0:F]        (L, F)   (halves swapped for SMOE_ACT_SILU_GATE_FIRST)
 * W (E,K,2F) any of the two contiguous layouts, b (E,2F) or NULL.  PRE may be NULL (inference: the
 * pre-activation is not stored).  H is computed from the pre-activation rounded to `dtype`, i.e. PRE is
 * bit-identical to smoe_scatter2scatter and H equals smoe_glu_fwd of it up to one unit in the last place on
 * rare rounding ties of the exponential.  bf16 / fp16 only; returns
 * SMOE_ERR_UNSUPPORTED (nothing launched) where the matrix-core path does not apply.
 */
int smoe_scatter2scatter_glu(const void* X, int64_t sxm, int64_t sxk,
                             const void* W, int64_t swe, int64_t swk, int64_t swn,
                             const void* b, int64_t sbe, int64_t sbn,
                             void* PRE, int64_t spm, void* H, int64_t shm,
                             const int64_t* eid, const int64_t* idx, const int64_t* off,
                             int64_t L, int64_t K, int64_t F, int E, int fan_out, int x_grouped,
                             int act, int dtype, void* stream);

/*
 * Backward counterpart: the input gradient of layer 2 (scattermoe/parallel_experts.py:108-123, the
 * scatter2scatter on the transposed weights with grouped rows in and out) fused with the gradient of the gated
 * linear unit:   dH = DY @ W[e]  (L, F), never stored;   DPRE (L, 2F) from dH and the saved PRE as smoe_glu_bwd.
 * DY (L,K) grouped rows, W (E,K,F), PRE / DPRE (L,2F) with row strides spm / sdpm.  dH is rounded to `dtype`
 * first, so the result equals smoe_scatter2scatter + smoe_glu_bwd up to one unit in the last place.  Returns SMOE_ERR_UNSUPPORTED where the matrix-core path does not apply.
 */
int smoe_scatter2scatter_glu_bwd(const void* DY, int64_t sdm, int64_t sdk,
                                 const void* W, int64_t swe, int64_t swk, int64_t swn,
                                 const void* PRE, int64_t spm, void* DPRE, int64_t sdpm,
                                 const int64_t* eid, const int64_t* idx, const int64_t* off,
                                 int64_t L, int64_t K, int64_t F, int E, int act, int dtype, void* stream);

/*
 * The same two fusions for the gpt-oss experts (scattermoe/utils/replace_moe.py:31-43 and the layer-2 input
 * gradient of parallel_experts.py:108-123): W holds 2F columns of (gate, up) pairs, PRE (may be NULL in the forward)
 * is (L, 2F) in that interleaved layout, H (L, F); alpha / limit as for smoe_gpt_oss_glu_fwd.  bf16 / fp16 only;
 * SMOE_ERR_UNSUPPORTED where there is no fused kernel (float32, rows that are not 16-byte multiples).
 */
int smoe_scatter2scatter_oss_glu(const void* X, int64_t sxm, int64_t sxk, const void* W, int64_t swe, int64_t swk,
                                 int64_t swn, const void* b, int64_t sbe, int64_t sbn, void* PRE, int64_t spm, void* H,
                                 int64_t shm, const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L,
                                 int64_t K, int64_t F, int E, int fan_out, int x_grouped, float alpha, float limit,
                                 int dtype, void* stream);
int smoe_scatter2scatter_oss_glu_bwd(const void* DY, int64_t sdm, int64_t sdk, const void* W, int64_t swe, int64_t swk,
                                     int64_t swn, const void* PRE, int64_t spm, void* DPRE, int64_t sdpm,
                                     const int64_t* eid, const int64_t* idx, const int64_t* off, int64_t L, int64_t K,
                                     int64_t F, int E, float alpha, float limit, int dtype, void* stream);

/*
 * Gated unit of the gpt-oss experts and its gradient, one pass each (scattermoe/utils/replace_moe.py:39-43, five
 * elementwise torch launches on strided slices there).  pre (rows, 2f), row stride spm, holds (gate, up) pairs in
 * adjacent columns:  g = min(gate, limit), u = clamp(up, -limit, limit), h[n, c] = (u + 1) * g * sigmoid(alpha * g).
 * h / dh (rows, f) row strides shm / sdhm; dpre (rows, 2f) row stride sdpm in the layout of pre.  Clamped inputs
 * receive no gradient (torch.clamp semantics: the bounds themselves still do).
 */
int smoe_gpt_oss_glu_fwd(const void* pre, int64_t spm, void* h, int64_t shm, int64_t rows, int64_t f, float alpha,
                         float limit, int dtype, void* stream);
int smoe_gpt_oss_glu_bwd(const void* pre, int64_t spm, const void* dh, int64_t sdhm, void* dpre, int64_t sdpm,
                         int64_t rows, int64_t f, float alpha, float limit, int dtype, void* stream);

/*
 * Decode step of a gated MLP, forward only: OUT[t] = sum_j gates[t,j] * ( W2[e] glu(W1[e] X[t] + b1[e]) + b2[e] ),
 * e = experts[t,j], for at most 8 (token, slot) rows, in two launches and without a routing triple (every
 * workgroup orders the handful of expert ids itself).  Replaces GLUMLP.forward (scattermoe/mlp.py:74-95: the
 * flatten_sort_count of parallel_experts.py:14-21, two scatter2scatter launches, chunk / activation / multiply,
 * and the gate bmm of parallel_experts.py:38-46) at decode sizes; bit-identical to smoe_route +
 * smoe_scatter2scatter_glu + smoe_scatter2scatter + smoe_combine on the same inputs.
 * X (T,d) row stride sxm; experts (T,k) int64 strides set,sek (ids outside [0,E) drop their row); gates (T,k)
 * strides sgt,sgk; W1 (E,2F,d) strides sw1e,sw1n (d contiguous); W2 (E,d,F) strides sw2e,sw2n (F contiguous);
 * b1 (E,2F) / b2 (E,d) or NULL; H (T*k,F) row stride shm: workspace for the hidden rows; OUT (T,d) row stride som.
 * `act` as for smoe_glu_fwd.  Returns SMOE_ERR_UNSUPPORTED (nothing launched) for float32, more than 8 rows, or
 * operands whose rows are not 16-byte aligned: the caller then issues the general sequence.
 */
int smoe_decode_glu_mlp(const void* X, int64_t sxm, const int64_t* experts, int64_t set, int64_t sek, const void* gates,
                        int64_t sgt, int64_t sgk, const void* W1, int64_t sw1e, int64_t sw1n, const void* b1,
                        int64_t sb1e, int64_t sb1n, const void* W2, int64_t sw2e, int64_t sw2n, const void* b2,
                        int64_t sb2e, int64_t sb2n, void* H, int64_t shm, void* OUT, int64_t som, int64_t T, int k,
                        int64_t d, int64_t F, int E, int act, int dtype, void* stream);

/*
 * Router front end: weights, experts = topk(softmax(logits.float(), -1), k) [; weights /= weights.sum(-1)].
 * Replaces the softmax / topk / renormalise sequence of scattermoe/utils/replace_moe.py:67-71 (the routing of the
 * Hugging Face blocks the reference patches).  logits (T,E) strides slt,sle, dtype `dtype`; weights_out (T,k)
 * float32 strides swt,swk, selected in descending order of probability; idx_out (T,k) int64 strides sit,sik.
 * Among equal probabilities the lowest expert id is selected first.  E <= 512, k <= 64.
 * NOT-A-NUMBER LOGITS, a deliberate divergence from the torch composition: torch.softmax turns a row with one NaN
 * into all NaN and torch.topk ranks NaN above every number, so the reference hands NaN weights (and whatever ids
 * topk picks) to the expert kernels, where out-of-range or repeated ids are undefined behaviour.  Here a NaN logit
 * counts as -inf (its expert gets probability 0 and is picked last), and a row that is all NaN / all -inf gets the
 * uniform distribution: ids are always valid and distinct, weights always finite.  A caller that wants to see a
 * blown-up router must test the logits itself (torch.isfinite) - this entry point does not report it.
 */
int smoe_topk_softmax(const void* logits, int64_t slt, int64_t sle, int64_t T, int E, int k, int renormalize,
                      float* weights_out, int64_t swt, int64_t swk, int64_t* idx_out, int64_t sit, int64_t sik,
                      int dtype, void* stream);


#ifdef __cplusplus
}
#endif
#endif /* SCATTERMOE_AMD_H */
