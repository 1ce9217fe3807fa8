// HBM-bound passes around the expert GEMMs, each one read + one write instead of a library bmm or a
// chain of elementwise launches:
//   combine    out[t,:]  = sum_j gates[t,j] * Y[t*k+j,:]        (reference: parallel_experts.py:44-46, a bmm;
//                                                                 without gates: the `.sum(-2)` of :120-123)
//   gate_grad  dg[t,j]   = <Y[t*k+j,:], dOut[t,:]>              (reference: parallel_experts.py:79, a bmm)
//   glu_fwd    h         = act(pre[:, f:]) * pre[:, :f]          (reference: mlp.py:81-87, chunk + act + mul)
//   glu_bwd    dpre      = [dh * act(g), dh * lin * act'(g)]     (autograd of the same expression)
// All arithmetic in fp32, one rounding to the tensor dtype on store.
#include "common.hpp"

namespace smoe {

template <typename T> struct Pack { static constexpr int n = 16 / sizeof(T); T v[16 / sizeof(T)]; };

// 16-byte accesses with the non-temporal hint, for data a pass touches exactly once (it should not displace what
// the neighbouring GEMM launches keep in the caches)
typedef int nt_i32x4 __attribute__((ext_vector_type(4)));
template <typename P>
__device__ __forceinline__ P stream_load16(const void* p) {
  static_assert(sizeof(P) == 16, "16-byte packs only");
  return __builtin_bit_cast(P, __builtin_nontemporal_load((const nt_i32x4*)p));
}
template <typename P>
__device__ __forceinline__ void stream_store16(void* p, const P& x) {
  static_assert(sizeof(P) == 16, "16-byte packs only");
  __builtin_nontemporal_store(__builtin_bit_cast(nt_i32x4, x), (nt_i32x4*)p);
}

// ---- combine -------------------------------------------------------------------------------------------
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void combine_kernel(const T* __restrict__ Y, int64_t sy, const T* __restrict__ G,
                                                     int64_t sgt, int64_t sgk, T* __restrict__ O, int64_t so,
                                                     int k, int N) {
  const int64_t t = blockIdx.x;
  const T* y0 = Y + t * k * sy;
  if (VEC) {
    typedef Pack<T> P;
    for (int c = threadIdx.x; c < N / P::n; c += 256) {
      float acc[P::n];
#pragma unroll
      for (int q = 0; q < P::n; ++q) acc[q] = 0.0f;
      // four slots' loads in flight at a time; the sum runs over the slots in order either way
      int j = 0;
      for (; j + 4 <= k; j += 4) {
        P x[4];
        float g[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          x[u] = stream_load16<P>(y0 + (j + u) * sy + (int64_t)c * P::n);
          g[u] = G ? to_f32(G[t * sgt + (j + u) * sgk]) : 1.0f;       // no gates: plain sum over the k slots
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int q = 0; q < P::n; ++q) acc[q] = fmaf(g[u], to_f32(x[u].v[q]), acc[q]);
      }
      if (j + 2 <= k) {
        const P x0 = stream_load16<P>(y0 + j * sy + (int64_t)c * P::n);
        const P x1 = stream_load16<P>(y0 + (j + 1) * sy + (int64_t)c * P::n);
        const float g0 = G ? to_f32(G[t * sgt + j * sgk]) : 1.0f, g1 = G ? to_f32(G[t * sgt + (j + 1) * sgk]) : 1.0f;
#pragma unroll
        for (int q = 0; q < P::n; ++q) acc[q] = fmaf(g0, to_f32(x0.v[q]), acc[q]);
#pragma unroll
        for (int q = 0; q < P::n; ++q) acc[q] = fmaf(g1, to_f32(x1.v[q]), acc[q]);
        j += 2;
      }
      if (j < k) {
        const float g = G ? to_f32(G[t * sgt + j * sgk]) : 1.0f;
        const P x = stream_load16<P>(y0 + j * sy + (int64_t)c * P::n);
#pragma unroll
        for (int q = 0; q < P::n; ++q) acc[q] = fmaf(g, to_f32(x.v[q]), acc[q]);
      }
      P o;
#pragma unroll
      for (int q = 0; q < P::n; ++q) o.v[q] = from_f32<T>(acc[q]);
      *(P*)(O + t * so + (int64_t)c * P::n) = o;
    }
  } else {
    for (int n = threadIdx.x; n < N; n += 256) {
      float acc = 0.0f;
      for (int j = 0; j < k; ++j) acc = fmaf(G ? to_f32(G[t * sgt + j * sgk]) : 1.0f, to_f32(y0[j * sy + n]), acc);
      O[t * so + n] = from_f32<T>(acc);
    }
  }
}

// ---- gate gradient --------------------------------------------------------------------------------------
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void gate_grad_kernel(const T* __restrict__ Y, int64_t sy, const T* __restrict__ D,
                                                       int64_t sd, T* __restrict__ DG, int64_t sgt, int64_t sgk,
                                                       int k, int N) {
  __shared__ float part[4];
  const int64_t t = blockIdx.x;
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  for (int j = 0; j < k; ++j) {
    const T* y = Y + (t * k + j) * sy;
    const T* d = D + t * sd;
    float acc = 0.0f;
    if (VEC) {
      typedef Pack<T> P;
      for (int c = threadIdx.x; c < N / P::n; c += 256) {
        const P a = stream_load16<P>(y + (int64_t)c * P::n);
        const P b = *(const P*)(d + (int64_t)c * P::n);
#pragma unroll
        for (int q = 0; q < P::n; ++q) acc = fmaf(to_f32(a.v[q]), to_f32(b.v[q]), acc);
      }
    } else {
      for (int n = threadIdx.x; n < N; n += 256) acc = fmaf(to_f32(y[n]), to_f32(d[n]), acc);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (lane == 0) part[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) DG[t * sgt + j * sgk] = from_f32<T>((part[0] + part[1]) + (part[2] + part[3]));
    __syncthreads();
  }
}

// ---- gate gradient + scaled gather of the output gradient, one pass ------------------------------------
// The backward pass of a gate-weighted expert layer walks the (L, N) expert outputs for the gate gradient and
// writes an (L, N) matrix of scaled output-gradient rows in expert-sorted order (reference parallel_experts.py:
// 76-93: a bmm, then group with coefficients).  Here one wave owns one (token, slot) row s = t * k + j: it reads
// dOut[t] (its k readers run side by side, so the memory side sees it once) and Y[s], adds up their dot product,
// and writes dOut[t] * gates[t, j] to row inv[s] of dY - which therefore is a buffer of its own: row s of Y may
// still be unread when some other wave's row of dY lands on it.  inv = inverse of the routing permutation
// (launch_invert_index); a row whose inverse entry does not point back at it is not written, as in
// group_by_source.  The product dOut * gate is rounded once, like group's; the dot product is added up in float32
// by one wave in a fixed order.
template <typename T, int P>
__global__ __launch_bounds__(256) void gate_grad_group_kernel(const T* __restrict__ Y, int64_t sy, const T* __restrict__ D,
                                                             int64_t sd, const T* __restrict__ G, int64_t sgt, int64_t sgk,
                                                             const int64_t* __restrict__ idx, const int* __restrict__ inv,
                                                             T* __restrict__ DY, int64_t sdy, T* __restrict__ DG,
                                                             int64_t sdgt, int64_t sdgk, int64_t L, int k, int N) {
  typedef Pack<T> V;
  const int lane = lane_id(), wave = threadIdx.x >> 6;
  const int nv = N / V::n;
  for (int64_t s = (int64_t)blockIdx.x * 4 + wave; s < L; s += (int64_t)gridDim.x * 4) {
    const int64_t t = s / k;
    const int j = (int)(s - t * k);
    const int q = inv[s];
    const bool mine = (unsigned)q < (uint64_t)L && idx[q] == s;
    const float c = to_f32(G[t * sgt + j * sgk]);
    const T* __restrict__ y = Y + s * sy;
    const T* __restrict__ d = D + t * sd;
    T* __restrict__ o = DY + (int64_t)(mine ? q : 0) * sdy;
    float acc = 0.0f;
    for (int j0 = 0; j0 < nv; j0 += 64 * P) {
      V a[P], b[P];
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const int c16 = j0 + p * 64 + lane;
        if (c16 < nv) {
          a[p] = stream_load16<V>(y + (int64_t)c16 * V::n);
          b[p] = *(const V*)(d + (int64_t)c16 * V::n);
        }
      }
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const int c16 = j0 + p * 64 + lane;
        if (c16 >= nv) continue;
        V w;
#pragma unroll
        for (int e = 0; e < V::n; ++e) {
          const float dv = to_f32(b[p].v[e]);
          acc = fmaf(to_f32(a[p].v[e]), dv, acc);
          w.v[e] = from_f32<T>(dv * c);
        }
        if (mine) stream_store16(o + (int64_t)c16 * V::n, w);
      }
    }
#pragma unroll
    for (int sh = 32; sh > 0; sh >>= 1) acc += __shfl_xor(acc, sh, 64);
    if (lane == 0) DG[t * sdgt + j * sdgk] = from_f32<T>(acc);
  }
}

// ---- gated linear unit -----------------------------------------------------------------------------------
// sigmoidf_, act_f, act_df: common.hpp

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void glu_fwd_kernel(const T* __restrict__ pre, int64_t sp, T* __restrict__ h,
                                                     int64_t sh, int64_t rows, int f, int act) {
  constexpr int W = VEC ? Pack<T>::n : 1;
  const int64_t per_row = f / W;
  const int64_t total = rows * per_row;
  const bool gf = (act & 1) != 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / per_row, c = (i % per_row) * W;
    if (VEC) {
      typedef Pack<T> P;
      const P lin = stream_load16<P>(pre + r * sp + (gf ? f : 0) + c);
      const P gat = stream_load16<P>(pre + r * sp + (gf ? 0 : f) + c);
      P o;
#pragma unroll
      for (int q = 0; q < P::n; ++q) o.v[q] = from_f32<T>(glu_h(act, to_f32(gat.v[q]), to_f32(lin.v[q])));
      stream_store16(h + r * sh + c, o);
    } else {
      h[r * sh + c] = from_f32<T>(glu_h(act, to_f32(pre[r * sp + (gf ? 0 : f) + c]), to_f32(pre[r * sp + (gf ? f : 0) + c])));
    }
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void glu_bwd_kernel(const T* __restrict__ pre, int64_t sp, const T* __restrict__ dh,
                                                     int64_t sdh, T* __restrict__ dpre, int64_t sdp, int64_t rows,
                                                     int f, int act) {
  constexpr int W = VEC ? Pack<T>::n : 1;
  const int64_t per_row = f / W;
  const int64_t total = rows * per_row;
  const bool gf = (act & 1) != 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / per_row, c = (i % per_row) * W;
    if (VEC) {
      typedef Pack<T> P;
      const P lin = stream_load16<P>(pre + r * sp + (gf ? f : 0) + c);
      const P gat = stream_load16<P>(pre + r * sp + (gf ? 0 : f) + c);
      const P d = stream_load16<P>(dh + r * sdh + c);
      P ol, og;
#pragma unroll
      for (int q = 0; q < P::n; ++q) {
        const float g = to_f32(gat.v[q]), dv = to_f32(d.v[q]);
        ol.v[q] = from_f32<T>(glu_dlin(act, dv, g));
        og.v[q] = from_f32<T>(glu_dgat(act, dv, g, to_f32(lin.v[q])));
      }
      stream_store16(dpre + r * sdp + (gf ? f : 0) + c, ol);
      stream_store16(dpre + r * sdp + (gf ? 0 : f) + c, og);
    } else {
      const float g = to_f32(pre[r * sp + (gf ? 0 : f) + c]), dv = to_f32(dh[r * sdh + c]);
      dpre[r * sdp + (gf ? f : 0) + c] = from_f32<T>(glu_dlin(act, dv, g));
      dpre[r * sdp + (gf ? 0 : f) + c] = from_f32<T>(glu_dgat(act, dv, g, to_f32(pre[r * sp + (gf ? f : 0) + c])));
    }
  }
}

// ---- gpt-oss gated unit ------------------------------------------------------------------------------------
// pre (rows, 2f) holds (gate, up) pairs in adjacent columns:
//   g = min(gate, limit); u = clamp(up, -limit, limit); h = (u + 1) * g * sigmoid(alpha * g)
// (scattermoe/utils/replace_moe.py:39-43).  One pass each way; clamped inputs pass no gradient, as with torch.clamp
// (the bounds themselves still do).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void oss_glu_fwd_kernel(const T* __restrict__ pre, int64_t sp, T* __restrict__ h,
                                                         int64_t sh, int64_t rows, int f, float alpha, float limit) {
  constexpr int W = VEC ? Pack<T>::n / 2 : 1;            // hidden columns per thread and step
  const int64_t per_row = f / W, total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / per_row, c = (i % per_row) * W;
    if (VEC) {
      struct Half { T v[W]; };
      const Pack<T> p = stream_load16<Pack<T>>(pre + r * sp + 2 * c);
      Half o;
#pragma unroll
      for (int q = 0; q < W; ++q) o.v[q] = from_f32<T>(oss_h(to_f32(p.v[2 * q]), to_f32(p.v[2 * q + 1]), alpha, limit));
      *(Half*)(h + r * sh + c) = o;
    } else {
      h[r * sh + c] = from_f32<T>(oss_h(to_f32(pre[r * sp + 2 * c]), to_f32(pre[r * sp + 2 * c + 1]), alpha, limit));
    }
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void oss_glu_bwd_kernel(const T* __restrict__ pre, int64_t sp, const T* __restrict__ dh,
                                                         int64_t sdh, T* __restrict__ dpre, int64_t sdp, int64_t rows,
                                                         int f, float alpha, float limit) {
  constexpr int W = VEC ? Pack<T>::n / 2 : 1;
  const int64_t per_row = f / W, total = rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / per_row, c = (i % per_row) * W;
    if (VEC) {
      struct Half { T v[W]; };
      const Pack<T> p = stream_load16<Pack<T>>(pre + r * sp + 2 * c);
      const Half d = *(const Half*)(dh + r * sdh + c);
      Pack<T> o;
#pragma unroll
      for (int q = 0; q < W; ++q) {
        float dg, du;
        oss_grad(to_f32(p.v[2 * q]), to_f32(p.v[2 * q + 1]), to_f32(d.v[q]), alpha, limit, dg, du);
        o.v[2 * q] = from_f32<T>(dg);
        o.v[2 * q + 1] = from_f32<T>(du);
      }
      stream_store16(dpre + r * sdp + 2 * c, o);
    } else {
      float dg, du;
      oss_grad(to_f32(pre[r * sp + 2 * c]), to_f32(pre[r * sp + 2 * c + 1]), to_f32(dh[r * sdh + c]), alpha, limit, dg, du);
      dpre[r * sdp + 2 * c] = from_f32<T>(dg);
      dpre[r * sdp + 2 * c + 1] = from_f32<T>(du);
    }
  }
}

static bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }
static unsigned ew_grid(int64_t total) {
  int64_t b = cdiv64(total, 256);
  return (unsigned)(b > 256 * 32 ? 256 * 32 : (b < 1 ? 1 : b));
}

template <typename T>
static int combine_t(const void* Y, int64_t sy, const void* G, int64_t sgt, int64_t sgk, void* O, int64_t so,
                     int64_t Tn, int k, int N, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = N % vn == 0 && sy % vn == 0 && so % vn == 0 && al16(Y) && al16(O);
  if (vec) hipLaunchKernelGGL((combine_kernel<T, true>), dim3((unsigned)Tn), dim3(256), 0, st, (const T*)Y, sy, (const T*)G, sgt, sgk, (T*)O, so, k, N);
  else hipLaunchKernelGGL((combine_kernel<T, false>), dim3((unsigned)Tn), dim3(256), 0, st, (const T*)Y, sy, (const T*)G, sgt, sgk, (T*)O, so, k, N);
  return launch_status("combine_kernel");
}

template <typename T>
static int gate_grad_t(const void* Y, int64_t sy, const void* D, int64_t sd, void* DG, int64_t sgt, int64_t sgk,
                       int64_t Tn, int k, int N, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = N % vn == 0 && sy % vn == 0 && sd % vn == 0 && al16(Y) && al16(D);
  if (vec) hipLaunchKernelGGL((gate_grad_kernel<T, true>), dim3((unsigned)Tn), dim3(256), 0, st, (const T*)Y, sy, (const T*)D, sd, (T*)DG, sgt, sgk, k, N);
  else hipLaunchKernelGGL((gate_grad_kernel<T, false>), dim3((unsigned)Tn), dim3(256), 0, st, (const T*)Y, sy, (const T*)D, sd, (T*)DG, sgt, sgk, k, N);
  return launch_status("gate_grad_kernel");
}

template <typename T>
static int glu_fwd_t(const void* pre, int64_t sp, void* h, int64_t sh, int64_t rows, int f, int act, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = f % vn == 0 && sp % vn == 0 && sh % vn == 0 && al16(pre) && al16(h);
  const int64_t total = rows * (f / (vec ? vn : 1));
  if (vec) hipLaunchKernelGGL((glu_fwd_kernel<T, true>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (T*)h, sh, rows, f, act);
  else hipLaunchKernelGGL((glu_fwd_kernel<T, false>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (T*)h, sh, rows, f, act);
  return launch_status("glu_fwd_kernel");
}

template <typename T>
static int glu_bwd_t(const void* pre, int64_t sp, const void* dh, int64_t sdh, void* dpre, int64_t sdp, int64_t rows,
                     int f, int act, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = f % vn == 0 && sp % vn == 0 && sdh % vn == 0 && sdp % vn == 0 && al16(pre) && al16(dh) && al16(dpre);
  const int64_t total = rows * (f / (vec ? vn : 1));
  if (vec) hipLaunchKernelGGL((glu_bwd_kernel<T, true>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (const T*)dh, sdh, (T*)dpre, sdp, rows, f, act);
  else hipLaunchKernelGGL((glu_bwd_kernel<T, false>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (const T*)dh, sdh, (T*)dpre, sdp, rows, f, act);
  return launch_status("glu_bwd_kernel");
}

template <typename T>
static int gate_grad_group_t(const void* Y, int64_t sy, const void* D, int64_t sd, const void* G, int64_t sgt, int64_t sgk,
                             const int64_t* idx, int* inv, void* DY, int64_t sdy, void* DG, int64_t sdgt, int64_t sdgk,
                             int64_t Tn, int k, int N, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = N % vn == 0 && sy % vn == 0 && sd % vn == 0 && sdy % vn == 0 && al16(Y) && al16(D) && al16(DY);
  const int64_t L = Tn * k;
  if (!vec || L > 0x7fffffffLL) return SMOE_ERR_UNSUPPORTED;
  if (const int rc = launch_invert_index(idx, L, inv, st)) return rc;
  int64_t blocks = cdiv64(L, 4);
  if (blocks > 256 * 64) blocks = 256 * 64;
  hipLaunchKernelGGL((gate_grad_group_kernel<T, 4>), dim3((unsigned)blocks), dim3(256), 0, st, (const T*)Y, sy, (const T*)D, sd,
                     (const T*)G, sgt, sgk, idx, (const int*)inv, (T*)DY, sdy, (T*)DG, sdgt, sdgk, L, k, N);
  return launch_status("gate_grad_group_kernel");
}

#define SMOE_DISPATCH(dtype, CALL)                                              \
  switch (dtype) {                                                              \
    case SMOE_F32: { typedef float T; return CALL; }                            \
    case SMOE_BF16: { typedef bf16_t T; return CALL; }                          \
    case SMOE_F16: { typedef f16_t T; return CALL; }                            \
    default: set_error("unknown dtype %d", dtype); return SMOE_ERR_DTYPE;       \
  }

int launch_combine(const void* Y, int64_t sy, const void* G, int64_t sgt, int64_t sgk, void* O, int64_t so,
                   int64_t Tn, int k, int N, int dtype, hipStream_t st) {
  SMOE_DISPATCH(dtype, combine_t<T>(Y, sy, G, sgt, sgk, O, so, Tn, k, N, st));
}
int launch_gate_grad(const void* Y, int64_t sy, const void* D, int64_t sd, void* DG, int64_t sgt, int64_t sgk,
                     int64_t Tn, int k, int N, int dtype, hipStream_t st) {
  SMOE_DISPATCH(dtype, gate_grad_t<T>(Y, sy, D, sd, DG, sgt, sgk, Tn, k, N, st));
}
int launch_gate_grad_group(const void* Y, int64_t sy, const void* D, int64_t sd, const void* G, int64_t sgt, int64_t sgk,
                           const int64_t* idx, int* inv, void* DY, int64_t sdy, void* DG, int64_t sdgt, int64_t sdgk,
                           int64_t Tn, int k, int N, int dtype, hipStream_t st) {
  SMOE_DISPATCH(dtype, gate_grad_group_t<T>(Y, sy, D, sd, G, sgt, sgk, idx, inv, DY, sdy, DG, sdgt, sdgk, Tn, k, N, st));
}
int launch_glu_fwd(const void* pre, int64_t sp, void* h, int64_t sh, int64_t rows, int f, int act, int dtype, hipStream_t st) {
  SMOE_DISPATCH(dtype, glu_fwd_t<T>(pre, sp, h, sh, rows, f, act, st));
}
int launch_glu_bwd(const void* pre, int64_t sp, const void* dh, int64_t sdh, void* dpre, int64_t sdp, int64_t rows,
                   int f, int act, int dtype, hipStream_t st) {
  SMOE_DISPATCH(dtype, glu_bwd_t<T>(pre, sp, dh, sdh, dpre, sdp, rows, f, act, st));
}

template <typename T>
static int oss_glu_fwd_t(const void* pre, int64_t sp, void* h, int64_t sh, int64_t rows, int f, float alpha,
                         float limit, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = f % (vn / 2) == 0 && sp % vn == 0 && sh % (vn / 2) == 0 && al16(pre) && ((uintptr_t)h & 7) == 0;
  const int64_t total = rows * (f / (vec ? vn / 2 : 1));
  if (vec) hipLaunchKernelGGL((oss_glu_fwd_kernel<T, true>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (T*)h, sh, rows, f, alpha, limit);
  else hipLaunchKernelGGL((oss_glu_fwd_kernel<T, false>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (T*)h, sh, rows, f, alpha, limit);
  return launch_status("oss_glu_fwd_kernel");
}

template <typename T>
static int oss_glu_bwd_t(const void* pre, int64_t sp, const void* dh, int64_t sdh, void* dpre, int64_t sdp, int64_t rows,
                         int f, float alpha, float limit, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = f % (vn / 2) == 0 && sp % vn == 0 && sdp % vn == 0 && sdh % (vn / 2) == 0 && al16(pre) && al16(dpre) &&
                   ((uintptr_t)dh & 7) == 0;
  const int64_t total = rows * (f / (vec ? vn / 2 : 1));
  if (vec) hipLaunchKernelGGL((oss_glu_bwd_kernel<T, true>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (const T*)dh, sdh, (T*)dpre, sdp, rows, f, alpha, limit);
  else hipLaunchKernelGGL((oss_glu_bwd_kernel<T, false>), dim3(ew_grid(total)), dim3(256), 0, st, (const T*)pre, sp, (const T*)dh, sdh, (T*)dpre, sdp, rows, f, alpha, limit);
  return launch_status("oss_glu_bwd_kernel");
}

int launch_oss_glu_fwd(const void* pre, int64_t sp, void* h, int64_t sh, int64_t rows, int f, float alpha, float limit,
                       int dtype, hipStream_t st) {
  SMOE_DISPATCH(dtype, oss_glu_fwd_t<T>(pre, sp, h, sh, rows, f, alpha, limit, st));
}
int launch_oss_glu_bwd(const void* pre, int64_t sp, const void* dh, int64_t sdh, void* dpre, int64_t sdp, int64_t rows,
                       int f, float alpha, float limit, int dtype, hipStream_t st) {
  SMOE_DISPATCH(dtype, oss_glu_bwd_t<T>(pre, sp, dh, sdh, dpre, sdp, rows, f, alpha, limit, st));
}

}  // namespace smoe
