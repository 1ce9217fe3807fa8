// groupXtY, layout-agnostic path: DW[e] = X[rows(e)]^T DY[rows(e)], Db[e] = sum DY[rows(e)].
// Counterpart of _groupXtY / _xty_and_bias (scattermoe/kernels/ops.py:242-366).
// One block owns a 64(k) x 64(n) tile of one expert and walks that expert's rows in order, so the
// summation order is fixed; empty experts get explicit zeros (the reference pre-fills with torch.zeros).
#include "common.hpp"

namespace smoe {

static constexpr int XK = 64, XN = 64, XR = 16, XT = 256;

template <typename T>
__global__ __launch_bounds__(XT) void xty_generic_kernel(XtYArgs a, int k_tiles, int n_tiles) {
  __shared__ float sX[XR][XK + 4];
  __shared__ float sDY[XR][XN + 4];
  int b = blockIdx.x;
  const int n_tile = b % n_tiles; b /= n_tiles;
  const int k_tile = b % k_tiles; b /= k_tiles;
  const int e = b;
  const int r_lo = e ? (int)a.off[e - 1] : 0;
  const int r_hi = (int)a.off[e];
  const T* __restrict__ X = (const T*)a.X;
  const T* __restrict__ DY = (const T*)a.DY;
  T* __restrict__ DW = (T*)a.DW + (int64_t)e * a.sdwe;
  const int tid = threadIdx.x;
  const int k0 = k_tile * XK, n0 = n_tile * XN;
  const int ty = tid / 16, tx = tid % 16;   // thread owns k rows ty*4.., n cols tx*4..
  float acc[4][4] = {};
  float db = 0.0f;                          // thread tid < XN sums column n0 + tid
  const bool want_db = a.Db != nullptr && k_tile == 0;

  for (int r0 = r_lo; r0 < r_hi; r0 += XR) {
#pragma unroll
    for (int i = 0; i < (XR * XK) / XT; ++i) {
      const int lin = tid + i * XT;
      const int kk = lin % XK, rr = lin / XK;
      const int r = r0 + rr, k = k0 + kk;
      sX[rr][kk] = (r < r_hi && k < a.K) ? to_f32(X[(int64_t)r * a.sxm + (int64_t)k * a.sxk]) : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < (XR * XN) / XT; ++i) {
      const int lin = tid + i * XT;
      const int nn = lin % XN, rr = lin / XN;
      const int r = r0 + rr, n = n0 + nn;
      sDY[rr][nn] = (r < r_hi && n < a.N) ? to_f32(DY[(int64_t)r * a.sdym + (int64_t)n * a.sdyn]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int rr = 0; rr < XR; ++rr) {
      float xv[4], dv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) xv[i] = sX[rr][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) dv[j] = sDY[rr][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(xv[i], dv[j], acc[i][j]);
    }
    if (want_db && tid < XN) {
#pragma unroll
      for (int rr = 0; rr < XR; ++rr) db += sDY[rr][tid];
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = k0 + ty * 4 + i;
    if (k >= a.K) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < a.N) DW[(int64_t)k * a.sdwk + (int64_t)n * a.sdwn] = from_f32<T>(acc[i][j]);
    }
  }
  if (want_db && tid < XN && n0 + tid < a.N)
    ((T*)a.Db)[(int64_t)e * a.sdbe + (int64_t)(n0 + tid) * a.sdbn] = from_f32<T>(db);
}

template <typename T>
static int launch_t(const XtYArgs& a, hipStream_t st) {
  const int k_tiles = (a.K + XK - 1) / XK, n_tiles = (a.N + XN - 1) / XN;
  const int64_t grid = (int64_t)a.E * k_tiles * n_tiles;
  if (grid == 0) return 0;
  if (grid > 0x7fffffffLL) { set_error("smoe_groupXtY: grid too large"); return SMOE_ERR_RANGE; }
  hipLaunchKernelGGL(xty_generic_kernel<T>, dim3((unsigned)grid), dim3(XT), 0, st, a, k_tiles, n_tiles);
  return launch_status("xty_generic_kernel");
}

int launch_xty_generic(const XtYArgs& a, int dtype, hipStream_t st) {
  switch (dtype) {
    case SMOE_F32: return launch_t<float>(a, st);
    case SMOE_BF16: return launch_t<bf16_t>(a, st);
    case SMOE_F16: return launch_t<f16_t>(a, st);
    default: set_error("smoe_groupXtY: unknown dtype %d", dtype); return SMOE_ERR_DTYPE;
  }
}

}  // namespace smoe
