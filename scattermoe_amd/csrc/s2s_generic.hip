// scatter2scatter, layout-agnostic path: any dtype (fp32 / bf16 / fp16), any strides, any sizes.
// Counterpart of _scatter2scatter (scattermoe/kernels/ops.py:50-118, inner loop :11-42).
// 64x64 output tiles that never straddle experts, fp32 FMA accumulation through LDS tiles.
// This is the fallback for the shapes and layouts the MFMA paths (bf16 / fp16 / fp32) decline.
#include "common.hpp"

namespace smoe {

static constexpr int GBM = 64, GBN = 64, GBK = 16, GT = 256;

template <typename T>
__global__ __launch_bounds__(GT) void s2s_generic_kernel(S2SArgs a, int n_tiles) {
  __shared__ float sA[GBK][GBM + 4];
  __shared__ float sB[GBK][GBN + 4];
  __shared__ int64_t sSrc[GBM];
  __shared__ int64_t sDst[GBM];

  const int m_tile = blockIdx.x / n_tiles;
  const int n_tile = blockIdx.x % n_tiles;
  int e, row0, rows;
  if (!find_tile<GBM>(a.off, a.E, m_tile, e, row0, rows)) return;

  const T* __restrict__ X = (const T*)a.X;
  const T* __restrict__ W = (const T*)a.W + (int64_t)e * a.swe;
  T* __restrict__ Y = (T*)a.Y;
  const int tid = threadIdx.x;
  if (tid < GBM) {
    int64_t src = -1, dst = -1;
    if (tid < rows) {
      const int64_t n = row0 + tid;
      const int64_t i = a.idx[n];
      src = a.x_grouped ? n : i / a.fan_out;
      dst = a.y_grouped ? n : i;
    }
    sSrc[tid] = src;
    sDst[tid] = dst;
  }
  __syncthreads();

  const int n0 = n_tile * GBN;
  const int ty = tid / 16, tx = tid % 16;   // thread owns rows ty*4.., cols tx*4..
  float acc[4][4] = {};
  const bool w_n_fast = a.swn == 1;

  for (int k0 = 0; k0 < a.K; k0 += GBK) {
    // A tile: k fastest across threads (contiguous when sxk == 1)
#pragma unroll
    for (int i = 0; i < (GBM * GBK) / GT; ++i) {
      const int lin = tid + i * GT;
      const int kk = lin % GBK, mm = lin / GBK;
      const int64_t src = sSrc[mm];
      const int k = k0 + kk;
      sA[kk][mm] = (src >= 0 && k < a.K) ? to_f32(X[src * a.sxm + (int64_t)k * a.sxk]) : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < (GBN * GBK) / GT; ++i) {
      const int lin = tid + i * GT;
      int kk, nn;
      if (w_n_fast) { nn = lin % GBN; kk = lin / GBN; } else { kk = lin % GBK; nn = lin / GBK; }
      const int k = k0 + kk, n = n0 + nn;
      sB[kk][nn] = (k < a.K && n < a.N) ? to_f32(W[(int64_t)k * a.swk + (int64_t)n * a.swn]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GBK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = sA[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = sB[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }

  const T* __restrict__ B = (const T*)a.b;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t dst = sDst[ty * 4 + i];
    if (dst < 0) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < a.N) {
        float v = acc[i][j];
        if (B) v += to_f32(B[(int64_t)e * a.sbe + (int64_t)n * a.sbn]);
        Y[dst * a.sym + (int64_t)n * a.syn] = from_f32<T>(v);
      }
    }
  }
}

template <typename T>
static int launch_t(const S2SArgs& a, hipStream_t st) {
  const int n_tiles = (a.N + GBN - 1) / GBN;
  const int64_t m_tiles = max_tiles(a.L, a.E, GBM);
  const int64_t grid = m_tiles * n_tiles;
  if (grid > 0x7fffffffLL) { set_error("smoe_scatter2scatter: grid too large"); return SMOE_ERR_RANGE; }
  hipLaunchKernelGGL(s2s_generic_kernel<T>, dim3((unsigned)grid), dim3(GT), 0, st, a, n_tiles);
  return launch_status("s2s_generic_kernel");
}

int launch_s2s_generic(const S2SArgs& a, int dtype, hipStream_t st) {
  switch (dtype) {
    case SMOE_F32: return launch_t<float>(a, st);
    case SMOE_BF16: return launch_t<bf16_t>(a, st);
    case SMOE_F16: return launch_t<f16_t>(a, st);
    default: set_error("smoe_scatter2scatter: unknown dtype %d", dtype); return SMOE_ERR_DTYPE;
  }
}

}  // namespace smoe
