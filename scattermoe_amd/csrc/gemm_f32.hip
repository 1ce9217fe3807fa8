// float32 MFMA paths of scatter2scatter and groupXtY for gfx950: true fp32 products and fp32 accumulation
// (v_mfma_f32_32x32x2_f32; gfx950 has no TF32 mode), for operands whose rows are 16-byte aligned.  Everything else
// in float32 runs on the any-layout FMA kernels.
//
// One workgroup (4 waves, 2 x 2) owns one 128 x 128 output tile that never straddles two experts; each wave a
// 64 x 64 quarter as 2 x 2 MFMA blocks.  The contraction is walked in slices of 16 through two LDS buffers, both
// operands stored [k][row] so that an MFMA operand (lane = row, lanes 32..63 the second k) is one conflict-free
// ds_read_b32.  Global loads are 16 bytes per thread, fetched into registers one slice ahead of the MFMAs; an
// operand with contiguous contraction axis is transposed on its way into LDS.  The fp32 matrix pipe is 16 times
// slower than the bf16 one, so this simple pipeline already keeps it busy.
//
// Counterparts in the reference: _scatter2scatter (scattermoe/kernels/ops.py:50-118) and _groupXtY
// (ops.py:242-366) with float32 tensors (where Triton would use TF32 products under ALLOW_TF32).
#include "common.hpp"

namespace smoe {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

static constexpr int FBM = 128, FBN = 128, FBK = 16, FNT = 256;
static constexpr int FLD = FBM + 4;                 // LDS row length in floats: 16-byte aligned rows, spread banks
static_assert(FBM == FBN, "one LDS row length for both operands");

// Operand tile of 128 rows x 16 contraction elements, held by a thread as two 16-byte pieces.
struct Piece2 { f32x4 v[2]; };

// rows contiguous along the contraction: element (row, k) at rowp[row] + k
// thread piece p = t + 256 j: row = p / 4, contraction quad = p % 4
__device__ __forceinline__ Piece2 load_kc(const float* const* rowp_lds, const bool* ok_lds, int k0, int K) {
  Piece2 r;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int p = threadIdx.x + j * FNT, row = p >> 2, kq = p & 3;
    const int k = k0 + kq * 4;
    r.v[j] = (ok_lds[row] && k < K) ? *(const f32x4*)(rowp_lds[row] + k) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  return r;
}
__device__ __forceinline__ void store_kc(float (*s)[FLD], const Piece2& r) {
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int p = threadIdx.x + j * FNT, row = p >> 2, kq = p & 3;
#pragma unroll
    for (int c = 0; c < 4; ++c) s[kq * 4 + c][row] = r.v[j][c];
  }
}
// rows of the tile contiguous along the tile's row axis: element (k, n) at base + k * ld + n
// thread piece p = t + 256 j: k = p / 32, column quad = p % 32
__device__ __forceinline__ Piece2 load_nc(const float* base, int64_t ld, int k0, int kend, int n0, int ncols) {
  Piece2 r;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int p = threadIdx.x + j * FNT, kk = p >> 5, nq = p & 31;
    const int k = k0 + kk, n = n0 + nq * 4;
    r.v[j] = (k < kend && n < ncols) ? *(const f32x4*)(base + (int64_t)k * ld + n) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  return r;
}
__device__ __forceinline__ void store_nc(float (*s)[FLD], const Piece2& r) {
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int p = threadIdx.x + j * FNT, kk = p >> 5, nq = p & 31;
    *(f32x4*)&s[kk][nq * 4] = r.v[j];
  }
}

// 16-deep slice held in LDS: acc[i][j] += A-block i x B-block j for this wave's 64 x 64 quarter
__device__ __forceinline__ void mma_slice(const float (*sa)[FLD], const float (*sb)[FLD], int wm, int wn,
                                          f32x16 (&acc)[2][2]) {
  const int l = lane_id(), half = l >> 5, r = l & 31;
#pragma unroll
  for (int s = 0; s < FBK / 2; ++s) {
    float a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = sa[2 * s + half][wm * 64 + i * 32 + r];
#pragma unroll
    for (int j = 0; j < 2; ++j) b[j] = sb[2 * s + half][wn * 64 + j * 32 + r];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
  }
}

// =====================================================================================================
// scatter2scatter
// =====================================================================================================
template <bool W_KC>
__global__ __launch_bounds__(FNT) void s2s_f32_kernel(S2SArgs a, int n_tiles) {
  __shared__ __attribute__((aligned(16))) float sA[2][FBK][FLD];
  __shared__ __attribute__((aligned(16))) float sB[2][FBK][FLD];
  __shared__ const float* rowA[FBM];
  __shared__ const float* rowB[FBN];
  __shared__ bool okA[FBM], okB[FBN];
  __shared__ int64_t sDst[FBM];

  const int m_tile = blockIdx.x / n_tiles, n_tile = blockIdx.x % n_tiles;
  int e, row0, rows;
  if (!find_tile<FBM>(a.off, a.E, m_tile, e, row0, rows)) return;
  const int n0 = n_tile * FBN;
  const float* X = (const float*)a.X;
  const float* W = (const float*)a.W + (int64_t)e * a.swe;
  for (int m = threadIdx.x; m < FBM; m += FNT) {
    const bool ok = m < rows;
    int64_t src = 0, dst = -1;
    if (ok) {
      const int64_t n = row0 + m;
      src = n; dst = n;
      if (!a.x_grouped || !a.y_grouped) {
        const int64_t i = a.idx[n];
        if (!a.x_grouped) src = i / a.fan_out;
        if (!a.y_grouped) dst = i;
      }
    }
    rowA[m] = X + src * a.sxm;
    okA[m] = ok;
    sDst[m] = ok ? dst * a.sym : -1;
    if (W_KC) {
      rowB[m] = W + (int64_t)(n0 + m < a.N ? n0 + m : 0) * a.swn;
      okB[m] = n0 + m < a.N;
    }
  }
  __syncthreads();

  const int wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int K = a.K, nk = (K + FBK - 1) / FBK;
  Piece2 ra = load_kc(rowA, okA, 0, K);
  Piece2 rb = W_KC ? load_kc(rowB, okB, 0, K) : load_nc(W, a.swk, 0, K, n0, a.N);
  store_kc(sA[0], ra);
  if (W_KC) store_kc(sB[0], rb); else store_nc(sB[0], rb);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) {
      ra = load_kc(rowA, okA, (kt + 1) * FBK, K);
      rb = W_KC ? load_kc(rowB, okB, (kt + 1) * FBK, K) : load_nc(W, a.swk, (kt + 1) * FBK, K, n0, a.N);
    }
    mma_slice(sA[cur], sB[cur], wm, wn, acc);
    if (kt + 1 < nk) {
      store_kc(sA[cur ^ 1], ra);
      if (W_KC) store_kc(sB[cur ^ 1], rb); else store_nc(sB[cur ^ 1], rb);
    }
    __syncthreads();
  }

  // accumulator register r of a lane: row (r / 4) * 8 + (lane / 32) * 4 + r % 4, column lane % 32 of the block
  const int l = lane_id();
  const float* bias = a.b ? (const float*)a.b + (int64_t)e * a.sbe : nullptr;
  float* Y = (float*)a.Y;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn * 64 + j * 32 + (l & 31);
    if (n >= a.N) continue;
    const float bv = bias ? bias[(int64_t)n * a.sbn] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = wm * 64 + i * 32 + (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
        const int64_t d = sDst[m];
        if (d >= 0) Y[d + n] = acc[i][j][r] + bv;
      }
  }
}

static bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

bool try_s2s_f32(const S2SArgs& a, hipStream_t st, int& rc) {
  if (a.glu != 0) return false;
  if (a.sxk != 1 || a.syn != 1 || a.K % 4 != 0 || a.sxm % 4 != 0 || !al16(a.X) || !al16(a.W) || a.swe % 4 != 0)
    return false;
  bool w_kc;
  if (a.swk == 1 && a.swn % 4 == 0) w_kc = true;
  else if (a.swn == 1 && a.swk % 4 == 0 && a.N % 4 == 0) w_kc = false;
  else return false;
  const int n_tiles = (a.N + FBN - 1) / FBN;
  const int64_t grid = max_tiles(a.L, a.E, FBM) * n_tiles;
  if (grid > 0x7fffffffLL) { set_error("smoe_scatter2scatter: grid too large"); rc = SMOE_ERR_RANGE; return true; }
  if (w_kc) hipLaunchKernelGGL(s2s_f32_kernel<true>, dim3((unsigned)grid), dim3(FNT), 0, st, a, n_tiles);
  else hipLaunchKernelGGL(s2s_f32_kernel<false>, dim3((unsigned)grid), dim3(FNT), 0, st, a, n_tiles);
  rc = launch_status("s2s_f32_kernel");
  return true;
}

// =====================================================================================================
// groupXtY:  OUT[e] (P x Q, Q contiguous) = sum over the expert's rows r of  Pm[r, :]^T  Qm[r, :]
// =====================================================================================================
struct XtYPlanF32 {
  const float* P; int64_t ldp; int np;
  const float* Q; int64_t ldq; int nq;
  float* OUT; int64_t soe, sop;
  const int64_t* off;
};

__global__ __launch_bounds__(FNT) void xty_f32_kernel(XtYPlanF32 a, int p_tiles, int q_tiles) {
  __shared__ __attribute__((aligned(16))) float sA[2][FBK][FLD];
  __shared__ __attribute__((aligned(16))) float sB[2][FBK][FLD];
  int b = blockIdx.x;
  const int q_tile = b % q_tiles; b /= q_tiles;
  const int p_tile = b % p_tiles;
  const int e = b / p_tiles;
  const int r_lo = e ? (int)a.off[e - 1] : 0, r_hi = (int)a.off[e];
  const int p0 = p_tile * FBM, q0 = q_tile * FBN;
  const float* P = a.P + (int64_t)r_lo * a.ldp;
  const float* Q = a.Q + (int64_t)r_lo * a.ldq;
  const int klen = r_hi - r_lo, nk = (klen + FBK - 1) / FBK;

  const int wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  if (nk > 0) {
    Piece2 ra = load_nc(P, a.ldp, 0, klen, p0, a.np), rb = load_nc(Q, a.ldq, 0, klen, q0, a.nq);
    store_nc(sA[0], ra);
    store_nc(sB[0], rb);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
      const int cur = kt & 1;
      if (kt + 1 < nk) {
        ra = load_nc(P, a.ldp, (kt + 1) * FBK, klen, p0, a.np);
        rb = load_nc(Q, a.ldq, (kt + 1) * FBK, klen, q0, a.nq);
      }
      mma_slice(sA[cur], sB[cur], wm, wn, acc);
      if (kt + 1 < nk) {
        store_nc(sA[cur ^ 1], ra);
        store_nc(sB[cur ^ 1], rb);
      }
      __syncthreads();
    }
  }
  // empty experts write zeros
  const int l = lane_id();
  float* O = a.OUT + (int64_t)e * a.soe;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int q = q0 + wn * 64 + j * 32 + (l & 31);
    if (q >= a.nq) continue;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int p = p0 + wm * 64 + i * 32 + (r >> 2) * 8 + (l >> 5) * 4 + (r & 3);
        if (p < a.np) O[(int64_t)p * a.sop + q] = acc[i][j][r];
      }
  }
}

// bias gradient: column sums of dY per expert segment.  A workgroup owns 256 columns of one expert: 64 column threads
// (16 bytes = 4 columns each) x 4 row lanes; the 4 partial sums of a column are added in a fixed order.
__global__ __launch_bounds__(256) void colsum_f32_kernel(const float* __restrict__ DY, int64_t ld, int N,
                                                        const int64_t* __restrict__ off, float* __restrict__ Db,
                                                        int64_t sdbe, int64_t sdbn) {
  __shared__ float part[4][256];
  const int e = blockIdx.y;
  const int c4 = threadIdx.x & 63, rg = threadIdx.x >> 6;
  const int n = (blockIdx.x * 64 + c4) * 4;
  const int r_lo = e ? (int)off[e - 1] : 0, r_hi = (int)off[e];
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
  if (n < N)
    for (int r = r_lo + rg; r < r_hi; r += 4) s += *(const f32x4*)(DY + (int64_t)r * ld + n);
#pragma unroll
  for (int q = 0; q < 4; ++q) part[rg][c4 * 4 + q] = s[q];
  __syncthreads();
  const int col = blockIdx.x * 256 + threadIdx.x;
  if (col < N) Db[(int64_t)e * sdbe + (int64_t)col * sdbn] = ((part[0][threadIdx.x] + part[1][threadIdx.x]) +
                                                               part[2][threadIdx.x]) + part[3][threadIdx.x];
}

bool try_xty_f32(const XtYArgs& a, hipStream_t st, int& rc) {
  rc = 0;
  if (a.sdyn != 1 || a.sxk != 1 || a.sdym % 4 != 0 || a.sxm % 4 != 0 || a.K % 4 != 0 || a.N % 4 != 0) return false;
  if (!al16(a.DY) || !al16(a.X) || !al16(a.DW) || a.sdwe % 4 != 0) return false;
  XtYPlanF32 p;
  if (a.sdwk == 1 && a.sdwn % 4 == 0) {            // output rows = N index, K contiguous
    p.P = (const float*)a.DY; p.ldp = a.sdym; p.np = a.N;
    p.Q = (const float*)a.X; p.ldq = a.sxm; p.nq = a.K;
    p.sop = a.sdwn;
  } else if (a.sdwn == 1 && a.sdwk % 4 == 0) {     // output rows = K index, N contiguous
    p.P = (const float*)a.X; p.ldp = a.sxm; p.np = a.K;
    p.Q = (const float*)a.DY; p.ldq = a.sdym; p.nq = a.N;
    p.sop = a.sdwk;
  } else return false;
  p.OUT = (float*)a.DW; p.soe = a.sdwe; p.off = a.off;
  const int p_tiles = (p.np + FBM - 1) / FBM, q_tiles = (p.nq + FBN - 1) / FBN;
  const int64_t grid = (int64_t)a.E * p_tiles * q_tiles;
  if (grid > 0x7fffffffLL) { set_error("smoe_groupXtY: grid too large"); rc = SMOE_ERR_RANGE; return true; }
  if (grid > 0) {
    hipLaunchKernelGGL(xty_f32_kernel, dim3((unsigned)grid), dim3(FNT), 0, st, p, p_tiles, q_tiles);
    rc = launch_status("xty_f32_kernel");
    if (rc != 0) return true;
  }
  if (a.Db != nullptr && a.N > 0) {
    hipLaunchKernelGGL(colsum_f32_kernel, dim3((a.N + 255) / 256, a.E), dim3(256), 0, st, (const float*)a.DY,
                       a.sdym, a.N, a.off, (float*)a.Db, a.sdbe, a.sdbn);
    rc = launch_status("colsum_f32_kernel");
  }
  return true;
}

}  // namespace smoe
