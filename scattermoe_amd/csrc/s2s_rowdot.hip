// scatter2scatter for a handful of rows (single-token and few-token decode): every weight element is used by at
// most four rows, so the launch is a stream over the weights of the experts that were hit and nothing else
// matters.  No LDS tiles and no MFMA: each wave reads whole 16-byte pieces of K-contiguous weight rows with
// plain coalesced loads (a wave instruction covers 1 KB of one weight row), multiplies them with the matching
// pieces of up to four input rows by packed dot products, and the partial sums are reduced across lanes once at
// the end.  Many small waves per CU keep far more bytes in flight than the ring-buffered MFMA tiles can.
//
// Work split: a workgroup (4 waves) owns C = 8 output columns of one tile of up to R = 4 expert-sorted rows; its
// waves take the contraction pieces round-robin (piece p of 512 elements goes to wave p % 4), so the four waves
// together read 4 KB runs of each weight row.  A workgroup walks `gpw` consecutive column groups.
//
// Counterparts in the reference: _single2scatter (scattermoe/kernels/single.py:5-59), and _scatter2scatter
// (scattermoe/kernels/ops.py:50-118) for the row/column conventions, bias and the fused GLU of mlp.py:81-87.
#include "common.hpp"

namespace smoe {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Pair;
template <> struct Pair<bf16_t> {
  typedef __bf16 v2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ float dot(unsigned a, unsigned b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
  }
};
template <> struct Pair<f16_t> {
  typedef _Float16 v2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ float dot(unsigned a, unsigned b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(v2, a), __builtin_bit_cast(v2, b), c, false);
  }
};

// Sum each of the N = 32 per-lane values over the 64 lanes of the wave with 32 exchanges: every step halves the
// number of values a lane carries (the lane keeps the half selected by one bit of its id and adds the partner's
// copy of it).  Afterwards lanes 2j and 2j+1 hold the total of value j in v[0].
template <int HALF, int OFF, int N>
__device__ __forceinline__ void transpose_sum_step(float (&v)[N], int lane) {
  const bool up = (lane & OFF) != 0;
#pragma unroll
  for (int i = 0; i < HALF; ++i) {
    const float keep = up ? v[i + HALF] : v[i];
    const float send = up ? v[i] : v[i + HALF];
    v[i] = keep + __shfl_xor(send, OFF, 64);
  }
  if constexpr (HALF > 1) transpose_sum_step<HALF / 2, OFF / 2>(v, lane);
}
template <int N>
__device__ __forceinline__ void wave_transpose_sum(float (&v)[N]) {
  static_assert(N == 32, "written for 32 values over 64 lanes");
  transpose_sum_step<N / 2, 32>(v, lane_id());
  v[0] += __shfl_xor(v[0], 1, 64);
}

static constexpr int ROWDOT_MAX_ROWS = 8;   // launches with more rows than this go to the MFMA tiles
static constexpr int RD_R = 4;        // rows per tile
static constexpr int RD_C = 8;        // columns per workgroup pass
static constexpr int RD_WAVES = 4;
static constexpr int RD_PIECE = 512;  // contraction elements one wave instruction covers (64 lanes x 8)

// One column group: the C weight rows `wp` against the R input rows at byte offsets `xoff` of `Xb`, contraction
// length K.  Leaves the R*C totals in part[0][r*C + c] (visible to the whole workgroup on return).
template <typename T, int R, int C, int NW>
__device__ __forceinline__ void rowdot_pass(const char* Xb, const int64_t (&xoff)[R], const char* const (&wp)[C],
                                            int K, float (&part)[NW][R * C]) {
  const int wave = threadIdx.x >> 6, lane = lane_id();
  float acc[R * C];
#pragma unroll
  for (int i = 0; i < R * C; ++i) acc[i] = 0.0f;

  for (int k = (wave * 64 + lane) * 8; k < K; k += NW * RD_PIECE) {
    u32x4 w[C], x[R];
#pragma unroll
    for (int c = 0; c < C; ++c) w[c] = __builtin_nontemporal_load((const u32x4*)(wp[c] + (int64_t)k * 2));   // read once
#pragma unroll
    for (int r = 0; r < R; ++r) x[r] = *(const u32x4*)(Xb + xoff[r] + (int64_t)k * 2);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int c = 0; c < C; ++c)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[r * C + c] = Pair<T>::dot(x[r][q], w[c][q], acc[r * C + c]);
  }

  wave_transpose_sum<R * C>(acc);
  __syncthreads();                               // the previous pass has read `part`
  if ((lane & 1) == 0) part[wave][lane >> 1] = acc[0];
  __syncthreads();
  if (threadIdx.x < R * C) {
    float v = 0.0f;
#pragma unroll
    for (int w_ = 0; w_ < NW; ++w_) v += part[w_][threadIdx.x];
    part[0][threadIdx.x] = v;                    // only this thread read column threadIdx.x of `part`
  }
  __syncthreads();
}

template <typename T, bool GLU>
__global__ __launch_bounds__(RD_WAVES * 64) void s2s_rowdot_kernel(S2SArgs a, int n_groups, int gpw) {
  constexpr int R = RD_R, C = RD_C;
  __shared__ float part[RD_WAVES][R * C];
  const int wave = threadIdx.x >> 6, lane = lane_id();
  int e, row0, rows;
  if (!find_tile<R>(a.off, a.E, blockIdx.y, e, row0, rows)) return;

  // source rows of X and destination rows of Y (uniform over the workgroup)
  int64_t xoff[R], dst[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t n = row0 + (r < rows ? r : rows - 1);
    int64_t src = n, d = n;
    if (!a.x_grouped || !a.y_grouped) {
      const int64_t i = a.idx[n];
      if (!a.x_grouped) src = i / a.fan_out;
      if (!a.y_grouped) d = i;
    }
    xoff[r] = src * a.sxm * 2;
    dst[r] = d;
  }
  const char* Xb = (const char*)a.X;
  const char* Wb = (const char*)a.W + (int64_t)e * a.swe * 2;
  const T* bias = a.b ? (const T*)a.b + (int64_t)e * a.sbe : nullptr;
  const int F = a.N;                         // GLU: hidden width (the weights have 2F columns)
  const int K = a.K;

  for (int g = blockIdx.x * gpw; g < min(n_groups, (int)(blockIdx.x + 1) * gpw); ++g) {
    // column c of the pass -> weight column
    int col[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
      if (GLU) {
        const int hc = g * (C / 2) + c % (C / 2);
        col[c] = hc < F ? hc + (c >= C / 2 ? F : 0) : 0;
      } else {
        const int n = g * C + c;
        col[c] = n < F ? n : 0;
      }
    }
    const char* wp[C];
#pragma unroll
    for (int c = 0; c < C; ++c) wp[c] = Wb + (int64_t)col[c] * a.swn * 2;
    rowdot_pass<T, R, C, RD_WAVES>(Xb, xoff, wp, K, part);
    if (!GLU) {
      if (threadIdx.x < R * C) {
        const int r = threadIdx.x / C, c = threadIdx.x % C;
        const int n = g * C + c;
        if (r < rows && n < F) {
          float v = part[0][threadIdx.x];
          if (bias != nullptr) v += to_f32(bias[(int64_t)n * a.sbn]);
          ((T*)a.Y)[dst[r] * a.sym + n] = from_f32<T>(v);
        }
      }
    } else {
      // both halves are rounded to the storage type first and the hidden value is computed from the rounded values
      if (threadIdx.x < R * (C / 2)) {
        const int r = threadIdx.x / (C / 2), c = threadIdx.x % (C / 2);
        const int n = g * (C / 2) + c;
        if (r < rows && n < F) {
          float v1 = part[0][r * C + c], v2 = part[0][r * C + C / 2 + c];
          if (bias != nullptr) {
            v1 += to_f32(bias[(int64_t)n * a.sbn]);
            v2 += to_f32(bias[(int64_t)(F + n) * a.sbn]);
          }
          const T first = from_f32<T>(v1), second = from_f32<T>(v2);
          const bool gf = (a.act & 1) != 0;
          const float lin = to_f32(gf ? second : first), gat = to_f32(gf ? first : second);
          const int64_t row = row0 + r;            // the fused form works on rows in grouped order
          if (a.Y != nullptr) {
            ((T*)a.Y)[row * a.sym + n] = first;
            ((T*)a.Y)[row * a.sym + F + n] = second;
          }
          ((T*)a.H)[row * a.shm + n] = from_f32<T>(glu_h(a.act, gat, lin));
        }
      }
    }
  }
}

// Called with the operand checks of the MFMA path already done (K-contiguous weights, 16-byte aligned rows,
// K a multiple of 8).  Returns false when the shape is not this kernel's.
bool try_s2s_rowdot(const S2SArgs& a, int dtype, hipStream_t st, int& rc) {
  if (a.glu >= 2 || a.L > ROWDOT_MAX_ROWS) return false;
  const int64_t m_tiles = max_tiles(a.L, a.E, RD_R);
  const int n_groups = a.glu == 1 ? (a.N + RD_C / 2 - 1) / (RD_C / 2) : (a.N + RD_C - 1) / RD_C;
  // enough workgroups to give every CU several, few enough that the tile lookup is amortised
  int gpw = 1;
  while (gpw < 8 && m_tiles * ((n_groups + 2 * gpw - 1) / (2 * gpw)) >= 2048) gpw *= 2;
  const dim3 grid((unsigned)((n_groups + gpw - 1) / gpw), (unsigned)m_tiles), block(RD_WAVES * 64);
  if (dtype == SMOE_BF16) {
    if (a.glu) hipLaunchKernelGGL((s2s_rowdot_kernel<bf16_t, true>), grid, block, 0, st, a, n_groups, gpw);
    else hipLaunchKernelGGL((s2s_rowdot_kernel<bf16_t, false>), grid, block, 0, st, a, n_groups, gpw);
  } else {
    if (a.glu) hipLaunchKernelGGL((s2s_rowdot_kernel<f16_t, true>), grid, block, 0, st, a, n_groups, gpw);
    else hipLaunchKernelGGL((s2s_rowdot_kernel<f16_t, false>), grid, block, 0, st, a, n_groups, gpw);
  }
  rc = launch_status("s2s_rowdot_kernel");
  return true;
}

// =====================================================================================================
// The whole gated MLP of a decode step (at most 8 (token, slot) rows, forward only) in two launches: layer 1 with
// its GLU, then layer 2 with the gate-weighted combine.  Neither needs the routing triple: every workgroup sorts
// the handful of expert ids itself (stable, so rows of one expert keep slot order and share one pass over that
// expert's weights, four rows at a time).  Hidden rows travel between the launches in slot order (row t*k + j).
// Same arithmetic, in the same order, as the general path (row-dot scatter2scatter launches + combine), so the
// results are bit-identical to it.
// Reference: GLUMLP.forward, scattermoe/mlp.py:74-95, with flatten_sort_count (parallel_experts.py:14-21) and
// the gate combine of ParallelLinear.forward (parallel_experts.py:38-46) folded in.
// =====================================================================================================
struct SortedRows {
  int e[DECODE_MAX_ROWS];        // expert ids, ascending
  int slot[DECODE_MAX_ROWS];     // slot t*k + j of each sorted row
};

__device__ __forceinline__ void sort_rows(const DecodeArgs& a, SortedRows& s, int* raw) {
  const int L = a.T * a.k;
  if (threadIdx.x < L) raw[threadIdx.x] = (int)a.experts[(threadIdx.x / a.k) * a.set + (threadIdx.x % a.k) * a.sek];
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 0; i < L; ++i) {                 // stable insertion sort
      const int ei = raw[i];
      int j = i;
      while (j > 0 && s.e[j - 1] > ei) {
        s.e[j] = s.e[j - 1];
        s.slot[j] = s.slot[j - 1];
        --j;
      }
      s.e[j] = ei;
      s.slot[j] = i;
    }
  }
  __syncthreads();
}

// Tile `want` of the sorted rows: runs of one expert, at most RD_R rows each.  Returns false past the last tile.
__device__ __forceinline__ bool decode_tile(const SortedRows& s, int L, int want, int& start, int& rows) {
  start = 0;
  for (int t = 0; start < L; ++t) {
    const int e = s.e[start];
    rows = 1;
    while (start + rows < L && rows < RD_R && s.e[start + rows] == e) ++rows;
    if (t == want) return true;
    start += rows;
  }
  return false;
}

template <typename T>
__global__ __launch_bounds__(RD_WAVES * 64) void decode_l1_kernel(DecodeArgs a, int n_groups, int gpw) {
  constexpr int R = RD_R, C = RD_C;
  __shared__ float part[RD_WAVES][R * C];
  __shared__ SortedRows srt;
  __shared__ int raw[DECODE_MAX_ROWS];
  sort_rows(a, srt, raw);
  const int L = a.T * a.k;
  int start, rows;
  if (!decode_tile(srt, L, blockIdx.y, start, rows)) return;
  const int e = srt.e[start];
  if (e < 0 || e >= a.E) return;                     // rows with an invalid expert id are dropped
  int64_t xoff[R];
  int slot[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    slot[r] = srt.slot[start + (r < rows ? r : rows - 1)];
    xoff[r] = (int64_t)(slot[r] / a.k) * a.sxm * 2;
  }
  const char* Wb = (const char*)a.W1 + (int64_t)e * a.sw1e * 2;
  const T* bias = a.b1 ? (const T*)a.b1 + (int64_t)e * a.sb1e : nullptr;
  const int F = a.F;
  for (int g = blockIdx.x * gpw; g < min(n_groups, (int)(blockIdx.x + 1) * gpw); ++g) {
    const char* wp[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
      const int hc = g * (C / 2) + c % (C / 2);
      const int col = hc < F ? hc + (c >= C / 2 ? F : 0) : 0;
      wp[c] = Wb + (int64_t)col * a.sw1n * 2;
    }
    rowdot_pass<T, R, C, RD_WAVES>((const char*)a.X, xoff, wp, a.d, part);
    if (threadIdx.x < R * (C / 2)) {
      const int r = threadIdx.x / (C / 2), c = threadIdx.x % (C / 2);
      const int n = g * (C / 2) + c;
      if (r < rows && n < F) {
        float v1 = part[0][r * C + c], v2 = part[0][r * C + C / 2 + c];
        if (bias != nullptr) {
          v1 += to_f32(bias[(int64_t)n * a.sb1n]);
          v2 += to_f32(bias[(int64_t)(F + n) * a.sb1n]);
        }
        const T first = from_f32<T>(v1), second = from_f32<T>(v2);
        const bool gf = (a.act & 1) != 0;
        const float lin = to_f32(gf ? second : first), gat = to_f32(gf ? first : second);
        ((T*)a.H)[(int64_t)slot[r] * a.shm + n] = from_f32<T>(glu_h(a.act, gat, lin));
      }
    }
  }
}

template <typename T, int NW>
__global__ __launch_bounds__(NW * 64) void decode_l2_kernel(DecodeArgs a) {
  constexpr int R = RD_R, C = RD_C;
  __shared__ float part[NW][R * C];
  __shared__ float ybuf[DECODE_MAX_ROWS][C];         // layer-2 outputs of every slot, rounded to the storage type
  __shared__ SortedRows srt;
  __shared__ int raw[DECODE_MAX_ROWS];
  sort_rows(a, srt, raw);
  const int L = a.T * a.k;
  if (threadIdx.x < DECODE_MAX_ROWS * C) ybuf[threadIdx.x / C][threadIdx.x % C] = 0.0f;
  const int n0 = blockIdx.x * C;
  int start, rows;
  for (int t = 0; decode_tile(srt, L, t, start, rows); ++t) {
    const int e = srt.e[start];
    if (e < 0 || e >= a.E) continue;
    int64_t xoff[R];
    int slot[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      slot[r] = srt.slot[start + (r < rows ? r : rows - 1)];
      xoff[r] = (int64_t)slot[r] * a.shm * 2;
    }
    const char* Wb = (const char*)a.W2 + (int64_t)e * a.sw2e * 2;
    const char* wp[C];
#pragma unroll
    for (int c = 0; c < C; ++c) wp[c] = Wb + (int64_t)(n0 + c < a.d ? n0 + c : 0) * a.sw2n * 2;
    rowdot_pass<T, R, C, NW>((const char*)a.H, xoff, wp, a.F, part);
    if (threadIdx.x < R * C) {
      const int r = threadIdx.x / C, c = threadIdx.x % C;
      if (r < rows && n0 + c < a.d) {
        float v = part[0][threadIdx.x];
        if (a.b2 != nullptr) v += to_f32(((const T*)a.b2)[(int64_t)e * a.sb2e + (int64_t)(n0 + c) * a.sb2n]);
        ybuf[slot[r]][c] = to_f32(from_f32<T>(v));
      }
    }
  }
  __syncthreads();
  if (threadIdx.x < a.T * C) {
    const int t = threadIdx.x / C, c = threadIdx.x % C;
    if (n0 + c < a.d) {
      float acc = 0.0f;
      for (int j = 0; j < a.k; ++j)
        acc = fmaf(to_f32(((const T*)a.gates)[(int64_t)t * a.sgt + (int64_t)j * a.sgk]), ybuf[t * a.k + j][c], acc);
      ((T*)a.OUT)[(int64_t)t * a.som + n0 + c] = from_f32<T>(acc);
    }
  }
}

int launch_decode_glu_mlp(const DecodeArgs& a, int dtype, hipStream_t st) {
  const int L = a.T * a.k;
  const int n_groups = (a.F + RD_C / 2 - 1) / (RD_C / 2);
  int gpw = 1;
  while (gpw < 8 && (int64_t)L * ((n_groups + 2 * gpw - 1) / (2 * gpw)) >= 2048) gpw *= 2;
  const dim3 grid1((unsigned)((n_groups + gpw - 1) / gpw), (unsigned)L), grid2((unsigned)((a.d + RD_C - 1) / RD_C));
  const dim3 block(RD_WAVES * 64);
  // same split of the contraction over the waves as the general path's launches: that is what keeps the results
  // bit-identical to it (eight waves for layer 2 measured no faster)
  constexpr int L2_WAVES = RD_WAVES;
  if (dtype == SMOE_BF16) {
    hipLaunchKernelGGL(decode_l1_kernel<bf16_t>, grid1, block, 0, st, a, n_groups, gpw);
    hipLaunchKernelGGL((decode_l2_kernel<bf16_t, L2_WAVES>), grid2, dim3(L2_WAVES * 64), 0, st, a);
  } else {
    hipLaunchKernelGGL(decode_l1_kernel<f16_t>, grid1, block, 0, st, a, n_groups, gpw);
    hipLaunchKernelGGL((decode_l2_kernel<f16_t, L2_WAVES>), grid2, dim3(L2_WAVES * 64), 0, st, a);
  }
  return launch_status("decode_glu_mlp kernels");
}

}  // namespace smoe
