// Row gather into expert-sorted order, optionally scaled by a per-row coefficient.
// Counterpart of group (scattermoe/kernels/ops.py:377-410) and its kernel _group (ops.py:413-457):
//   Y[n, :] = A[idx[n] / fan_out, :] * coeff[idx[n]]
// Pure HBM traffic: one wave moves one row in 16-byte pieces when rows are contiguous and aligned,
// element-wise otherwise.  The product is formed in fp32 and rounded once to the tensor dtype.
#include "common.hpp"

namespace smoe {

static constexpr int kGroupThreads = 256;
static constexpr int kGroupRowsPerBlock = kGroupThreads / 64;

template <typename T> struct Vec16 { static constexpr int n = 16 / sizeof(T); T v[16 / sizeof(T)]; };

template <typename T, bool VEC>
__global__ __launch_bounds__(kGroupThreads) void group_kernel(GroupArgs a) {
  const T* __restrict__ A = (const T*)a.A;
  const T* __restrict__ coeff = (const T*)a.coeff;
  T* __restrict__ Y = (T*)a.Y;
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  for (int64_t n = (int64_t)blockIdx.x * kGroupRowsPerBlock + wave; n < a.L;
       n += (int64_t)gridDim.x * kGroupRowsPerBlock) {
    const int64_t i = a.idx[n];
    const int64_t src = i / a.fan_out;
    const float c = coeff ? to_f32(coeff[i]) : 1.0f;
    const T* __restrict__ s = A + src * a.sam;
    T* __restrict__ d = Y + n * a.sym;
    if (VEC) {
      typedef Vec16<T> V;
      typedef int VV __attribute__((ext_vector_type(4)));
      const int nv = a.K / V::n;
      for (int j = lane; j < nv; j += 64) {
        V x = *(const V*)(s + (int64_t)j * V::n);
        if (coeff) {
#pragma unroll
          for (int q = 0; q < V::n; ++q) x.v[q] = from_f32<T>(to_f32(x.v[q]) * c);
        }
        __builtin_nontemporal_store(*(const VV*)&x, (VV*)(d + (int64_t)j * V::n));
      }
    } else {
      for (int j = lane; j < a.K; j += 64) {
        const float x = to_f32(s[(int64_t)j * a.sak]);
        d[(int64_t)j * a.syk] = coeff ? from_f32<T>(x * c) : from_f32<T>(x);
      }
    }
  }
}

template <typename T>
static int launch_group_t(const GroupArgs& a, hipStream_t st) {
  if (a.L == 0 || a.K == 0) return 0;
  constexpr int vn = 16 / sizeof(T);
  const bool vec = a.sak == 1 && a.syk == 1 && a.K % vn == 0 && a.sam % vn == 0 && a.sym % vn == 0 &&
                   ((uintptr_t)a.A % 16 == 0) && ((uintptr_t)a.Y % 16 == 0);
  int64_t blocks = cdiv64(a.L, kGroupRowsPerBlock);
  if (blocks > 256 * 64) blocks = 256 * 64;   // grid-stride beyond 64 blocks per CU
  if (vec)
    hipLaunchKernelGGL((group_kernel<T, true>), dim3((unsigned)blocks), dim3(kGroupThreads), 0, st, a);
  else
    hipLaunchKernelGGL((group_kernel<T, false>), dim3((unsigned)blocks), dim3(kGroupThreads), 0, st, a);
  return launch_status("group_kernel");
}

// ---- the same rows, walked by source row -------------------------------------------------------------
// With a coefficient per slot the gather above reads every source row fan_out times (from different workgroups, at
// different times: from the memory-side cache at best).  When idx is a permutation of [0, L) - what the routing
// produces - the walk can go by source row instead: a wave reads row t once and writes its fan_out scaled copies to
// the rows inv[t * fan_out + f], inv being the inverse permutation (built by the first launch into a caller
// workspace of L ints).  A slot whose inverse entry does not point back at it (idx not a permutation, stale
// workspace) is skipped, so nothing is ever written outside Y; same arithmetic, hence the same bits, as the gather.
__global__ __launch_bounds__(256) void invert_index_kernel(const int64_t* __restrict__ idx, int L, int* __restrict__ inv) {
  const int r = blockIdx.x * 256 + threadIdx.x;
  if (r >= L) return;
  const int64_t s = idx[r];
  if ((uint64_t)s < (uint64_t)L) inv[s] = r;
}

int launch_invert_index(const int64_t* idx, int64_t L, int* inv, hipStream_t st) {
  if (L == 0) return 0;
  hipLaunchKernelGGL(invert_index_kernel, dim3((unsigned)cdiv64(L, 256)), dim3(256), 0, st, idx, (int)L, inv);
  return launch_status("invert_index_kernel");
}

template <typename T, int P>
__global__ __launch_bounds__(kGroupThreads) void group_by_source_kernel(GroupArgs a, const int* __restrict__ inv) {
  typedef Vec16<T> V;
  typedef int VV __attribute__((ext_vector_type(4)));
  const T* __restrict__ A = (const T*)a.A;
  const T* __restrict__ coeff = (const T*)a.coeff;
  T* __restrict__ Y = (T*)a.Y;
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int nv = a.K / V::n;                       // 16-byte pieces per row
  const int64_t rows = a.L / a.fan_out;
  for (int64_t t = (int64_t)blockIdx.x * kGroupRowsPerBlock + wave; t < rows;
       t += (int64_t)gridDim.x * kGroupRowsPerBlock) {
    // lane f < fan_out looks up where copy f of the row goes, and whether that row of Y is really its own
    int pos = -1;
    float c = 1.0f;
    if (lane < a.fan_out) {
      const int64_t slot = t * a.fan_out + lane;
      const int q = inv[slot];
      if ((unsigned)q < (unsigned)a.L && a.idx[q] == slot) {
        pos = q;
        if (coeff) c = to_f32(coeff[slot]);
      }
    }
    const T* __restrict__ s = A + t * a.sam;
    for (int j0 = 0; j0 < nv; j0 += 64 * P) {
      V x[P];
#pragma unroll
      for (int p = 0; p < P; ++p) {
        const int j = j0 + p * 64 + lane;
        if (j < nv) x[p] = *(const V*)(s + (int64_t)j * V::n);
      }
      for (int f = 0; f < a.fan_out; ++f) {
        const int dst = __shfl(pos, f, 64);
        if (dst < 0) continue;
        const float cf = __shfl(c, f, 64);
        T* __restrict__ d = Y + (int64_t)dst * a.sym;
#pragma unroll
        for (int p = 0; p < P; ++p) {
          const int j = j0 + p * 64 + lane;
          if (j >= nv) continue;
          V y = x[p];
          if (coeff) {
#pragma unroll
            for (int q = 0; q < V::n; ++q) y.v[q] = from_f32<T>(to_f32(y.v[q]) * cf);
          }
          __builtin_nontemporal_store(*(const VV*)&y, (VV*)(d + (int64_t)j * V::n));
        }
      }
    }
  }
}

template <typename T>
static int launch_group_by_source_t(const GroupArgs& a, int* inv, hipStream_t st) {
  constexpr int vn = 16 / sizeof(T);
  const bool vec = a.sak == 1 && a.syk == 1 && a.K % vn == 0 && a.sam % vn == 0 && a.sym % vn == 0 &&
                   ((uintptr_t)a.A % 16 == 0) && ((uintptr_t)a.Y % 16 == 0);
  if (!vec || a.fan_out > 64 || a.L % a.fan_out != 0) return SMOE_ERR_UNSUPPORTED;
  if (a.L == 0 || a.K == 0) return 0;
  hipLaunchKernelGGL(invert_index_kernel, dim3((unsigned)cdiv64(a.L, 256)), dim3(256), 0, st, a.idx, a.L, inv);
  int64_t blocks = cdiv64(a.L / a.fan_out, kGroupRowsPerBlock);
  if (blocks > 256 * 64) blocks = 256 * 64;
  hipLaunchKernelGGL((group_by_source_kernel<T, 4>), dim3((unsigned)blocks), dim3(kGroupThreads), 0, st, a, (const int*)inv);
  return launch_status("group_by_source_kernel");
}

int launch_group_by_source(const GroupArgs& a, int* inv, int dtype, hipStream_t st) {
  switch (dtype) {
    case SMOE_F32: return launch_group_by_source_t<float>(a, inv, st);
    case SMOE_BF16: return launch_group_by_source_t<bf16_t>(a, inv, st);
    case SMOE_F16: return launch_group_by_source_t<f16_t>(a, inv, st);
    default: set_error("smoe_group_by_source: unknown dtype %d", dtype); return SMOE_ERR_DTYPE;
  }
}

int launch_group(const GroupArgs& a, int dtype, hipStream_t st) {
  switch (dtype) {
    case SMOE_F32: return launch_group_t<float>(a, st);
    case SMOE_BF16: return launch_group_t<bf16_t>(a, st);
    case SMOE_F16: return launch_group_t<f16_t>(a, st);
    default: set_error("smoe_group: unknown dtype %d", dtype); return SMOE_ERR_DTYPE;
  }
}

}  // namespace smoe
