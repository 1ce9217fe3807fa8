// Routing prep: deterministic stable counting sort of flattened expert ids + inclusive offsets.
// Counterpart of flatten_sort_count (scattermoe/parallel_experts.py:14-21), which runs
// torch.sort + bincount + cumsum.  Keys are tiny (expert ids), so a counting sort with an LDS
// histogram per block and a wavefront match/rank scatter replaces the generic 64-bit radix sort.
//
// Inputs of up to 16384 rows (one workgroup of 4 or 16 waves) run in ONE launch; larger ones in three:
//   hist    : per-chunk LDS histogram                       -> counts[chunk][E]
//   scan    : exclusive scan over (expert-major, chunk)     -> bases[chunk][E], off[E]
//   scatter : stable rank inside the chunk + base           -> eid_out, idx_out
// The result is independent of scheduling: every output position is a pure function of the input.
#include "common.hpp"
#include <mutex>

namespace smoe {

static constexpr int kRouteThreads = 256;
static constexpr int kRouteWaves = kRouteThreads / 64;
static constexpr int kRouteChunk = 4096;       // elements per block
static constexpr int kRouteMaxE = 2048;        // LDS: (waves+1) * E ints
static constexpr int kRouteFusedMax = 16384;   // rows one workgroup of 1024 threads sorts by itself (32768 rows take it
                                               // 33 us, the three launches 28 us) ...
static constexpr int kRouteFusedMaxE = 512;    // ... for at most this many experts (17 * E ints of LDS)

template <typename I>
__device__ __forceinline__ int load_id(const I* p, int64_t i) { return (int)p[i]; }

// Lanes of the wave that hold the same key as this lane (keys < 2^nbits), inactive lanes excluded.
__device__ __forceinline__ unsigned long long match_any(int key, int nbits, bool active) {
  unsigned long long m = __ballot(active);
  for (int b = 0; b < nbits; ++b) {
    const bool bit = (key >> b) & 1;
    const unsigned long long v = __ballot(bit);
    m &= bit ? v : ~v;
  }
  return m;
}

__device__ __forceinline__ int bits_for(int E) {
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  return nbits;
}

// Per-wave histogram of the wave's contiguous segment of the chunk.  wave w owns
// [chunk_lo + w*seg, chunk_lo + (w+1)*seg) ∩ [0, L).
template <typename I>
__device__ __forceinline__ void wave_histogram(const I* __restrict__ ids, int64_t seg_lo, int64_t seg_hi,
                                               int E, int* __restrict__ hist_w) {
  const int lane = lane_id();
  for (int64_t p = seg_lo + lane; p < seg_hi; p += 64) {
    const int e = load_id(ids, p);
    if ((unsigned)e < (unsigned)E) atomicAdd(&hist_w[e], 1);
  }
}

// Stable scatter of one wave's segment.  base_w[e] holds the output position of the wave's next row
// of expert e and is advanced as rounds of 64 consecutive elements are placed.
template <typename I>
__device__ __forceinline__ void wave_scatter(const I* __restrict__ ids, int64_t seg_lo, int64_t seg_hi,
                                             int E, int nbits, int* __restrict__ base_w,
                                             int64_t* __restrict__ eid_out, int64_t* __restrict__ idx_out) {
  const int lane = lane_id();
  const unsigned long long lt = (1ull << lane) - 1ull;
  for (int64_t p0 = seg_lo; p0 < seg_hi; p0 += 64) {
    const int64_t p = p0 + lane;
    const bool in = p < seg_hi;
    int e = in ? load_id(ids, p) : 0;
    const bool ok = in && (unsigned)e < (unsigned)E;
    if (!ok) e = 0;
    const unsigned long long same = match_any(e, nbits, ok);
    const int rank = __popcll(same & lt);
    const int leader = __ffsll((long long)same) - 1;   // -1 only for lanes with ok == false
    int first = 0;
    if (ok && lane == leader) first = atomicAdd(&base_w[e], __popcll(same));
    first = __shfl(first, leader < 0 ? 0 : leader, 64);
    if (ok) {
      const int pos = first + rank;
      eid_out[pos] = (int64_t)e;
      idx_out[pos] = p;
    }
  }
}

// ---- single-launch path: whole input in one block ------------------------------------------------
template <typename I, int THREADS>
__global__ __launch_bounds__(THREADS) void route_fused_kernel(
    const I* __restrict__ ids, int L, int E, int64_t* __restrict__ eid_out,
    int64_t* __restrict__ idx_out, int64_t* __restrict__ off_out) {
  constexpr int kRouteThreads = THREADS, kRouteWaves = THREADS / 64;      // this kernel's own block shape
  extern __shared__ int lds[];          // [kRouteWaves][E] wave histograms/bases, then [E] totals
  int* hist = lds;
  int* total = lds + kRouteWaves * E;
  const int tid = threadIdx.x, w = tid >> 6;
  for (int i = tid; i < (kRouteWaves + 1) * E; i += kRouteThreads) lds[i] = 0;
  __syncthreads();
  const int seg = (L + kRouteWaves - 1) / kRouteWaves;
  const int64_t lo = min((int64_t)w * seg, (int64_t)L), hi = min(lo + seg, (int64_t)L);
  wave_histogram(ids, lo, hi, E, hist + w * E);
  __syncthreads();
  // per expert: exclusive prefix over waves, total count
  for (int e = tid; e < E; e += kRouteThreads) {
    int run = 0;
    for (int ww = 0; ww < kRouteWaves; ++ww) {
      const int c = hist[ww * E + e];
      hist[ww * E + e] = run;
      run += c;
    }
    total[e] = run;
  }
  __syncthreads();
  // exclusive scan of totals over experts (wave 0, 64 experts per step), inclusive offsets out
  if (w == 0) {
    const int lane = lane_id();
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int c = e < E ? total[e] : 0;
      int incl = c;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        int v = __shfl_up(incl, d, 64);
        if (lane >= d) incl += v;
      }
      if (e < E) {
        total[e] = carry + incl - c;           // exclusive base of expert e
        off_out[e] = (int64_t)(carry + incl);  // inclusive end
      }
      carry += __shfl(incl, 63, 64);
    }
  }
  __syncthreads();
  for (int i = tid; i < kRouteWaves * E; i += kRouteThreads) hist[i] += total[i % E];
  __syncthreads();
  wave_scatter(ids, lo, hi, E, bits_for(E), hist + w * E, eid_out, idx_out);
}

// ---- three-launch path ------------------------------------------------------------------------------
template <typename I>
__global__ __launch_bounds__(kRouteThreads) void route_hist_kernel(
    const I* __restrict__ ids, int64_t L, int E, int* __restrict__ counts /*[nchunk][E]*/) {
  extern __shared__ int lds[];  // [E]
  const int tid = threadIdx.x;
  for (int i = tid; i < E; i += kRouteThreads) lds[i] = 0;
  __syncthreads();
  const int64_t lo = (int64_t)blockIdx.x * kRouteChunk;
  const int64_t hi = min(lo + kRouteChunk, L);
  for (int64_t p = lo + tid; p < hi; p += kRouteThreads) {
    const int e = load_id(ids, p);
    if ((unsigned)e < (unsigned)E) atomicAdd(&lds[e], 1);
  }
  __syncthreads();
  for (int i = tid; i < E; i += kRouteThreads) counts[(int64_t)blockIdx.x * E + i] = lds[i];
}

// One block of 16 waves.  counts[c][e] -> exclusive position of chunk c's first row of expert e.
// A wave takes the experts e = wave, wave + 16, ...; its lanes take 64 chunks at a time (wave-wide scan, carry
// between the groups of 64), so the walk over the chunks of an expert is 64 wide instead of serial.
__global__ __launch_bounds__(1024) void route_scan_kernel(int* __restrict__ counts, int nchunk, int E,
                                                         int64_t* __restrict__ off_out) {
  extern __shared__ int total[];  // [E]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  for (int e = w; e < E; e += 16) {
    int run = 0;
    for (int c0 = 0; c0 < nchunk; c0 += 64) {
      const int c = c0 + lane;
      const int v = c < nchunk ? counts[(int64_t)c * E + e] : 0;
      int incl = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        int u = __shfl_up(incl, d, 64);
        if (lane >= d) incl += u;
      }
      if (c < nchunk) counts[(int64_t)c * E + e] = run + incl - v;
      run += __shfl(incl, 63, 64);
    }
    if (lane == 0) total[e] = run;
  }
  __syncthreads();
  if (tid < 64) {
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int c = e < E ? total[e] : 0;
      int incl = c;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        int v = __shfl_up(incl, d, 64);
        if (lane >= d) incl += v;
      }
      if (e < E) {
        total[e] = carry + incl - c;
        off_out[e] = (int64_t)(carry + incl);
      }
      carry += __shfl(incl, 63, 64);
    }
  }
  __syncthreads();
  for (int64_t i = tid; i < (int64_t)nchunk * E; i += blockDim.x) counts[i] += total[i % E];
}

template <typename I>
__global__ __launch_bounds__(kRouteThreads) void route_scatter_kernel(
    const I* __restrict__ ids, int64_t L, int E, const int* __restrict__ bases /*[nchunk][E]*/,
    int64_t* __restrict__ eid_out, int64_t* __restrict__ idx_out) {
  extern __shared__ int lds[];  // [kRouteWaves][E]
  const int tid = threadIdx.x, w = tid >> 6;
  for (int i = tid; i < kRouteWaves * E; i += kRouteThreads) lds[i] = 0;
  __syncthreads();
  constexpr int seg = kRouteChunk / kRouteWaves;
  const int64_t chunk_lo = (int64_t)blockIdx.x * kRouteChunk;
  const int64_t lo = min(chunk_lo + (int64_t)w * seg, L), hi = min(lo + seg, L);
  wave_histogram(ids, lo, hi, E, lds + w * E);
  __syncthreads();
  for (int e = tid; e < E; e += kRouteThreads) {
    int run = bases[(int64_t)blockIdx.x * E + e];
    for (int ww = 0; ww < kRouteWaves; ++ww) {
      const int c = lds[ww * E + e];
      lds[ww * E + e] = run;
      run += c;
    }
  }
  __syncthreads();
  wave_scatter(ids, lo, hi, E, bits_for(E), lds + w * E, eid_out, idx_out);
}

size_t route_workspace_bytes(int64_t L, int E) {
  if (L <= kRouteChunk || (L <= kRouteFusedMax && E <= kRouteFusedMaxE)) return 0;
  return (size_t)cdiv64(L, kRouteChunk) * (size_t)E * sizeof(int);
}

template <typename I>
static int launch_route_t(const I* ids, int64_t L, int E, int64_t* eid_out, int64_t* idx_out,
                          int64_t* off_out, void* ws, hipStream_t st) {
  if (L <= kRouteChunk) {
    const size_t lds = (size_t)(kRouteWaves + 1) * E * sizeof(int);
    hipLaunchKernelGGL((route_fused_kernel<I, kRouteThreads>), dim3(1), dim3(kRouteThreads), lds, st, ids, (int)L, E,
                       eid_out, idx_out, off_out);
    return launch_status("route_fused_kernel");
  }
  if (L <= kRouteFusedMax && E <= kRouteFusedMaxE) {
    // one workgroup of 16 waves: a launch costs more than sorting 2048 rows per wave does
    const size_t lds = (size_t)(1024 / 64 + 1) * E * sizeof(int);
    hipLaunchKernelGGL((route_fused_kernel<I, 1024>), dim3(1), dim3(1024), lds, st, ids, (int)L, E,
                       eid_out, idx_out, off_out);
    return launch_status("route_fused_kernel");
  }
  const int nchunk = (int)cdiv64(L, kRouteChunk);
  int* counts = (int*)ws;
  hipLaunchKernelGGL(route_hist_kernel<I>, dim3(nchunk), dim3(kRouteThreads), (size_t)E * sizeof(int), st,
                     ids, L, E, counts);
  hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), (size_t)E * sizeof(int), st, counts, nchunk,
                     E, off_out);
  hipLaunchKernelGGL(route_scatter_kernel<I>, dim3(nchunk), dim3(kRouteThreads),
                     (size_t)kRouteWaves * E * sizeof(int), st, ids, L, E, (const int*)counts, eid_out,
                     idx_out);
  return launch_status("route_scatter_kernel");
}

// ---- routing without a caller workspace -----------------------------------------------------------------
// The per-chunk histograms of the three-launch path live in a fixed device array instead of caller memory, for
// callers that can neither allocate nor bring a workspace (code under stream capture, serving loops).  Each GPU
// holds its own copy of the array at its own address; `scratch_ptr` resolves and caches that address once per
// device.  The array keeps the previous call's contents; nothing has to start at zero, because the histogram
// launch writes every entry the later launches read.  Calls that overlap on one GPU share the array and race.
static __device__ __align__(256) unsigned char route_scratch[SMOE_ROUTE_STATIC_BYTES];

static constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

// Device address of this GPU's copy of `route_scratch` (the array's name is only a host-side handle).
static int scratch_ptr(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("smoe_route_static: cannot identify the current device (%s)", hipGetErrorString(e));
    return e != hipSuccess ? (int)e : SMOE_ERR_RANGE;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(route_scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("smoe_route_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return e != hipSuccess ? (int)e : SMOE_ERR_NULL;
    }
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

int route_static_init() {
  void* p = nullptr;
  return scratch_ptr(&p);
}

int launch_route(const void* ids, int idx_dtype, int64_t L, int E, int64_t* eid_out, int64_t* idx_out,
                 int64_t* off_out, void* ws, hipStream_t st);

int launch_route_static(const void* ids, int idx_dtype, int64_t L, int E, int64_t* eid_out, int64_t* idx_out,
                        int64_t* off_out, hipStream_t st) {
  if (E > kRouteMaxE) {          // before the buffer check: too many experts is a range error, not a workspace one
    set_error("smoe_route_static: E=%d exceeds the supported maximum %d", E, kRouteMaxE);
    return SMOE_ERR_RANGE;
  }
  const size_t need = route_workspace_bytes(L, E);
  if (need > (size_t)SMOE_ROUTE_STATIC_BYTES) {
    set_error("smoe_route_static: L=%lld rows over E=%d experts need %zu bytes of histograms, the built-in buffer "
              "holds %d (use smoe_route with a workspace)", (long long)L, E, need, SMOE_ROUTE_STATIC_BYTES);
    return SMOE_ERR_WORKSPACE;
  }
  void* ws = nullptr;
  if (need > 0) {
    if (const int rc = scratch_ptr(&ws)) return rc;
  }
  return launch_route(ids, idx_dtype, L, E, eid_out, idx_out, off_out, ws, st);
}

int launch_route(const void* ids, int idx_dtype, int64_t L, int E, int64_t* eid_out, int64_t* idx_out,
                 int64_t* off_out, void* ws, hipStream_t st) {
  if (E > kRouteMaxE) {
    set_error("smoe_route: E=%d exceeds the supported maximum %d", E, kRouteMaxE);
    return SMOE_ERR_RANGE;
  }
  switch (idx_dtype) {
    case SMOE_I64: return launch_route_t((const int64_t*)ids, L, E, eid_out, idx_out, off_out, ws, st);
    case SMOE_I32: return launch_route_t((const int32_t*)ids, L, E, eid_out, idx_out, off_out, ws, st);
    case SMOE_I16: return launch_route_t((const int16_t*)ids, L, E, eid_out, idx_out, off_out, ws, st);
    case SMOE_U8: return launch_route_t((const uint8_t*)ids, L, E, eid_out, idx_out, off_out, ws, st);
    default: set_error("smoe_route: unknown index dtype %d", idx_dtype); return SMOE_ERR_DTYPE;
  }
}

// off[e] = number of rows with id <= e, from an ascending id vector.  Boundary n (between rows n-1
// and n, with virtual ids -1 before the first row and E after the last) owns the experts in
// [eid[n-1], eid[n]) and writes n to each, so every off[e] is written exactly once.
__global__ __launch_bounds__(256) void offsets_from_sorted_kernel(const int64_t* __restrict__ eid, int64_t L,
                                                                 int E, int64_t* __restrict__ off) {
  const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n > L) return;
  int64_t lo = n > 0 ? eid[n - 1] : 0;
  int64_t cur = n < L ? eid[n] : (int64_t)E;
  if (lo < 0) lo = 0;
  if (cur > E) cur = E;
  for (int64_t e = lo; e < cur; ++e) off[e] = n;
}

int launch_offsets_from_sorted(const int64_t* eid, int64_t L, int E, int64_t* off, hipStream_t st) {
  const int64_t n = L + 1;
  hipLaunchKernelGGL(offsets_from_sorted_kernel, dim3((unsigned)cdiv64(n, 256)), dim3(256), 0, st, eid, L, E, off);
  return launch_status("offsets_from_sorted_kernel");
}

}  // namespace smoe
