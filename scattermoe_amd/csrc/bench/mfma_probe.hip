// Measurement aid of bench.py, built into a library of its own (libsmoe_bench_probe.so): not part of the MoE path,
// not in the product library or its header.  What the matrix pipe of this GPU sustains on its own.  One wave per
// SIMD on every CU issues independent 32x32x16 bf16 MFMAs on operands that stay in registers - no memory traffic,
// no LDS - so the rate is the shader clock the power management grants, and that clock depends on the operand bits
// (all-zero operands run near the nominal clock, operands with random signs and mantissas 15-25 % below it).
// bench.py reports both rates beside the roofline fraction, which is priced against the nominal peak.
#include <hip/hip_runtime.h>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned probe_u32x4;

static constexpr int PROBE_WGS = 256, PROBE_THREADS = 256, PROBE_MFMAS = 64;

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

__global__ __launch_bounds__(PROBE_THREADS) void mfma_rate_kernel(float* out, int iters, int random_operands) {
  const int t = threadIdx.x + blockIdx.x * PROBE_THREADS;
  probe_bf16x8 a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    probe_u32x4 ua, ub;
    for (int e = 0; e < 4; ++e) {
      // pairs of bf16 with exponents of values in [0.5, 2), random sign and mantissa - or zeros
      const unsigned ra = (probe_hash(t * 64 + i * 8 + e) & 0x807f807fU) | 0x3f003f00U;
      const unsigned rb = (probe_hash(t * 64 + i * 8 + e + 4) & 0x807f807fU) | 0x3f003f00U;
      ua[e] = random_operands ? ra : 0u;
      ub[e] = random_operands ? rb : 0u;
    }
    a[i] = __builtin_bit_cast(probe_bf16x8, ua);
    b[i] = __builtin_bit_cast(probe_bf16x8, ub);
  }
  probe_f32x16 acc[16];
  for (int i = 0; i < 16; ++i)
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < PROBE_MFMAS; ++m)
      acc[m & 15] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(m >> 2) & 7], b[(m + (m >> 4)) & 7], acc[m & 15], 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 16; ++i)
    for (int e = 0; e < 16; ++e) s += acc[i][e];
  out[t] = s;
}

}  // namespace

// out: 65536 floats of device memory (overwritten); *flop_out: flop count of the launch.  0 = launched,
// -1 = NULL pointer, -5 = iters out of range, > 0 = hipError_t of the launch.
extern "C" int smoe_bench_mfma_rate(float* out, int iters, int random_operands, double* flop_out, void* stream) {
  if (!out) return -1;
  if (iters < 1 || iters > (1 << 22)) return -5;
  if (flop_out) *flop_out = (double)PROBE_WGS * (PROBE_THREADS / 64) * (double)iters * PROBE_MFMAS * (2.0 * 32 * 32 * 16);
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(PROBE_WGS), dim3(PROBE_THREADS), 0, (hipStream_t)stream, out, iters,
                     random_operands != 0);
  return (int)hipGetLastError();
}
