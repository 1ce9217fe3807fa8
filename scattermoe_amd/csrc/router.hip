// Router front end: softmax over the expert logits of every token, top-k selection and optional renormalisation
// of the selected probabilities, in one pass over the (T, E) logits.
//
// Counterpart in the reference: the three torch calls of the Granite injection,
// scattermoe/utils/replace_moe.py:67-71 (softmax in float -> topk -> divide by the sum of the selected ones);
// every Hugging Face MoE block the reference patches computes its routing weights this way.
//
// One wave per token.  Lane l holds logits l, l+64, ... (at most 8 per lane, i.e. E <= 512).  Selection is k
// rounds of a wave-wide arg-max; among equal values the lowest expert id wins.  All arithmetic in fp32.
// Every id written is a valid expert id whatever the logits hold: a NaN logit counts as -inf, and a row without
// any usable logit is routed as if all its logits were equal.
#include "common.hpp"

namespace smoe {

static constexpr int ROUTER_MAX_PER_LANE = 8;

template <typename T>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const T* __restrict__ logits, int64_t slt, int64_t sle,
                                                          float* __restrict__ w_out, int64_t swt, int64_t swk,
                                                          int64_t* __restrict__ i_out, int64_t sit, int64_t sik,
                                                          int64_t Tn, int E, int k, int renorm) {
  const int lane = lane_id();
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= Tn) return;
  float v[ROUTER_MAX_PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int q = 0; q < ROUTER_MAX_PER_LANE; ++q) {
    const int e = q * 64 + lane;
    v[q] = e < E ? to_f32(logits[t * slt + e * sle]) : -INFINITY;
    if (v[q] != v[q]) v[q] = -INFINITY;                        // a NaN logit never wins: its expert gets probability 0
    mx = fmaxf(mx, v[q]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  const bool none = !(mx > -INFINITY);                         // no usable logit in the row: uniform probabilities
  float sum = 0.0f;
#pragma unroll
  for (int q = 0; q < ROUTER_MAX_PER_LANE; ++q) {
    float p = none ? 1.0f : __expf(v[q] - mx);
    if (p != p) p = 1.0f;                                      // +inf - +inf: the logit is the maximum
    v[q] = q * 64 + lane < E ? p : -1.0f;                      // -1: not a candidate (probabilities are >= 0)
    sum += fmaxf(v[q], 0.0f);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
  const float inv = 1.0f / sum;
  float picked = 0.0f;          // lane j keeps the j-th selected probability (k <= 64)
  float sel_sum = 0.0f;
  for (int j = 0; j < k; ++j) {
    float best = -1.0f;
    int be = 0x7fffffff;
#pragma unroll
    for (int q = 0; q < ROUTER_MAX_PER_LANE; ++q) {
      const int e = q * 64 + lane;
      if (v[q] > best) { best = v[q]; be = e; }                // ascending e inside a lane: first maximum wins
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      if (ob > best || (ob == best && oe < be)) { best = ob; be = oe; }
    }
    const float pr = best * inv;
    if (lane == j) picked = pr;
    sel_sum += pr;
    if (lane == 0) i_out[t * sit + j * sik] = be;
    if ((be & 63) == lane) {
#pragma unroll
      for (int q = 0; q < ROUTER_MAX_PER_LANE; ++q)
        if (q == (be >> 6)) v[q] = -1.0f;                       // taken
    }
  }
  if (lane < k) w_out[t * swt + lane * swk] = renorm ? picked / sel_sum : picked;
}

int launch_topk_softmax(const void* logits, int64_t slt, int64_t sle, float* w, int64_t swt, int64_t swk,
                        int64_t* idx, int64_t sit, int64_t sik, int64_t Tn, int E, int k, int renorm, int dtype,
                        hipStream_t st) {
  const dim3 grid((unsigned)((Tn + 3) / 4)), block(256);
  switch (dtype) {
    case SMOE_F32:
      hipLaunchKernelGGL(topk_softmax_kernel<float>, grid, block, 0, st, (const float*)logits, slt, sle, w, swt, swk,
                         idx, sit, sik, Tn, E, k, renorm);
      break;
    case SMOE_BF16:
      hipLaunchKernelGGL(topk_softmax_kernel<bf16_t>, grid, block, 0, st, (const bf16_t*)logits, slt, sle, w, swt, swk,
                         idx, sit, sik, Tn, E, k, renorm);
      break;
    case SMOE_F16:
      hipLaunchKernelGGL(topk_softmax_kernel<f16_t>, grid, block, 0, st, (const f16_t*)logits, slt, sle, w, swt, swk,
                         idx, sit, sik, Tn, E, k, renorm);
      break;
    default:
      set_error("unknown dtype %d", dtype);
      return SMOE_ERR_DTYPE;
  }
  return launch_status("topk_softmax_kernel");
}

}  // namespace smoe
