// Mixture-of-experts routing: softmax over all experts (fp32), an additive selection
// bias that does not enter the weights, group-limited selection (only the experts of
// the `keep` best of `groups` equal groups of neighbours stay eligible; a group's score
// is its best biased score; excluded experts count as -infinity), then the `top`
// eligible experts with the largest biased scores.  Weights = the chosen experts'
// unbiased softmax scores, not renormalised.  One wave per token; ties go to the lower
// index.  A second router (moe_top_logits) chooses on the logits and renormalises over
// the chosen ones.
#include "mx_common.h"

namespace mx {

struct Best {
  float v;
  int i;
};

__device__ __forceinline__ Best better(Best a, Best b) {
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__device__ __forceinline__ Best wave_best(Best x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Best y;
    y.v = __shfl_xor(x.v, o, 64);
    y.i = __shfl_xor(x.i, o, 64);
    x = better(x, y);
  }
  return x;
}

__global__ void __launch_bounds__(64)
moe_topk_kernel(int* __restrict__ idx, float* __restrict__ wts, const float* __restrict__ z,
                const float* __restrict__ corr, int experts, int top, int groups, int keep) {
  extern __shared__ float sm[];
  float* s = sm;                    // softmax scores
  float* ch = sm + experts;         // biased scores, -inf once excluded or taken
  float* gs = sm + 2 * experts;     // group scores
  const long row = blockIdx.x;
  const int lane = threadIdx.x;
  const float* zr = z + row * experts;
  float mx_ = -INFINITY;
  for (int e = lane; e < experts; e += 64) mx_ = fmaxf(mx_, zr[e]);
  mx_ = ft::wave_max(mx_);
  float sum = 0.f;
  for (int e = lane; e < experts; e += 64) {
    const float p = expf(zr[e] - mx_);
    s[e] = p;
    sum += p;
  }
  sum = ft::wave_sum(sum);
  for (int e = lane; e < experts; e += 64) {
    const float p = s[e] / sum;
    s[e] = p;
    ch[e] = p + corr[e];
  }
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int gsz = experts / groups;
    for (int g = lane; g < groups; g += 64) {
      float b = -INFINITY;
      for (int e = g * gsz; e < (g + 1) * gsz; ++e) b = fmaxf(b, ch[e]);
      gs[g] = b;
    }
    __syncthreads();
    // the keep best groups get +inf as a mark; the others' experts are excluded
    for (int k = 0; k < keep; ++k) {
      Best b{-INFINITY, 1 << 30};
      for (int g = lane; g < groups; g += 64)
        if (gs[g] != INFINITY) b = better(b, Best{gs[g], g});
      b = wave_best(b);
      if (lane == 0 && b.i < groups) gs[b.i] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < experts; e += 64)
      if (gs[e / gsz] != INFINITY) ch[e] = -INFINITY;
    __syncthreads();
  }
  for (int k = 0; k < top; ++k) {
    Best b{-INFINITY, 1 << 30};
    for (int e = lane; e < experts; e += 64) b = better(b, Best{ch[e], e});
    b = wave_best(b);
    const int e = b.i < experts ? b.i : 0;
    if (lane == 0) {
      idx[row * top + k] = e;
      wts[row * top + k] = s[e];
      ch[e] = -INFINITY;
    }
    __syncthreads();
  }
}

// Routing on the logits themselves: the `top` largest logits of a row are chosen (ties to
// the lower index) and weighted by the softmax over just those.  One wave per token.
__global__ void __launch_bounds__(64)
moe_top_logits_kernel(int* __restrict__ idx, float* __restrict__ wts, const float* __restrict__ z, int experts,
                      int top) {
  extern __shared__ float sm[];
  float* ch = sm;                   // logits, -inf once taken
  float* val = sm + experts;        // the chosen logits, largest first
  const long row = blockIdx.x;
  const int lane = threadIdx.x;
  const float* zr = z + row * experts;
  for (int e = lane; e < experts; e += 64) ch[e] = zr[e];
  __syncthreads();
  for (int k = 0; k < top; ++k) {
    Best b{-INFINITY, 1 << 30};
    for (int e = lane; e < experts; e += 64) b = better(b, Best{ch[e], e});
    b = wave_best(b);
    const int e = b.i < experts ? b.i : 0;
    if (lane == 0) {
      idx[row * top + k] = e;
      val[k] = b.v;
      ch[e] = -INFINITY;
    }
    __syncthreads();
  }
  float sum = 0.f;
  for (int k = lane; k < top; k += 64) sum += expf(val[k] - val[0]);
  sum = ft::wave_sum(sum);
  for (int k = lane; k < top; k += 64) wts[row * top + k] = expf(val[k] - val[0]) / sum;
}

}  // namespace mx

extern "C" int mx_moe_top_logits(int* idx, float* wts, const float* z, long rows, int experts, int top,
                                 hipStream_t s) {
  if (rows <= 0) return 0;
  if (experts < 1 || top < 1 || top > experts) return -1;
  const size_t lds = (size_t)(experts + top) * sizeof(float);
  if (lds > 60 * 1024) return -2;
  hipLaunchKernelGGL(mx::moe_top_logits_kernel, dim3((unsigned)rows), dim3(64), lds, s, idx, wts, z, experts, top);
  return (int)hipGetLastError();
}

extern "C" int mx_moe_topk(int* idx, float* wts, const float* z, const float* corr, long rows, int experts,
                           int top, int groups, int keep, hipStream_t s) {
  if (rows <= 0) return 0;
  if (experts < 1 || top < 1 || top > experts || groups < 1 || experts % groups || keep < 1 || keep > groups)
    return -1;
  const size_t lds = (size_t)(2 * experts + groups) * sizeof(float);
  if (lds > 60 * 1024) return -2;
  hipLaunchKernelGGL(mx::moe_topk_kernel, dim3((unsigned)rows), dim3(64), lds, s, idx, wts, z, corr, experts,
                     top, groups, keep);
  return (int)hipGetLastError();
}
