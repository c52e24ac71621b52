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

// four consecutive activations as fp32
__device__ __forceinline__ void load4(const float* p, float* v) {
  const float4 u = *reinterpret_cast<const float4*>(p);
  v[0] = u.x; v[1] = u.y; v[2] = u.z; v[3] = u.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float* v) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(u.x << 16);
  v[1] = __uint_as_float(u.x & 0xffff0000u);
  v[2] = __uint_as_float(u.y << 16);
  v[3] = __uint_as_float(u.y & 0xffff0000u);
}

// The same router with its logits computed here, for few rows (decode steps): z = W h + b
// in fp32 (W, b fp32; h fp32 or bf16), one workgroup of sixteen waves per token, a wave
// per expert in turn with the lanes along the width (four elements per lane and pass when
// the rows allow 16-byte loads, several passes in flight); then wave 0 chooses as above.
constexpr int kRouteWaves = 16;

template <typename T>
__global__ void __launch_bounds__(64 * kRouteWaves)
moe_route_top_logits_kernel(int* __restrict__ idx, float* __restrict__ wts, const T* __restrict__ h, long h_stride,
                            const float* __restrict__ router, const float* __restrict__ bias, int experts,
                            int width, int top, int vec) {
  extern __shared__ float sm[];
  float* ch = sm;
  float* val = sm + experts;
  const long row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* hr = h + row * h_stride;
  for (int e = wave; e < experts; e += kRouteWaves) {
    const float* wr = router + (long)e * width;
    float acc = 0.f;
    if (vec) {
#pragma unroll 4
      for (int i = lane * 4; i < width; i += 256) {
        float x[4];
        load4(hr + i, x);
        const float4 w4 = *reinterpret_cast<const float4*>(wr + i);
        acc += x[0] * w4.x + x[1] * w4.y + x[2] * w4.z + x[3] * w4.w;
      }
    } else {
      for (int i = lane; i < width; i += 64) acc += ld(hr, i) * wr[i];
    }
    acc = ft::wave_sum(acc);
    if (lane == 0) ch[e] = acc + (bias != nullptr ? bias[e] : 0.f);
  }
  __syncthreads();
  if (wave != 0) return;
  // one wave from here on: lane 0's LDS writes are made visible to the wave's other lanes
  // by a wave-level fence instead of a workgroup barrier
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
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  float sum = 0.f;
  for (int k = lane; k < top; k += 64) sum += expf(val[k] - val[0]);
  sum = ft::wave_sum(sum);
  for (int k = lane; k < top; k += 64) wts[row * top + k] = expf(val[k] - val[0]) / sum;
}

}  // namespace mx

extern "C" int mx_moe_route_top_logits(int* idx, float* wts, const void* h, int bf16, long h_stride,
                                       const float* router, const float* bias, long rows, int experts, int width,
                                       int top, hipStream_t s) {
  if (rows <= 0) return 0;
  if (experts < 1 || top < 1 || top > experts || width < 1) return -1;
  const size_t lds = (size_t)(experts + top) * sizeof(float);
  if (lds > 60 * 1024) return -2;
  const long es = bf16 ? 2 : 4;
  const int vec = width % 4 == 0 && h_stride % 4 == 0 && ((uintptr_t)h) % (4 * es) == 0 &&
                  ((uintptr_t)router) % 16 == 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((mx::moe_route_top_logits_kernel<T>), dim3((unsigned)rows),
                                         dim3(64 * mx::kRouteWaves), lds, s, idx, wts, (const T*)h, h_stride, router,
                                         bias, experts, width, top, vec));
  return (int)hipGetLastError();
}

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
