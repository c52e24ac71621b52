// Mixture-of-experts for few rows (decode steps, hipGraph-capturable: nothing is read
// back on the host): every (row, chosen expert) pair streams its expert's weights.
//
//   moe_gu_pairs:   y[pair, c] = glu(W_gate[e] h, W_up[e] h)[c]      (clamped GLU fused)
//                   or, for experts without a gate, y[pair, c] = relu(W_up[e] h)[c]^2
//   moe_down_pairs: out[row, c] += sum_k w[row, k] * (W_down[e_k] y[row, k])[c]   (fp32)
//
// One wave per output column, lanes along the reduction axis with 16-byte loads where
// the row length allows; the few rows' activations stay in L1/L2 while each expert
// matrix is read once per pair that chose it.
#include "mx_common.h"

namespace mx {

template <typename T> struct Vec;
template <> struct Vec<float> { static constexpr int N = 4; using V = float4; };
template <> struct Vec<bf16_t> { static constexpr int N = 8; using V = uint4; };

__device__ __forceinline__ float dot_vec(const float4& a, const float4& b) {
  return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}
__device__ __forceinline__ float dot_vec(const uint4& a, const uint4& b) {
  float x[8], y[8];
  ft::load8(a, x);
  ft::load8(b, y);
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) s += x[i] * y[i];
  return s;
}

// per-lane partial of a . b over n elements (wave-strided); vec: n % N == 0 and both
// rows 16-byte aligned
template <typename T>
__device__ __forceinline__ float dot_part(const T* a, const T* b, int n, int lane, bool vec) {
  float s = 0.f;
  if (vec) {
    using V = typename Vec<T>::V;
    const V* av = reinterpret_cast<const V*>(a);
    const V* bv = reinterpret_cast<const V*>(b);
    for (int i = lane; i < n / Vec<T>::N; i += 64) s += dot_vec(av[i], bv[i]);
  } else {
    for (int i = lane; i < n; i += 64) s += ld(a, i) * ld(b, i);
  }
  return s;
}

// grid (ceil(ff / 4), pairs), 256 threads: wave w -> column 4 * blockIdx.x + w
template <typename T>
__global__ void __launch_bounds__(256)
moe_gu_pairs_kernel(T* __restrict__ y, const T* __restrict__ h, long h_stride, const int* __restrict__ idx,
                    const T* __restrict__ wgu, int top, int experts, int ff, int width, float limit,
                    int vec, int relu_sq) {
  const int pair = blockIdx.y;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= ff) return;
  const int lane = threadIdx.x & 63;
  int e = idx[pair];
  if (e < 0 || e >= experts) e = 0;
  const T* hr = h + (long)(pair / top) * h_stride;
  if (relu_sq) {
    // one matrix [ff, width] per expert
    const float u0 = ft::wave_sum(dot_part(hr, wgu + ((long)e * ff + c) * width, width, lane, vec));
    if (lane == 0) {
      T tmp[1];
      st(tmp, 0, u0);
      const float u = fmaxf(ld(tmp, 0), 0.f);
      st(y, (long)pair * ff + c, u * u);
    }
    return;
  }
  const T* wg = wgu + ((long)e * 2 * ff + c) * width;
  const T* wu = wg + (long)ff * width;
  const float g0 = ft::wave_sum(dot_part(hr, wg, width, lane, vec));
  const float u0 = ft::wave_sum(dot_part(hr, wu, width, lane, vec));
  if (lane == 0) {
    // the products leave the matrix unit in the activation dtype, like the tiled path
    T tmp[2];
    st(tmp, 0, g0);
    st(tmp, 1, u0);
    const float g = fminf(ld(tmp, 0), limit);
    const float u = fminf(fmaxf(ld(tmp, 1), -limit), limit);
    st(y, (long)pair * ff + c, g * sigmoidf_(1.702f * g) * (u + 1.0f));
  }
}

// grid (ceil(width / 4), rows)
template <typename T>
__global__ void __launch_bounds__(256)
moe_down_pairs_kernel(float* __restrict__ out, const T* __restrict__ y, const int* __restrict__ idx,
                      const float* __restrict__ wts, const T* __restrict__ wdown, int top, int experts,
                      int ff, int width, int vec) {
  const int row = blockIdx.y;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= width) return;
  const int lane = threadIdx.x & 63;
  float acc = 0.f;
  for (int k = 0; k < top; ++k) {
    int e = idx[row * top + k];
    if (e < 0 || e >= experts) e = 0;
    const float d = ft::wave_sum(dot_part(y + ((long)row * top + k) * ff, wdown + ((long)e * width + c) * ff,
                                          ff, lane, vec));
    T tmp[1];
    st(tmp, 0, d);
    acc += wts[row * top + k] * ld(tmp, 0);
  }
  if (lane == 0) out[(long)row * width + c] += acc;
}

}  // namespace mx

using namespace mx;

extern "C" int mx_moe_pairs(float* out, void* y, const void* h, int bf16, long h_stride, const int* idx,
                            const float* wts, const void* wgu, const void* wdown, long rows, int top,
                            int experts, int ff, int width, float limit, int relu_sq, hipStream_t s) {
  if (rows <= 0) return 0;
  const long pairs = rows * top;
  if (pairs > 65535 || rows > 65535) return -1;
  const int n = bf16 ? 8 : 4;
  const int vec_gu = (width % n == 0 && (h_stride * (bf16 ? 2 : 4)) % 16 == 0) ? 1 : 0;
  const int vec_dn = (ff % n == 0) ? 1 : 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((moe_gu_pairs_kernel<T>), dim3((ff + 3) / 4, (unsigned)pairs), dim3(256),
                                         0, s, (T*)y, (const T*)h, h_stride, idx, (const T*)wgu, top, experts, ff,
                                         width, limit, vec_gu, relu_sq));
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((moe_down_pairs_kernel<T>), dim3((width + 3) / 4, (unsigned)rows),
                                         dim3(256), 0, s, out, (const T*)y, idx, wts, (const T*)wdown, top,
                                         experts, ff, width, vec_dn));
  return (int)hipGetLastError();
}
