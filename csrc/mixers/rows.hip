// Row-wise kernels around an fp32 residual stream: embedding rows (optionally with a
// sinusoidal position vector), the fused "post-norm add + next pre-norm" step, the layer
// norm (weight and bias) that adds a sublayer's output to the residual, the tanh cap of
// the logits, per-head gated output norm, activations
// (relu^2, clamped GLU, gelu GLU, gelu * token-side embedding) and the weighted row scatter-add
// that combines expert outputs.
#include "mx_common.h"

namespace mx {

// out = table[id] * scale (+ a sinusoidal position vector when freqs is given: column 2i
// gets sin(p f_i), column 2i+1 cos(p f_i), with the angle p f_i formed in fp32)
template <typename T>
__global__ void embed_rows_kernel(float* __restrict__ out, const int* __restrict__ ids,
                                  const T* __restrict__ table, int width, int vocab, float scale,
                                  const int* __restrict__ positions, const float* __restrict__ freqs) {
  const int row = blockIdx.x;
  int id = ids[row];
  if (id < 0 || id >= vocab) id = 0;
  const float p = freqs != nullptr ? (float)positions[row] : 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = ld(table, (long)id * width + i) * scale;
    if (freqs != nullptr) {
      const float a = p * freqs[i >> 1];
      v += (i & 1) ? cosf(a) : sinf(a);
    }
    out[(long)row * width + i] = v;
  }
}

// layer norm with weight and bias, ln(u) = (u - mean) / sqrt(var + eps) * w + b with var
// the mean squared deviation (two passes), around an fp32 residual x:
//   y given:            x += ln(y);  cast = x
//   y null, out null:   x  = ln(x);  cast = x
//   y null, out given:  out = ln(x)  (x untouched)
template <typename TY, typename TO, int NT>
__global__ void layer_norm_kernel(float* __restrict__ x, const TY* __restrict__ y, long y_stride,
                                  const float* __restrict__ w, const float* __restrict__ b,
                                  TO* __restrict__ out, TO* __restrict__ cast, int width, float eps) {
  __shared__ float red[NT / 64];
  const long row = blockIdx.x;
  float* xr = x + row * width;
  const TY* yr = y != nullptr ? y + row * y_stride : nullptr;
  auto src = [&](int i) { return yr != nullptr ? ld(yr, i) : xr[i]; };
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) sum += src(i);
  const float mean = block_sum<NT>(sum, red) / (float)width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float d = src(i) - mean;
    ss += d * d;
  }
  const float r = 1.0f / sqrtf(block_sum<NT>(ss, red) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += NT) {
    const float v = (src(i) - mean) * r * w[i] + b[i];
    if (out != nullptr) {
      st(out, row * width + i, v);
    } else {
      const float nx = yr != nullptr ? xr[i] + v : v;
      xr[i] = nx;
      if (cast != nullptr) st(cast, row * width + i, nx);
    }
  }
}

// x <- cap * tanh(x / cap); infinite entries stay
__global__ void tanh_cap_kernel(float* __restrict__ x, long n, float cap) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float v = x[i];
    if (isfinite(v)) x[i] = cap * tanhf(v / cap);
  }
}

// residual (fp32, in place): x += rms_norm(y) * wb (+ add_vec);
// out = rms_norm(x) * next_w (TO);  cast = x (TO).  Every part is optional.
template <typename TY, typename TO, int NT>
__global__ void add_rms_norm_kernel(float* __restrict__ x, const TY* __restrict__ y, long y_stride,
                                    const float* __restrict__ wb, const float* __restrict__ add_vec,
                                    const float* __restrict__ next_w, TO* __restrict__ out,
                                    TO* __restrict__ cast, int width, float eps) {
  __shared__ float red[NT / 64];
  const long row = blockIdx.x;
  float* xr = x + row * width;
  if (y != nullptr) {
    const TY* yr = y + row * y_stride;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += NT) {
      const float v = ld(yr, i);
      ss += v * v;
    }
    ss = block_sum<NT>(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += NT) {
      float v = xr[i] + ld(yr, i) * r * wb[i];
      if (add_vec != nullptr) v += add_vec[i];
      xr[i] = v;
    }
  } else if (add_vec != nullptr) {
    for (int i = threadIdx.x; i < width; i += NT) xr[i] += add_vec[i];
  }
  // each thread re-reads only what it wrote itself: no barrier needed
  if (out != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += NT) {
      const float v = xr[i];
      ss += v * v;
    }
    ss = block_sum<NT>(ss, red);
    const float r = 1.0f / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += NT) st(out, row * width + i, xr[i] * r * next_w[i]);
  }
  if (cast != nullptr)
    for (int i = threadIdx.x; i < width; i += NT) st(cast, row * width + i, xr[i]);
}

// one wave per (row, head): out = o / rms(o) * w * sigmoid(gate)
template <typename TG, typename TO>
__global__ void head_rms_gate_kernel(TO* __restrict__ out, const float* __restrict__ o,
                                     const float* __restrict__ w, const TG* __restrict__ gate,
                                     long gate_stride, long pairs, int heads, int dv, float eps) {
  const long pair = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long row = pair / heads;
  const int h = (int)(pair % heads);
  const float* op = o + (row * heads + h) * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += 64) ss += op[i] * op[i];
  ss = ft::wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int i = lane; i < dv; i += 64) {
    const float g = sigmoidf_(ld(gate, row * gate_stride + (long)h * dv + i));
    st(out, (row * heads + h) * dv + i, op[i] * r * w[i] * g);
  }
}

template <typename T>
__global__ void relu_sq_kernel(T* __restrict__ x, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float v = fmaxf(ld(x, i), 0.f);
    st(x, i, v * v);
  }
}

// out[r, c] = relu(u[r, c])^2 for the first ff columns of wider rows
template <typename T>
__global__ void relu_sq_rows_kernel(T* __restrict__ out, const T* __restrict__ u, long u_stride, long rows, int ff) {
  const long n = rows * ff;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float v = fmaxf(ld(u, (i / ff) * u_stride + i % ff), 0.f);
    st(out, i, v * v);
  }
}

// out[row] += sum_k w[row, k] * y[idx[row, k]]: combines the outputs of the experts each
// row chose, y being in another row order (sorted by expert).  grid rows.
template <typename TY>
__global__ void gather_add_rows_kernel(float* __restrict__ out, const TY* __restrict__ y,
                                       const int* __restrict__ idx, const float* __restrict__ w, int top,
                                       int width, long y_rows) {
  const long row = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const long src = idx[row * top + k];
      if (src >= 0 && src < y_rows) acc += w[row * top + k] * ld(y, src * width + c);
    }
    out[row * width + c] += acc;
  }
}

// rows [gate (ff) | up (ff) | ...]: g = min(gate, limit), u = clamp(up, +-limit),
// out = g * sigmoid(1.702 g) * (u + 1)
template <typename T>
__global__ void clamp_swiglu_kernel(T* __restrict__ out, const T* __restrict__ gu, long gu_stride,
                                    long rows, int ff, float limit) {
  const long n = rows * ff;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long r = i / ff;
    const int c = (int)(i % ff);
    const float g = fminf(ld(gu, r * gu_stride + c), limit);
    const float u = fminf(fmaxf(ld(gu, r * gu_stride + ff + c), -limit), limit);
    st(out, i, g * sigmoidf_(1.702f * g) * (u + 1.0f));
  }
}

__device__ __forceinline__ float gelu_tanh_(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// rows [gate (ff) | up (ff)]: out = gelu_tanh(gate) * up
template <typename T>
__global__ void gelu_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, long gu_stride, long rows, int ff) {
  const long n = rows * ff;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long r = i / ff;
    const int c = (int)(i % ff);
    st(out, i, gelu_tanh_(ld(gu, r * gu_stride + c)) * ld(gu, r * gu_stride + ff + c));
  }
}

template <typename T>
__global__ void side_gate_kernel(T* __restrict__ out, const T* __restrict__ gpre,
                                 const T* __restrict__ table, long table_stride,
                                 const int* __restrict__ ids, int col0, long rows, int sd, int vocab) {
  const long n = rows * sd;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long r = i / sd;
    const int c = (int)(i % sd);
    int id = ids[r];
    if (id < 0 || id >= vocab) id = 0;
    st(out, i, gelu_tanh_(ld(gpre, i)) * ld(table, (long)id * table_stride + col0 + c));
  }
}

// out[rows[i]] += w_i * y[i]; rows == nullptr: identity.  No row repeats within a call.
template <typename TY, typename TW>
__global__ void scale_add_rows_kernel(float* __restrict__ out, const TY* __restrict__ y,
                                      const int* __restrict__ rows, const TW* __restrict__ weights,
                                      int sigmoid, int width, int out_rows) {
  const long i = blockIdx.x;
  const long dst = rows != nullptr ? rows[i] : i;
  if (dst < 0 || dst >= out_rows) return;
  float w = ld(weights, i);
  if (sigmoid) w = sigmoidf_(w);
  for (int c = threadIdx.x; c < width; c += blockDim.x)
    out[dst * width + c] += w * ld(y, i * width + c);
}

}  // namespace mx

using namespace mx;

extern "C" int mx_embed_rows(float* out, const int* ids, const void* table, int bf16, int rows,
                             int width, int vocab, float scale, const int* positions, const float* freqs,
                             hipStream_t s) {
  if (rows <= 0) return 0;
  if (freqs != nullptr && positions == nullptr) return -1;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((embed_rows_kernel<T>), dim3(rows), dim3(256), 0, s, out, ids,
                                         (const T*)table, width, vocab, scale, positions, freqs));
  return (int)hipGetLastError();
}

template <typename TY, typename TO>
static void launch_layer_norm(float* x, const void* y, long ys, const float* w, const float* b, void* out,
                              void* cast, int rows, int width, float eps, hipStream_t s) {
  hipLaunchKernelGGL((layer_norm_kernel<TY, TO, 256>), dim3(rows), dim3(256), 0, s, x, (const TY*)y, ys, w, b,
                     (TO*)out, (TO*)cast, width, eps);
}

extern "C" int mx_layer_norm(float* x, const void* y, int y_bf16, long y_stride, const float* w, const float* b,
                             void* out, void* cast, int out_bf16, int rows, int width, float eps, hipStream_t s) {
  if (rows <= 0) return 0;
  if (y != nullptr && out != nullptr) return -1;
  if (y_bf16) {
    if (out_bf16) launch_layer_norm<bf16_t, bf16_t>(x, y, y_stride, w, b, out, cast, rows, width, eps, s);
    else launch_layer_norm<bf16_t, float>(x, y, y_stride, w, b, out, cast, rows, width, eps, s);
  } else {
    if (out_bf16) launch_layer_norm<float, bf16_t>(x, y, y_stride, w, b, out, cast, rows, width, eps, s);
    else launch_layer_norm<float, float>(x, y, y_stride, w, b, out, cast, rows, width, eps, s);
  }
  return (int)hipGetLastError();
}

template <typename TY, typename TO>
static void launch_add_rms(float* x, const void* y, long ys, const float* wb, const float* av,
                           const float* nw, void* out, void* cast, int rows, int width, float eps,
                           hipStream_t s) {
  hipLaunchKernelGGL((add_rms_norm_kernel<TY, TO, 256>), dim3(rows), dim3(256), 0, s, x, (const TY*)y,
                     ys, wb, av, nw, (TO*)out, (TO*)cast, width, eps);
}

extern "C" int mx_add_rms_norm(float* x, const void* y, int y_bf16, long y_stride, const float* wb,
                               const float* add_vec, const float* next_w, void* out, void* cast,
                               int out_bf16, int rows, int width, float eps, hipStream_t s) {
  if (rows <= 0) return 0;
  if (y_bf16) {
    if (out_bf16) launch_add_rms<bf16_t, bf16_t>(x, y, y_stride, wb, add_vec, next_w, out, cast, rows, width, eps, s);
    else launch_add_rms<bf16_t, float>(x, y, y_stride, wb, add_vec, next_w, out, cast, rows, width, eps, s);
  } else {
    if (out_bf16) launch_add_rms<float, bf16_t>(x, y, y_stride, wb, add_vec, next_w, out, cast, rows, width, eps, s);
    else launch_add_rms<float, float>(x, y, y_stride, wb, add_vec, next_w, out, cast, rows, width, eps, s);
  }
  return (int)hipGetLastError();
}

extern "C" int mx_head_rms_gate(void* out, int out_bf16, const float* o, const float* w,
                                const void* gate, int gate_bf16, long gate_stride, long rows, int heads,
                                int dv, float eps, hipStream_t s) {
  const long pairs = rows * heads;
  if (pairs <= 0) return 0;
  const dim3 grid((unsigned)((pairs + 3) / 4)), block(256);
  if (gate_bf16 && out_bf16)
    hipLaunchKernelGGL((head_rms_gate_kernel<bf16_t, bf16_t>), grid, block, 0, s, (bf16_t*)out, o, w,
                       (const bf16_t*)gate, gate_stride, pairs, heads, dv, eps);
  else if (!gate_bf16 && !out_bf16)
    hipLaunchKernelGGL((head_rms_gate_kernel<float, float>), grid, block, 0, s, (float*)out, o, w,
                       (const float*)gate, gate_stride, pairs, heads, dv, eps);
  else
    return -1;
  return (int)hipGetLastError();
}

static inline unsigned ew_grid(long n) {
  long g = (n + 255) / 256;
  return (unsigned)(g < 1 ? 1 : g > 65535 ? 65535 : g);
}

extern "C" int mx_tanh_cap(float* x, long n, float cap, hipStream_t s) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return -1;
  hipLaunchKernelGGL(tanh_cap_kernel, dim3(ew_grid(n)), dim3(256), 0, s, x, n, cap);
  return (int)hipGetLastError();
}

extern "C" int mx_relu_sq(void* x, int bf16, long n, hipStream_t s) {
  if (n <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((relu_sq_kernel<T>), dim3(ew_grid(n)), dim3(256), 0, s, (T*)x, n));
  return (int)hipGetLastError();
}

extern "C" int mx_relu_sq_rows(void* out, const void* u, int bf16, long u_stride, long rows, int ff, hipStream_t s) {
  if (rows * ff <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((relu_sq_rows_kernel<T>), dim3(ew_grid(rows * ff)), dim3(256), 0, s,
                                         (T*)out, (const T*)u, u_stride, rows, ff));
  return (int)hipGetLastError();
}

extern "C" int mx_gather_add_rows(float* out, const void* y, int y_bf16, const int* idx, const float* w, long rows,
                                  int top, int width, long y_rows, hipStream_t s) {
  if (rows <= 0 || top <= 0) return 0;
  if (rows > 0x7fffffffL) return -1;
  MX_DISPATCH_T(y_bf16, hipLaunchKernelGGL((gather_add_rows_kernel<T>), dim3((unsigned)rows), dim3(256), 0, s, out,
                                           (const T*)y, idx, w, top, width, y_rows));
  return (int)hipGetLastError();
}

extern "C" int mx_clamp_swiglu(void* out, const void* gu, int bf16, long gu_stride, long rows, int ff,
                               float limit, hipStream_t s) {
  if (rows * ff <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((clamp_swiglu_kernel<T>), dim3(ew_grid(rows * ff)), dim3(256), 0,
                                         s, (T*)out, (const T*)gu, gu_stride, rows, ff, limit));
  return (int)hipGetLastError();
}

extern "C" int mx_gelu_glu(void* out, const void* gu, int bf16, long gu_stride, long rows, int ff, hipStream_t s) {
  if (rows * ff <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((gelu_glu_kernel<T>), dim3(ew_grid(rows * ff)), dim3(256), 0, s, (T*)out,
                                         (const T*)gu, gu_stride, rows, ff));
  return (int)hipGetLastError();
}

extern "C" int mx_side_gate(void* out, const void* gpre, const void* table, int bf16, long table_stride,
                            const int* ids, int col0, long rows, int sd, int vocab, hipStream_t s) {
  if (rows * sd <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((side_gate_kernel<T>), dim3(ew_grid(rows * sd)), dim3(256), 0, s,
                                         (T*)out, (const T*)gpre, (const T*)table, table_stride, ids, col0,
                                         rows, sd, vocab));
  return (int)hipGetLastError();
}

extern "C" int mx_scale_add_rows(float* out, const void* y, int y_bf16, const int* rows,
                                 const void* weights, int w_bf16, int sigmoid, long n, int width,
                                 int out_rows, hipStream_t s) {
  if (n <= 0) return 0;
  const dim3 grid((unsigned)n), block(256);
  if (y_bf16 && w_bf16)
    hipLaunchKernelGGL((scale_add_rows_kernel<bf16_t, bf16_t>), grid, block, 0, s, out, (const bf16_t*)y,
                       rows, (const bf16_t*)weights, sigmoid, width, out_rows);
  else if (y_bf16)
    hipLaunchKernelGGL((scale_add_rows_kernel<bf16_t, float>), grid, block, 0, s, out, (const bf16_t*)y,
                       rows, (const float*)weights, sigmoid, width, out_rows);
  else if (w_bf16)
    return -1;
  else
    hipLaunchKernelGGL((scale_add_rows_kernel<float, float>), grid, block, 0, s, out, (const float*)y,
                       rows, (const float*)weights, sigmoid, width, out_rows);
  return (int)hipGetLastError();
}
