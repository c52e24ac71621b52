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

// a value of a row that is fp32 or bf16, decided at run time (uniform over the launch)
__device__ __forceinline__ float ldx(const void* p, int bf16, long i) {
  return bf16 ? ft::bf16_to_f32(((const bf16_t*)p)[i]) : ((const float*)p)[i];
}

// x (fp32 residual) = embed[cur] * scale + table[hash] per row (without `embed`: x +=
// table[hash]), hash = (prev * mul_prev + cur * mul_cur) mod
// buckets with prev the token before the row's own in its sequence: the row above within a
// segment, last_tok[slot] for a segment's first row (pos0 > 0), and for a sequence's first
// token row `buckets` instead.  One workgroup per row; pair_last_kernel stores each
// segment's last token afterwards (a second launch: another row of the segment may still
// be reading the old one).
template <typename T>
__global__ void pair_embed_add_kernel(float* __restrict__ x, const int* __restrict__ ids,
                                      const T* __restrict__ table, int width, long mul_prev, long mul_cur,
                                      int buckets, const int* __restrict__ start, const int* __restrict__ pos0,
                                      const int* __restrict__ slot, int num_segs, const int* __restrict__ last_tok,
                                      int num_slots, const T* __restrict__ embed, int vocab, float scale) {
  const int row = blockIdx.x;
  if (embed != nullptr) {                 // every row gets its embedding row, padding rows too
    int id = ids[row];
    if (id < 0 || id >= vocab) id = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x)
      x[(long)row * width + i] = ld(embed, (long)id * width + i) * scale;
  }
  if (row >= start[num_segs]) return;
  int lo_s = 0, hi_s = num_segs;
  while (hi_s - lo_s > 1) {
    const int mid = (lo_s + hi_s) >> 1;
    if (start[mid] <= row) lo_s = mid; else hi_s = mid;
  }
  const int sg = lo_s;
  const int sl = slot[sg];
  if (sl < 0 || sl >= num_slots) return;
  long prev;
  if (row > start[sg]) prev = ids[row - 1];
  else prev = pos0[sg] > 0 ? last_tok[sl] : -1;
  long idx = buckets;
  if (prev >= 0) {
    idx = (prev * mul_prev + (long)ids[row] * mul_cur) % buckets;
    if (idx < 0) idx += buckets;
  }
  for (int i = threadIdx.x; i < width; i += blockDim.x) x[(long)row * width + i] += ld(table, idx * width + i);
}

__global__ void pair_last_kernel(const int* __restrict__ ids, const int* __restrict__ start,
                                 const int* __restrict__ slot, int num_segs, int* __restrict__ last_tok,
                                 int num_slots) {
  const int sg = blockIdx.x * blockDim.x + threadIdx.x;
  if (sg >= num_segs) return;
  const int sl = slot[sg];
  const int a = start[sg], b = start[sg + 1];
  if (sl < 0 || sl >= num_slots || b <= a) return;
  last_tok[sl] = ids[b - 1];
}

// residual (fp32, in place): x += mult * (y1 + y2);  out = rms_norm(x) * next_w (TO).
// y1 / y2 are fp32 or bf16 each and optional, as is out.
template <typename TO, int NT>
__global__ void add_scaled_rms_norm_kernel(float* __restrict__ x, const void* __restrict__ y1, int y1_bf16,
                                           long y1_stride, const void* __restrict__ y2, int y2_bf16,
                                           long y2_stride, float mult, const float* __restrict__ next_w,
                                           TO* __restrict__ out, int width, float eps) {
  __shared__ float red[NT / 64];
  const long row = blockIdx.x;
  float* xr = x + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    float v = xr[i];
    if (y1 != nullptr) {
      float y = ldx(y1, y1_bf16, row * y1_stride + i);
      if (y2 != nullptr) y += ldx(y2, y2_bf16, row * y2_stride + i);
      v += mult * y;
      xr[i] = v;
    }
    ss += v * v;
  }
  if (out == nullptr) return;
  ss = block_sum<NT>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)width + eps);
  // each thread re-reads only what it wrote itself
  for (int i = threadIdx.x; i < width; i += NT) st(out, row * width + i, xr[i] * r * next_w[i]);
}

// out (fp32) = scale * (a / rms(a) * wa + b / rms(b) * wb), one workgroup per row
template <typename T, int NT>
__global__ void dual_rms_mean_kernel(float* __restrict__ out, const T* __restrict__ a, long a_stride,
                                     const T* __restrict__ b, long b_stride, const float* __restrict__ wa,
                                     const float* __restrict__ wb, int width, float eps, float scale) {
  __shared__ float red[NT / 64];
  const long row = blockIdx.x;
  const T* ar = a + row * a_stride;
  const T* br = b + row * b_stride;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float u = ld(ar, i), v = ld(br, i);
    sa += u * u;
    sb += v * v;
  }
  sa = block_sum<NT>(sa, red);
  sb = block_sum<NT>(sb, red);
  const float ra = 1.0f / sqrtf(sa / (float)width + eps), rb = 1.0f / sqrtf(sb / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += NT)
    out[row * width + i] = scale * (ld(ar, i) * ra * wa[i] + ld(br, i) * rb * wb[i]);
}

// out = o * sigmoid(g), o fp32 dense rows, g rows g_stride apart
template <typename TG, typename TO>
__global__ void sigmoid_gate_kernel(TO* __restrict__ out, const float* __restrict__ o, const TG* __restrict__ g,
                                    long g_stride, long rows, int n) {
  const long total = rows * n;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long r = i / n;
    const int c = (int)(i % n);
    st(out, i, o[i] * sigmoidf_(ld(g, r * g_stride + c)));
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

// one wave per (row, head): out = o / rms(o) * w * sigmoid(gate), or * silu(gate)
template <typename TG, typename TO>
__global__ void head_rms_gate_kernel(TO* __restrict__ out, const float* __restrict__ o,
                                     const float* __restrict__ w, const TG* __restrict__ gate,
                                     long gate_stride, long pairs, int heads, int dv, float eps, int silu) {
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
    const float gp = ld(gate, row * gate_stride + (long)h * dv + i);
    const float g = silu ? gp * sigmoidf_(gp) : sigmoidf_(gp);
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

// rows [gate (ff) | up (ff)]: out = gelu_tanh(gate) * up, or relu(gate) * up
template <typename T>
__global__ void gelu_glu_kernel(T* __restrict__ out, const T* __restrict__ gu, long gu_stride, long rows, int ff,
                                int relu) {
  const long n = rows * ff;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const long r = i / ff;
    const int c = (int)(i % ff);
    const float g = ld(gu, r * gu_stride + c);
    st(out, i, (relu ? fmaxf(g, 0.f) : gelu_tanh_(g)) * ld(gu, r * gu_stride + ff + c));
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
                                int dv, float eps, int silu, hipStream_t s) {
  const long pairs = rows * heads;
  if (pairs <= 0) return 0;
  const dim3 grid((unsigned)((pairs + 3) / 4)), block(256);
  if (gate_bf16 && out_bf16)
    hipLaunchKernelGGL((head_rms_gate_kernel<bf16_t, bf16_t>), grid, block, 0, s, (bf16_t*)out, o, w,
                       (const bf16_t*)gate, gate_stride, pairs, heads, dv, eps, silu);
  else if (!gate_bf16 && !out_bf16)
    hipLaunchKernelGGL((head_rms_gate_kernel<float, float>), grid, block, 0, s, (float*)out, o, w,
                       (const float*)gate, gate_stride, pairs, heads, dv, eps, silu);
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

extern "C" int mx_gelu_glu(void* out, const void* gu, int bf16, long gu_stride, long rows, int ff, int relu,
                           hipStream_t s) {
  if (rows * ff <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((gelu_glu_kernel<T>), dim3(ew_grid(rows * ff)), dim3(256), 0, s, (T*)out,
                                         (const T*)gu, gu_stride, rows, ff, relu));
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

extern "C" int mx_pair_embed_add(float* x, const int* ids, const void* table, int bf16, int rows, int width,
                                 long mul_prev, long mul_cur, int buckets, const int* start, const int* pos0,
                                 const int* slot, int num_segs, int* last_tok, int num_slots, const void* embed,
                                 int vocab, float scale, hipStream_t s) {
  if (rows <= 0 || num_segs <= 0) return 0;
  if (buckets < 1 || width < 1) return -1;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((pair_embed_add_kernel<T>), dim3(rows), dim3(256), 0, s, x, ids,
                                         (const T*)table, width, mul_prev, mul_cur, buckets, start, pos0, slot,
                                         num_segs, last_tok, num_slots, (const T*)embed, vocab, scale));
  hipLaunchKernelGGL(pair_last_kernel, dim3((num_segs + 63) / 64), dim3(64), 0, s, ids, start, slot, num_segs, last_tok,
                     num_slots);
  return (int)hipGetLastError();
}

extern "C" int mx_add_scaled_rms_norm(float* x, const void* y1, int y1_bf16, long y1_stride, const void* y2,
                                      int y2_bf16, long y2_stride, float mult, const float* next_w, void* out,
                                      int out_bf16, int rows, int width, float eps, hipStream_t s) {
  if (rows <= 0) return 0;
  if (y1 == nullptr && (y2 != nullptr || out == nullptr)) return -1;
  if (out_bf16)
    hipLaunchKernelGGL((add_scaled_rms_norm_kernel<bf16_t, 256>), dim3(rows), dim3(256), 0, s, x, y1, y1_bf16,
                       y1_stride, y2, y2_bf16, y2_stride, mult, next_w, (bf16_t*)out, width, eps);
  else
    hipLaunchKernelGGL((add_scaled_rms_norm_kernel<float, 256>), dim3(rows), dim3(256), 0, s, x, y1, y1_bf16,
                       y1_stride, y2, y2_bf16, y2_stride, mult, next_w, (float*)out, width, eps);
  return (int)hipGetLastError();
}

extern "C" int mx_dual_rms_mean(float* out, const void* a, long a_stride, const void* b, long b_stride, int bf16,
                                const float* wa, const float* wb, int rows, int width, float eps, float scale,
                                hipStream_t s) {
  if (rows <= 0) return 0;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((dual_rms_mean_kernel<T, 256>), dim3(rows), dim3(256), 0, s, out,
                                         (const T*)a, a_stride, (const T*)b, b_stride, wa, wb, width, eps, scale));
  return (int)hipGetLastError();
}

extern "C" int mx_sigmoid_gate(void* out, int out_bf16, const float* o, const void* g, int g_bf16, long g_stride,
                               long rows, int n, hipStream_t s) {
  if (rows * n <= 0) return 0;
  const dim3 grid(ew_grid(rows * n)), block(256);
  if (g_bf16 && out_bf16)
    hipLaunchKernelGGL((sigmoid_gate_kernel<bf16_t, bf16_t>), grid, block, 0, s, (bf16_t*)out, o, (const bf16_t*)g,
                       g_stride, rows, n);
  else if (!g_bf16 && !out_bf16)
    hipLaunchKernelGGL((sigmoid_gate_kernel<float, float>), grid, block, 0, s, (float*)out, o, (const float*)g,
                       g_stride, rows, n);
  else
    return -1;
  return (int)hipGetLastError();
}
