// Short causal convolution + SiLU with a per-slot input history, and the gated delta
// rule with one decay per head and key channel over fp32 state slots.
//
// A step's rows come in segments (one per sequence): rows [start[s], start[s+1]) are
// consecutive positions pos0[s].. of the sequence that owns state slot slot[s].  A
// segment at position 0 starts from zeros (the slot's old contents are not read), so a
// slot needs no clearing when it changes hands.  slot < 0 marks a padding segment.
//
// Recurrence per head, S [dk, dv] fp32:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// Columns of S (the dv axis) are independent, so a workgroup owns 32 columns of one
// head of one sequence: 8 lanes share a column (each holds dk/8 consecutive rows in
// registers, the two dot products are reduced over those 8 lanes), and the rows of a
// segment are walked in order.  q, k (unit-normalised), g and beta are prepared for all
// rows at once by delta_prep_kernel, so the sequential loop only streams them.
#include "mx_common.h"

namespace mx {

constexpr int kMaxTaps = 16;

// out[row, c] = silu(bias[c] + sum_j w[c, j] * in(row - (taps-1) + j, c)), inputs before
// the segment's first row come from the slot's history (zeros at position 0); rows of x
// are x_stride apart (a column range of a wider product), rows of out are dense
template <typename T>
__global__ void short_conv_kernel(T* __restrict__ out, const T* __restrict__ x, long x_stride,
                                  const float* __restrict__ w, const float* __restrict__ bias,
                                  const float* __restrict__ hist, const int* __restrict__ start,
                                  const int* __restrict__ pos0, const int* __restrict__ slot, int channels,
                                  int taps, int num_slots) {
  const int s = blockIdx.z;
  const int r0 = start[s], n = start[s + 1] - r0;
  const int rel = blockIdx.y;
  if (rel >= n) return;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int sl = slot[s];
  const long row = r0 + rel;
  if (sl < 0 || sl >= num_slots) {
    st(out, row * channels + c, 0.f);
    return;
  }
  const bool fresh = pos0[s] <= 0;
  const float* h = hist + (long)sl * (taps - 1) * channels;
  float acc = bias != nullptr ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int src = rel - (taps - 1) + j;
    float v;
    if (src >= 0) v = ld(x, (long)(r0 + src) * x_stride + c);
    else v = fresh ? 0.f : h[(long)(taps - 1 + src) * channels + c];
    acc += v * w[(long)c * taps + j];
  }
  st(out, row * channels + c, acc * sigmoidf_(acc));
}

// history <- the segment's last taps-1 inputs (older ones shift out); runs after
// short_conv_kernel, one thread per (segment, channel)
template <typename T>
__global__ void conv_hist_kernel(const T* __restrict__ x, long x_stride, float* __restrict__ hist,
                                 const int* __restrict__ start, const int* __restrict__ pos0,
                                 const int* __restrict__ slot, int channels, int taps, int num_slots) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int sl = slot[s];
  const int r0 = start[s], n = start[s + 1] - r0;
  if (sl < 0 || sl >= num_slots || n <= 0) return;
  const bool fresh = pos0[s] <= 0;
  float* h = hist + (long)sl * (taps - 1) * channels;
  float keep[kMaxTaps];
  for (int m = 0; m < taps - 1; ++m) {
    const int src = n - (taps - 1) + m;
    if (src >= 0) keep[m] = ld(x, (long)(r0 + src) * x_stride + c);
    else keep[m] = fresh ? 0.f : h[(long)(taps - 1 + src) * channels + c];
  }
  for (int m = 0; m < taps - 1; ++m) h[(long)m * channels + c] = keep[m];
}

// per row: qn / kn = unit vectors per kv head (q also * dk^-1/2), g = exp(-exp(A) *
// softplus(a + dt_bias)), beta = sigmoid(b).  One wave per (row, item), items = kv
// heads (q, k) then heads (g, beta).
template <typename T>
__global__ void delta_prep_kernel(float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ g,
                                  float* __restrict__ beta, const T* __restrict__ qkv, long qkv_stride,
                                  const T* __restrict__ a, long a_stride, const T* __restrict__ b,
                                  long b_stride, const float* __restrict__ a_log,
                                  const float* __restrict__ dt_bias, long rows, int heads, int kv_heads,
                                  int dk) {
  const int items = kv_heads + heads;
  const long w = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (w >= rows * items) return;
  const int lane = threadIdx.x & 63;
  const long row = w / items;
  const int it = (int)(w % items);
  if (it < kv_heads) {
    const T* q = qkv + row * qkv_stride + (long)it * dk;
    const T* k = q + (long)kv_heads * dk;
    float sq = 0.f, sk = 0.f;
    for (int i = lane; i < dk; i += 64) {
      const float qv = ld(q, i), kv = ld(k, i);
      sq += qv * qv;
      sk += kv * kv;
    }
    sq = ft::wave_sum(sq);
    sk = ft::wave_sum(sk);
    const float rq = 1.0f / sqrtf(sq + 1e-6f) * (1.0f / sqrtf((float)dk));
    const float rk = 1.0f / sqrtf(sk + 1e-6f);
    for (int i = lane; i < dk; i += 64) {
      qn[(row * kv_heads + it) * dk + i] = ld(q, i) * rq;
      kn[(row * kv_heads + it) * dk + i] = ld(k, i) * rk;
    }
  } else {
    const int h = it - kv_heads;
    const float rate = expf(a_log[h]);
    for (int i = lane; i < dk; i += 64) {
      const float z = ld(a, row * a_stride + (long)h * dk + i) + dt_bias[(long)h * dk + i];
      g[(row * heads + h) * dk + i] = expf(-rate * softplusf_(z));
    }
    if (lane == 0) beta[row * heads + h] = sigmoidf_(ld(b, row * b_stride + h));
  }
}

constexpr int kKL = 8;        // lanes that share one state column
constexpr int kCols = 32;     // state columns per workgroup (256 threads)

// sum over the 8 adjacent lanes that share a column, on the VALU's lane-permute path
// (quad swaps, then the mirrored half row): every lane of the group gets the total
__device__ __forceinline__ float sum8(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // lanes ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // lanes ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // 7 - lane
  return v;
}

// grid (dv tiles, heads, segments), 256 threads.  Lane group member kl holds the state
// rows kl, kl + 8, ... of its column (dk <= 8 R).
//
// The per-row inputs (k, q, decay: dk floats each; v: this tile's 32 columns; beta) are
// staged through LDS in chunks of TT rows, double buffered: all 256 threads issue the
// next chunk's global loads before the current chunk's rows are walked and park them in
// LDS afterwards, so the sequential loop reads LDS only and one memory latency is paid
// per TT rows, overlapped with the walk.
template <int R>
struct DeltaTile {
  static constexpr int TT = R <= 16 ? 16 : 8;                 // rows per chunk
  static constexpr int DKP = 8 * R;                           // padded key size
  static constexpr int ROWF = 3 * DKP + kCols + 1;            // floats per staged row
  static constexpr int NLD = (TT * 3 * DKP + 255) / 256;      // k/q/g loads per thread and chunk
  static constexpr int NV = (TT * kCols + 255) / 256;         // v loads per thread and chunk
};

template <typename T, int R>
__global__ void __launch_bounds__(256)
delta_rule_kernel(float* __restrict__ o, const float* __restrict__ qn, const float* __restrict__ kn,
                  const float* __restrict__ g, const float* __restrict__ beta, const T* __restrict__ qkv,
                  long qkv_stride, float* __restrict__ state, const int* __restrict__ start,
                  const int* __restrict__ pos0, const int* __restrict__ slot, int heads, int kv_heads,
                  int dk, int dv, int num_slots) {
  using P = DeltaTile<R>;
  __shared__ float stage[2][P::TT * P::ROWF];
  const int s = blockIdx.z, h = blockIdx.y;
  const int sl = slot[s];
  const int r0 = start[s], n = start[s + 1] - r0;
  const int tid = threadIdx.x;
  const int kl = tid & (kKL - 1);
  const int cl = tid >> 3;                // column within the tile
  const int col = blockIdx.x * kCols + cl;
  const bool live = col < dv;
  const int c = live ? col : dv - 1;      // dead lanes shadow the last column, store nothing
  const long o_stride = (long)heads * dv;
  if (sl < 0 || sl >= num_slots) {
    if (live && kl == 0)
      for (int t = 0; t < n; ++t) o[(long)(r0 + t) * o_stride + (long)h * dv + col] = 0.f;
    return;
  }
  if (n <= 0) return;
  const int kh = h / (heads / kv_heads);
  // rows kl, kl + 8, ...: the 8 lanes of a column read 8 consecutive LDS banks
  float* S = state + (((long)sl * heads + h) * dk) * dv;
  float st_[R];
  const bool fresh = pos0[s] <= 0;
#pragma unroll
  for (int r = 0; r < R; ++r) st_[r] = (!fresh && kl + kKL * r < dk) ? S[(long)(kl + kKL * r) * dv + c] : 0.f;
  const long voff = 2L * kv_heads * dk + (long)h * dv + (long)blockIdx.x * kCols;

  float ld_[P::NLD], lv_[P::NV], lb_ = 0.f;
  // issue the global loads of the chunk that starts at row t0 (cnt rows)
  auto fetch = [&](int t0, int cnt) {
#pragma unroll
    for (int u = 0; u < P::NLD; ++u) {
      const int e = tid + 256 * u;                  // (row tt, array a, entry i) of the chunk
      const int tt = e / (3 * P::DKP), rem = e % (3 * P::DKP);
      const int a = rem / P::DKP, i = rem % P::DKP;
      float v = 0.f;
      if (tt < cnt && i < dk) {
        const long row = r0 + t0 + tt;
        v = a == 0 ? kn[(row * kv_heads + kh) * dk + i]
          : a == 1 ? qn[(row * kv_heads + kh) * dk + i]
                   : g[(row * heads + h) * dk + i];
      }
      ld_[u] = v;
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      const int tt = e / kCols, cc = e % kCols;
      lv_[u] = (tt < cnt && blockIdx.x * kCols + cc < dv)
                   ? ld(qkv, (long)(r0 + t0 + tt) * qkv_stride + voff + cc) : 0.f;
    }
    lb_ = tid < cnt ? beta[(long)(r0 + t0 + tid) * heads + h] : 0.f;
  };
  auto park = [&](float* buf) {
#pragma unroll
    for (int u = 0; u < P::NLD; ++u) {
      const int e = tid + 256 * u;
      const int tt = e / (3 * P::DKP), rem = e % (3 * P::DKP);
      if (tt < P::TT) buf[tt * P::ROWF + rem] = ld_[u];
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      if (e < P::TT * kCols) buf[(e / kCols) * P::ROWF + 3 * P::DKP + e % kCols] = lv_[u];
    }
    if (tid < P::TT) buf[tid * P::ROWF + 3 * P::DKP + kCols] = lb_;
  };

  fetch(0, min(P::TT, n));
  park(stage[0]);
  __syncthreads();
  int cur = 0;
  for (int t0 = 0; t0 < n; t0 += P::TT) {
    const int cnt = min(P::TT, n - t0);
    const bool more = t0 + P::TT < n;
    if (more) fetch(t0 + P::TT, min(P::TT, n - t0 - P::TT));
    const float* buf = stage[cur];
    for (int t = 0; t < cnt; ++t) {
      const float* rw = buf + t * P::ROWF;
      float kk[R], qq[R];
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        kk[r] = rw[kl + kKL * r];
        qq[r] = rw[P::DKP + kl + kKL * r];
        st_[r] *= rw[2 * P::DKP + kl + kKL * r];
        dot += st_[r] * kk[r];
      }
      dot = sum8(dot);
      const float u = rw[3 * P::DKP + kCols] * (rw[3 * P::DKP + cl] - dot);
      float out = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        st_[r] += kk[r] * u;
        out += st_[r] * qq[r];
      }
      out = sum8(out);
      if (live && kl == 0) o[(long)(r0 + t0 + t) * o_stride + (long)h * dv + col] = out;
    }
    if (more) park(stage[cur ^ 1]);
    __syncthreads();
    cur ^= 1;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (kl + kKL * r < dk) S[(long)(kl + kKL * r) * dv + col] = st_[r];
  }
}

}  // namespace mx

using namespace mx;

extern "C" int mx_short_conv_silu(void* out, const void* x, int bf16, long x_stride, const float* w,
                                  const float* bias, float* hist,
                                  const int* start, const int* pos0, const int* slot, int num_segs,
                                  int max_rows, int channels, int taps, int num_slots, hipStream_t s) {
  if (num_segs <= 0 || max_rows <= 0 || channels <= 0) return 0;
  if (taps < 1 || taps > kMaxTaps) return -1;
  const dim3 block(256);
  const dim3 grid((channels + 255) / 256, max_rows, num_segs);
  if (grid.y > 65535 || grid.z > 65535) return -2;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((short_conv_kernel<T>), grid, block, 0, s, (T*)out, (const T*)x, x_stride,
                                         w, bias, hist, start, pos0, slot, channels, taps, num_slots));
  if (taps > 1)
    MX_DISPATCH_T(bf16, hipLaunchKernelGGL((conv_hist_kernel<T>), dim3((channels + 255) / 256, num_segs),
                                           block, 0, s, (const T*)x, x_stride, hist, start, pos0, slot,
                                           channels, taps, num_slots));
  return (int)hipGetLastError();
}

// history update alone, for kernels that fuse the convolution into a larger step
extern "C" int mx_conv_hist(const void* x, int bf16, long x_stride, float* hist, const int* start, const int* pos0,
                            const int* slot, int num_segs, int channels, int taps, int num_slots, hipStream_t s) {
  if (num_segs <= 0 || channels <= 0 || taps <= 1) return 0;
  if (taps > kMaxTaps || num_segs > 65535) return -1;
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((conv_hist_kernel<T>), dim3((channels + 255) / 256, num_segs), dim3(256),
                                         0, s, (const T*)x, x_stride, hist, start, pos0, slot, channels, taps,
                                         num_slots));
  return (int)hipGetLastError();
}

extern "C" int mx_delta_prep(float* qn, float* kn, float* g, float* beta, const void* qkv, int bf16,
                             long qkv_stride, const void* a, long a_stride, const void* b, long b_stride,
                             const float* a_log, const float* dt_bias, long rows, int heads, int kv_heads,
                             int dk, hipStream_t s) {
  const long waves = rows * (heads + kv_heads);
  if (waves <= 0) return 0;
  const dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  MX_DISPATCH_T(bf16, hipLaunchKernelGGL((delta_prep_kernel<T>), grid, block, 0, s, qn, kn, g, beta,
                                         (const T*)qkv, qkv_stride, (const T*)a, a_stride, (const T*)b,
                                         b_stride, a_log, dt_bias, rows, heads, kv_heads, dk));
  return (int)hipGetLastError();
}

template <typename T, int R>
static void launch_delta(dim3 grid, hipStream_t s, float* o, const float* qn, const float* kn,
                         const float* g, const float* beta, const void* qkv, long qkv_stride, float* state,
                         const int* start, const int* pos0, const int* slot, int heads, int kv_heads, int dk,
                         int dv, int num_slots) {
  hipLaunchKernelGGL((delta_rule_kernel<T, R>), grid, dim3(256), 0, s, o, qn, kn, g, beta, (const T*)qkv,
                     qkv_stride, state, start, pos0, slot, heads, kv_heads, dk, dv, num_slots);
}

extern "C" int mx_delta_max_dk() { return kKL * 32; }

extern "C" int mx_delta_rule(float* o, const float* qn, const float* kn, const float* g, const float* beta,
                             const void* qkv, int bf16, long qkv_stride, float* state, const int* start,
                             const int* pos0, const int* slot, int num_segs, int heads, int kv_heads, int dk,
                             int dv, int num_slots, hipStream_t s) {
  if (num_segs <= 0) return 0;
  if (dk < 1 || dk > mx_delta_max_dk() || dv < 1 || heads % kv_heads) return -1;
  const dim3 grid((dv + kCols - 1) / kCols, heads, num_segs);
  if (grid.z > 65535) return -2;
  const int need = (dk + kKL - 1) / kKL;
#define MX_DELTA(R)                                                                                  \
  MX_DISPATCH_T(bf16, launch_delta<T, R>(grid, s, o, qn, kn, g, beta, qkv, qkv_stride, state, start, \
                                         pos0, slot, heads, kv_heads, dk, dv, num_slots))
  if (need <= 2) MX_DELTA(2);
  else if (need <= 4) MX_DELTA(4);
  else if (need <= 8) MX_DELTA(8);
  else if (need <= 16) MX_DELTA(16);
  else MX_DELTA(32);
#undef MX_DELTA
  return (int)hipGetLastError();
}
