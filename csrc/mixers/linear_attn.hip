// Gated linear attention with one decay per head and key channel over fp32 state slots.
//
// Rows come in segments as in delta_rule.hip (start / pos0 / slot; a segment at position
// 0 starts from zeros; slot < 0 is padding).  Rows of the fused projection are
// [q (heads*dk) | k (heads*dk) | v (heads*dv) | ...]; `a` holds the decay's pre-activation
// [heads*dk] per row.  Per head, S [dk, dv] fp32:
//   g = sigmoid(a + bias)^(1/tau) = exp(-softplus(-(a + bias)) / tau)
//   S <- diag(g) S + k v^T;   o = S^T (q dk^-1/2)
// Columns of S are independent and, unlike the delta rule, the update of an entry needs
// nothing from other entries, so only the output dot product crosses lanes.  What bounds
// the walk is LDS traffic: a lane needs its own k, q and decay values for every state row it
// holds, whatever the column.  So a lane holds a block of R state rows x C columns (C = 1 or 2) in
// registers (12 R + 4 C bytes read from LDS per C R entries and row); 32 lanes share a
// group of C columns (dk <= 32 R), a workgroup of 256 threads owns 8 C columns of one head
// of one sequence, and each column's output is reduced over the 16 lanes of a DPP row
// and then across the two rows (lane-permute adds only).  A segment's rows are walked in order with the per-row
// inputs staged through LDS in chunks.  The raw q, k and a of the next two chunks are in
// flight (two register sets) while the current chunk is walked, and are turned into
// scaled q, k and decay (fp32) when they are parked in LDS, so no separate preparation
// pass and no fp32 copies of q, k and the decays exist.
#include "mx_common.h"

namespace mx {

constexpr int kGL = 32;        // lanes that share a group of state columns (two DPP rows)
// State columns per lane, C, are 2 (16 columns per workgroup) when the step has enough
// (sequence, head, column tile) triples to fill the chip, else 1 (8 columns per workgroup,
// twice the workgroups, half the work per row and wave): a single sequence's walk is bound by
// the latency of one wave's row, not by throughput.

__device__ __forceinline__ float gla_sum16(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // lanes ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // lanes ^ 2
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // 7 - lane (halves)
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));  // 15 - lane
  return v;
}

// sum over the 32 lanes of a column group (an aligned pair of DPP rows); the lanes of the
// pair's upper row (kl >= 16) get it: after the sums within each row, lane 15 of a row is
// added into the row above (rows 1 and 3 of the wave), all on the VALU's lane-permute path
__device__ __forceinline__ float gla_sum32_upper(float v) {
  v = gla_sum16(v);
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x142, 0xA, 0xF, false));
  return v;
}

// SHORT: the form for steps whose segments have at most kGlaShortRows rows (decode): small
// chunks, so few registers and several workgroups per CU
constexpr int kGlaShortRows = 4;

template <int R, bool SHORT, int C>
struct GlaTile {
  static constexpr int COLS = (256 / kGL) * C;                // state columns per workgroup
  static constexpr int TT = SHORT ? kGlaShortRows : R <= 4 ? 16 : 8;   // rows per chunk
  static constexpr int NP = kGL * R;                          // padded key size
  static constexpr int SR = R + (R >= 8 ? 4 : 0);             // floats between two lanes' runs
  static constexpr int BP = kGL * SR;                         // floats of a staged k (or q, or decay)
  static constexpr int ROWF = 3 * BP + 16;                   // floats per staged row: k | q | decay | v
  static constexpr int NLD = (TT * 3 * NP + 255) / 256;       // k/q/a loads per thread and chunk
  static constexpr int NV = (TT * COLS + 255) / 256;        // v loads per thread and chunk
};

template <int R>
__device__ __forceinline__ void gla_run(const float* p, float* v) {
  if constexpr (R >= 4) {
#pragma unroll
    for (int i = 0; i < R / 4; ++i) {
      const float4 u = reinterpret_cast<const float4*>(p)[i];
      v[4 * i] = u.x; v[4 * i + 1] = u.y; v[4 * i + 2] = u.z; v[4 * i + 3] = u.w;
    }
  } else if constexpr (R == 2) {
    const float2 u = *reinterpret_cast<const float2*>(p);
    v[0] = u.x; v[1] = u.y;
  } else {
    v[0] = p[0];
  }
}

// sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau) in fp32 on the hardware's exp2 / log2:
// softplus(-z) = log(1 + e) with e = exp(-z); for small e the series e - e^2/2 keeps the
// digits that 1 + e would drop.  The absolute error of the decay's logarithm stays near
// 1e-7, the spacing of fp32 numbers below 1.
__device__ __forceinline__ float gla_decay(float z, float inv_tau) {
  const float e = __expf(-z);
  const float sp = e < 1e-3f ? e * (1.0f - 0.5f * e) : __logf(1.0f + e);
  return __expf(-sp * inv_tau);
}

// 16 bytes of a row, widened to floats
template <typename T> struct GlaVec;
template <> struct GlaVec<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void widen(const uint4& u, float* f) {
    f[0] = __uint_as_float(u.x); f[1] = __uint_as_float(u.y); f[2] = __uint_as_float(u.z); f[3] = __uint_as_float(u.w);
  }
};
template <> struct GlaVec<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void widen(const uint4& u, float* f) {
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

// A chunk's raw inputs, as loaded from global memory (two such sets are in flight): q, k
// and a either entry by entry (ld) or in 16-byte pieces (lw, the VEC form), v entry by entry.
template <typename T, int R, bool SHORT, int C>
struct GlaRegs {
  using P = GlaTile<R, SHORT, C>;
  static constexpr int NLW = (P::TT * 3 * P::NP / GlaVec<T>::N + 255) / 256;
  T ld[P::NLD];
  uint4 lw[NLW];
  T lv[P::NV];
};

// VEC: dk, the row strides and the base addresses are whole 16-byte pieces, so q, k and a
// are staged with one 16-byte load per 8 bf16 (4 fp32) entries
template <typename T, int R, bool SHORT, bool VEC, int C>
__global__ void __launch_bounds__(256)
gla_scan_kernel(float* __restrict__ o, const T* __restrict__ qkv, long qkv_stride, const T* __restrict__ a,
                long a_stride, const float* __restrict__ a_bias, float inv_tau, float* __restrict__ state,
                const int* __restrict__ start, const int* __restrict__ pos0, const int* __restrict__ slot,
                int heads, int dk, int dv, int num_slots) {
  using P = GlaTile<R, SHORT, C>;
  using Regs = GlaRegs<T, R, SHORT, C>;
  constexpr int kGC = C, kGCols = P::COLS;
  __shared__ __attribute__((aligned(16))) float stage[P::TT * P::ROWF];
  __shared__ __attribute__((aligned(16))) float out_s[P::TT * kGCols];   // a chunk's outputs, written out after the walk
  __shared__ float bias_s[P::NP];                // the head's decay bias (read when a chunk is parked)
  const int s = blockIdx.z, h = blockIdx.y;
  const int sl = slot[s];
  const int r0 = start[s], rows = start[s + 1] - r0;
  const int tid = threadIdx.x;
  const int kl = tid & (kGL - 1);
  const int cl = tid / kGL;                       // column group within the workgroup
  const int col0 = blockIdx.x * kGCols + cl * kGC;  // this lane's first column
  const long o_stride = (long)heads * dv;
  if (sl < 0 || sl >= num_slots) {
    if (tid < kGCols && blockIdx.x * kGCols + tid < dv)
      for (int t = 0; t < rows; ++t) o[(long)(r0 + t) * o_stride + (long)h * dv + blockIdx.x * kGCols + tid] = 0.f;
    return;
  }
  if (rows <= 0) return;
  for (int i = tid; i < P::NP; i += 256) bias_s[i] = i < dk ? a_bias[(long)h * dk + i] : 0.f;
  float* S = state + (((long)sl * heads + h) * dk) * dv;
  float st_[kGC][R];
  const bool fresh = pos0[s] <= 0;
#pragma unroll
  for (int j = 0; j < kGC; ++j)
#pragma unroll
    for (int r = 0; r < R; ++r)          // columns past dv and rows past dk stay zero and are not stored
      st_[j][r] = (!fresh && kl * R + r < dk && col0 + j < dv) ? S[(long)(kl * R + r) * dv + col0 + j] : 0.f;
  const long qoff = (long)h * dk, koff = (long)heads * dk + qoff;
  const long voff = 2L * heads * dk + (long)h * dv + (long)blockIdx.x * kGCols;
  const float qscale = 1.0f / sqrtf((float)dk);

  // issue the loads of the chunk that starts at row t0 (nothing is waited for here)
  auto fetch = [&](Regs& g, int t0) {
    const int cnt = min(P::TT, rows - t0);       // <= 0 past the end: nothing is loaded
    if constexpr (VEC) {
      constexpr int V = GlaVec<T>::N, PV = 3 * P::NP / V;   // pieces per staged row
#pragma unroll
      for (int u = 0; u < Regs::NLW; ++u) {
        const int e = tid + 256 * u;                // (row tt, array w, piece) of the chunk
        const int tt = e / PV, rem = e % PV;
        const int w = rem / (P::NP / V), i0 = (rem % (P::NP / V)) * V;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (tt < cnt && i0 < dk) {
          const long row = r0 + t0 + tt;
          const T* src = w == 2 ? a + row * a_stride + qoff + i0 : qkv + row * qkv_stride + (w == 0 ? koff : qoff) + i0;
          v = *reinterpret_cast<const uint4*>(src);
        }
        g.lw[u] = v;
      }
    } else {
#pragma unroll
      for (int u = 0; u < P::NLD; ++u) {
        const int e = tid + 256 * u;                // (row tt, array w, entry i) of the chunk
        const int tt = e / (3 * P::NP), rem = e % (3 * P::NP);
        const int w = rem / P::NP, i = rem % P::NP;
        T v = T(0);
        if (tt < cnt && i < dk) {
          const long row = r0 + t0 + tt;
          v = w == 2 ? a[row * a_stride + qoff + i] : qkv[row * qkv_stride + (w == 0 ? koff : qoff) + i];
        }
        g.ld[u] = v;
      }
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      const int tt = e / kGCols, cc = e % kGCols;
      g.lv[u] = (tt < cnt && blockIdx.x * kGCols + cc < dv) ? qkv[(long)(r0 + t0 + tt) * qkv_stride + voff + cc]
                                                            : T(0);
    }
  };
  // convert and park a loaded chunk in LDS: k as it is, q scaled, the decay from its pre-activation
  auto park = [&](const Regs& g) {
    if constexpr (VEC) {
      constexpr int V = GlaVec<T>::N, PV = 3 * P::NP / V;
#pragma unroll
      for (int u = 0; u < Regs::NLW; ++u) {
        const int e = tid + 256 * u;
        const int tt = e / PV, rem = e % PV;
        const int w = rem / (P::NP / V), i0 = (rem % (P::NP / V)) * V;
        if (tt < P::TT) {
          float f[V];
          GlaVec<T>::widen(g.lw[u], f);
          if (w == 1) {
#pragma unroll
            for (int j = 0; j < V; ++j) f[j] *= qscale;
          } else if (w == 2) {
#pragma unroll
            for (int j = 0; j < V; ++j) f[j] = i0 < dk ? gla_decay(f[j] + bias_s[i0 + j], inv_tau) : 0.f;
          }
          // a piece lies within one lane's run (or the runs are not padded apart): V floats in a row
          float4* dst = reinterpret_cast<float4*>(stage + tt * P::ROWF + w * P::BP + (i0 / R) * P::SR + i0 % R);
#pragma unroll
          for (int j = 0; j < V / 4; ++j) dst[j] = make_float4(f[4 * j], f[4 * j + 1], f[4 * j + 2], f[4 * j + 3]);
        }
      }
    } else {
#pragma unroll
      for (int u = 0; u < P::NLD; ++u) {
        const int e = tid + 256 * u;
        const int tt = e / (3 * P::NP), rem = e % (3 * P::NP);
        const int w = rem / P::NP, i = rem % P::NP;
        if (tt < P::TT) {
          float v = ld(&g.ld[u], 0);
          if (w == 1) v *= qscale;
          else if (w == 2) v = i < dk ? gla_decay(v + bias_s[i], inv_tau) : 0.f;
          stage[tt * P::ROWF + w * P::BP + (i / R) * P::SR + i % R] = v;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < P::NV; ++u) {
      const int e = tid + 256 * u;
      if (e < P::TT * kGCols) stage[(e / kGCols) * P::ROWF + 3 * P::BP + e % kGCols] = ld(&g.lv[u], 0);
    }
  };
  // one row of the chunk in LDS: update the state, return the columns' outputs (complete in
  // the lanes kl >= 16)
  auto walk = [&](int t, float* out) {
    const float* rw = stage + t * P::ROWF;
    float kk[R], qq[R], gg[R];
    gla_run<R>(rw + kl * P::SR, kk);
    gla_run<R>(rw + P::BP + kl * P::SR, qq);
    gla_run<R>(rw + 2 * P::BP + kl * P::SR, gg);
    float vv[kGC];
#pragma unroll
    for (int j = 0; j < kGC; ++j) vv[j] = rw[3 * P::BP + cl * kGC + j];
#pragma unroll
    for (int j = 0; j < kGC; ++j) {
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        st_[j][r] = gg[r] * st_[j][r] + kk[r] * vv[j];
        acc += st_[j][r] * qq[r];
      }
      out[j] = gla_sum32_upper(acc);
    }
  };
  // walk the chunk in LDS (rows t0 ..), then replace it by the chunk waiting in `next`
  // and send the outputs off in coalesced stores (rows of 8 C columns).  A full chunk's walk
  // is straight-line code: its outputs wait in registers and are written to LDS in one
  // go, so no per-row branch keeps the next rows' LDS reads from being issued early.
  auto turn = [&](int t0, const Regs& next) {
    const int cnt = min(P::TT, rows - t0);
    if (cnt == P::TT) {
      float outs[P::TT][kGC];
#pragma unroll
      for (int t = 0; t < P::TT; ++t) walk(t, outs[t]);
      if (kl == 16) {
#pragma unroll
        for (int t = 0; t < P::TT; ++t)
#pragma unroll
          for (int j = 0; j < kGC; ++j) out_s[t * kGCols + cl * kGC + j] = outs[t][j];
      }
    } else {
      for (int t = 0; t < cnt; ++t) {
        float out[kGC];
        walk(t, out);
        if (kl == 16) {
#pragma unroll
          for (int j = 0; j < kGC; ++j) out_s[t * kGCols + cl * kGC + j] = out[j];
        }
      }
    }
    __syncthreads();
    if (t0 + P::TT < rows) park(next);
    for (int e = tid; e < cnt * kGCols; e += 256) {
      const int tt = e / kGCols, cc = e % kGCols;
      if (blockIdx.x * kGCols + cc < dv)
        o[(long)(r0 + t0 + tt) * o_stride + (long)h * dv + blockIdx.x * kGCols + cc] = out_s[e];
    }
    __syncthreads();
  };

  // Two register sets keep the loads of the next two chunks in flight while a chunk is
  // walked: a set is loaded two chunk walks before it is parked.
  Regs ga, gb;
  fetch(ga, 0);
  fetch(gb, P::TT);
  __syncthreads();                               // bias_s
  park(ga);
  __syncthreads();
  fetch(ga, 2 * P::TT);
  for (int t0 = 0; t0 < rows; t0 += 2 * P::TT) {
    turn(t0, gb);                                // chunk at t0; then the chunk at t0 + TT is parked
    fetch(gb, t0 + 3 * P::TT);
    if (t0 + P::TT >= rows) break;
    turn(t0 + P::TT, ga);                        // then the chunk at t0 + 2 TT is parked
    fetch(ga, t0 + 4 * P::TT);
  }
#pragma unroll
  for (int j = 0; j < kGC; ++j)
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (kl * R + r < dk && col0 + j < dv) S[(long)(kl * R + r) * dv + col0 + j] = st_[j][r];
}

}  // namespace mx

using namespace mx;

extern "C" int mx_gla_max_dk() { return kGL * 8; }

template <typename T, int R, bool VEC, int C>
static void launch_gla(dim3 grid, hipStream_t s, bool few, float* o, const void* qkv, long qkv_stride, const void* a,
                       long a_stride, const float* a_bias, float inv_tau, float* state, const int* start,
                       const int* pos0, const int* slot, int heads, int dk, int dv, int num_slots) {
  if (few)
    hipLaunchKernelGGL((gla_scan_kernel<T, R, true, VEC, C>), grid, dim3(256), 0, s, o, (const T*)qkv, qkv_stride,
                       (const T*)a, a_stride, a_bias, inv_tau, state, start, pos0, slot, heads, dk, dv, num_slots);
  else
    hipLaunchKernelGGL((gla_scan_kernel<T, R, false, VEC, C>), grid, dim3(256), 0, s, o, (const T*)qkv, qkv_stride,
                       (const T*)a, a_stride, a_bias, inv_tau, state, start, pos0, slot, heads, dk, dv, num_slots);
}

extern "C" int mx_gla_scan(float* o, const void* qkv, int bf16, long qkv_stride, const void* a, long a_stride,
                           const float* a_bias, float tau, float* state, const int* start, const int* pos0,
                           const int* slot, int num_segs, int max_rows, int heads, int dk, int dv, int num_slots,
                           hipStream_t s) {
  if (num_segs <= 0) return 0;
  const bool few = max_rows > 0 && max_rows <= kGlaShortRows;   // the longest segment of the step (0: unknown)
  if (dk < 1 || dk > mx_gla_max_dk() || dv < 1 || heads < 1 || !(tau > 0.f)) return -1;
  // two columns per lane when that still gives at least two workgroups per CU's worth of them
  const long wide = (long)((dv + 15) / 16) * heads * num_segs;
  const int cpl = wide >= 512 ? 2 : 1;
  const int cols = 256 / kGL * cpl;
  const dim3 grid((dv + cols - 1) / cols, heads, num_segs);
  if (grid.z > 65535 || grid.y > 65535) return -2;
  const int need = (dk + kGL - 1) / kGL;
  const int piece = bf16 ? 8 : 4;                // entries per 16 bytes
  const bool vec = dk % piece == 0 && qkv_stride % piece == 0 && a_stride % piece == 0 &&
                   ((uintptr_t)qkv) % 16 == 0 && ((uintptr_t)a) % 16 == 0;
#define MX_GLA_C(R, V, C)                                                                                        \
  MX_DISPATCH_T(bf16, launch_gla<T, R, V, C>(grid, s, few, o, qkv, qkv_stride, a, a_stride, a_bias, 1.0f / tau, state, \
                                             start, pos0, slot, heads, dk, dv, num_slots))
#define MX_GLA(R)                                   \
  do {                                              \
    if (vec && cpl == 2) MX_GLA_C(R, true, 2);      \
    else if (vec) MX_GLA_C(R, true, 1);             \
    else if (cpl == 2) MX_GLA_C(R, false, 2);       \
    else MX_GLA_C(R, false, 1);                     \
  } while (0)
  if (need <= 1) MX_GLA(1);
  else if (need <= 2) MX_GLA(2);
  else if (need <= 4) MX_GLA(4);
  else MX_GLA(8);
#undef MX_GLA
#undef MX_GLA_C
  return (int)hipGetLastError();
}
