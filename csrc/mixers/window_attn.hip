// Windowed grouped-query attention over a paged key cache and a paged value cache:
// softmax or sigmoid weights, an optional logarithmic distance bias, and several score
// maps per head that share the head's values (differential attention).
//
// Query head a = h * maps + m (head h, map m) reads key head (h / rep) * maps + m and
// value head h / rep, rep = heads / kv_heads.  Position i sees key j iff 0 <= i - j
// (< window when window > 0); with `blocks` the window is a block of the sequence instead
// (j <= i and i / window == j / window, blocks counted from position 0); with
// keep_first = f > 0 the positions j < f stay visible whatever the window.
// s = q.k * scale, capped to softcap tanh(s / softcap) when softcap > 0;
// score = s - r1[a] ln(1 + r2[a] (i - j)) + dist_bias[min(i - j, nd - 1)][a]; weight =
// softmax over the visible keys, or sigmoid(score + pb[a]) unnormalised.  A softmax may carry a sink: one more
// term exp(sink) in its denominator, a key that is always visible and has no value.
// Queries, scores, weights and sums are fp32; the caches hold fp32 or bf16 rows.
//
// Kernels: attn_prep (whole-projection RMS norms, rotary positions, cache writes),
// conv_attn_prep (short causal convolution over time, per-head RMS norms, cache writes),
// window_attn (one workgroup per (row, query head): decode rows and short segments),
// band_weights (scores -> weights for the banded matrix products of long segments) and
// diff_combine (two maps -> one gated, normed head output).
#include "mx_common.h"

namespace mx {

// ---------------------------------------------------------------------------------
// one workgroup per row of the fused [q | k | v] projection
// ---------------------------------------------------------------------------------
template <typename T, typename TC, int NT>
__global__ void attn_prep_kernel(float* __restrict__ q_out, const T* __restrict__ qkv, long stride,
                                 int nq, int nk, int nv, const float* __restrict__ wq,
                                 const float* __restrict__ wk, float eps, const float* __restrict__ table,
                                 int table_rows, int rot_dims, int head_dim,
                                 const int* __restrict__ positions, const int* __restrict__ slots,
                                 TC* __restrict__ k_cache, TC* __restrict__ v_cache, long num_slots) {
  __shared__ float red[NT / 64];
  const long row = blockIdx.x;
  const T* in = qkv + row * stride;
  float rq = 1.f, rk = 1.f;
  if (wq != nullptr) {
    float ss = 0.f;
    for (int e = threadIdx.x; e < nq; e += NT) {
      const float v = ld(in, e);
      ss += v * v;
    }
    ss = block_sum<NT>(ss, red);
    rq = 1.0f / sqrtf(ss / (float)nq + eps);
  }
  if (wk != nullptr) {
    float ss = 0.f;
    for (int e = threadIdx.x; e < nk; e += NT) {
      const float v = ld(in, nq + e);
      ss += v * v;
    }
    ss = block_sum<NT>(ss, red);
    rk = 1.0f / sqrtf(ss / (float)nk + eps);
  }
  int pos = positions[row];
  const bool rot = table != nullptr && rot_dims > 0;
  if (pos < 0 || pos >= table_rows) pos = 0;
  const float* cs = rot ? table + (long)pos * rot_dims : nullptr;
  const int half = rot_dims / 2;
  const long slot = slots[row];
  const bool keep = slot >= 0 && slot < num_slots;
  // q entries, then k entries
  for (int e = threadIdx.x; e < nq + nk; e += NT) {
    const bool is_q = e < nq;
    const int off = is_q ? e : e - nq;
    const float* w = is_q ? wq : wk;
    const float r = is_q ? rq : rk;
    const T* src = in + (is_q ? 0 : nq);
    float v = ld(src, off) * (w != nullptr ? r * w[off] : 1.f);
    if (rot) {
      const int d = off % head_dim;
      if (d < rot_dims) {
        const int i = d < half ? d : d - half;
        const int po = d < half ? off + half : off - half;
        const float pv = ld(src, po) * (w != nullptr ? r * w[po] : 1.f);
        const float c = cs[i], s = cs[half + i];
        v = d < half ? v * c - pv * s : v * c + pv * s;
      }
    }
    if (is_q) q_out[row * nq + off] = v;
    else if (keep) st(k_cache, slot * nk + off, v);
  }
  if (keep)
    for (int e = threadIdx.x; e < nv; e += NT) st(v_cache, slot * nv + e, ld(in, nq + nk + e));
}

// ---------------------------------------------------------------------------------
// one wave per (row, chunk) of the fused [q | k | v] projection, a chunk being one head
// of q or k (head_dim channels) or up to head_dim channels of v: a causal convolution
// over time on every channel (taps along the row axis, the last tap on the row itself;
// rows before the segment's first come from the state slot's history, zeros at position
// 0), then, for q and k, the head's RMS norm with one weight vector shared by the heads,
// fp32 throughout.  The convolved chunk waits in the wave's LDS strip between the two
// passes.  q leaves as fp32, k and v go to the row's cache slot.  The history is
// updated afterwards by mx_conv_hist.  grid (rows, ceil(chunks / 4)), 4 waves.
// ---------------------------------------------------------------------------------
template <typename T, typename TC>
__global__ void __launch_bounds__(256)
conv_attn_prep_kernel(float* __restrict__ q_out, const T* __restrict__ qkv, long stride, int nq, int nk, int nv,
                      const float* __restrict__ conv_w, int taps, const float* __restrict__ hist,
                      const int* __restrict__ start, const int* __restrict__ pos0, const int* __restrict__ slot,
                      int num_segs, int num_state_slots, const float* __restrict__ wq,
                      const float* __restrict__ wk, float eps, int head_dim, const int* __restrict__ slots,
                      TC* __restrict__ k_cache, TC* __restrict__ v_cache, long num_slots) {
  extern __shared__ float smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* y = smem + wave * head_dim;
  const int channels = nq + nk + nv;
  const int qk_chunks = (nq + nk) / head_dim;
  const int chunks = qk_chunks + (nv + head_dim - 1) / head_dim;
  const int ch = blockIdx.y * 4 + wave;
  const int row = blockIdx.x;
  if (ch >= chunks || row >= start[num_segs]) return;
  int lo_s = 0, hi_s = num_segs;
  while (hi_s - lo_s > 1) {
    const int mid = (lo_s + hi_s) >> 1;
    if (start[mid] <= row) lo_s = mid; else hi_s = mid;
  }
  const int s = lo_s;
  const int r0 = start[s], rel = row - r0;
  const int sl = slot[s];
  const bool old = sl >= 0 && sl < num_state_slots && pos0[s] > 0;   // the slot's history counts
  const float* h = hist + (long)(old ? sl : 0) * (taps - 1) * channels;
  const int c0 = ch * head_dim;
  const int len = min(head_dim, channels - c0);
  float ss = 0.f;
  for (int i = lane; i < len; i += 64) {
    const int c = c0 + i;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int src = rel - (taps - 1) + j;
      float v;
      if (src >= 0) v = ld(qkv, (long)(r0 + src) * stride + c);
      else v = old ? h[(long)(taps - 1 + src) * channels + c] : 0.f;
      acc += v * conv_w[(long)c * taps + j];
    }
    y[i] = acc;                        // each lane re-reads only what it wrote itself
    ss += acc * acc;
  }
  const long cs = slots[row];
  const bool keep = cs >= 0 && cs < num_slots;
  if (ch < qk_chunks) {
    const bool is_q = c0 < nq;
    const float* w = is_q ? wq : wk;
    float r = 1.f;
    if (w != nullptr) r = 1.0f / sqrtf(ft::wave_sum(ss) / (float)head_dim + eps);
    for (int i = lane; i < len; i += 64) {
      const float v = w != nullptr ? y[i] * r * w[i] : y[i];
      if (is_q) q_out[(long)row * nq + c0 + i] = v;
      else if (keep) st(k_cache, cs * nk + (c0 - nq) + i, v);
    }
  } else if (keep) {
    for (int i = lane; i < len; i += 64) st(v_cache, cs * nv + (c0 - nq - nk) + i, y[i]);
  }
}

// ---------------------------------------------------------------------------------
// per-row attention: grid (rows, query heads), 256 threads = 4 waves.  A wave takes
// every fourth chunk of 64 keys: lane = key for the scores (each lane walks its key's
// cached row in 16-byte pieces), online softmax per wave, waves merged through LDS.
// The weighted sums of the value rows come in two forms:
//  * VEC (value rows are whole 16-byte pieces): a lane owns one 16-byte piece of the
//    row (8 bf16 / 4 fp32 columns) of every (64 / LPK)-th key, LPK = pieces per row
//    rounded up to a power of two; a pass loads 64 / LPK whole rows with one 16-byte
//    load per lane, branch-free (a key past the chunk's end reads row 0 with weight 0),
//    so several passes are in flight; the lanes that share a piece are summed at the end;
//  * otherwise lane = value column, one key at a time.
// ---------------------------------------------------------------------------------
constexpr int kWaves = 4;
constexpr int kMaxVCols = 8;          // value columns per lane (scalar form): dv <= 512

template <typename TC> struct Piece;
template <> struct Piece<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void load(const float* p, float* v) {
    const float4 u = *reinterpret_cast<const float4*>(p);
    v[0] = u.x; v[1] = u.y; v[2] = u.z; v[3] = u.w;
  }
};
template <> struct Piece<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void load(const bf16_t* p, float* v) {
    const uint4 u = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

template <typename TC>
__device__ __forceinline__ float dot_row(const TC* __restrict__ kp, const float* __restrict__ q, int dk, bool vec);

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ kp, const float* __restrict__ q, int dk,
                                                bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int d = 0; d < dk; d += 4) {
      const float4 k4 = *reinterpret_cast<const float4*>(kp + d);
      acc += q[d] * k4.x + q[d + 1] * k4.y + q[d + 2] * k4.z + q[d + 3] * k4.w;
    }
  } else {
    for (int d = 0; d < dk; ++d) acc += q[d] * kp[d];
  }
  return acc;
}

template <>
__device__ __forceinline__ float dot_row<bf16_t>(const bf16_t* __restrict__ kp, const float* __restrict__ q, int dk,
                                                 bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int d = 0; d < dk; d += 8) {
      const uint4 u = *reinterpret_cast<const uint4*>(kp + d);
      const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        acc += q[d + 2 * p] * __uint_as_float(w[p] << 16);
        acc += q[d + 2 * p + 1] * __uint_as_float(w[p] & 0xffff0000u);
      }
    }
  } else {
    for (int d = 0; d < dk; ++d) acc += q[d] * ld(kp, d);
  }
  return acc;
}

template <typename TC, bool VEC>
__global__ void __launch_bounds__(64 * kWaves)
window_attn_kernel(float* __restrict__ out, const float* __restrict__ q, const TC* __restrict__ k_cache,
                   const TC* __restrict__ v_cache, const int* __restrict__ start, const int* __restrict__ pos0,
                   const int* __restrict__ kv_len, const int* __restrict__ bt, int bt_stride, int num_segs,
                   int heads, int maps, int kv_heads, int dk, int dv, int window, float scale, int sigmoid,
                   const float* __restrict__ r1, const float* __restrict__ r2, const float* __restrict__ pb,
                   int block_size, int num_blocks, int skip_from, int vec, int lpk, float softcap, int has_sink,
                   float sink, int blocks, int keep_first, const float* __restrict__ dist_bias, int nd) {
  extern __shared__ float smem[];
  const int row = blockIdx.x, a = blockIdx.y;
  const int hq = heads * maps;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // the segment that owns this row: the last s with start[s] <= row
  int lo_s = 0, hi_s = num_segs;
  while (hi_s - lo_s > 1) {
    const int mid = (lo_s + hi_s) >> 1;
    if (start[mid] <= row) lo_s = mid; else hi_s = mid;
  }
  const int s = lo_s;
  const int r0 = start[s], n = start[s + 1] - r0;
  if (row >= start[num_segs] || (skip_from > 0 && n >= skip_from)) return;
  float* q_s = smem;                         // [dk]
  float* o_s = smem + dk;                    // [kWaves][dv]
  float* ml_s = o_s + kWaves * dv;           // [kWaves][2]
  const float* qp = q + ((long)row * hq + a) * dk;
  for (int d = tid; d < dk; d += blockDim.x) q_s[d] = qp[d];
  __syncthreads();
  const int h = a / maps, m = a % maps, rep = heads / kv_heads;
  const int kh = (h / rep) * maps + m, vh = h / rep;
  const long nk = (long)kv_heads * maps * dk, nv = (long)kv_heads * dv;
  const int i = pos0[s] + (row - r0);
  const int last = min(i, kv_len[s] - 1);    // padding rows (empty context) see nothing
  const int first = window > 0 ? (blocks ? (i / window) * window : max(0, i - window + 1)) : 0;
  // kept first positions that lie before the window: keys 0 .. ext-1 go in front of the band
  const int ext = window > 0 ? max(0, min(min(keep_first, first), last + 1)) : 0;
  const int nkeys = ext + max(0, last - first + 1);
  const float c1 = r1 != nullptr ? r1[a] : 0.f, c2 = r1 != nullptr ? r2[a] : 0.f;
  const float bias = (sigmoid && pb != nullptr) ? pb[a] : 0.f;
  const int* table = bt + (long)s * bt_stride;

  constexpr int NO = VEC ? Piece<TC>::N : kMaxVCols;
  float o[NO];
#pragma unroll
  for (int u = 0; u < NO; ++u) o[u] = 0.f;
  // VEC: this lane's piece of the value row and which key of a pass it reads
  const int pieces = dv / Piece<TC>::N;
  const int sg = lane & (lpk - 1), sub = lane / lpk, kpp = 64 / lpk;
  const bool has_piece = sg < pieces;
  float mx_ = -INFINITY, l_ = 0.f;
  for (int c0 = wave * 64; c0 < nkeys; c0 += 64 * kWaves) {
    const int cnt = min(64, nkeys - c0);
    const int cc = c0 + lane;
    const int j = cc < ext ? cc : first + cc - ext;
    int slot = -1;
    float z = -INFINITY;
    if (lane < cnt) {
      const int blk = table[j / block_size];
      if (blk >= 0 && blk < num_blocks) {
        slot = blk * block_size + j % block_size;
        z = dot_row<TC>(k_cache + (long)slot * nk + (long)kh * dk, q_s, dk, vec != 0) * scale;
        if (softcap > 0.f) z = softcap * tanhf(z / softcap);
        if (r1 != nullptr) z -= c1 * logf(1.0f + c2 * (float)(i - j));
        if (dist_bias != nullptr) z += dist_bias[(long)min(i - j, nd - 1) * hq + a];
      }
    }
    float p;
    if (sigmoid) {
      p = slot >= 0 ? sigmoidf_(z + bias) : 0.f;
    } else {
      const float mn = fmaxf(mx_, ft::wave_max(z));
      const float resc = mx_ == -INFINITY ? 0.f : expf(mx_ - mn);
      p = (slot >= 0 && mn != -INFINITY) ? expf(z - mn) : 0.f;
      l_ = l_ * resc + ft::wave_sum(p);
#pragma unroll
      for (int u = 0; u < NO; ++u) o[u] *= resc;
      mx_ = mn;
    }
    if constexpr (VEC) {
      const int passes = (cnt + kpp - 1) / kpp;
#pragma unroll 4
      for (int ps = 0; ps < passes; ++ps) {
        const int jj = ps * kpp + sub;                  // < 64: a lane past cnt has weight 0, slot -1
        const float pj = __shfl(p, jj);
        const int sj = __shfl(slot, jj);
        const bool ok = sj >= 0 && has_piece;
        const TC* vp = v_cache + (ok ? (long)sj * nv + (long)vh * dv + sg * Piece<TC>::N : 0L);
        float v[Piece<TC>::N];
        Piece<TC>::load(vp, v);
        const float w = ok ? pj : 0.f;
#pragma unroll
        for (int u = 0; u < Piece<TC>::N; ++u) o[u] += w * v[u];
      }
    } else {
      for (int jj = 0; jj < cnt; ++jj) {
        const float pj = __shfl(p, jj);
        const int sj = __shfl(slot, jj);
        if (sj < 0) continue;
        const TC* vp = v_cache + (long)sj * nv + (long)vh * dv;
#pragma unroll
        for (int u = 0; u < kMaxVCols; ++u) {
          const int c = lane + 64 * u;
          if (c < dv) o[u] += pj * ld(vp, c);
        }
      }
    }
  }
  if constexpr (VEC) {
    // lanes sub = 0, 1, ... hold partial sums of the same piece
    for (int off = lpk; off < 64; off <<= 1) {
#pragma unroll
      for (int u = 0; u < NO; ++u) o[u] += __shfl_xor(o[u], off);
    }
    if (sub == 0 && has_piece) {
#pragma unroll
      for (int u = 0; u < NO; ++u) o_s[wave * dv + sg * Piece<TC>::N + u] = o[u];
    }
  } else {
#pragma unroll
    for (int u = 0; u < kMaxVCols; ++u) {
      const int c = lane + 64 * u;
      if (c < dv) o_s[wave * dv + c] = o[u];
    }
  }
  if (lane == 0) {
    ml_s[2 * wave] = mx_;
    ml_s[2 * wave + 1] = l_;
  }
  __syncthreads();
  float* op = out + ((long)row * hq + a) * dv;
  for (int c = tid; c < dv; c += blockDim.x) {
    float acc = 0.f;
    if (sigmoid) {
#pragma unroll
      for (int w = 0; w < kWaves; ++w) acc += o_s[w * dv + c];
    } else {
      float mm = has_sink ? sink : -INFINITY;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) mm = fmaxf(mm, ml_s[2 * w]);
      float l = has_sink ? expf(sink - mm) : 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        const float f = ml_s[2 * w] == -INFINITY ? 0.f : expf(ml_s[2 * w] - mm);
        l += ml_s[2 * w + 1] * f;
        acc += o_s[w * dv + c] * f;
      }
      acc = l > 0.f ? acc / l : 0.f;
    }
    op[c] = acc;
  }
}

// ---------------------------------------------------------------------------------
// scores -> weights in place for the banded products.  S [gk = (g, m)] [(r, t)] [keys]:
// the rep query heads of a key head stacked along the rows.  grid (rep * rows, gk).
// The first `ext` columns are the positions 0 .. ext-1 (kept first tokens that lie before
// the band), column c >= ext is position key0 + c - ext.  A row's visible columns are
// the kept ones [0, ka) and its window (or block) [c_lo, c_hi].
// ---------------------------------------------------------------------------------
template <int NT>
__global__ void band_weights_kernel(float* __restrict__ S, int rows, int keys, int first_pos, int key0,
                                    int heads, int maps, int kv_heads, int window, float scale, int sigmoid,
                                    const float* __restrict__ r1, const float* __restrict__ r2,
                                    const float* __restrict__ pb, float softcap, int has_sink, float sink,
                                    int blocks, int keep_first, int ext, const float* __restrict__ dist_bias,
                                    int nd) {
  __shared__ float red[NT / 64];
  const int rep = heads / kv_heads;
  const int rr = blockIdx.x, gk = blockIdx.y;
  const int r = rr / rows, t = rr % rows;
  const int g = gk / maps, m = gk % maps;
  const int a = (g * rep + r) * maps + m;
  const int i = first_pos + t;
  float* sp = S + ((long)gk * rep * rows + rr) * keys;
  // visible columns [0, ka) and [c_lo, c_hi]
  const int hq = heads * maps;
  const int first_i = window > 0 ? (blocks ? (i / window) * window : max(0, i - window + 1)) : 0;
  const int c_hi = min(keys - 1, i - key0 + ext);
  const int c_lo = max(ext, first_i - key0 + ext);
  const int ka = window > 0 ? min(c_lo, ext + max(0, keep_first - key0)) : 0;
  const int nvis = ka + max(0, c_hi - c_lo + 1);
  const float c1 = r1 != nullptr ? r1[a] : 0.f, c2 = r1 != nullptr ? r2[a] : 0.f;
  auto score = [&](int c) {
    const int d = i - (c < ext ? c : key0 + c - ext);
    float z = sp[c] * scale;
    if (softcap > 0.f) z = softcap * tanhf(z / softcap);
    if (r1 != nullptr) z -= c1 * logf(1.0f + c2 * (float)d);
    if (dist_bias != nullptr) z += dist_bias[(long)min(d, nd - 1) * hq + a];
    return z;
  };
  for (int c = ka + threadIdx.x; c < min(c_lo, keys); c += NT) sp[c] = 0.f;
  for (int c = max(c_hi + 1, ka) + threadIdx.x; c < keys; c += NT) sp[c] = 0.f;
  if (sigmoid) {
    const float bias = pb != nullptr ? pb[a] : 0.f;
    for (int u = threadIdx.x; u < nvis; u += NT) {
      const int c = u < ka ? u : c_lo + u - ka;
      sp[c] = sigmoidf_(score(c) + bias);
    }
    return;
  }
  float mx_ = -INFINITY;
  for (int u = threadIdx.x; u < nvis; u += NT) {
    const int c = u < ka ? u : c_lo + u - ka;
    const float z = score(c);
    sp[c] = z;                         // each thread re-reads only its own columns
    mx_ = fmaxf(mx_, z);
  }
  mx_ = ft::wave_max(mx_);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx_;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) mx_ = fmaxf(mx_, red[w]);
  if (has_sink) mx_ = fmaxf(mx_, sink);
  float sum = 0.f;
  for (int u = threadIdx.x; u < nvis; u += NT) {
    const int c = u < ka ? u : c_lo + u - ka;
    const float p = expf(sp[c] - mx_);
    sp[c] = p;
    sum += p;
  }
  sum = block_sum<NT>(sum, red);
  if (has_sink) sum += expf(sink - mx_);
  const float inv = sum > 0.f ? 1.0f / sum : 0.f;
  for (int u = threadIdx.x; u < nvis; u += NT) {
    const int c = u < ka ? u : c_lo + u - ka;
    sp[c] *= inv;
  }
}

// one wave per (row, head): o = a1 - lam a2; o / rms(o) * post * sigmoid(gate)
template <typename TG, typename TO>
__global__ void diff_combine_kernel(TO* __restrict__ out, const float* __restrict__ a, const TG* __restrict__ gate,
                                    long gate_stride, long pairs, int heads, int dv, float lam, float post,
                                    float eps) {
  const long pair = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (pair >= pairs) return;
  const int lane = threadIdx.x & 63;
  const long row = pair / heads;
  const int h = (int)(pair % heads);
  const float* a1 = a + ((row * heads + h) * 2) * dv;
  const float* a2 = a1 + dv;
  float ss = 0.f;
  for (int c = lane; c < dv; c += 64) {
    const float o = a1[c] - lam * a2[c];
    ss += o * o;
  }
  ss = ft::wave_sum(ss);
  const float f = 1.0f / sqrtf(ss / (float)dv + eps) * post * sigmoidf_(ld(gate, row * gate_stride + h));
  for (int c = lane; c < dv; c += 64) st(out, (row * heads + h) * dv + c, (a1[c] - lam * a2[c]) * f);
}

}  // namespace mx

using namespace mx;

extern "C" int mx_attn_prep(float* q_out, const void* qkv, int bf16, long stride, int nq, int nk, int nv,
                            const float* wq, const float* wk, float eps, const float* table, int table_rows,
                            int rot_dims, int head_dim, const int* positions, const int* slots, void* k_cache,
                            void* v_cache, int cache_bf16, long num_slots, long rows, hipStream_t s) {
  if (rows <= 0) return 0;
  if (head_dim < 1 || rot_dims < 0 || rot_dims > head_dim || rot_dims % 2 || nq % head_dim || nk % head_dim) return -1;
  const dim3 grid((unsigned)rows), block(256);
#define MX_PREP(T, TC)                                                                                     \
  hipLaunchKernelGGL((attn_prep_kernel<T, TC, 256>), grid, block, 0, s, q_out, (const T*)qkv, stride, nq, nk, \
                     nv, wq, wk, eps, table, table_rows, rot_dims, head_dim, positions, slots, (TC*)k_cache,  \
                     (TC*)v_cache, num_slots)
  if (bf16 && cache_bf16) MX_PREP(bf16_t, bf16_t);
  else if (bf16) MX_PREP(bf16_t, float);
  else if (cache_bf16) MX_PREP(float, bf16_t);
  else MX_PREP(float, float);
#undef MX_PREP
  return (int)hipGetLastError();
}

extern "C" int mx_conv_hist(const void* x, int bf16, long x_stride, float* hist, const int* start, const int* pos0,
                            const int* slot, int num_segs, int channels, int taps, int num_slots, hipStream_t s);

extern "C" int mx_conv_attn_prep(float* q_out, const void* qkv, int bf16, long stride, int nq, int nk, int nv,
                                 const float* conv_w, int taps, float* hist, const int* start, const int* pos0,
                                 const int* slot, int num_segs, int num_state_slots, const float* wq,
                                 const float* wk, float eps, int head_dim, const int* slots, void* k_cache,
                                 void* v_cache, int cache_bf16, long num_slots, long rows, hipStream_t s) {
  if (rows <= 0 || num_segs <= 0) return 0;
  if (head_dim < 1 || nq % head_dim || nk % head_dim || taps < 1 || nv < 0) return -1;
  const int channels = nq + nk + nv;
  const size_t shm = (size_t)4 * head_dim * sizeof(float);
  const int chunks = (nq + nk) / head_dim + (nv + head_dim - 1) / head_dim;
  if (shm > 64 * 1024 || rows > 0x7fffffffL || (chunks + 3) / 4 > 65535) return -3;
  const dim3 grid((unsigned)rows, (unsigned)((chunks + 3) / 4)), block(256);
#define MX_CPREP(T, TC)                                                                                       \
  hipLaunchKernelGGL((conv_attn_prep_kernel<T, TC>), grid, block, shm, s, q_out, (const T*)qkv, stride, nq, nk, \
                     nv, conv_w, taps, hist, start, pos0, slot, num_segs, num_state_slots, wq, wk, eps,         \
                     head_dim, slots, (TC*)k_cache, (TC*)v_cache, num_slots)
  if (bf16 && cache_bf16) MX_CPREP(bf16_t, bf16_t);
  else if (bf16) MX_CPREP(bf16_t, float);
  else if (cache_bf16) MX_CPREP(float, bf16_t);
  else MX_CPREP(float, float);
#undef MX_CPREP
  int rc = (int)hipGetLastError();
  if (rc == 0 && taps > 1)
    rc = mx_conv_hist(qkv, bf16, stride, hist, start, pos0, slot, num_segs, channels, taps, num_state_slots, s);
  return rc;
}

extern "C" int mx_window_max_dv() { return 64 * kMaxVCols; }

extern "C" int mx_window_attention(float* out, const float* q, const void* k_cache, const void* v_cache,
                                   int cache_bf16, const int* start, const int* pos0, const int* kv_len,
                                   const int* bt, int bt_stride, int num_segs, long total_rows, int heads, int maps,
                                   int kv_heads, int dk, int dv, int window, float scale, int sigmoid,
                                   const float* r1, const float* r2, const float* pb, int block_size,
                                   int num_blocks, int skip_from, float softcap, int has_sink, float sink,
                                   int blocks, int keep_first, const float* dist_bias, int nd, hipStream_t s) {
  if (num_segs <= 0 || total_rows <= 0) return 0;
  if (dv < 1 || dv > mx_window_max_dv() || dk < 1 || heads % kv_heads || maps < 1) return -1;
  if (keep_first < 0 || (dist_bias != nullptr && nd < 1) || (blocks && window < 1)) return -1;
  const int hq = heads * maps;
  if (total_rows > 0x7fffffffL || hq > 65535) return -2;
  const long es = cache_bf16 ? 2 : 4;
  const long nk = (long)kv_heads * maps * dk;
  const int vec = (dk * es) % 16 == 0 && (nk * es) % 16 == 0 && ((uintptr_t)k_cache) % 16 == 0;
  // value rows in whole 16-byte pieces, at most 64 per row: the vector form of the sums
  const long nv = (long)kv_heads * dv;
  const long pieces = dv * es / 16;
  const bool vecv = (dv * es) % 16 == 0 && (nv * es) % 16 == 0 && ((uintptr_t)v_cache) % 16 == 0 && pieces <= 64;
  int lpk = 1;
  while (lpk < pieces) lpk <<= 1;
  const size_t shm = (size_t)(dk + kWaves * dv + 2 * kWaves) * sizeof(float);
  if (shm > 64 * 1024) return -3;
  const dim3 grid((unsigned)total_rows, (unsigned)hq), block(64 * kWaves);
#define MX_WATTN(V)                                                                                          \
  MX_DISPATCH_T(cache_bf16, hipLaunchKernelGGL((window_attn_kernel<T, V>), grid, block, shm, s, out, q,         \
                                               (const T*)k_cache, (const T*)v_cache, start, pos0, kv_len, bt,  \
                                               bt_stride, num_segs, heads, maps, kv_heads, dk, dv, window, scale, \
                                               sigmoid, r1, r2, pb, block_size, num_blocks, skip_from, vec, lpk,  \
                                               softcap, has_sink, sink, blocks, keep_first, dist_bias, nd))
  if (vecv) MX_WATTN(true);
  else MX_WATTN(false);
#undef MX_WATTN
  return (int)hipGetLastError();
}

extern "C" int mx_band_weights(float* S, int gk, int rep_rows_total, int rows, int keys, int first_pos, int key0,
                               int heads, int maps, int kv_heads, int window, float scale, int sigmoid,
                               const float* r1, const float* r2, const float* pb, float softcap, int has_sink,
                               float sink, int blocks, int keep_first, int ext, const float* dist_bias, int nd,
                               hipStream_t s) {
  if (gk <= 0 || rep_rows_total <= 0 || keys <= 0) return 0;
  if (heads % kv_heads || gk != kv_heads * maps || rep_rows_total != heads / kv_heads * rows || gk > 65535) return -1;
  if (keep_first < 0 || ext < 0 || ext > keys || ext > key0 || (dist_bias != nullptr && nd < 1) ||
      (blocks && window < 1))
    return -1;
  hipLaunchKernelGGL((band_weights_kernel<256>), dim3((unsigned)rep_rows_total, (unsigned)gk), dim3(256), 0, s, S,
                     rows, keys, first_pos, key0, heads, maps, kv_heads, window, scale, sigmoid, r1, r2, pb, softcap,
                     has_sink, sink, blocks, keep_first, ext, dist_bias, nd);
  return (int)hipGetLastError();
}

extern "C" int mx_diff_combine(void* out, int out_bf16, const float* a, const void* gate, int gate_bf16,
                               long gate_stride, long rows, int heads, int dv, float lam, float post, float eps,
                               hipStream_t s) {
  const long pairs = rows * heads;
  if (pairs <= 0) return 0;
  const dim3 grid((unsigned)((pairs + 3) / 4)), block(256);
  if (gate_bf16 && out_bf16)
    hipLaunchKernelGGL((diff_combine_kernel<bf16_t, bf16_t>), grid, block, 0, s, (bf16_t*)out, a,
                       (const bf16_t*)gate, gate_stride, pairs, heads, dv, lam, post, eps);
  else if (!gate_bf16 && !out_bf16)
    hipLaunchKernelGGL((diff_combine_kernel<float, float>), grid, block, 0, s, (float*)out, a, (const float*)gate,
                       gate_stride, pairs, heads, dv, lam, post, eps);
  else
    return -1;
  return (int)hipGetLastError();
}
