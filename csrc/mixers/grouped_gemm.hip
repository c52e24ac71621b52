// Grouped matrix product for the experts of a mixture layer on many rows (prefill):
// the rows of A [M, K] are sorted by group, group g owns the rows up to offs[g] (running
// sums of the group sizes, read on the device: no host round trip), and
//     C[rows of g] = A[rows of g] . W[g]^T,      W [G, N, K], bf16 in, fp32 accumulate, bf16 out.
//
// A workgroup of four waves owns a 64 x 64 tile of C inside one group (blockIdx.y walks
// the groups' row tiles; slots past the last tile exit at once), K in steps of 64 through
// LDS with the next step's 16-byte global loads in flight during the MFMAs
// (v_mfma_f32_16x16x32_bf16; a wave owns 32 x 32 = 2 x 2 tiles).  Rows past a group's end,
// columns past N and k past K are zero-filled on load and not stored.
#include "mx_common.h"

namespace mx {

typedef __bf16 gg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gg_f32x4 __attribute__((ext_vector_type(4)));

constexpr int kGM = 64, kGN = 64, kGK = 64;
constexpr int kGLd = kGK + 8;        // LDS row stride (bf16): 144 bytes, keeps 16-byte alignment

__global__ void __launch_bounds__(256)
grouped_gemm_kernel(bf16_t* __restrict__ C, const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                    const int* __restrict__ offs, int groups, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) bf16_t As[kGM * kGLd];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[kGN * kGLd];
  // this workgroup's group and row tile
  int g = 0, row0 = 0, end = 0;
  {
    int t = blockIdx.y, prev = 0;
    bool found = false;
    for (g = 0; g < groups; ++g) {
      end = min(max(offs[g], prev), M);
      const int tiles = (end - prev + kGM - 1) / kGM;
      if (t < tiles) {
        row0 = prev + t * kGM;
        found = true;
        break;
      }
      t -= tiles;
      prev = end;
    }
    if (!found) return;
  }
  const int n0 = blockIdx.x * kGN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l15 = lane & 15, g4 = lane >> 4;
  const bf16_t* Wg = W + (long)g * N * K;

  uint4 ra[2], rw[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int piece = tid + 256 * p;
      const int r = piece >> 3, k = k0 + (piece & 7) * 8;
      const int row = row0 + r, col = n0 + r;
      ra[p] = (row < end && k < K) ? *reinterpret_cast<const uint4*>(A + (long)row * K + k) : uint4{0, 0, 0, 0};
      rw[p] = (col < N && k < K) ? *reinterpret_cast<const uint4*>(Wg + (long)col * K + k) : uint4{0, 0, 0, 0};
    }
  };
  gg_f32x4 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = gg_f32x4{0.f, 0.f, 0.f, 0.f};

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += kGK) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int piece = tid + 256 * p;
      const int off = (piece >> 3) * kGLd + (piece & 7) * 8;
      *reinterpret_cast<uint4*>(As + off) = ra[p];
      *reinterpret_cast<uint4*>(Ws + off) = rw[p];
    }
    __syncthreads();
    if (k0 + kGK < K) fetch(k0 + kGK);
#pragma unroll
    for (int ks = 0; ks < kGK / 32; ++ks) {
      uint4 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a[i] = *reinterpret_cast<const uint4*>(As + (wm * 32 + i * 16 + l15) * kGLd + ks * 32 + g4 * 8);
        b[i] = *reinterpret_cast<const uint4*>(Ws + (wn * 32 + i * 16 + l15) * kGLd + ks * 32 + g4 * 8);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(gg_bf16x8, a[i]),
                                                              __builtin_bit_cast(gg_bf16x8, b[j]), acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // lane (g4, l15) holds rows 4 g4 .. 4 g4 + 3 of column l15 of each 16 x 16 tile
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 32 + j * 16 + l15;
      if (col >= N) continue;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int row = row0 + wm * 32 + i * 16 + 4 * g4 + v;
        if (row < end) C[(long)row * N + col] = ft::f32_to_bf16(acc[i][j][v]);
      }
    }
}

}  // namespace mx

extern "C" int mx_grouped_gemm(void* C, const void* A, const void* W, const int* offs, int groups, long M, int N,
                               int K, hipStream_t s) {
  if (M <= 0 || N <= 0 || groups <= 0) return 0;
  if (K < 8 || K % 8 || M > 0x7fffffffL) return -1;
  if (((uintptr_t)A) % 16 || ((uintptr_t)W) % 16) return -2;
  const long tiles = (M + mx::kGM - 1) / mx::kGM + groups;
  if (tiles > 65535) return -3;
  const dim3 grid((unsigned)((N + mx::kGN - 1) / mx::kGN), (unsigned)tiles), block(256);
  hipLaunchKernelGGL(mx::grouped_gemm_kernel, grid, block, 0, s, (mx::bf16_t*)C, (const mx::bf16_t*)A,
                     (const mx::bf16_t*)W, offs, groups, (int)M, N, K);
  return (int)hipGetLastError();
}
