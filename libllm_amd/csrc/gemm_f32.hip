// True 32-bit matrix product C[M,N] = A[M,K] * W[N,K]^T with float32 storage and float32 FMA
// accumulation in a fixed order over K (no matrix-core reduced-precision mode).  Tiled through
// shared memory: 64x64 output tile per block of 256 threads, 4x4 outputs per thread.
//
// The sum over K is formed in three levels: 16 terms in a row, 16 such sums, and the sums of
// those (256 terms each).  One running sum over all of K loses about sqrt(K) * 2^-24 of the
// terms' size (with K = 8,200 the logits of a two-layer model were 2.3e-5 off in a row's L2
// norm against a float64 computation, three times what a blocked sum gives); the order is still
// fixed by K alone, so a row's bits do not depend on what else a step holds.
#include "common.h"

template <int BM, int BN, int BK>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A,
                                                        const float* __restrict__ W,
                                                        float* __restrict__ C, int M, int N, int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[4][4], mid[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = mid[i][j] = 0.f;

  int tile = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
    float part[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[i][j] = 0.f;
#pragma unroll
    for (int e = tid; e < BM * BK; e += 256) {
      const int r = e / BK, c = e % BK;
      const int gm = m0 + r, gk = k0 + c;
      As[c][r] = (gm < M && gk < K) ? A[(size_t)gm * K + gk] : 0.f;
    }
#pragma unroll
    for (int e = tid; e < BN * BK; e += 256) {
      const int r = e / BK, c = e % BK;
      const int gn = n0 + r, gk = k0 + c;
      Ws[c][r] = (gn < N && gk < K) ? W[(size_t)gn * K + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
    }
    const bool fold = (++tile % 16) == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        mid[i][j] += part[i][j];
        if (fold) {
          acc[i][j] += mid[i][j];
          mid[i][j] = 0.f;
        }
      }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] += mid[i][j];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) C[(size_t)gm * N + gn] = acc[i][j];
    }
  }
}

// The same sums for up to 16 rows of A (decode steps): a block of 256 threads takes 16 rows of W,
// one output a thread, and 64 elements of K between barriers, loaded 16 bytes a thread.  A block of
// the kernel above would compute 64 rows of A of which up to 16 exist, and a weight of 2,048 rows
// would give 32 blocks for 256 compute units.  The terms are added in the same order (16 in a row,
// 16 such sums, the sums of those), so a row's bits are the same from either kernel.
template <int BK>
__global__ __launch_bounds__(256) void gemm_f32_few_rows_kernel(const float* __restrict__ A,
                                                                 const float* __restrict__ W,
                                                                 float* __restrict__ C, int M, int N, int K,
                                                                 int vec) {
  __shared__ float As[16][BK + 1];
  __shared__ float Ws[16][BK + 1];
  const int tid = threadIdx.x;
  const int n = tid % 16, m = tid / 16;
  const int n0 = blockIdx.x * 16;
  const int lr = tid / (BK / 4), lc = (tid % (BK / 4)) * 4;      // the row and the 4 elements this thread loads
  float acc = 0.f, mid = 0.f;
  int tile = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int r = lr; r < 16; r += 256 / (BK / 4)) {
      const int gk = k0 + lc;
      float4 a = make_float4(0.f, 0.f, 0.f, 0.f), w = make_float4(0.f, 0.f, 0.f, 0.f);
      if (vec && gk + 3 < K) {
        if (r < M) a = *reinterpret_cast<const float4*>(A + (size_t)r * K + gk);
        if (n0 + r < N) w = *reinterpret_cast<const float4*>(W + (size_t)(n0 + r) * K + gk);
      } else {
        float av[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (r < M && gk + e < K) av[e] = A[(size_t)r * K + gk + e];
          if (n0 + r < N && gk + e < K) wv[e] = W[(size_t)(n0 + r) * K + gk + e];
        }
        a = make_float4(av[0], av[1], av[2], av[3]);
        w = make_float4(wv[0], wv[1], wv[2], wv[3]);
      }
      As[r][lc] = a.x; As[r][lc + 1] = a.y; As[r][lc + 2] = a.z; As[r][lc + 3] = a.w;
      Ws[r][lc] = w.x; Ws[r][lc + 1] = w.y; Ws[r][lc + 2] = w.z; Ws[r][lc + 3] = w.w;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < BK; c += 16) {
      if (k0 + c < K) {                      // (a tile of 16 that lies beyond K does not exist in the kernel above either)
        float part = 0.f;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) part = fmaf(As[m][c + kk], Ws[n][c + kk], part);
        mid += part;
        if ((++tile % 16) == 0) {
          acc += mid;
          mid = 0.f;
        }
      }
    }
    __syncthreads();
  }
  acc += mid;
  if (m < M && n0 + n < N) C[(size_t)m * N + n0 + n] = acc;
}

extern "C" int llm_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K,
                            hipStream_t stream) {
  if (M <= 0 || N <= 0) return LLM_OK;
  if (K <= 0) return LLM_ERR_ARG;
  if (M <= 16) {
    const int vec = (K % 4 == 0) && ((((uintptr_t)A) | ((uintptr_t)W)) & 15) == 0;
    gemm_f32_few_rows_kernel<64><<<(N + 15) / 16, 256, 0, stream>>>(A, W, C, M, N, K, vec);
    return llm_launch_status();
  }
  const int gy = (M + 63) / 64, gx = (N + 63) / 64;
  if (gy > 65535) return LLM_ERR_ARG;
  gemm_f32_kernel<64, 64, 16><<<dim3(gx, gy), 256, 0, stream>>>(A, W, C, M, N, K);
  return llm_launch_status();
}
