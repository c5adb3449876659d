// C[M,N] = X[M,K] * W[N,K]^T for few rows (M <= 64): the decode-time matrix product, bound by the
// one pass over W.  bfloat16 inputs, float32 accumulation on the matrix cores, output bfloat16 or
// float32.  (The reference's counterpart for one row is src/flint/cuda/matvec.cu:61-87.)
//
// A block owns 16*RT rows of W and splits K over its waves in blocks of 128; every lane reads 64
// contiguous bytes of one W row per block, and the X fragments it needs from cache.  W rows are
// the A operand, X rows the B operand, so lane l ends with C[n = 4*(l/16)+e][m = l%16].  Partial
// sums of the waves are added through shared memory in a fixed order: an output does not depend on
// M or on which other rows are in the batch.
#include "mfma.h"

template <int MT, int RT, int WAVES, typename OutT>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                 const bf16_t* __restrict__ W,
                                                                 OutT* __restrict__ C, int M, int N,
                                                                 int K) {
  __shared__ float red[WAVES][RT * MT * 4][64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * RT);

  f32x4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bf16_t* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n = n0 + rt * 16 + r;
    if (n > N - 1) n = N - 1;                   // rows past the end read the last row; not stored
    wrow[rt] = W + (size_t)n * K;
  }
  const bf16_t* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    xok[mt] = m < M;
    xrow[mt] = X + (size_t)(xok[mt] ? m : 0) * K;
  }

  const int nkb = (K + 127) / 128;
  for (int kb = wave; kb < nkb; kb += WAVES) {
    const int k = kb * 128 + g * 32;
    Frag a[RT][4], b[MT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = k + j * 8;
      const bool in = kk < K;                   // K is a multiple of 8: a piece is whole or absent
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) a[rt][j] = in ? frag_load(wrow[rt] + kk) : frag_zero();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[mt][j] = (in && xok[mt]) ? frag_load(xrow[mt] + kk) : frag_zero();
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = mfma_bf16(a[rt][j], b[mt][j], acc[rt][mt]);
  }

#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[wave][(rt * MT + mt) * 4 + e][lane] = acc[rt][mt][e];
  __syncthreads();
  for (int it = threadIdx.x; it < RT * MT * 4 * 64; it += WAVES * 64) {
    const int idx = it >> 6, ln = it & 63;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) sum += red[w][idx][ln];
    const int rt = idx / (MT * 4), mt = (idx >> 2) % MT, e = idx & 3;
    const int n = n0 + rt * 16 + 4 * (ln >> 4) + e;
    const int m = mt * 16 + (ln & 15);
    if (n < N && m < M) Conv<OutT>::store(C + (size_t)m * N + n, sum);
  }
}

template <int MT, int RT, typename OutT>
static int launch_skinny(const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K,
                         hipStream_t stream) {
  constexpr int WAVES = 4;
  const int blocks = (N + 16 * RT - 1) / (16 * RT);
  gemm_skinny_kernel<MT, RT, WAVES, OutT><<<blocks, WAVES * 64, 0, stream>>>(X, W, C, M, N, K);
  return llm_launch_status();
}

template <int MT, typename OutT>
static int pick_rt(const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int rt,
                   hipStream_t stream) {
  if constexpr (MT <= 2) {
    if (rt >= 4) return launch_skinny<MT, 4, OutT>(X, W, C, M, N, K, stream);
  }
  if (rt >= 2) return launch_skinny<MT, 2, OutT>(X, W, C, M, N, K, stream);
  return launch_skinny<MT, 1, OutT>(X, W, C, M, N, K, stream);
}

template <typename OutT>
static int pick_mt(const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int rt,
                   hipStream_t stream) {
  switch ((M + 15) / 16) {
    case 1: return pick_rt<1, OutT>(X, W, C, M, N, K, rt, stream);
    case 2: return pick_rt<2, OutT>(X, W, C, M, N, K, rt, stream);
    case 3: return pick_rt<3, OutT>(X, W, C, M, N, K, rt, stream);
    case 4: return pick_rt<4, OutT>(X, W, C, M, N, K, rt, stream);
  }
  return LLM_ERR_ARG;
}

// rows_per_block: 0 lets the library choose; otherwise 16, 32 or 64 rows of W per block.
extern "C" int llm_gemm_skinny_bf16(const void* X, const void* W, void* C, int out_dtype, int M, int N,
                                    int K, int rows_per_block, hipStream_t stream) {
  if (M <= 0 || N <= 0) return LLM_OK;
  if (M > 64 || K <= 0 || (K & 7)) return LLM_ERR_ARG;
  if ((((uintptr_t)X) | ((uintptr_t)W)) & 15) return LLM_ERR_ARG;
  int rt = rows_per_block / 16;
  if (rows_per_block == 0) rt = (N >= 32768) ? 4 : (N >= 8192 ? 2 : 1);
  if (out_dtype == LLM_DTYPE_BF16)
    return pick_mt<bf16_t>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, N, K, rt, stream);
  if (out_dtype == LLM_DTYPE_F32)
    return pick_mt<float>((const bf16_t*)X, (const bf16_t*)W, (float*)C, M, N, K, rt, stream);
  return LLM_ERR_ARG;
}
