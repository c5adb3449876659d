// C[M,N] = X[M,K] * W[N,K]^T for few rows (M <= 64): the decode-time matrix product, bound by the
// one pass over W.  bfloat16 inputs, float32 accumulation on the matrix cores, output bfloat16 or
// float32.  (The reference's counterpart for one row is src/flint/cuda/matvec.cu:61-87.)
//
// A block of WN x 8 waves owns 16*RT*WN rows of W.  The 8 waves of a row group split K: step s
// (32 elements) belongs to wave (s / 2) % 8, so the block reads 1 KB of every row at a time.  W
// fragments go from global memory straight to registers (W rows are the A operand, lane l holds
// row l % 16); the rows of X, which every wave needs, are staged through shared memory one chunk
// of K at a time and read from there as B operands, so lane l ends with C[n = 4*(l/16)+e][m = l%16].
// Partial sums of the 8 waves are added through shared memory in a fixed order.  Which wave adds
// which step does not depend on M or on the tile shape: an output is the same bits whatever else
// is in the batch.
//
// Epilogues: plain store, or SwiGLU over a stacked [gate; up] weight (out[m, i] =
// silu(gate_i) * up_i, src/flint/cuda/swiglu.cu:44-49), where a wave owns a gate tile and the up
// tile of the same columns; gate and up are rounded to the activation dtype first, as the
// unfused path stores them.
#include "mfma.h"

#define SK_WK 8            // waves that split K
#define SK_EPI_NONE 0
#define SK_EPI_SWIGLU 1

// MT: 16-row tiles of X; RT: 16-row tiles of W per wave; WN: row groups per block; G: granules of
// 2 steps that a wave takes per chunk (a chunk is 512*G elements of K).
template <int MT, int RT, int WN, int G, int EPI, typename OutT>
__global__ __launch_bounds__(WN* SK_WK * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                      const bf16_t* __restrict__ W,
                                                                      OutT* __restrict__ C, int M,
                                                                      int N, int K, int n_out) {
  constexpr int NT = WN * SK_WK * 64;
  constexpr int CK = 512 * G;                    // elements of K per chunk
  constexpr int ROW_B = CK * 2;                  // bytes of a staged row; 16-byte pieces are swizzled
  constexpr int X_BYTES = 16 * MT * ROW_B;
  constexpr int RED_BYTES = SK_WK * WN * RT * MT * 1024;
  constexpr int LDS_BYTES = X_BYTES > RED_BYTES ? X_BYTES : RED_BYTES;
  constexpr int XV = CK / 8;                     // 16-byte pieces of a staged row
  constexpr int ROWS_PASS = NT / XV;             // rows staged per pass of the block
  constexpr int PASSES = (16 * MT + ROWS_PASS - 1) / ROWS_PASS;
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave / SK_WK, wk = wave % SK_WK;
  const int r = lane & 15, g = lane >> 4;
  const int group = blockIdx.x * WN + wn;                       // row group of this wave
  const int n_steps = (K + 31) / 32;
  const int n_chunks = (K + CK - 1) / CK;

  // first row of each of this wave's tiles
  int tile_row[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (EPI == SK_EPI_SWIGLU)
      tile_row[rt] = (rt & 1) * n_out + (group * (RT / 2) + (rt >> 1)) * 16;
    else
      tile_row[rt] = (group * RT + rt) * 16;
  }
  const bf16_t* wp[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int n = tile_row[rt] + r;
    if (n > N - 1) n = N - 1;                   // rows past the end read the last row; not stored
    wp[rt] = W + (size_t)n * K + g * 8;
  }

  f32x4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // staging of X: thread t carries piece (t % XV) of rows (t / XV) + p * ROWS_PASS
  const int x_col = tid % XV, x_row0 = tid / XV;
  uint4 xr[PASSES];
  auto load_x = [&](int chunk) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int row = x_row0 + p * ROWS_PASS;
      const int k = chunk * CK + x_col * 8;
      xr[p] = (row < M && k < K) ? *reinterpret_cast<const uint4*>(X + (size_t)row * K + k)
                                 : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  auto store_x = [&]() {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int row = x_row0 + p * ROWS_PASS;
      if (row < 16 * MT) *reinterpret_cast<uint4*>(lds + row * ROW_B + ((x_col ^ (row & 7)) * 16)) = xr[p];
    }
  };
  Frag a[2][G][2][RT];
  auto load_w = [&](int chunk, Frag (&dst)[G][2][RT]) {
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int s = chunk * (CK / 32) + gi * 16 + wk * 2 + u;
        const bool in = s < n_steps && (s * 32 + g * 8) < K;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) dst[gi][u][rt] = in ? frag_load(wp[rt] + s * 32) : frag_zero();
      }
  };
  auto compute = [&](Frag (&src)[G][2][RT]) {
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int piece = (gi * 16 + wk * 2 + u) * 4 + g;         // 16-byte piece of the chunk
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          Frag b;
          b.u = *reinterpret_cast<const uint4*>(lds + (mt * 16 + r) * ROW_B + ((piece ^ (r & 7)) * 16));
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) acc[rt][mt] = mfma_bf16(src[gi][u][rt], b, acc[rt][mt]);
        }
      }
  };

  load_x(0);
  load_w(0, a[0]);
  for (int c = 0; c < n_chunks; c += 2) {
    // even chunk from a[0], odd chunk from a[1]
    store_x();
    __syncthreads();
    if (c + 1 < n_chunks) {
      load_x(c + 1);
      load_w(c + 1, a[1]);
    }
    compute(a[0]);
    __syncthreads();
    if (c + 1 >= n_chunks) break;
    store_x();
    __syncthreads();
    if (c + 2 < n_chunks) {
      load_x(c + 2);
      load_w(c + 2, a[0]);
    }
    compute(a[1]);
    __syncthreads();
  }

  // ---- add the partial sums of the 8 waves in order, apply the epilogue, store
  float* red = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      *reinterpret_cast<float4*>(red + ((((wk * WN + wn) * RT + rt) * MT + mt) * 64 + lane) * 4) =
          make_float4(acc[rt][mt][0], acc[rt][mt][1], acc[rt][mt][2], acc[rt][mt][3]);
  __syncthreads();
  constexpr int OUT_RT = (EPI == SK_EPI_SWIGLU) ? RT / 2 : RT;
  constexpr int ITEMS = WN * OUT_RT * MT * 64;
  const int ldc = (EPI == SK_EPI_SWIGLU) ? n_out : N;
  for (int it = tid; it < ITEMS; it += NT) {
    const int ln = it & 63;
    const int mt = (it >> 6) % MT;
    const int ort = (it / (64 * MT)) % OUT_RT;
    const int w_n = it / (64 * MT * OUT_RT);
    float v[4];
    int n;
    if (EPI == SK_EPI_SWIGLU) {
      float gsum[4] = {0.f, 0.f, 0.f, 0.f}, usum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < SK_WK; ++w) {
        const float4 pg = *reinterpret_cast<const float4*>(
            red + ((((w * WN + w_n) * RT + 2 * ort) * MT + mt) * 64 + ln) * 4);
        const float4 pu = *reinterpret_cast<const float4*>(
            red + ((((w * WN + w_n) * RT + 2 * ort + 1) * MT + mt) * 64 + ln) * 4);
        gsum[0] += pg.x; gsum[1] += pg.y; gsum[2] += pg.z; gsum[3] += pg.w;
        usum[0] += pu.x; usum[1] += pu.y; usum[2] += pu.z; usum[3] += pu.w;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float gt = bf16_to_f32(f32_to_bf16(gsum[e])), up = bf16_to_f32(f32_to_bf16(usum[e]));
        v[e] = up * gt / (1.0f + expf(-gt));
      }
      n = ((blockIdx.x * WN + w_n) * OUT_RT + ort) * 16 + 4 * (ln >> 4);
    } else {
      float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < SK_WK; ++w) {
        const float4 p = *reinterpret_cast<const float4*>(
            red + ((((w * WN + w_n) * RT + ort) * MT + mt) * 64 + ln) * 4);
        sum[0] += p.x; sum[1] += p.y; sum[2] += p.z; sum[3] += p.w;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = sum[e];
      n = ((blockIdx.x * WN + w_n) * RT + ort) * 16 + 4 * (ln >> 4);
    }
    const int m = mt * 16 + (ln & 15);
    if (m >= M || n >= ldc) continue;
    OutT* dst = C + (size_t)m * ldc + n;
    if (n + 3 < ldc && (ldc & 3) == 0) {
      if (sizeof(OutT) == 2) {
        uint2 pk;
        pk.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        pk.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        *reinterpret_cast<uint2*>(dst) = pk;
      } else {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < ldc) Conv<OutT>::store(dst + e, v[e]);
    }
  }
}

template <int MT, int RT, int WN, int G, int EPI, typename OutT>
static int launch_skinny(const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int n_out,
                         hipStream_t stream) {
  const int rows = (EPI == SK_EPI_SWIGLU) ? n_out : N;
  const int tiles = (rows + 15) / 16;
  constexpr int OUT_RT = (EPI == SK_EPI_SWIGLU) ? RT / 2 : RT;
  const int blocks = (tiles + OUT_RT * WN - 1) / (OUT_RT * WN);
  gemm_skinny_kernel<MT, RT, WN, G, EPI, OutT>
      <<<blocks, WN * SK_WK * 64, 0, stream>>>(X, W, C, M, N, K, n_out);
  return llm_launch_status();
}

template <int EPI, typename OutT>
static int pick_shape(const bf16_t* X, const bf16_t* W, OutT* C, int M, int N, int K, int n_out,
                      hipStream_t stream) {
  constexpr int RT = (EPI == SK_EPI_SWIGLU) ? 2 : 1;
  switch ((M + 15) / 16) {
    case 1: return launch_skinny<1, RT, 1, 2, EPI, OutT>(X, W, C, M, N, K, n_out, stream);
    case 2: return launch_skinny<2, RT, 2 / RT, 1, EPI, OutT>(X, W, C, M, N, K, n_out, stream);
    case 3: return launch_skinny<3, RT, 2 / RT, 1, EPI, OutT>(X, W, C, M, N, K, n_out, stream);
    case 4: return launch_skinny<4, RT, 2 / RT, 1, EPI, OutT>(X, W, C, M, N, K, n_out, stream);
  }
  return LLM_ERR_ARG;
}

static bool skinny_args_ok(const void* X, const void* W, const void* C, int M, int K) {
  if (M > 64 || K <= 0 || (K & 7)) return false;
  if ((((uintptr_t)X) | ((uintptr_t)W) | ((uintptr_t)C)) & 15) return false;
  return true;
}

extern "C" int llm_gemm_skinny_bf16(const void* X, const void* W, void* C, int out_dtype, int M, int N,
                                    int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return LLM_OK;
  if (!skinny_args_ok(X, W, C, M, K)) return LLM_ERR_ARG;
  if (out_dtype == LLM_DTYPE_BF16)
    return pick_shape<SK_EPI_NONE, bf16_t>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, N, K, N, stream);
  if (out_dtype == LLM_DTYPE_F32)
    return pick_shape<SK_EPI_NONE, float>((const bf16_t*)X, (const bf16_t*)W, (float*)C, M, N, K, N, stream);
  return LLM_ERR_ARG;
}

// out[M, I] = silu(X Wg^T) * (X Wu^T) with W = [Wg; Wu] stacked, [2I, K]; I a multiple of 16.
extern "C" int llm_gemm_skinny_swiglu_bf16(const void* X, const void* W, void* C, int M, int I, int K,
                                           hipStream_t stream) {
  if (M <= 0 || I <= 0) return LLM_OK;
  if (!skinny_args_ok(X, W, C, M, K) || (I & 15)) return LLM_ERR_ARG;
  return pick_shape<SK_EPI_SWIGLU, bf16_t>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, 2 * I, K, I,
                                            stream);
}
