// C[M,N] = X[M,K] * W[N,K]^T for 33 to 256 rows: still bound by the one pass over W, but with too
// many rows for a block to stage all of them per 16 rows of W, as the product for few rows does.
// bfloat16 inputs, float32 accumulation on the matrix cores.  (Up to 128 rows a block takes all
// the rows; beyond, two blocks take a slab of rows each, see the kernel's first lines.)
//
// A block owns 64 rows of W over all of K or one slice of it.  Four of its eight waves compute:
// two pairs of waves with two tiles of 16 rows each (what a wave reads of X from shared memory
// serves both tiles), the first wave of a pair taking the first two steps (of 32 elements) of
// every chunk of 128, the second the other two.  W is the copy tiled for the matrix cores
// (llm_pack_weight): a wave's fragment of a step is 1 KiB in a row, and goes from global memory
// straight to registers, three chunks ahead (four register stages: with six and five chunks
// ahead the kernel needs 164 registers instead of 128, one block instead of two fits a compute
// unit, and it is 3 to 7 % slower).  The rows of X go through shared memory, a chunk at a
// time, in two buffers filled in turns (one barrier a chunk), and the other four waves do nothing
// but that: a wave's loads complete in the order they were asked for, so a wave that waited for
// the rows of the next chunk would wait for every fragment of W asked for before them (with
// every wave doing both, a chunk took 1.9 us instead of 1.5).  The waves that compute read the
// rows as B operands, so lane l ends with C[m = 16 mt + l % 16][n = 4 (l / 16) + e] for the 16
// rows n of a tile of W.  The two waves of a pair add their sums through shared memory, first
// wave first: a row's bits do not depend on the other rows.
//
// Epilogues: plain store as bfloat16; with slices of K (grid height > 1), float32 matrices
// [slice, M, N] that the caller adds in order; or SwiGLU over a stacked [gate; up] weight
// (src/flint/cuda/swiglu.cu:44-49): a wave's two tiles are a gate tile and the up tile of the
// same columns, gate and up rounded to bfloat16 first, as the unfused path stores them.
#include "mfma.h"

#define MID_EPI_NONE 0
#define MID_EPI_SWIGLU 1
#define MID_EPI_GATED 2      // as SwiGLU, the gate through the activation that the arguments name (common.h)
#define MID_IS_GATED(E) ((E) == MID_EPI_SWIGLU || (E) == MID_EPI_GATED)
#define MID_CK 128          // elements of K per chunk
#define MID_STEPS 4         // steps of 32 per chunk
#define MID_STAGES 4        // chunks of W in registers
#define MID_WK 2            // waves that share a tile of W, splitting each chunk's steps
#define MID_NT 512          // threads of a block: four waves that compute, four that stage X
#define MID_RT 2            // tiles of W a wave owns

// Loads whose completion this file counts itself.  With ordinary loads the compiler makes a wave
// wait for all of its loads once a chunk (it does not count loads across the loop's branches),
// which puts a trip to memory into every chunk.  The compiler does not see these, so every wave
// issues the same number per chunk, also past the end (there from one line that all lanes share),
// and waits by count.  A register such a load fills must not be read, copied or spilled before
// the wait that covers it: the waits name those registers as operands, and no form of the kernel
// may spill (a test compiles this file and checks that; others compare every form with float64,
// and bit for bit across row counts).
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void load16_uncounted(u32x4v& dst, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(dst) : "v"(p) : "memory");
}

// The same with the non-temporal hint, for the weights, which are read once: they then do not push
// the rows of X out of the chiplet's cache (1 to 2 % of a decode step at batches of 96 and 128).
__device__ __forceinline__ void load16_uncounted_stream(u32x4v& dst, const void* p) {
  asm volatile("global_load_dwordx4 %0, %1, off nt" : "=&v"(dst) : "v"(p) : "memory");
}

template <int MT, int EPI, typename OutT>
__global__ __launch_bounds__(MID_NT, 2) void gemm_mid_kernel(const bf16_t* __restrict__ X,
                                                             const bf16_t* __restrict__ W,
                                                             OutT* __restrict__ C, int M, int N, int K,
                                                             int ldx, int w_steps, int n_out, int act,
                                                             int slab_rows, int n_tiles) {
  constexpr int ROW_B = MID_CK * 2;                  // bytes of a staged row: 16 pieces of 16 bytes, swizzled
  constexpr int BUF = 16 * MT * ROW_B;
  constexpr int PASSES = MT;                         // 256 threads carry 16 rows a pass
  constexpr int US = MID_STEPS / MID_WK;             // steps of a chunk that a wave takes
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * BUF];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave >> 1, wk = wave & 1;
  const int r = lane & 15, g = lane >> 4;
  // More than 128 rows go in two slabs of slab_rows rows, a block each.  The two blocks of a tile
  // of W are neighbours among the blocks that one chiplet gets (block b goes to chiplet b % 8),
  // so they run side by side and the second finds the tile in the chiplet's cache.
  int bx = blockIdx.x, m0 = 0;
  if (slab_rows < M) {
    const int i = bx >> 3;
    bx = (i >> 1) * 8 + (bx & 7);
    m0 = (i & 1) * slab_rows;
  }
  if (bx >= n_tiles) return;                         // (the grid is rounded up to whole rounds of the chiplets)
  const int m_total = M;
  M = (M - m0 < slab_rows) ? M - m0 : slab_rows;     // this block's rows
  const int k0 = blockIdx.y * K;                     // this block's slice of K (K elements, a multiple of 32 if sliced)
  X += k0 + (size_t)m0 * ldx;
  const int n_chunks = K / MID_CK;                   // K is a multiple of the chunk

  // first rows of W of this wave's tiles
  int tile_row[MID_RT];
  const bf16_t* wp[MID_RT];
#pragma unroll
  for (int rt = 0; rt < MID_RT; ++rt) {
    if (MID_IS_GATED(EPI))
      tile_row[rt] = rt * n_out + (bx * 2 + wn) * 16;
    else
      tile_row[rt] = ((bx * 2 + wn) * MID_RT + rt) * 16;
    int t = tile_row[rt] / 16;
    if (t > (N - 1) / 16) t = (N - 1) / 16;          // tiles past the end read the last one; not stored
    wp[rt] = W + ((size_t)t * w_steps * 64 + lane) * 8 + (size_t)(k0 / 32) * 512;
  }

  f32x4 acc[MID_RT][MT];
#pragma unroll
  for (int rt = 0; rt < MID_RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  float* ex = reinterpret_cast<float*>(lds);
  if (wave >= 4) {
    // ---- the waves that stage X: chunk c + 1 goes to its buffer while chunk c is computed on; the
    // loads are asked for two chunks before.  A row's 16 pieces are stored at piece ^ (row % 16):
    // the 16 lanes of a read, one row each, then fall into 16 different groups of banks.
    const int t2 = tid - 256, x_col = t2 & 15, x_row0 = t2 >> 4;
    static_assert(PASSES <= 8, "the waits below name eight registers");
    u32x4v xr[2][8];
    const int last = n_chunks - 1;
    auto load_x = [&](int chunk, u32x4v (&dst)[8]) {
      const int k = chunk * MID_CK + x_col * 8;
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const int row = x_row0 + p * 16;
        const bf16_t* src = (p < PASSES && row < M && chunk <= last) ? X + (size_t)row * ldx + k : X;
        load16_uncounted(dst[p], src);
      }
    };
    auto store_x = [&](int buf, u32x4v (&src)[8]) {
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        const int row = x_row0 + p * 16;
        *reinterpret_cast<u32x4v*>(lds + buf * BUF + row * ROW_B + ((x_col ^ (row & 15)) * 16)) = src[p];
      }
    };
    // all but the newest eight loads have arrived: the registers named are then valid
#define MID_WAIT_X(R)                                                                              \
  asm volatile("s_waitcnt vmcnt(8)"                                                                \
               : "+v"(R[0]), "+v"(R[1]), "+v"(R[2]), "+v"(R[3]), "+v"(R[4]), "+v"(R[5]), "+v"(R[6]), \
                 "+v"(R[7])::"memory")
    load_x(0, xr[0]);
    load_x(1, xr[1]);
    MID_WAIT_X(xr[0]);
    store_x(0, xr[0]);
    load_x(2, xr[0]);
#define MID_STAGE(C, CUR)                  \
  __syncthreads();                         \
  MID_WAIT_X(CUR);                         \
  store_x(((C) + 1) & 1, CUR);             \
  load_x((C) + 3, CUR);                    \
  if ((C) + 1 >= n_chunks) break;
    for (int c = 0;; c += 2) {
      MID_STAGE(c, xr[1])
      MID_STAGE(c + 1, xr[0])
    }
#undef MID_STAGE
#undef MID_WAIT_X
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // nothing of this wave's is in flight when it ends
    __syncthreads();
    __syncthreads();
    return;
  }

  static_assert(US == 2 && MID_RT == 2 && MID_STAGES == 4, "the waits below name four registers and count twelve loads");
  u32x4v a[MID_STAGES][US][MID_RT];
  const int last = n_chunks - 1;
  auto load_w = [&](int chunk, u32x4v (&dst)[US][MID_RT]) {
    const int s0 = chunk * MID_STEPS + wk * US;
#pragma unroll
    for (int u = 0; u < US; ++u)
#pragma unroll
      for (int rt = 0; rt < MID_RT; ++rt)
        load16_uncounted_stream(dst[u][rt], chunk <= last ? wp[rt] + (size_t)(s0 + u) * 512 : W);
  };
  auto compute = [&](int buf, u32x4v (&src)[US][MID_RT]) {
#pragma unroll
    for (int u = 0; u < US; ++u) {
      const int piece = (wk * US + u) * 4 + g;
      Frag b[MT];                                      // all of a step's reads before its matrix instructions
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        b[mt].u = *reinterpret_cast<const uint4*>(lds + buf * BUF + (mt * 16 + r) * ROW_B + ((piece ^ r) * 16));
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int rt = 0; rt < MID_RT; ++rt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, src[u][rt]), b[mt].v,
                                                                acc[rt][mt], 0, 0, 0);
    }
  };
  // all but the newest twelve loads (three chunks) have arrived
#define MID_WAIT_W(R) \
  asm volatile("s_waitcnt vmcnt(12)" : "+v"(R[0][0]), "+v"(R[0][1]), "+v"(R[1][0]), "+v"(R[1][1])::"memory")

#pragma unroll
  for (int c = 0; c < MID_STAGES - 1; ++c) load_w(c, a[c]);
  // iteration c: chunk c of X lies in buffer c % 2
#define MID_STEP(C, CUR, NXT)                 \
  __syncthreads();                            \
  load_w((C) + MID_STAGES - 1, NXT);          \
  MID_WAIT_W(CUR);                            \
  compute((C) & 1, CUR);                      \
  if ((C) + 1 >= n_chunks) break;
  for (int c = 0;; c += 4) {
    MID_STEP(c, a[0], a[3])
    MID_STEP(c + 1, a[1], a[0])
    MID_STEP(c + 2, a[2], a[1])
    MID_STEP(c + 3, a[3], a[2])
  }
#undef MID_WAIT_W
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // nothing of this wave's is in flight past here
#undef MID_STEP

  // ---- the second wave of a pair hands its sums to the first through shared memory
  __syncthreads();                                     // every wave is done with the staged rows
  if (wk == 1) {
#pragma unroll
    for (int rt = 0; rt < MID_RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        *reinterpret_cast<float4*>(ex + (((wn * MID_RT + rt) * MT + mt) * 64 + lane) * 4) =
            make_float4(acc[rt][mt][0], acc[rt][mt][1], acc[rt][mt][2], acc[rt][mt][3]);
  }
  __syncthreads();
  if (wk == 1) return;
#pragma unroll
  for (int rt = 0; rt < MID_RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const float4 v = *reinterpret_cast<const float4*>(ex + (((wn * MID_RT + rt) * MT + mt) * 64 + lane) * 4);
      acc[rt][mt] += f32x4{v.x, v.y, v.z, v.w};
    }

  if (MID_IS_GATED(EPI)) {
    const int n = tile_row[0] + 4 * g;                 // output column: the gate tile's rows
    if (n >= n_out) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      if (m >= M) continue;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float gt = bf16_to_f32(f32_to_bf16(acc[0][mt][e])), u = bf16_to_f32(f32_to_bf16(acc[1][mt][e]));
        v[e] = (EPI == MID_EPI_SWIGLU) ? u * gt / (1.0f + expf(-gt)) : llm_gated(act, gt, u);
      }
      uint2 pk;
      pk.x = pack2_bf16(v[0], v[1]);
      pk.y = pack2_bf16(v[2], v[3]);
      *reinterpret_cast<uint2*>(C + (size_t)(m0 + m) * n_out + n) = pk;       // n_out is a multiple of 16
    }
    return;
  }

#pragma unroll
  for (int rt = 0; rt < MID_RT; ++rt) {
    const int n = tile_row[rt] + 4 * g;
    if (n >= N) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      if (m >= M) continue;
      const f32x4 sum = acc[rt][mt];
      OutT* dst = C + ((size_t)blockIdx.y * m_total + m0 + m) * N + n;
      if (n + 3 < N && (N & 3) == 0) {
        if (sizeof(OutT) == 2) {
          uint2 pk;
          pk.x = pack2_bf16(sum[0], sum[1]);
          pk.y = pack2_bf16(sum[2], sum[3]);
          *reinterpret_cast<uint2*>(dst) = pk;
        } else {
          *reinterpret_cast<float4*>(dst) = make_float4(sum[0], sum[1], sum[2], sum[3]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) Conv<OutT>::store(dst + e, sum[e]);
      }
    }
  }
}

template <int EPI, typename OutT>
static int launch_mid(const bf16_t* X, const bf16_t* W, void* C, int M, int N, int K, int ldx,
                      int k_split, int act, hipStream_t stream) {
  const int n_out = (MID_IS_GATED(EPI)) ? N / 2 : N;
  const int per_block = (MID_IS_GATED(EPI)) ? 32 : 64;
  const int n_tiles = (n_out + per_block - 1) / per_block;
  // up to 128 rows: a block a tile of W; beyond: two slabs of rows, evenly, in whole tiles of 16
  const int slab_rows = (M <= 128) ? M : ((M + 31) / 32) * 16;
  const dim3 grid((M <= 128) ? n_tiles : 2 * ((n_tiles + 7) / 8) * 8, k_split);
  const int w_steps = (K + 31) / 32;
#define MID_CASE(T)                                                                                  \
  case T:                                                                                            \
    gemm_mid_kernel<T, EPI, OutT><<<grid, MID_NT, 0, stream>>>(X, W, (OutT*)C, M, N, K / k_split, ldx,  \
                                                            w_steps, n_out, act, slab_rows, n_tiles); \
    break;
  switch ((slab_rows + 15) / 16) {
    MID_CASE(3)
    MID_CASE(4)
    MID_CASE(5)
    MID_CASE(6)
    MID_CASE(7)
    MID_CASE(8)
    default: return LLM_ERR_ARG;
  }
#undef MID_CASE
  return llm_launch_status();
}

// X [M, K] bfloat16 with rows ldx apart, 33 <= M <= 256 (beyond 128 in two slabs of rows that
// share every tile of W through the chiplet's cache); W the tiled copy of a [N, K] matrix.
// epilogue 0: C [M, N] bfloat16, or with k_split > 1 float32 [k_split, M, N], the products over
// the slices of K; K is a multiple of 128 * k_split; epilogue 1 (1 | act << 4 for another activation of the gate, common.h): C [M, N/2] bfloat16, SwiGLU over
// W = [Wg; Wu], N/2 a multiple of 16.
extern "C" int llm_gemm_mid_bf16(const void* X, int ldx, const void* W_tiled, void* C, int epilogue,
                                 int out_dtype, int M, int N, int K, int k_split, hipStream_t stream) {
  const int act = epilogue >> 4;                 // the gate's activation rides above the epilogue's code
  epilogue &= 15;
  if (act < 0 || act >= LLM_ACT_COUNT || (act != 0 && epilogue != MID_EPI_SWIGLU)) return LLM_ERR_ARG;
  if (M < 33 || M > 256 || N <= 0 || K <= 0 || (K & 7) || ldx < K || (ldx & 7) || k_split < 1)
    return LLM_ERR_ARG;
  if (X == nullptr || W_tiled == nullptr || C == nullptr) return LLM_ERR_ARG;
  if ((((uintptr_t)X) | ((uintptr_t)W_tiled) | ((uintptr_t)C)) & 15) return LLM_ERR_ARG;
  if (k_split > 65535 || K % (k_split * MID_CK) != 0) return LLM_ERR_ARG;
  if (epilogue == MID_EPI_NONE) {
    if (k_split == 1 && out_dtype == LLM_DTYPE_BF16)
      return launch_mid<MID_EPI_NONE, bf16_t>((const bf16_t*)X, (const bf16_t*)W_tiled, C, M, N, K, ldx, 1, 0, stream);
    if (out_dtype == LLM_DTYPE_F32)
      return launch_mid<MID_EPI_NONE, float>((const bf16_t*)X, (const bf16_t*)W_tiled, C, M, N, K, ldx, k_split, 0, stream);
    return LLM_ERR_ARG;
  }
  if (epilogue == MID_EPI_SWIGLU) {
    if ((N & 31) || out_dtype != LLM_DTYPE_BF16 || k_split != 1) return LLM_ERR_ARG;
    if (act != LLM_ACT_SILU)      // SiLU keeps the kernel that knows nothing else
      return launch_mid<MID_EPI_GATED, bf16_t>((const bf16_t*)X, (const bf16_t*)W_tiled, C, M, N, K, ldx, 1, act, stream);
    return launch_mid<MID_EPI_SWIGLU, bf16_t>((const bf16_t*)X, (const bf16_t*)W_tiled, C, M, N, K, ldx, 1, 0, stream);
  }
  return LLM_ERR_ARG;
}
