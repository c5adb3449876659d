// C = X[M,K] * W[N,K]^T for many rows (prompt steps), where the product is bound by the matrix
// cores and by what a compute unit can pull from the caches, not by one pass over W.  bfloat16
// inputs, float32 sums (v_mfma_f32_16x16x32_bf16), bfloat16 output; plain, or SwiGLU over a stacked
// [gate; up] weight (out[m, i] = silu(gate_i) * up_i, src/flint/cuda/swiglu.cu:44-49), which saves
// the pass of a kernel of its own over gate and up (100 MB a layer at 2,048 rows of the 1B shape).
//
// A block of 8 waves owns 256 rows of X and 256 rows of W (SwiGLU: 128 gate rows and the 128 up
// rows of the same columns): at that size a unit reads 64 KiB for 64 elements of K, which the
// caches deliver in about the time the matrix cores need for them.  A wave owns 64 x 128 of the
// tile (SwiGLU: 64 x (64 gate + 64 up)): 32 sums of 16 x 16, with W as the A operand, so that a
// lane ends with four consecutive columns of one row of C.  A second form takes 128 rows of X a
// block (a wave 64 x 64): half the arithmetic for three quarters of the bytes, but twice the
// blocks, for steps whose tiles of 256 rows would leave compute units idle.
//
// Tiles of 64 elements of K go from global memory straight into LDS (global_load_lds_dwordx4, no
// registers in between), two buffers of 64 (48) KiB.  A row of a tile is 128 bytes in 8 pieces of 16;
// piece p of row r lies at p ^ (r & 7), so that the 16 rows a fragment read touches fall into
// different banks; the swizzle is applied on the global side, since a direct load fills LDS in lane
// order.  The fragments of a step of 32 are read into registers one step ahead of the matrix
// instructions that use them (two sets of 12 or 8), and the direct loads of the tile after next go out
// between matrix instructions: one barrier per tile of K.
//
// Blocks are numbered so that the blocks of a chiplet (every eighth) share operands in its cache:
// a chiplet takes every eighth tile of W rows and, at a time, a band of 8 tiles of X rows.
#include "mfma.h"

#define WD_BN 256          // rows of W a block
#define WD_BK 64           // elements of K a tile
#define WD_NT 512          // threads of a block
#define WD_EPI_NONE 0
#define WD_EPI_SWIGLU 1
#define WD_EPI_GATED 2       // as SwiGLU, the gate through the activation that the arguments name (common.h)
#define WD_IS_GATED(E) ((E) == WD_EPI_SWIGLU || (E) == WD_EPI_GATED)

template <int EPI, int BM>
__global__ __launch_bounds__(WD_NT) void gemm_wide_kernel(const bf16_t* __restrict__ X, int ldx,
                                                          const bf16_t* __restrict__ W, int ldw,
                                                          bf16_t* __restrict__ C, int M, int N, int K,
                                                          int n_out, int m_tiles, int n_tiles, int act) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  static_assert(BM == 256 || BM == 128, "rows of X a block");
  constexpr int OPER = 256 * 128;                 // bytes of W's tile; X's follows it
  constexpr int BUF = OPER + BM * 128;
  constexpr int WM = BM / 64, WNW = 8 / WM;       // waves along the rows of X and of W
  constexpr int NTW = 256 / WNW / 16;             // tiles of 16 rows of W a wave: 8 or 4
  constexpr int XP = BM / 64;                     // pieces of X a thread loads per tile of K
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int wm = wave % WM, wn = wave / WM;

  // blocks i, i + 8, ... share a chiplet: a chiplet takes every eighth tile of W rows and, at a
  // time, a band of 8 tiles of X rows; its 32 units then share 8 tiles of X and 4 of W whatever
  // the number of rows
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int n_per = (n_tiles + 7) >> 3;                      // tiles of W rows a chiplet
  const int band = j / (8 * n_per), jj = j - band * (8 * n_per);
  const int band_rows = (m_tiles - band * 8 < 8) ? m_tiles - band * 8 : 8;     // the last band may be short
  const int mt_blk = band * 8 + jj % band_rows, nt_blk = (jj / band_rows) * 8 + xcd;
  if (nt_blk >= n_tiles || jj >= band_rows * n_per) return;
  const int m0 = mt_blk * BM;

  // global -> LDS without registers in between: a wave's load instruction fills 1 KiB of LDS in
  // lane order, 8 rows of 8 pieces; lane l fills slot (l & 7) of row (l >> 3) and so fetches
  // piece (l & 7) ^ (row & 7) of that row.  A thread carries rows (tid >> 3) + 64 p of both operands.
  const int row0 = tid >> 3, piece = (tid & 7) ^ (row0 & 7);
  const bf16_t* xp[XP];
  const bf16_t* wp[4];
#pragma unroll
  for (int p = 0; p < XP; ++p) {
    int m = m0 + row0 + 64 * p;
    if (m > M - 1) m = M - 1;
    xp[p] = X + (size_t)m * ldx + piece * 8;
  }
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int row = row0 + 64 * p;
    int n;
    if (WD_IS_GATED(EPI)) {
      n = nt_blk * 128 + (row & 127);
      if (n > n_out - 1) n = n_out - 1;
      n += (row >> 7) * n_out;
    } else {
      n = nt_blk * WD_BN + row;
      if (n > N - 1) n = N - 1;
    }
    wp[p] = W + (size_t)n * ldw + piece * 8;
  }
  // The loads are written in assembly: the compiler would make every read of LDS wait for all of
  // them (it cannot tell that they fill the other buffer).  It does not count them either: the
  // kernel waits for them itself, before the barrier that hands a buffer over.
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
  // wave w fills rows 8 w .. 8 w + 7 of each group of 64 rows: 1 KiB at (64 p + 8 w) * 128
  // (the instruction takes its place in LDS from M0, which is put back afterwards: the compiler
  // need not know)
#define WD_LOAD1(GP, LA)                                                                          \
  {                                                                                               \
    uint32_t m0_was;                                                                              \
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0" \
                 : "=&s"(m0_was) : "s"(LA), "v"(GP) : "memory");                                  \
  }
#define WD_LOAD(KT, BUFI)                                                                         \
  {                                                                                               \
    const size_t ko = (size_t)(KT) * WD_BK;                                                      \
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds0 + (BUFI) * BUF + wave * 1024);      \
    _Pragma("unroll") for (int p = 0; p < 4; ++p) WD_LOAD1(wp[p] + ko, base + p * 8192)           \
    _Pragma("unroll") for (int p = 0; p < XP; ++p) WD_LOAD1(xp[p] + ko, base + OPER + p * 8192)   \
  }

  f32x4 acc[NTW][4];
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // rows of this wave's tiles within the block's operands
  int a_row[NTW], b_row[4];
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt)
    a_row[nt] = (WD_IS_GATED(EPI)) ? ((nt / (NTW / 2)) * 128 + wn * (NTW / 2) * 16 + (nt % (NTW / 2)) * 16 + r)
                                       : (wn * NTW * 16 + nt * 16 + r);
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) b_row[mt] = wm * 64 + mt * 16 + r;

  const int n_kt = K / WD_BK;
  Frag f0a[NTW], f0b[4], f1a[NTW], f1b[4];
#define WD_READ(FA, FB, BUFI, KS)                                                                 \
  {                                                                                               \
    const unsigned char* la = lds + (BUFI) * BUF;                                                 \
    const unsigned char* lb = la + OPER;                                                          \
    _Pragma("unroll") for (int mt = 0; mt < 4; ++mt)                                              \
      FB[mt].u = *reinterpret_cast<const uint4*>(lb + b_row[mt] * 128 + ((((KS) * 4 + g) ^ (r & 7)) * 16)); \
    _Pragma("unroll") for (int nt = 0; nt < NTW; ++nt)                                            \
      FA[nt].u = *reinterpret_cast<const uint4*>(la + a_row[nt] * 128 + ((((KS) * 4 + g) ^ (r & 7)) * 16)); \
  }
  WD_LOAD(0, 0)
  if (n_kt > 1) WD_LOAD(1, 1)
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");     // everything this wave asked for has arrived
  __syncthreads();
  WD_READ(f0a, f0b, 0, 0)
  // Round kt: the fragments of the tile's first step are in registers.  Those of the second step
  // are asked for while the first step's matrix instructions run, three after every eight, so that
  // the eight waves do not all come to LDS at once; behind the barrier (every wave has read all
  // of tile kt, tile kt + 1 lies in the other buffer) the second step runs, and between its matrix
  // instructions go the reads of the first fragments of tile kt + 1 and the direct loads of tile
  // kt + 2 into the buffer that tile kt leaves (a wave that issued all of them in a row would hold
  // its matrix instructions back for as long).
  // fragment q of a step's: 0..3 of X, then those of W
  constexpr int R = 4 + NTW;                      // fragments a step
  constexpr int L = 4 + XP;                       // direct loads a thread and tile: 0..3 of W, then those of X
#define WD_READ1(FA, FB, BUFI, KS, Q)                                                             \
  {                                                                                               \
    const unsigned char* la = lds + (BUFI) * BUF;                                                 \
    if ((Q) < 4)                                                                                  \
      FB[(Q)].u = *reinterpret_cast<const uint4*>(la + OPER + b_row[(Q)] * 128 + ((((KS) * 4 + g) ^ (r & 7)) * 16)); \
    else                                                                                          \
      FA[(Q) - 4].u = *reinterpret_cast<const uint4*>(la + a_row[(Q) - 4] * 128 + ((((KS) * 4 + g) ^ (r & 7)) * 16)); \
  }
  // NTW groups of four matrix instructions a step; the reads (and loads) are dealt out over them
  for (int kt = 0; kt < n_kt; ++kt) {
    const int buf = kt & 1;
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = (R * nt) / NTW; q < (R * (nt + 1)) / NTW; ++q) WD_READ1(f1a, f1b, buf, 1, q)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = mfma_bf16(f0a[nt], f0b[mt], acc[nt][mt]);
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    {
      const bool more = kt + 2 < n_kt, next = kt + 1 < n_kt;
      const size_t ko = (size_t)(more ? kt + 2 : kt) * WD_BK;
      const uint32_t base = __builtin_amdgcn_readfirstlane(lds0 + buf * BUF + wave * 1024);
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt) {
        __builtin_amdgcn_sched_barrier(0);
        if (next) {
#pragma unroll
          for (int q = (R * nt) / NTW; q < (R * (nt + 1)) / NTW; ++q) WD_READ1(f0a, f0b, buf ^ 1, 0, q)
        }
        if (more) {
#pragma unroll
          for (int j = (L * nt) / NTW; j < (L * (nt + 1)) / NTW; ++j) {
            if (j < 4) { WD_LOAD1(wp[j] + ko, base + j * 8192) }
            else { WD_LOAD1(xp[j - 4] + ko, base + OPER + (j - 4) * 8192) }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) acc[nt][mt] = mfma_bf16(f1a[nt], f1b[mt], acc[nt][mt]);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- epilogue: lane holds C[m = .. + r][n = .. + 4 g + e].  Each wave turns its tile (64 rows
  // of its outputs) round through a region of LDS of its own, rows 16
  // bytes longer than they are so that the 16 rows of a store fall into different banks, and then
  // stores whole rows, 16 bytes a lane.
  __syncthreads();                                   // every wave has read the last tile
  constexpr int OUT_T = (WD_IS_GATED(EPI)) ? NTW / 2 : NTW;   // tiles of 16 outputs of a wave
  constexpr int OUT_COLS = OUT_T * 16;
  constexpr int ROW_B = OUT_COLS * 2 + 16;
  unsigned char* mine = lds + wave * (64 * ROW_B);
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int nt = 0; nt < OUT_COLS / 16; ++nt) {
      uint2 pk;
      if (WD_IS_GATED(EPI)) {
        // gate and up rounded to bfloat16 first, as the unfused path stores them; the exponential
        // and the reciprocal by the hardware's instructions (their error is far below the rounding
        // of the result)
        const uint32_t g01 = pack2_bf16(acc[nt][mt][0], acc[nt][mt][1]), g23 = pack2_bf16(acc[nt][mt][2], acc[nt][mt][3]);
        const uint32_t u01 = pack2_bf16(acc[nt + NTW / 2][mt][0], acc[nt + NTW / 2][mt][1]), u23 = pack2_bf16(acc[nt + NTW / 2][mt][2], acc[nt + NTW / 2][mt][3]);
        const float gt[4] = {__uint_as_float(g01 << 16), __uint_as_float(g01 & 0xffff0000u), __uint_as_float(g23 << 16), __uint_as_float(g23 & 0xffff0000u)};
        const float up[4] = {__uint_as_float(u01 << 16), __uint_as_float(u01 & 0xffff0000u), __uint_as_float(u23 << 16), __uint_as_float(u23 & 0xffff0000u)};
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
          v[e] = (EPI == WD_EPI_SWIGLU) ? up[e] * gt[e] * __builtin_amdgcn_rcpf(1.0f + fast_exp2(-1.4426950408889634f * gt[e]))
                                        : llm_gated(act, gt[e], up[e]);
        pk.x = pack2_bf16(v[0], v[1]);
        pk.y = pack2_bf16(v[2], v[3]);
      } else {
        pk.x = pack2_bf16(acc[nt][mt][0], acc[nt][mt][1]);
        pk.y = pack2_bf16(acc[nt][mt][2], acc[nt][mt][3]);
      }
      *reinterpret_cast<uint2*>(mine + (mt * 16 + r) * ROW_B + (nt * 16 + 4 * g) * 2) = pk;
    }
  // (a wave reads only what it wrote itself: the compiler's wait for its stores is enough)
  constexpr int LPR = OUT_COLS / 8;                  // lanes a row
  constexpr int RPP = 64 / LPR;                      // rows a pass
  const int ldc = (WD_IS_GATED(EPI)) ? n_out : N;
  const int n_wave = (WD_IS_GATED(EPI)) ? nt_blk * 128 + wn * OUT_COLS : nt_blk * WD_BN + wn * OUT_COLS;
  const int col = (lane % LPR) * 8;
#pragma unroll
  for (int pass = 0; pass < 64 / RPP; ++pass) {
    const int row = pass * RPP + lane / LPR;
    const int m = m0 + wm * 64 + row, n = n_wave + col;
    const uint4 v = *reinterpret_cast<const uint4*>(mine + row * ROW_B + col * 2);
    if (m < M && n < ldc) {
      bf16_t* dst = C + (size_t)m * ldc + n;
      if (n + 7 < ldc && (ldc & 7) == 0) {
        *reinterpret_cast<uint4*>(dst) = v;
      } else {
        const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (n + e < ldc) dst[e] = (bf16_t)(w4[e >> 1] >> (16 * (e & 1)));
      }
    }
  }
}

template <int EPI, int BM>
static int launch_wide(const void* X, int ldx, const void* W, int ldw, void* C, int M, int N, int K,
                       int n_out, int act, hipStream_t stream) {
  const int m_tiles = (M + BM - 1) / BM;
  const int per = (WD_IS_GATED(EPI)) ? 128 : WD_BN;
  const int n_tiles = (n_out + per - 1) / per;
  const long long blocks = 8LL * ((m_tiles + 7) / 8) * 8 * ((n_tiles + 7) / 8);   // bands of 8 tiles of X rows; surplus blocks leave at once
  if (blocks > 0x7fffffffLL) return LLM_ERR_ARG;
  // the two buffers of the loop, or the epilogue's regions (8 waves x 64 rows of up to 272 bytes)
  const int lds_bytes = (2 * (256 + BM) * 128 > 8 * 64 * 272) ? 2 * (256 + BM) * 128 : 8 * 64 * 272;
  // more than 64 KiB of LDS has to be asked for, once per device and kernel
  static bool asked[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return LLM_ERR_LAUNCH;
  if (!asked[dev]) {
    if (hipFuncSetAttribute((const void*)gemm_wide_kernel<EPI, BM>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            lds_bytes) != hipSuccess)
      return LLM_ERR_LAUNCH;
    asked[dev] = true;
  }
  gemm_wide_kernel<EPI, BM><<<(unsigned)blocks, WD_NT, lds_bytes, stream>>>(
      (const bf16_t*)X, ldx, (const bf16_t*)W, ldw, (bf16_t*)C, M, N, K, n_out, m_tiles, n_tiles, act);
  return llm_launch_status();
}

// X [M, K] rows ldx apart, W [N, K] rows ldw apart (both bfloat16, K a multiple of 64, 16-byte aligned rows);
// epilogue 0: C [M, N]; 1: C [M, N/2], SwiGLU over W = [Wg; Wu], N/2 a multiple of 16 (1 | act << 4:
// the gate through another activation of common.h).
// block_rows: rows of X a block takes, 256 or 128 (half the arithmetic per byte a unit reads, twice
// the blocks: for steps whose tiles of 256 rows would leave units idle).
extern "C" int llm_gemm_wide_bf16(const void* X, int ldx, const void* W, int ldw, void* C, int epilogue,
                                  int block_rows, int M, int N, int K, hipStream_t stream) {
  const int act = epilogue >> 4;                 // the gate's activation rides above the epilogue's code
  epilogue &= 15;
  if (act < 0 || act >= LLM_ACT_COUNT || (act != 0 && epilogue != WD_EPI_SWIGLU)) return LLM_ERR_ARG;
  if (M <= 0 || N <= 0 || K < WD_BK || (K % WD_BK) || ldx < K || ldw < K || (ldx & 7) || (ldw & 7)) return LLM_ERR_ARG;
  if ((((uintptr_t)X) | ((uintptr_t)W) | ((uintptr_t)C)) & 15) return LLM_ERR_ARG;
  if (epilogue != WD_EPI_NONE && epilogue != WD_EPI_SWIGLU) return LLM_ERR_ARG;
  if (block_rows != 256 && block_rows != 128) return LLM_ERR_ARG;
  if (X == nullptr || W == nullptr || C == nullptr) return LLM_ERR_ARG;
  const int n_out = (epilogue == WD_EPI_SWIGLU) ? N / 2 : N;
  if (epilogue == WD_EPI_SWIGLU && (N & 31)) return LLM_ERR_ARG;
  if (n_out & 3) return LLM_ERR_ARG;
  if (epilogue == WD_EPI_SWIGLU && act != LLM_ACT_SILU)       // SiLU keeps the kernel that knows nothing else
    return block_rows == 256 ? launch_wide<WD_EPI_GATED, 256>(X, ldx, W, ldw, C, M, N, K, n_out, act, stream)
                             : launch_wide<WD_EPI_GATED, 128>(X, ldx, W, ldw, C, M, N, K, n_out, act, stream);
  if (epilogue == WD_EPI_SWIGLU)
    return block_rows == 256 ? launch_wide<WD_EPI_SWIGLU, 256>(X, ldx, W, ldw, C, M, N, K, n_out, 0, stream)
                             : launch_wide<WD_EPI_SWIGLU, 128>(X, ldx, W, ldw, C, M, N, K, n_out, 0, stream);
  return block_rows == 256 ? launch_wide<WD_EPI_NONE, 256>(X, ldx, W, ldw, C, M, N, K, n_out, 0, stream)
                           : launch_wide<WD_EPI_NONE, 128>(X, ldx, W, ldw, C, M, N, K, n_out, 0, stream);
}
