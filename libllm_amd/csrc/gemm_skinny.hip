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
// Epilogues: plain store; SwiGLU over a stacked [gate; up] weight (out[m, i] =
// silu(gate_i) * up_i, src/flint/cuda/swiglu.cu:44-49), where a wave owns a gate tile and the up
// tile of the same columns, gate and up rounded to the activation dtype first, as the unfused path
// stores them; or accumulation into a float32 matrix (the residual stream).
//
// Rotary epilogue for a stacked q|k|v projection whose q and k rows were reordered so that the two
// dims of a rotating pair are neighbours (pair j of a head at 2j, 2j+1): bias, rotation at the
// token's position (src/libllm/llama.cc:151-176 pairs j with j + rot_dim/2; the reordering only
// moves them side by side), rotated q to the output, rotated k and v to the token's place in the
// paged cache (laid out as common.h says).
//
// An RMS norm between two such products needs no kernel of its own (up to 16 rows): y = x w s with
// s = rsqrt(mean(x^2) + eps) a factor of the whole row, so (x w s) W^T = s ((x w) W^T).  The
// product that adds into the stream also stores the new stream times the next norm's weight,
// rounded to bfloat16, and the sums of squares of the new stream over its tiles of 16 columns; the
// product that follows takes those rows as its X, adds the sums of squares of a row in a fixed
// order, and multiplies its sums by s before its own epilogue.  The statistics are those of the
// 32-bit stream, as in the norm kernel (src/flint/cuda/rms_norm.cu:45-76); a row is rounded once,
// before instead of after its scale.
#include "mfma.h"

#define SK_WK 8            // waves that split K
#define SK_EPI_NONE 0
#define SK_EPI_SWIGLU 1
#define SK_EPI_ACCUM 2
#define SK_EPI_ROPE 3
#define SK_EPI_GATED 4       // as SwiGLU, the gate through the activation that the arguments name (common.h)
#define SK_IS_GATED(E) ((E) == SK_EPI_SWIGLU || (E) == SK_EPI_GATED)

// MT: 16-row tiles of X; RT: 16-row tiles of W per wave; WN: row groups per block; G: granules of
// 2 steps that a wave takes per chunk (a chunk is 512*G elements of K).
struct SkinnyRope {
  const float* bias;       // [N] or null
  const float* cos_t;      // [positions, rot_dim / 2]
  const float* sin_t;
  const int* tok_pos;      // [M] position of each row's token
  const int* tok_seq;      // [M] its sequence in the step
  const int* seq_slot;     // [sequences] slot of each sequence
  const int* table;        // [slots, table_stride] page of (slot, position / 64)
  bf16_t* k_pages;
  bf16_t* v_pages;
  int table_stride, n_heads, n_kv, hd, rot_dim, write_kv;
};

struct SkinnyNorm {
  const float* next_w;     // accumulating epilogue: weight [N] of the norm that reads the stream next, or null
  bf16_t* raw;             //   out [M, N]: the new stream times next_w
  float* ssq_out;          //   out [M, N / 16]: sums of squares of the new stream over tiles of 16 columns
  const float* ssq_in;     // [M, parts_in]: such sums for the rows of X, which still lack their scale; or null
  int parts_in;
  float eps;
  int act;                 // gated epilogue: the gate's activation (common.h); 0 is SiLU
};

template <int MT, int RT, int WN, int G, int EPI, typename OutT>
__global__ __launch_bounds__(WN* SK_WK * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                      const bf16_t* __restrict__ W,
                                                                      OutT* __restrict__ C, int M,
                                                                      int N, int K, int ldw,
                                                                      int n_out, int ldx, int w_steps,
                                                                      SkinnyRope rope, SkinnyNorm norm) {
  constexpr int NT = WN * SK_WK * 64;
  constexpr int CK = 512 * G;                    // elements of K per chunk
  constexpr int ROW_B = CK * 2;                  // bytes of a staged row; 16-byte pieces are swizzled
  constexpr int X_BYTES = 16 * MT * ROW_B;
  constexpr int RED_BYTES = SK_WK * WN * ((SK_IS_GATED(EPI)) ? 2 : 1) * MT * 1024;
  constexpr int LDS_BYTES = X_BYTES > RED_BYTES ? X_BYTES : RED_BYTES;
  constexpr int XV = CK / 8;                     // 16-byte pieces of a staged row
  constexpr int ROWS_PASS = NT / XV;             // rows staged per pass of the block
  constexpr int PASSES = (16 * MT + ROWS_PASS - 1) / ROWS_PASS;
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];
  __shared__ float s_scale[16 * MT];             // a row's rsqrt(mean(x^2) + eps) where X lacks it

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wn = wave / SK_WK, wk = wave % SK_WK;
  const int r = lane & 15, g = lane >> 4;
  const int group = blockIdx.x * WN + wn;                       // row group of this wave
  // K may be a slice of the rows of X and W: blockIdx.y counts the slices (K elements each, a
  // multiple of 32 then), rows of X lie ldx apart, a full row of W has w_steps steps of 32, and
  // each slice stores its sums to a matrix of its own (plain epilogue only).  Whoever adds the
  // matrices does it in a fixed order; one launch with a grid of height 1 is the whole product.
  const int k0 = blockIdx.y * K;
  X += k0;
  const int n_steps = (K + 31) / 32;
  const int n_chunks = (K + CK - 1) / CK;

  // first row of each of this wave's tiles
  int tile_row[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (SK_IS_GATED(EPI))
      tile_row[rt] = (rt & 1) * n_out + (group * (RT / 2) + (rt >> 1)) * 16;
    else
      tile_row[rt] = (group * RT + rt) * 16;
  }
  const bf16_t* wp[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (ldw == 0) {                             // tiled for the matrix cores: see llm_pack_weight
      int t = tile_row[rt] / 16;
      if (t > (N - 1) / 16) t = (N - 1) / 16;
      wp[rt] = W + ((size_t)t * w_steps * 64 + lane) * 8 + (size_t)(k0 / 32) * 512;
    } else {
      int n = tile_row[rt] + r;
      if (n > N - 1) n = N - 1;                 // rows past the end read the last row; not stored
      wp[rt] = W + (size_t)n * ldw + g * 8 + k0;
    }
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
    const int k = chunk * CK + x_col * 8;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int row = x_row0 + p * ROWS_PASS;
      xr[p] = (row < M && k < K) ? *reinterpret_cast<const uint4*>(X + (size_t)row * ldx + k)
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
  const int wstep = (ldw == 0) ? 512 : 32;       // elements between a lane's fragments of consecutive steps
  // Stages of W in registers: fragments are asked for ST - 1 chunks ahead.  Up to 48 rows of X one
  // chunk ahead is up to 3 % of a decode step faster than two (fewer registers, and the compiler
  // makes a wave wait for all its loads at every chunk anyway); from 49 rows on it is a third slower.
  constexpr int ST = (MT <= 3) ? 2 : 3;
  Frag a[ST][G][2][RT];
  auto load_w = [&](int chunk, Frag (&dst)[G][2][RT]) {
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int s = chunk * (CK / 32) + gi * 16 + wk * 2 + u;
        const bool in = s < n_steps && (s * 32 + g * 8) < K;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) dst[gi][u][rt] = in ? frag_load_stream(wp[rt] + (size_t)s * wstep) : frag_zero();
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

  // W fragments are fetched ST - 1 chunks ahead (the register stages in rotation), X one chunk
  load_x(0);
  load_w(0, a[0]);
  if (ST == 3 && 1 < n_chunks) load_w(1, a[1]);

  // What the epilogue needs from memory beside the sums is asked for now, behind the first loads:
  // a thread finishes at most one group of four outputs per round (ITEMS <= NT), and which one is
  // known from the start, so its position, cache page and rotation, or the values it adds to,
  // are in registers by the time the sums are (1 % of a decode step at up to 16 rows).
  constexpr int RPR = (SK_IS_GATED(EPI)) ? 2 : 1;    // W tiles of a row group per round
  constexpr int OUT_RT = RT / RPR;
  constexpr int ITEMS = WN * MT * 64;
  static_assert(ITEMS <= NT, "one item a thread");
  const int ldc = (SK_IS_GATED(EPI)) ? n_out : N;
  const int e_ln = tid & 63, e_mt = (tid >> 6) % MT, e_wn = tid / (64 * MT);
  const int e_m = e_mt * 16 + (e_ln & 15);
  const int e_n0 = (blockIdx.x * WN + e_wn) * OUT_RT * 16 + 4 * (e_ln >> 4);   // round ort adds 16 * ort
  const bool e_on = tid < ITEMS && e_m < M;
  int e_pos = 0, e_page = 0;
  float2 e_cos[EPI == SK_EPI_ROPE ? OUT_RT : 1], e_sin[EPI == SK_EPI_ROPE ? OUT_RT : 1];
  float e_prev[EPI == SK_EPI_ACCUM ? OUT_RT : 1][4], e_nw[EPI == SK_EPI_ACCUM ? OUT_RT : 1][4];
  if (EPI == SK_EPI_ROPE && e_on) {
    e_pos = rope.tok_pos[e_m];
    const int q_dim = rope.n_heads * rope.hd, kv_dim = rope.n_kv * rope.hd;
#pragma unroll
    for (int ort = 0; ort < OUT_RT; ++ort) {
      const int n = e_n0 + ort * 16, d = n % rope.hd;
      e_cos[ort] = make_float2(1.f, 1.f);
      e_sin[ort] = make_float2(0.f, 0.f);
      if (n < q_dim + kv_dim && d < rope.rot_dim) {       // rot_dim is even; d is a multiple of 4
        const float* cr = rope.cos_t + (size_t)e_pos * (rope.rot_dim / 2) + (d >> 1);
        const float* sr = rope.sin_t + (size_t)e_pos * (rope.rot_dim / 2) + (d >> 1);
        e_cos[ort].x = cr[0];
        e_sin[ort].x = sr[0];
        if (d + 2 < rope.rot_dim) {
          e_cos[ort].y = cr[1];
          e_sin[ort].y = sr[1];
        }
      }
    }
    if (rope.write_kv && e_n0 + (OUT_RT - 1) * 16 >= q_dim) {
      const int slot = rope.seq_slot[rope.tok_seq[e_m]];
      e_page = rope.table[(size_t)slot * rope.table_stride + e_pos / 64];
    }
  }
  if (EPI == SK_EPI_ACCUM && e_on) {
#pragma unroll
    for (int ort = 0; ort < OUT_RT; ++ort) {
      const int n = e_n0 + ort * 16;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        e_prev[ort][e] = (n + e < ldc) ? Conv<OutT>::load(C + (size_t)e_m * ldc + n + e) : 0.f;
        e_nw[ort][e] = (norm.next_w != nullptr && n + e < ldc) ? norm.next_w[n + e] : 0.f;
      }
    }
  }
  // The sums of squares of a row of X that still lacks its scale: TPR threads a row, each asks
  // for every TPR-th one now and adds them after the loop, when they have long arrived.
  constexpr int TPR = NT / 16, SS_AHEAD = 8;
  float e_ss[SS_AHEAD];
  const int ss_row = tid / TPR, ss_part = tid % TPR;
  if constexpr (MT == 1) {                       // (the host asks for it with up to 16 rows only)
    static_assert(TPR <= 64 && (TPR & (TPR - 1)) == 0, "the threads of a row lie in one wave");
    if (norm.ssq_in != nullptr) {
#pragma unroll
      for (int i = 0; i < SS_AHEAD; ++i) {
        const int p = ss_part + i * TPR;
        e_ss[i] = (ss_row < M && p < norm.parts_in) ? norm.ssq_in[(size_t)ss_row * norm.parts_in + p] : 0.f;
      }
    }
  }
#define SK_STEP(C, CUR, NXT)                    \
  store_x();                                    \
  __syncthreads();                              \
  if ((C) + 1 < n_chunks) load_x((C) + 1);      \
  if ((C) + ST - 1 < n_chunks) load_w((C) + ST - 1, NXT); \
  compute(CUR);                                 \
  __syncthreads();                              \
  if ((C) + 1 >= n_chunks) break;
  if constexpr (ST == 3) {
    for (int c = 0;; c += 3) {
      SK_STEP(c, a[0], a[2])
      SK_STEP(c + 1, a[1], a[0])
      SK_STEP(c + 2, a[ST - 1], a[1])
    }
  } else {
    for (int c = 0;; c += 2) {
      SK_STEP(c, a[0], a[1])
      SK_STEP(c + 1, a[1], a[0])
    }
  }
#undef SK_STEP

  if constexpr (MT == 1) {
    if (norm.ssq_in != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < SS_AHEAD; ++i) ss += e_ss[i];
      if (ss_row < M)                            // rows wider than 16 * SS_AHEAD * TPR columns
        for (int p = ss_part + SS_AHEAD * TPR; p < norm.parts_in; p += TPR)
          ss += norm.ssq_in[(size_t)ss_row * norm.parts_in + p];
#pragma unroll
      for (int off = TPR / 2; off >= 1; off >>= 1) ss += __shfl_xor(ss, off, 64);
      if (ss_part == 0) s_scale[ss_row] = rsqrtf(ss / (float)K + norm.eps);   // read behind the next barrier
    }
  }

  // ---- add the partial sums of the 8 waves in order, apply the epilogue, store: one output tile
  // of every row group a round (a gate and its up tile together), so that the buffer stays small
  float* red = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int ort = 0; ort < OUT_RT; ++ort) {
  if (ort > 0) __syncthreads();                          // the round before has been read
#pragma unroll
  for (int j = 0; j < RPR; ++j)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      *reinterpret_cast<float4*>(red + ((((wk * WN + wn) * RPR + j) * MT + mt) * 64 + lane) * 4) =
          make_float4(acc[ort * RPR + j][mt][0], acc[ort * RPR + j][mt][1], acc[ort * RPR + j][mt][2],
                      acc[ort * RPR + j][mt][3]);
  __syncthreads();
  if (tid < ITEMS) {
    const int ln = e_ln, mt = e_mt, w_n = e_wn;
    float v[4];
    const int n = e_n0 + ort * 16;
    if (SK_IS_GATED(EPI)) {
      float gsum[4] = {0.f, 0.f, 0.f, 0.f}, usum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < SK_WK; ++w) {
        const float4 pg = *reinterpret_cast<const float4*>(
            red + ((((w * WN + w_n) * RPR + 0) * MT + mt) * 64 + ln) * 4);
        const float4 pu = *reinterpret_cast<const float4*>(
            red + ((((w * WN + w_n) * RPR + 1) * MT + mt) * 64 + ln) * 4);
        gsum[0] += pg.x; gsum[1] += pg.y; gsum[2] += pg.z; gsum[3] += pg.w;
        usum[0] += pu.x; usum[1] += pu.y; usum[2] += pu.z; usum[3] += pu.w;
      }
      if (norm.ssq_in != nullptr) {
        const float sc = s_scale[e_m];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          gsum[e] *= sc;
          usum[e] *= sc;
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float gt = bf16_to_f32(f32_to_bf16(gsum[e])), up = bf16_to_f32(f32_to_bf16(usum[e]));
        v[e] = (EPI == SK_EPI_SWIGLU) ? up * gt / (1.0f + expf(-gt)) : llm_gated(norm.act, gt, up);
      }
    } else {
      float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < SK_WK; ++w) {
        const float4 p = *reinterpret_cast<const float4*>(
            red + (((w * WN + w_n) * MT + mt) * 64 + ln) * 4);
        sum[0] += p.x; sum[1] += p.y; sum[2] += p.z; sum[3] += p.w;
      }
      const float sc = (norm.ssq_in != nullptr) ? s_scale[e_m] : 1.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (norm.ssq_in != nullptr) ? sum[e] * sc : sum[e];
    }
    const int m = e_m;
    if (EPI == SK_EPI_ROPE) {
      if (m >= M || n >= N) continue;                 // N, hd are multiples of 16: four outputs, one head
      if (rope.bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += rope.bias[n + e];
      }
      const int q_dim = rope.n_heads * rope.hd, kv_dim = rope.n_kv * rope.hd;
      const int pos = e_pos;
      const int d = n % rope.hd;
      {                                               // q and k rotate; elsewhere the angle is zero
        const float c0 = e_cos[ort].x, s0 = e_sin[ort].x, c1 = e_cos[ort].y, s1 = e_sin[ort].y;
        const float a0 = v[0], a1 = v[1], a2 = v[2], a3 = v[3];
        v[0] = a0 * c0 - a1 * s0;
        v[1] = a1 * c0 + a0 * s0;
        v[2] = a2 * c1 - a3 * s1;
        v[3] = a3 * c1 + a2 * s1;
      }
      uint2 pk;
      pk.x = pack2_bf16(v[0], v[1]);
      pk.y = pack2_bf16(v[2], v[3]);
      if (n < q_dim) {
        *reinterpret_cast<uint2*>(C + (size_t)m * q_dim + n) = pk;
      } else if (rope.write_kv) {
        const int page = e_page;
        const int kn = n - q_dim;
        if (kn < kv_dim) {
          const int kvh = kn / rope.hd;
          *reinterpret_cast<uint2*>(rope.k_pages + ((size_t)page * rope.n_kv + kvh) * llm_key_block(rope.hd) +
                                    llm_key_offset(pos % 64, d)) = pk;
        } else {
          const int kvh = (kn - kv_dim) / rope.hd;
          bf16_t* vp = rope.v_pages + ((size_t)page * rope.n_kv + kvh) * llm_value_block(rope.hd) +
                       llm_value_offset(rope.hd, d, pos % 64);         // dims d .. d + 3 lie 32 apart
          vp[0] = (bf16_t)(pk.x & 0xffffu);
          vp[32] = (bf16_t)(pk.x >> 16);
          vp[64] = (bf16_t)(pk.y & 0xffffu);
          vp[96] = (bf16_t)(pk.y >> 16);
        }
      }
      continue;
    }
    if (EPI == SK_EPI_ACCUM && norm.next_w != nullptr) {
      // (N is a multiple of 16 here: a tile is whole or absent; every lane of the wave comes along)
      const bool on = m < M && n < ldc;
      float ss = 0.f;
      if (on) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] += e_prev[ort][e];
          ss += v[e] * v[e];
        }
        *reinterpret_cast<float4*>(C + (size_t)m * ldc + n) = make_float4(v[0], v[1], v[2], v[3]);
        uint2 pk;
        pk.x = pack2_bf16(v[0] * e_nw[ort][0], v[1] * e_nw[ort][1]);
        pk.y = pack2_bf16(v[2] * e_nw[ort][2], v[3] * e_nw[ort][3]);
        *reinterpret_cast<uint2*>(norm.raw + (size_t)m * ldc + n) = pk;
      }
      ss += __shfl_xor(ss, 16, 64);                  // the four lanes that hold a row's 16 columns
      ss += __shfl_xor(ss, 32, 64);
      if (on && (ln >> 4) == 0) norm.ssq_out[(size_t)m * (ldc / 16) + n / 16] = ss;
      continue;
    }
    if (m >= M || n >= ldc) continue;
    OutT* dst = C + ((size_t)blockIdx.y * M + m) * ldc + n;
    if (EPI == SK_EPI_ACCUM) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += e_prev[ort][e];
    }
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
}

struct SkinnyArgs {
  const bf16_t* X;
  const bf16_t* W;
  void* C;
  int M, N, K, ldw, n_out;     // ldw: elements between rows of W (a multiple of 8, at least K)
  int k_split;                 // slices of K, each to a result matrix of its own (1: the whole product)
  hipStream_t stream;
  SkinnyRope rope;
  SkinnyNorm norm;
};

template <int MT, int RT, int WN, int G, int EPI, typename OutT>
static int launch_skinny(const SkinnyArgs& a) {
  const int rows = (SK_IS_GATED(EPI)) ? a.n_out : a.N;
  const int tiles = (rows + 15) / 16;
  constexpr int OUT_RT = (SK_IS_GATED(EPI)) ? RT / 2 : RT;
  const int blocks = (tiles + OUT_RT * WN - 1) / (OUT_RT * WN);
  const dim3 grid(blocks, a.k_split);
  gemm_skinny_kernel<MT, RT, WN, G, EPI, OutT><<<grid, WN * SK_WK * 64, 0, a.stream>>>(
      a.X, a.W, (OutT*)a.C, a.M, a.N, a.K / a.k_split, a.ldw, a.n_out, a.K, (a.K + 31) / 32, a.rope,
      a.norm);
  return llm_launch_status();
}

template <int MT, int EPI, typename OutT>
static int pick_rows(const SkinnyArgs& a) {
  const int units = llm_compute_units();
  if constexpr (SK_IS_GATED(EPI)) {
    // four tiles a block (32 output columns) where that still leaves a block for every compute
    // unit; they pay from 33 rows of X on; at 17 to 32 rows two are 2 % of a decode step faster
    // (whole engines compared in one process; feed-forwards of 8,192 and 14,336 on 256 units)
    if (a.n_out >= 32 * units && MT >= 3) return launch_skinny<MT, 4, 1, 1, EPI, OutT>(a);
    return launch_skinny<MT, 2, 1, 1, EPI, OutT>(a);
  } else {
    // slices of K: 64 rows of W a block, so that a slice of X is staged for as many as possible
    if (a.k_split > 1) return launch_skinny<MT, 2, 2, 1, EPI, OutT>(a);
    // else as many rows of W a block (64, 32, 16) as leave blocks for half of the compute units,
    // for three quarters, or whatever there is (measured at 8,192, 6,144 and fewer rows on 256 units)
    if (a.N >= 32 * units) return launch_skinny<MT, 2, 2, 1, EPI, OutT>(a);
    if (a.N >= 24 * units) return launch_skinny<MT, 2, 1, 1, EPI, OutT>(a);
    return launch_skinny<MT, 1, 1, 1, EPI, OutT>(a);
  }
}

template <int EPI, typename OutT>
static int pick_shape(const SkinnyArgs& a) {
  constexpr int RT = (SK_IS_GATED(EPI)) ? 2 : 1;
  const int mt = (a.M + 15) / 16;
  switch (mt) {
    case 1:
      // no more tiles of W than compute units (so a block a unit at most): more of each row in
      // flight per wave.  Whole engines compared in one process on 256 units: 1 to 1.5 % of a decode
      // step with weights of 2,048 and 3,072 rows, nothing lost at 4,096; at 6,144 rows it costs 2.5 %.
      if constexpr (RT == 1) {
        if (a.N <= 16 * llm_compute_units()) return launch_skinny<1, RT, 1, 4, EPI, OutT>(a);
      }
      // gate/up has more blocks than the chip has compute units: with the narrow chunk a block
      // needs few enough registers for two of them to share a unit, and the tail of one overlaps
      // the head of the next (3 % of a decode step at the 1B and 8B shapes, whole engines compared)
      if constexpr (SK_IS_GATED(EPI)) return launch_skinny<1, RT, 1, 1, EPI, OutT>(a);
      // likewise any weight with more tiles than units whose K gives fewer than three chunks of
      // 1,024: with the narrow chunk a block still has loads ahead of its arithmetic (the head of
      // the 1B shape, K = 2,048: 0.829 against 0.838 ms a decode step at batch 1, 0.977 against
      // 0.985 at batch 8; with K = 3,072 and 4,096 the two are the same)
      if ((a.K + 1023) / 1024 < 3) return launch_skinny<1, RT, 1, 1, EPI, OutT>(a);
      return launch_skinny<1, RT, 1, 2, EPI, OutT>(a);
    // More rows of W per block where W has rows enough to fill the GPU with such blocks: the rows
    // of X are then staged once for 64 rows of W instead of 16.
    case 2: return pick_rows<2, EPI, OutT>(a);
    case 3: return pick_rows<3, EPI, OutT>(a);
    case 4: return pick_rows<4, EPI, OutT>(a);
  }
  return LLM_ERR_ARG;
}

// Rows of W lie ldw elements apart (ldw >= K, a multiple of 8); ldw == 0 says that W is the
// tiled copy that llm_pack_weight makes.
// With k_split > 1 (more than 16 rows, epilogue 0, float32) C is [k_split, M, N]: the products over
// the k_split slices of K, for the caller to add in order.
// C[M, N] (epilogue 0: stored as out_dtype; 2: added into the float32 C) or C[M, N/2] (epilogue 1, or 1 | act << 4 for another activation of the gate, common.h:
// SwiGLU over W = [Wg; Wu], N/2 a multiple of 16) from X[M, K] and W[N, K].  X is bfloat16.
static int skinny_product(const void* X, const void* W, void* C, int epilogue, int out_dtype, int M,
                          int N, int K, int ldw, int k_split, SkinnyNorm norm,
                          hipStream_t stream) {
  if (M <= 0 || N <= 0) return LLM_OK;
  norm.act = epilogue >> 4;                    // the gate's activation rides above the epilogue's code
  epilogue &= 15;
  if (norm.act < 0 || norm.act >= LLM_ACT_COUNT || (norm.act != 0 && epilogue != SK_EPI_SWIGLU)) return LLM_ERR_ARG;
  if (norm.act != LLM_ACT_SILU) epilogue = SK_EPI_GATED;       // SiLU keeps the kernel that knows nothing else
  // slices of K: more than 16 rows, plain epilogue, float32 results [k_split, M, N]
  if (k_split < 1 || (k_split > 1 && (M <= 16 || epilogue != SK_EPI_NONE || out_dtype != LLM_DTYPE_F32 ||
                                      K % (k_split * 32) != 0)))
    return LLM_ERR_ARG;
  if (M > 64 || K <= 0 || (K & 7) || (ldw != 0 && (ldw < K || (ldw & 7)))) return LLM_ERR_ARG;
  if (X == nullptr || W == nullptr || C == nullptr) return LLM_ERR_ARG;
  if ((((uintptr_t)X) | ((uintptr_t)W) | ((uintptr_t)C)) & 15) return LLM_ERR_ARG;
  SkinnyArgs a;
  a.X = (const bf16_t*)X;
  a.W = (const bf16_t*)W;
  a.C = C;
  a.M = M;
  a.N = N;
  a.K = K;
  a.ldw = ldw;
  a.n_out = N;
  a.k_split = k_split;
  a.stream = stream;
  a.rope = SkinnyRope{};
  a.norm = norm;
  if (epilogue == SK_EPI_NONE) {
    if (out_dtype == LLM_DTYPE_BF16) return pick_shape<SK_EPI_NONE, bf16_t>(a);
    if (out_dtype == LLM_DTYPE_F32) return pick_shape<SK_EPI_NONE, float>(a);
  } else if (SK_IS_GATED(epilogue)) {
    if ((N & 31) || out_dtype != LLM_DTYPE_BF16) return LLM_ERR_ARG;
    a.n_out = N / 2;
    return epilogue == SK_EPI_SWIGLU ? pick_shape<SK_EPI_SWIGLU, bf16_t>(a) : pick_shape<SK_EPI_GATED, bf16_t>(a);
  } else if (epilogue == SK_EPI_ACCUM) {
    if (out_dtype != LLM_DTYPE_F32) return LLM_ERR_ARG;
    return pick_shape<SK_EPI_ACCUM, float>(a);
  }
  return LLM_ERR_ARG;
}

extern "C" int llm_gemm_skinny_bf16(const void* X, const void* W, void* C,
                                    int epilogue, int out_dtype, int M, int N, int K, int ldw,
                                    int k_split, hipStream_t stream) {
  return skinny_product(X, W, C, epilogue, out_dtype, M, N, K, ldw, k_split, SkinnyNorm{}, stream);
}

// The same around an RMS norm that gets no kernel of its own (see the head of this file), for up
// to 16 rows.  Epilogue 2 with next_w: beside adding into the float32 stream C[M, N] (N a multiple
// of 16), raw[M, N] = bfloat16(C * next_w) and ssq_out[M, N / 16], the sums of squares of C over
// tiles of 16 columns, are written for the product after the norm whose weight next_w is.
// With ssq_in[M, parts_in]: X holds such rows, and the sums are multiplied by
// rsqrt(sum(ssq_in[m]) / K + eps) before the epilogue (0 or 1).
extern "C" int llm_gemm_skinny_norm_bf16(const void* X, const void* W, void* C, int epilogue,
                                         int out_dtype, int M, int N, int K, int ldw,
                                         const float* next_w, void* raw, float* ssq_out,
                                         const float* ssq_in, int parts_in, float eps,
                                         hipStream_t stream) {
  if (M > 16) return LLM_ERR_ARG;
  SkinnyNorm norm{};
  if (next_w != nullptr) {
    if (epilogue != SK_EPI_ACCUM || (N & 15) || raw == nullptr || ssq_out == nullptr || (((uintptr_t)raw) & 15))
      return LLM_ERR_ARG;
    norm.next_w = next_w;
    norm.raw = (bf16_t*)raw;
    norm.ssq_out = ssq_out;
  }
  if (ssq_in != nullptr) {
    if ((epilogue & 15) == SK_EPI_ACCUM || parts_in <= 0 || !(eps >= 0.f)) return LLM_ERR_ARG;
    norm.ssq_in = ssq_in;
    norm.parts_in = parts_in;
    norm.eps = eps;
  }
  return skinny_product(X, W, C, epilogue, out_dtype, M, N, K, ldw, 1, norm, stream);
}

// The stacked q|k|v projection with the rotary epilogue (see the head of this file): rotated q as
// bfloat16 [M, n_heads * hd] to `q_out`, k and v to the cache if write_kv.  N is
// (n_heads + 2 n_kv) * hd with write_kv, else n_heads * hd; hd a multiple of 16, rot_dim even.
extern "C" int llm_gemm_skinny_rope_bf16(const void* X, const void* W,
                                         const float* bias, void* q_out, int M, int K, int ldw, int n_heads,
                                         int n_kv, int hd, const float* cos_t, const float* sin_t,
                                         int rot_dim, const int* tok_pos, const int* tok_seq,
                                         const int* seq_slot, const int* table, int table_stride,
                                         void* k_pages, void* v_pages, int page_size, int write_kv,
                                         const float* ssq_in, int parts_in, float eps,
                                         hipStream_t stream) {
  if (M <= 0) return LLM_OK;
  // ssq_in: the rows of X still lack their norm's scale (see llm_gemm_skinny_norm_bf16), or null
  if (ssq_in != nullptr && (M > 16 || parts_in <= 0 || !(eps >= 0.f))) return LLM_ERR_ARG;
  if (M > 64 || K <= 0 || (K & 7) || (ldw != 0 && (ldw < K || (ldw & 7))) || n_heads <= 0 || n_kv < 0 || hd <= 0 || (hd & 15) || rot_dim < 0 ||
      rot_dim > hd || (rot_dim & 1) || page_size != 64)
    return LLM_ERR_ARG;
  if (X == nullptr || W == nullptr || q_out == nullptr || tok_pos == nullptr) return LLM_ERR_ARG;
  if ((((uintptr_t)X) | ((uintptr_t)W) | ((uintptr_t)q_out)) & 15) return LLM_ERR_ARG;
  if (rot_dim > 0 && (cos_t == nullptr || sin_t == nullptr)) return LLM_ERR_ARG;
  if (write_kv && (!k_pages || !v_pages || !table || !seq_slot || !tok_seq || n_kv <= 0 ||
                   ((((uintptr_t)k_pages) | ((uintptr_t)v_pages)) & 7)))
    return LLM_ERR_ARG;
  SkinnyArgs a;
  a.X = (const bf16_t*)X;
  a.W = (const bf16_t*)W;
  a.C = q_out;
  a.M = M;
  a.N = (n_heads + (write_kv ? 2 * n_kv : 0)) * hd;
  a.K = K;
  a.ldw = ldw;
  a.n_out = a.N;
  a.k_split = 1;
  a.stream = stream;
  a.rope.bias = bias;
  a.rope.cos_t = cos_t;
  a.rope.sin_t = sin_t;
  a.rope.tok_pos = tok_pos;
  a.rope.tok_seq = tok_seq;
  a.rope.seq_slot = seq_slot;
  a.rope.table = table;
  a.rope.k_pages = (bf16_t*)k_pages;
  a.rope.v_pages = (bf16_t*)v_pages;
  a.rope.table_stride = table_stride;
  a.rope.n_heads = n_heads;
  a.rope.n_kv = n_kv;
  a.rope.hd = hd;
  a.rope.rot_dim = rot_dim;
  a.rope.write_kv = write_kv;
  a.norm = SkinnyNorm{};
  a.norm.ssq_in = ssq_in;
  a.norm.parts_in = parts_in;
  a.norm.eps = eps;
  return pick_shape<SK_EPI_ROPE, bf16_t>(a);
}

// W[N, K] (rows ldw apart) into the layout the skinny product streams best: for every tile of 16
// rows and every step of 32 elements of K, the 64 fragments of 8 elements in lane order
// (lane l: row l % 16, elements 8 * (l / 16) .. + 7), so that a wave's load is 1 KiB in a row.
// Rows and elements past the end are zero.  out holds ceil(N/16) * ceil(K/32) * 512 elements.
__global__ void pack_weight_kernel(const bf16_t* __restrict__ W, bf16_t* __restrict__ out, int N, int K,
                                   int ldw) {
  const int n_steps = (K + 31) / 32;
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n = t * 16 + r;
  for (int s = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6); s < n_steps; s += gridDim.y * (blockDim.x >> 6)) {
    const int k = s * 32 + g * 8;
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (n < N && k < K) v = *reinterpret_cast<const uint4*>(W + (size_t)n * ldw + k);   // K is a multiple of 8
    *reinterpret_cast<uint4*>(out + (((size_t)t * n_steps + s) * 64 + lane) * 8) = v;
  }
}

extern "C" int llm_pack_weight(const void* W, void* out, int N, int K, int ldw, hipStream_t stream) {
  if (N <= 0 || K <= 0) return LLM_OK;
  if ((K & 7) || ldw < K || (ldw & 7) || ((((uintptr_t)W) | ((uintptr_t)out)) & 15)) return LLM_ERR_ARG;
  const int tiles = (N + 15) / 16;
  dim3 grid(tiles, 8);
  pack_weight_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)W, (bf16_t*)out, N, K, ldw);
  return llm_launch_status();
}
