// Matrix-core attention over the paged cache in bfloat16: a flash-style kernel for prompts (any
// number of new tokens per sequence) and a split-key kernel plus combine for single decoded tokens.
// Scores, the running softmax and the output accumulate in float32; probabilities are rounded to
// bfloat16 for the second product, as in the reference's fused path
// (src/flint/cuda/flash_attn.cc:101-186).
//
// Both kernels work on one page (64 keys) at a time through the same routine.  A wave holds up to
// 16 "queries" (16 consecutive tokens of one head for prompts; the query heads that share one kv
// head for decoding), one per lane column j = lane % 16:
//   S^T[key][query] = K[key][:] . Q[query][:]      A operand = K rows, B operand = Q rows
//   O^T[d][query]  += V^T[d][key] * P^T[key][query] A operand = V^T rows (values are stored
//                                                   transposed in the cache), B operand = P
// so every lane's scores, softmax state and output column belong to its own query.  The rows of a
// score tile are assigned to keys so that a lane ends with 8 consecutive keys of each 32-key block
// (tile t, row 4g+e  ->  key 8g + 4t + e), which is exactly the B fragment of the second product.
#include "mfma.h"

#define PAGE 64

// The largest of three in one instruction.  fmaxf first quiets a signalling NaN in every operand
// the compiler cannot prove clean (one more instruction each for sums that come off the matrix
// cores); the instruction alone gives the same result for everything but the NaN's payload.
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float max2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// The largest of x over the four lanes that share lane % 16, in all four: the halves of the wave
// swapped, then the rows of 16 lanes, in registers (a shuffle goes through shared memory).
__device__ __forceinline__ float max_over_lane_groups(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const uint32_t v = __float_as_uint(max2(__uint_as_float(h[0]), __uint_as_float(h[1])));
  const auto q = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  return max2(__uint_as_float(q[0]), __uint_as_float(q[1]));
}
// The sum likewise: neighbouring rows of 16 lanes first, then the halves of the wave.
__device__ __forceinline__ float sum_over_lane_groups(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto q = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const uint32_t v = __float_as_uint(__uint_as_float(q[0]) + __uint_as_float(q[1]));
  const auto h = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return __uint_as_float(h[0]) + __uint_as_float(h[1]);
}
__device__ __forceinline__ float max_of_16(const f32x4 (&s)[4]) {
  float mx = max3(s[0][0], s[0][1], s[0][2]);
  mx = max3(mx, s[0][3], s[1][0]);
  mx = max3(mx, s[1][1], s[1][2]);
  mx = max3(mx, s[1][3], s[2][0]);
  mx = max3(mx, s[2][1], s[2][2]);
  mx = max3(mx, s[2][3], s[3][0]);
  mx = max3(mx, s[3][1], s[3][2]);
  return max2(mx, s[3][3]);
}

template <int HD>
struct AttnState {
  f32x4 o[HD / 16];   // O^T[d = 16*dt + 4*(lane/16) + e][query = lane % 16]
  float m;            // running maximum of the scaled scores, in log2 units
  float l;            // running sum of exp2(score - m)
};

// One page of one kv head, laid out as common.h says.  q: B fragments of this lane's query;
// key0: absolute position of the page's first key; [kmin, kmax]: keys this lane's query may see.
template <int HD>
__device__ __forceinline__ void attn_page(const bf16_t* __restrict__ kpage,
                                          const bf16_t* __restrict__ vpage,
                                          const Frag (&q)[(HD + 31) / 32], float scale_log2,
                                          int key0, int kmin, int kmax, AttnState<HD>& st) {
  constexpr int KS = (HD + 31) / 32;
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  float s[4][4];
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4) {
    const int key_row = (t4 >> 1) * 32 + 8 * (r >> 2) + 4 * (t4 & 1) + (r & 3);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g * 8;
      const Frag a = (d < HD) ? frag_load(kpage + llm_key_offset(key_row, d)) : frag_zero();
      acc = mfma_bf16(a, q[ks], acc);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int key = key0 + (t4 >> 1) * 32 + 8 * g + 4 * (t4 & 1) + e;
      s[t4][e] = (key >= kmin && key <= kmax) ? acc[e] * scale_log2 : -INFINITY;
    }
  }
  float mx = -INFINITY;
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
    for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s[t4][e]);
  mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  const float m_new = fmaxf(st.m, mx);
  const bool any = m_new > -INFINITY;
  const float corr = (st.m > -INFINITY) ? exp2f(st.m - m_new) : 0.f;
  float sum = 0.f;
  Frag p[2];
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float pv = (any && s[t4][e] > -INFINITY) ? exp2f(s[t4][e] - m_new) : 0.f;
      const bf16_t pb = f32_to_bf16(pv);
      p[t4 >> 1].h[4 * (t4 & 1) + e] = pb;
      sum += bf16_to_f32(pb);          // the sum uses the rounded values that multiply V
    }
  sum += __shfl_xor(sum, 16, 64);
  sum += __shfl_xor(sum, 32, 64);
  st.l = st.l * corr + sum;
  st.m = m_new;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    f32x4 o = st.o[dt];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] *= corr;
    const bf16_t* vrow = vpage + llm_value_offset(HD, dt * 16 + r, 8 * g);
    o = mfma_bf16(frag_load(vrow), p[0], o);
    o = mfma_bf16(frag_load(vrow + HD * 32), p[1], o);      // the same dims of positions 32 ..
    st.o[dt] = o;
  }
}

template <int HD>
__device__ __forceinline__ void attn_init(AttnState<HD>& st) {
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) st.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m = -INFINITY;
  st.l = 0.f;
}

template <int HD>
__device__ __forceinline__ void load_query(const bf16_t* qrow, bool valid, Frag (&q)[(HD + 31) / 32]) {
  const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int ks = 0; ks < (HD + 31) / 32; ++ks) {
    const int d = ks * 32 + g * 8;
    q[ks] = (valid && d < HD) ? frag_load(qrow + d) : frag_zero();
  }
}

// ---------------------------------------------------------------------------------- prompts
// A block of 4 waves owns 64 * QT consecutive new tokens of one sequence and one query head; wave
// w owns QT tiles of 16 rows (query columns), tile t being rows 64t + 16w .. 64t + 16w + 15.  The
// block walks the pages its rows may see; a page's keys and values travel global memory ->
// registers (issued one page ahead) -> shared memory, where all four waves read their fragments,
// and a fragment read from shared memory serves all the wave's tiles.  16-byte pieces are
// swizzled in shared memory so that the 16 rows a fragment load touches fall on different banks.
// Blocks are numbered kv head first (consecutive blocks go to consecutive chiplets, so with 8 kv
// heads each chiplet's cache holds one head's keys and values), and long rows first, since later
// rows see more keys.
template <int HD>
struct KeyRow {            // bytes between staged key rows: a power of two of at least 128
  static constexpr int BYTES = (HD * 2 <= 128) ? 128 : ((HD * 2 <= 256) ? 256 : 512);
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// A page's keys and values: global memory -> registers (256 threads, 16 bytes each per round).
template <int HD>
__device__ __forceinline__ void fetch_page(const bf16_t* __restrict__ k_pages,
                                           const bf16_t* __restrict__ v_pages, int page, int n_kv,
                                           int kvh, u32x4 (&kreg)[(8 * HD + 255) / 256],
                                           u32x4 (&vreg)[(8 * HD + 255) / 256]) {
  constexpr int PIECES = 8 * HD, LOADS = (PIECES + 255) / 256;
  const size_t base = ((size_t)page * n_kv + kvh) * PAGE * HD;
  const u32x4* kp = reinterpret_cast<const u32x4*>(k_pages + base);
  const u32x4* vp = reinterpret_cast<const u32x4*>(v_pages + base);
#pragma unroll
  for (int j = 0; j < LOADS; ++j) {
    const int ci = threadIdx.x + j * 256;
    const int cc = (PIECES % 256 == 0 || ci < PIECES) ? ci : 0;     // a piece past the end is not staged
    kreg[j] = kp[cc];
    vreg[j] = vp[cc];
  }
}

// registers -> shared memory, 16-byte pieces swizzled within groups of 8.
template <int HD>
__device__ __forceinline__ void stage_page(unsigned char* k_lds, unsigned char* v_lds,
                                           const u32x4 (&kreg)[(8 * HD + 255) / 256],
                                           const u32x4 (&vreg)[(8 * HD + 255) / 256]) {
  constexpr int PIECES = 8 * HD, LOADS = (PIECES + 255) / 256, KRB = KeyRow<HD>::BYTES;
#pragma unroll
  for (int j = 0; j < LOADS; ++j) {
    const int ci = threadIdx.x + j * 256;
    if (PIECES % 256 == 0 || ci < PIECES) {
      // piece ci of the page as it lies in memory: keys in blocks of 16 dims (two pieces a key)
      const int krow = (ci & 127) >> 1, kc = ((ci >> 7) << 1) | (ci & 1);
      const int kf = (krow & 3) | (((krow >> 3) & 1) << 2);
      *reinterpret_cast<u32x4*>(k_lds + krow * KRB + (((kc & ~7) | ((kc & 7) ^ kf)) * 16)) = kreg[j];
      // values in halves of 32 positions (four pieces a dim and half)
      const int vrow = (ci % (4 * HD)) >> 2, vc = ((ci / (4 * HD)) << 2) | (ci & 3);
      *reinterpret_cast<u32x4*>(v_lds + vrow * 128 + ((vc ^ (vrow & 7)) * 16)) = vreg[j];
    }
  }
}

template <int HD, int QT>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, const int* __restrict__ table, int table_stride,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_pos0, bf16_t* __restrict__ out, int n_heads, int n_kv,
    float scale_log2, int window, int n_qblocks) {
  constexpr int KS = (HD + 31) / 32, DT = HD / 16, KRB = KeyRow<HD>::BYTES;
  constexpr int LOADS = (8 * HD + 255) / 256;    // 16-byte pieces of a page per thread
  constexpr int ROWS = 64 * QT;                  // rows of a block
  __shared__ __attribute__((aligned(16))) unsigned char k_lds[64 * KRB];
  __shared__ __attribute__((aligned(16))) unsigned char v_lds[HD * 128];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
  const int hi = blockIdx.x % n_heads, rest = blockIdx.x / n_heads;
  const int qb = n_qblocks - 1 - rest % n_qblocks, b = rest / n_qblocks;
  const int kvh = hi % n_kv, h = kvh * (n_heads / n_kv) + hi / n_kv;
  const int start = seq_start[b];
  const int n = seq_start[b + 1] - start;
  const int q0b = qb * ROWS;
  if (q0b >= n) return;                                          // the whole block leaves
  const int pos0 = seq_pos0[b], slot = seq_slot[b];
  // tile qt of wave w: rows q0b + 64 * qt + 16 * w .. + 15, so that every page staged for the
  // block's first 64 rows is used by all four waves
  int q0w[QT], row[QT], kmax[QT], kmin[QT];
  bool valid[QT];
  Frag qf[QT][KS];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    q0w[qt] = q0b + 64 * qt + wave * 16;
    row[qt] = q0w[qt] + r;
    valid[qt] = row[qt] < n;
    const int qpos = pos0 + row[qt];                             // rows past the end compute and are dropped
    kmax[qt] = qpos;
    kmin[qt] = (window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
    load_query<HD>(q + (size_t)(start + (valid[qt] ? row[qt] : n - 1)) * q_stride + (size_t)h * HD, valid[qt], qf[qt]);
  }

  // pages of the block, and of this wave's tiles
  const int last_row_b = (q0b + ROWS - 1 < n) ? q0b + ROWS - 1 : n - 1;
  const int pg_first = (window > 0 && pos0 + q0b - window + 1 > 0) ? (pos0 + q0b - window + 1) / PAGE : 0;
  const int pg_last = (pos0 + last_row_b) / PAGE;
  int wpg_first[QT], wpg_last[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int last_row_w = (q0w[qt] + 15 < n) ? q0w[qt] + 15 : n - 1;
    wpg_first[qt] = (window > 0 && pos0 + q0w[qt] - window + 1 > 0) ? (pos0 + q0w[qt] - window + 1) / PAGE : 0;
    wpg_last[qt] = (q0w[qt] < n) ? (pos0 + last_row_w) / PAGE : -1;
  }

  f32x4 o[QT][DT], l_acc[QT];           // every row of l_acc holds the running sum of its column
  float m_run[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m_run[qt] = -INFINITY;
    l_acc[qt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int* trow = table + (size_t)slot * table_stride;
  u32x4 kreg[LOADS], vreg[LOADS];
  fetch_page<HD>(k_pages, v_pages, trow[pg_first], n_kv, kvh, kreg, vreg);
  for (int pg = pg_first; pg <= pg_last; ++pg) {
    __syncthreads();                       // every wave is done with the page before
    stage_page<HD>(k_lds, v_lds, kreg, vreg);
    __syncthreads();
    if (pg < pg_last) fetch_page<HD>(k_pages, v_pages, trow[pg + 1], n_kv, kvh, kreg, vreg);
    // the last tile's rows are the latest and, with a window, a page of the first tile's is
    // one of the last's too unless the window is shorter than the block; a page outside a tile's
    // view is masked as a whole for it
    bool live = false;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) live = live || (pg >= wpg_first[qt] && pg <= wpg_last[qt]);
    if (!live) continue;
    const int key0 = pg * PAGE;

    // ---- scores S^T[key][query] for 64 keys and QT * 16 queries
    f32x4 sc[QT][4];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
      for (int t4 = 0; t4 < 4; ++t4) sc[qt][t4] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t4 = 0; t4 < 4; ++t4) {
      const int key_row = (t4 >> 1) * 32 + 8 * (r >> 2) + 4 * (t4 & 1) + (r & 3);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int c = ks * 4 + g;
        Frag a;
        if (ks * 32 + g * 8 < HD)
          a.u = *reinterpret_cast<const uint4*>(k_lds + key_row * KRB + (((c & ~7) | ((c & 7) ^ (r & 7))) * 16));
        else
          a = frag_zero();
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) sc[qt][t4] = mfma_bf16(a, qf[qt][ks], sc[qt][t4]);
      }
    }

    // ---- running softmax per query column, probabilities as B fragments.  Maxima are taken of
    // the raw scores (the scale is positive) and the scale goes into the exponent's multiply-add.
    Frag p[QT][2];
    float corr[QT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      // a page wholly inside every row's view needs no mask
      const bool mask = (key0 + 63 > pos0 + q0w[qt]) || (window > 0 && key0 < pos0 + q0w[qt] + 15 - window + 1);
      if (mask) {
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int key = key0 + (t4 >> 1) * 32 + 8 * g + 4 * (t4 & 1) + e;
            if (key < kmin[qt] || key > kmax[qt]) sc[qt][t4][e] = -INFINITY;
          }
      }
      const float mx = max_over_lane_groups(max_of_16(sc[qt]));
      const float m_new = max2(m_run[qt], mx * scale_log2);
      const float m_safe = (m_new > -INFINITY) ? m_new : 0.f;    // nothing seen yet: every p is 2^-inf = 0
      corr[qt] = fast_exp2(m_run[qt] - m_safe);
      m_run[qt] = m_new;
#pragma unroll
      for (int t4 = 0; t4 < 4; ++t4) {
        const float p0 = fast_exp2(fmaf(sc[qt][t4][0], scale_log2, -m_safe));
        const float p1 = fast_exp2(fmaf(sc[qt][t4][1], scale_log2, -m_safe));
        const float p2 = fast_exp2(fmaf(sc[qt][t4][2], scale_log2, -m_safe));
        const float p3 = fast_exp2(fmaf(sc[qt][t4][3], scale_log2, -m_safe));
        uint32_t* dst = reinterpret_cast<uint32_t*>(&p[qt][t4 >> 1].u) + 2 * (t4 & 1);
        dst[0] = pack2_bf16(p0, p1);
        dst[1] = pack2_bf16(p2, p3);
      }
    }

    // ---- O^T[d][query] += V^T[d][key] P^T[key][query]; a row of ones under V^T sums the rounded
    // probabilities of each query the same way
    Frag ones;
    ones.u = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      f32x4 acc = l_acc[qt];
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] *= corr[qt];
      acc = mfma_bf16(ones, p[qt][0], acc);
      acc = mfma_bf16(ones, p[qt][1], acc);
      l_acc[qt] = acc;
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int d = dt * 16 + r;
      Frag v0, v1;
      v0.u = *reinterpret_cast<const uint4*>(v_lds + d * 128 + ((g ^ (r & 7)) * 16));
      v1.u = *reinterpret_cast<const uint4*>(v_lds + d * 128 + (((g + 4) ^ (r & 7)) * 16));
#pragma unroll
      for (int qt = 0; qt < QT; ++qt) {
        f32x4 acc = o[qt][dt];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] *= corr[qt];
        acc = mfma_bf16(v0, p[qt][0], acc);
        acc = mfma_bf16(v1, p[qt][1], acc);
        o[qt][dt] = acc;
      }
    }
  }

#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    if (!valid[qt]) continue;
    const float inv = 1.0f / l_acc[qt][0];
    bf16_t* orow = out + (size_t)(start + row[qt]) * n_heads * HD + (size_t)h * HD;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uint2 pk;
      pk.x = (uint32_t)f32_to_bf16(o[qt][dt][0] * inv) | ((uint32_t)f32_to_bf16(o[qt][dt][1] * inv) << 16);
      pk.y = (uint32_t)f32_to_bf16(o[qt][dt][2] * inv) | ((uint32_t)f32_to_bf16(o[qt][dt][3] * inv) << 16);
      *reinterpret_cast<uint2*>(orow + dt * 16 + 4 * g) = pk;
    }
  }
}

// ---------------------------------------------------------------------------------- decoding
// One new token per sequence at position seq_pos0[b]; it sees keys kmin..pos.  grid (blocks, n_kv,
// sequences); a wave's 16 query columns are the query heads of the kv head's group (in blocks of 16
// if the group is larger).  The pages of the sequence are dealt out evenly to all waves of all
// blocks of a (sequence, kv head); a wave loads a whole page (keys and values) into registers
// before it computes; several blocks share a compute unit, so one's loads overlap another's
// arithmetic.  Where the whole grid fits at two blocks a compute unit, a wave also asks for its
// next page while it works on this one (AHEAD); with more blocks than that the registers this
// takes cost more in blocks per unit than the overlap gains.
// The waves of a block merge their (O, m, l)
// through shared memory; with several blocks each writes its merged partial to global memory and
// a second kernel merges the partials in block order.
template <int HD>
struct PageFrags {
  Frag k[4][(HD + 31) / 32];
  Frag v[HD / 16][2];
};

template <int HD>
__device__ __forceinline__ void load_keys(const bf16_t* __restrict__ kpage, PageFrags<HD>& f) {
  constexpr int KS = (HD + 31) / 32;
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4) {
    const int key_row = (t4 >> 1) * 32 + 8 * (r >> 2) + 4 * (t4 & 1) + (r & 3);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g * 8;
      f.k[t4][ks] = (d < HD) ? frag_load_stream(kpage + llm_key_offset(key_row, d)) : frag_zero();
    }
  }
}

template <int HD>
__device__ __forceinline__ void load_values(const bf16_t* __restrict__ vpage, PageFrags<HD>& f) {
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    const bf16_t* vrow = vpage + llm_value_offset(HD, dt * 16 + r, 8 * g);
    f.v[dt][0] = frag_load_stream(vrow);
    f.v[dt][1] = frag_load_stream(vrow + HD * 32);
  }
}

// Same arithmetic as attn_page, on fragments already loaded, in two halves: the scores, after
// which the keys' registers are free for the next page's, and the rest, after which the values' are.
template <int HD>
__device__ __forceinline__ void page_scores(const PageFrags<HD>& f, const Frag (&q)[(HD + 31) / 32],
                                            int key0, int kmin, int kmax, f32x4 (&s)[4]) {
  constexpr int KS = (HD + 31) / 32;
  const int lane = threadIdx.x & 63, g = lane >> 4;
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) acc = mfma_bf16(f.k[t4][ks], q[ks], acc);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int key = key0 + (t4 >> 1) * 32 + 8 * g + 4 * (t4 & 1) + e;
      if (key < kmin || key > kmax) acc[e] = -INFINITY;
    }
    s[t4] = acc;
  }
}

template <int HD>
__device__ __forceinline__ void page_values(const PageFrags<HD>& f, const f32x4 (&s)[4], float scale_log2,
                                            AttnState<HD>& st) {
  const float mx = max_over_lane_groups(max_of_16(s));
  const float m_new = max2(st.m, mx * scale_log2);
  const float m_safe = (m_new > -INFINITY) ? m_new : 0.f;      // nothing seen yet: every p is 0
  const float corr = fast_exp2(st.m - m_safe);
  float sum = 0.f;
  Frag p[2];
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4) {
    uint32_t* dst = reinterpret_cast<uint32_t*>(&p[t4 >> 1].u) + 2 * (t4 & 1);
#pragma unroll
    for (int e = 0; e < 4; e += 2) {
      const float p0 = fast_exp2(fmaf(s[t4][e], scale_log2, -m_safe));
      const float p1 = fast_exp2(fmaf(s[t4][e + 1], scale_log2, -m_safe));
      const uint32_t pk = pack2_bf16(p0, p1);
      dst[e >> 1] = pk;
      sum += __uint_as_float(pk << 16) + __uint_as_float(pk & 0xffff0000u);   // the rounded values
    }
  }
  st.l = st.l * corr + sum_over_lane_groups(sum);
  st.m = m_new;
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    f32x4 o = st.o[dt];
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] *= corr;
    o = mfma_bf16(f.v[dt][0], p[0], o);
    o = mfma_bf16(f.v[dt][1], p[1], o);
    st.o[dt] = o;
  }
}

// ---- work dealt out by length.  With sequences of very unequal lengths in one step, the same
// number of blocks for every (sequence, kv head) leaves the longest to a few blocks (64 sequences,
// one of 131,072 tokens among 63 of 2,048: one block a pair, 512 pages a wave, 13.4 ms a step
// where 3 would do).  Here the grid is flat, `budget` blocks and one more for every pair at most;
// every block works out its share from the lengths in device memory, so the same captured graph
// serves any lengths: the pages of all pairs are cut into chunks of C pages, C the least number
// that keeps the chunks within the budget; pair (b, kvh) has c_b = ceil(pages_b / C) chunks, in
// the order b, kvh, chunk.  A pair of one chunk writes its output itself; the others leave
// partials [chunk, head of the group] that the merge kernel below finds by the same sums.
__device__ __forceinline__ int attn_pages_of(int pos, int window, int& pg_first) {
  const int kmin = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  pg_first = kmin / PAGE;
  return pos / PAGE - pg_first + 1;
}

__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Pages of a chunk: from the lengths of all sequences.  Every lane returns the same.
__device__ __forceinline__ int attn_chunk_pages(const int* __restrict__ seq_pos0, int n_seqs, int n_kv,
                                                int window, int budget, int waves) {
  const int lane = threadIdx.x & 63;
  int total = 0, first;
  for (int i = lane; i < n_seqs; i += 64) total += attn_pages_of(seq_pos0[i], window, first);
  total = wave_sum_int(total);
  const long long units = (long long)total * n_kv;
  const int c = (int)((units + budget - 1) / budget);
  return c > waves ? c : waves;
}

// Chunks (per kv head) of the sequences before sequence b, and of b itself.
__device__ __forceinline__ void attn_chunks_before(const int* __restrict__ seq_pos0, int n_seqs, int window,
                                                   int chunk, int b, int& before, int& mine) {
  const int lane = threadIdx.x & 63;
  int sum = 0, first;
  for (int i = lane; i < b; i += 64) sum += (attn_pages_of(seq_pos0[i], window, first) + chunk - 1) / chunk;
  before = wave_sum_int(sum);
  mine = (attn_pages_of(seq_pos0[b], window, first) + chunk - 1) / chunk;
}

// The sequence whose chunks hold block g (counted over all kv heads), or -1 past the last chunk.
__device__ __forceinline__ int attn_locate(const int* __restrict__ seq_pos0, int n_seqs, int n_kv, int window,
                                           int chunk, int g, int& before, int& mine) {
  const int lane = threadIdx.x & 63;
  int run = 0, first;
  for (int i0 = 0; i0 < n_seqs; i0 += 64) {
    const int i = i0 + lane;
    const int c = (i < n_seqs) ? (attn_pages_of(seq_pos0[i], window, first) + chunk - 1) / chunk : 0;
    int incl = c;                                      // inclusive sums along the wave
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int up = __shfl_up(incl, off, 64);
      if (lane >= off) incl += up;
    }
    const bool here = c > 0 && g >= n_kv * (run + incl - c) && g < n_kv * (run + incl);
    const unsigned long long votes = __ballot(here);
    if (votes) {
      const int src = __ffsll((long long)votes) - 1;
      before = run + __shfl(incl - c, src, 64);
      mine = __shfl(c, src, 64);
      return i0 + src;
    }
    run += __shfl(incl, 63, 64);
  }
  return -1;
}

template <int HD, int WAVES, bool AHEAD>
__global__ __launch_bounds__(WAVES * 64, (HD <= 128) ? 2 : ((HD <= 192) ? 3 : 1)) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, const int* __restrict__ table, int table_stride,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0, float* __restrict__ part_o,
    float* __restrict__ part_ml, bf16_t* __restrict__ out, int n_heads, int n_kv, float scale_log2,
    int window, int budget, int n_seqs) {
  __shared__ float s_o[WAVES][HD][16];
  __shared__ float s_m[WAVES][16], s_l[WAVES][16];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
  const int group = n_heads / n_kv;
  // uniform: grid (blocks, n_kv, sequences), every pair cut into as many blocks;
  // by length (budget > 0): a flat grid, see above
  int blk = blockIdx.x, n_blk = gridDim.x, kvh = blockIdx.y, b = blockIdx.z;
  int chunk = 0, chunk_id = 0;
  if (budget > 0) {
    chunk = attn_chunk_pages(seq_pos0, n_seqs, n_kv, window, budget, WAVES);
    int before, mine;
    b = attn_locate(seq_pos0, n_seqs, n_kv, window, chunk, blockIdx.x, before, mine);
    if (b < 0) return;                               // past the last chunk (the whole block)
    const int rest = blockIdx.x - n_kv * before;
    kvh = rest / mine;
    blk = rest % mine;
    n_blk = mine;
    chunk_id = blockIdx.x;
  }
  const int pos = seq_pos0[b], slot = seq_slot[b];
  const int kmin = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int pg_first = kmin / PAGE, pg_last = pos / PAGE;
  int p0, p1;
  if (budget > 0) {
    const int c0 = pg_first + blk * chunk;
    const int c1 = (c0 + chunk < pg_last + 1) ? c0 + chunk : pg_last + 1;
    const int per = (c1 - c0 + WAVES - 1) / WAVES;
    p0 = c0 + wave * per;
    p1 = (p0 + per < c1) ? p0 + per : c1;
  } else {
    const int n_waves = n_blk * WAVES;
    const int per = (pg_last - pg_first + 1 + n_waves - 1) / n_waves;
    p0 = pg_first + (blk * WAVES + wave) * per;
    p1 = (p0 + per < pg_last + 1) ? p0 + per : pg_last + 1;
  }
  const int* trow = table + (size_t)slot * table_stride;

  for (int hb = 0; hb < group; hb += 16) {
    const bool valid = hb + r < group;
    const int h = kvh * group + (valid ? hb + r : 0);
    Frag qf[(HD + 31) / 32];
    load_query<HD>(q + (size_t)b * q_stride + (size_t)h * HD, valid, qf);
    AttnState<HD> st;
    attn_init<HD>(st);
    const int lo = valid ? kmin : 0x7fffffff, hi = valid ? pos : -1;
    {
      PageFrags<HD> f;
      for (int pg = p0; pg < p1; ++pg) {
        const size_t base = ((size_t)trow[pg] * n_kv + kvh) * PAGE * HD;
        if (HD <= 128) {
          f32x4 s[4];
          if (AHEAD) {
            // The next page's keys are asked for as soon as this page's scores stand, its values
            // as soon as this page's are used, so that a wave's pages overlap.  The compiler
            // takes further registers for it (169 instead of 119 at head size 64), which leaves
            // two blocks a compute unit: the host asks for this when the grid fits in that.
            if (pg == p0) {
              load_keys<HD>(k_pages + base, f);
              load_values<HD>(v_pages + base, f);
            }
            const size_t next = (pg + 1 < p1) ? ((size_t)trow[pg + 1] * n_kv + kvh) * PAGE * HD : 0;
            page_scores<HD>(f, qf, pg * PAGE, lo, hi, s);
            if (pg + 1 < p1) load_keys<HD>(k_pages + next, f);
            page_values<HD>(f, s, scale_log2, st);
            if (pg + 1 < p1) load_values<HD>(v_pages + next, f);
          } else {
            load_keys<HD>(k_pages + base, f);
            load_values<HD>(v_pages + base, f);
            page_scores<HD>(f, qf, pg * PAGE, lo, hi, s);
            page_values<HD>(f, s, scale_log2, st);
          }
        } else {
          attn_page<HD>(k_pages + base, v_pages + base, qf, scale_log2, pg * PAGE, lo, hi, st);
        }
      }
    }

    // ---- merge the waves of the block
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
      for (int e = 0; e < 4; ++e) s_o[wave][dt * 16 + 4 * g + e][r] = st.o[dt][e];
    if (g == 0) {
      s_m[wave][r] = st.m;
      s_l[wave][r] = st.l;
    }
    __syncthreads();
    for (int it = tid; it < 16 * HD; it += WAVES * 64) {
      const int j = it & 15, d = it >> 4;
      if (hb + j >= group) continue;
      float m = s_m[0][j];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) m = fmaxf(m, s_m[w][j]);
      float l = 0.f, o = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const float mw = s_m[w][j];
        const float wgt = (mw > -INFINITY) ? exp2f(mw - m) : 0.f;
        l += s_l[w][j] * wgt;
        o += s_o[w][d][j] * wgt;
      }
      const int hh = kvh * group + hb + j;
      if (n_blk == 1) {
        out[((size_t)b * n_heads + hh) * HD + d] = f32_to_bf16(o / l);
      } else {
        const size_t idx = (budget > 0) ? (size_t)chunk_id * group + hb + j
                                        : ((size_t)b * n_heads + hh) * n_blk + blk;
        part_o[idx * HD + d] = o;
        if (d == 0) {
          part_ml[idx * 2] = m;
          part_ml[idx * 2 + 1] = l;
        }
      }
    }
    __syncthreads();
  }
}

// out[b, h, :] = sum_s O_s 2^(m_s - m) / sum_s l_s 2^(m_s - m) over the blocks' partials, in block
// order; grid (n_heads, sequences), one thread per dimension.  Up to NB partials (the template's
// bound) are all fetched before any is used, so the kernel waits for memory once.
template <int NB>
__global__ void attn_decode_combine_kernel(const float* __restrict__ part_o,
                                           const float* __restrict__ part_ml,
                                           bf16_t* __restrict__ out, int n_heads, int hd, int n_blk) {
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const size_t idx0 = ((size_t)b * n_heads + h) * n_blk;
  const bool live = d < hd;
  float ms[NB], ls[NB], os[NB];
#pragma unroll
  for (int s = 0; s < NB; ++s) {
    const bool in = s < n_blk;
    const float2 ml = in ? *reinterpret_cast<const float2*>(part_ml + (idx0 + s) * 2) : make_float2(-INFINITY, 0.f);
    ms[s] = ml.x;
    ls[s] = ml.y;
    os[s] = (in && live) ? part_o[(idx0 + s) * hd + d] : 0.f;
  }
  float m = ms[0];
#pragma unroll
  for (int s = 1; s < NB; ++s) m = fmaxf(m, ms[s]);
  float l = 0.f, o = 0.f;
#pragma unroll
  for (int s = 0; s < NB; ++s) {
    const float w = (ms[s] > -INFINITY) ? exp2f(ms[s] - m) : 0.f;
    l += ls[s] * w;
    o += os[s] * w;
  }
  if (live) out[((size_t)b * n_heads + h) * hd + d] = f32_to_bf16(o / l);
}

// The same for any number of partials: block (dims, G groups); group g merges partials g, g+G, ...
// as they come (a running maximum), then the G groups are merged through shared memory.  G is 8
// for heads of up to 128 dims and 4 beyond, so that the block stays within 1,024 threads.
template <int G>
__global__ void attn_decode_combine_loop_kernel(const float* __restrict__ part_o,
                                                const float* __restrict__ part_ml,
                                                bf16_t* __restrict__ out, int n_heads, int hd,
                                                int n_blk) {
  __shared__ float s_m[G], s_l[G], s_o[G][256];
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x, grp = threadIdx.y;
  const size_t idx0 = ((size_t)b * n_heads + h) * n_blk;
  const bool live = d < hd;
  float m = -INFINITY, l = 0.f, o = 0.f;
#pragma unroll 4
  for (int s = grp; s < n_blk; s += G) {
    const float2 ml = *reinterpret_cast<const float2*>(part_ml + (idx0 + s) * 2);
    const float ov = live ? part_o[(idx0 + s) * hd + d] : 0.f;
    if (ml.x > -INFINITY) {
      const float m_new = fmaxf(m, ml.x);
      const float c_old = exp2f(m - m_new), c_new = exp2f(ml.x - m_new);   // exp2(-inf) = 0 at first
      l = l * c_old + ml.y * c_new;
      o = o * c_old + ov * c_new;
      m = m_new;
    }
  }
  if (d == 0) {
    s_m[grp] = m;
    s_l[grp] = l;
  }
  s_o[grp][d] = o;
  __syncthreads();
  if (grp != 0 || !live) return;
  float mm = s_m[0];
#pragma unroll
  for (int g = 1; g < G; ++g) mm = fmaxf(mm, s_m[g]);
  float lt = 0.f, ot = 0.f;
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const float w = (s_m[g] > -INFINITY) ? exp2f(s_m[g] - mm) : 0.f;
    lt += s_l[g] * w;
    ot += s_o[g][d] * w;
  }
  out[((size_t)b * n_heads + h) * hd + d] = f32_to_bf16(ot / lt);
}

// The same where the work was dealt out by length: block (dims, G groups) for (head, sequence)
// finds the pair's chunks by the sums that the attention kernel used; a pair of one chunk has
// written its output already.
template <int G>
__global__ void attn_decode_combine_by_length_kernel(const float* __restrict__ part_o,
                                                     const float* __restrict__ part_ml,
                                                     const int* __restrict__ seq_pos0, bf16_t* __restrict__ out,
                                                     int n_heads, int n_kv, int hd, int window, int budget,
                                                     int waves, int n_seqs) {
  __shared__ float s_m[G], s_l[G], s_o[G][256];
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x, grp = threadIdx.y;
  const int group = n_heads / n_kv, kvh = h / group;
  const int chunk = attn_chunk_pages(seq_pos0, n_seqs, n_kv, window, budget, waves);
  int before, mine;
  attn_chunks_before(seq_pos0, n_seqs, window, chunk, b, before, mine);
  if (mine == 1) return;
  const size_t first = (size_t)n_kv * before + (size_t)kvh * mine;       // the pair's first chunk
  const bool live = d < hd;
  float m = -INFINITY, l = 0.f, o = 0.f;
#pragma unroll 4
  for (int s = grp; s < mine; s += G) {
    const size_t idx = (first + s) * group + (h - kvh * group);
    const float2 ml = *reinterpret_cast<const float2*>(part_ml + idx * 2);
    const float ov = live ? part_o[idx * hd + d] : 0.f;
    if (ml.x > -INFINITY) {
      const float m_new = fmaxf(m, ml.x);
      const float c_old = exp2f(m - m_new), c_new = exp2f(ml.x - m_new);   // exp2(-inf) = 0 at first
      l = l * c_old + ml.y * c_new;
      o = o * c_old + ov * c_new;
      m = m_new;
    }
  }
  if (d == 0) {
    s_m[grp] = m;
    s_l[grp] = l;
  }
  s_o[grp][d] = o;
  __syncthreads();
  if (grp != 0 || !live) return;
  float mm = s_m[0];
#pragma unroll
  for (int gg = 1; gg < G; ++gg) mm = fmaxf(mm, s_m[gg]);
  float lt = 0.f, ot = 0.f;
#pragma unroll
  for (int gg = 0; gg < G; ++gg) {
    const float w = (s_m[gg] > -INFINITY) ? exp2f(s_m[gg] - mm) : 0.f;
    lt += s_l[gg] * w;
    ot += s_o[gg][d] * w;
  }
  out[((size_t)b * n_heads + h) * hd + d] = f32_to_bf16(ot / lt);
}

// ---------------------------------------------------------------------------------- entry points
#define FOR_HEAD_DIMS(X) X(16) X(32) X(48) X(64) X(80) X(96) X(112) X(128) X(144) X(160) X(176) X(192) X(208) X(224) X(240) X(256)

extern "C" int llm_attention_mfma_supported(int hd) {
#define CASE(D) if (hd == D) return 1;
  FOR_HEAD_DIMS(CASE)
#undef CASE
  return 0;
}

static bool attn_args_ok(const void* q, int q_stride, const void* k, const void* v, int n_heads,
                         int n_kv, int hd, int window) {
  if (n_heads <= 0 || n_kv <= 0 || n_heads % n_kv || window < 0) return false;
  if (hd % 16 || (q_stride % 8)) return false;         // 16-byte fragments of queries
  if ((((uintptr_t)q) | ((uintptr_t)k) | ((uintptr_t)v)) & 15) return false;
  return true;
}

extern "C" int llm_attention_prefill_bf16(const void* q, int q_stride, const void* k_pages,
                                          const void* v_pages, const int* table, int table_stride,
                                          int page_size, const int* seq_start, const int* seq_slot,
                                          const int* seq_pos0, void* out, int n_seqs, int max_new,
                                          int n_heads, int n_kv, int hd, float scale, int window,
                                          int tiles, hipStream_t stream) {
  if (n_seqs <= 0 || max_new <= 0) return LLM_OK;
  if ((tiles != 1 && tiles != 2) || page_size != PAGE || !attn_args_ok(q, q_stride, k_pages, v_pages, n_heads, n_kv, hd, window) ||
      n_heads > 65535 || n_seqs > 65535)
    return LLM_ERR_ARG;
  const float scale_log2 = scale * 1.4426950408889634f;
  // tiles: tiles of 16 rows a wave takes, so a block covers 64 or 128 rows.  Two halve the reads
  // from shared memory and the staging per row; the caller chooses (one balances short and long
  // rows better while the blocks are few).
  const int qt = tiles;
  const int n_qblocks = (max_new + 64 * qt - 1) / (64 * qt);
  const long long blocks = (long long)n_qblocks * n_heads * n_seqs;
  if (blocks > 0x7fffffffLL) return LLM_ERR_ARG;
#define LAUNCH(D, Q)                                                                              \
  attn_prefill_kernel<D, Q><<<(unsigned)blocks, 256, 0, stream>>>(                                \
      (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,          \
      table_stride, seq_start, seq_slot, seq_pos0, (bf16_t*)out, n_heads, n_kv, scale_log2,       \
      window, n_qblocks)
#define CASE(D)                                                                                   \
  if (hd == D) {                                                                                  \
    if (qt == 2)                                                                                  \
      LAUNCH(D, 2);                                                                               \
    else                                                                                          \
      LAUNCH(D, 1);                                                                               \
    return llm_launch_status();                                                                   \
  }
  FOR_HEAD_DIMS(CASE)
#undef CASE
#undef LAUNCH
  return LLM_ERR_ARG;
}

// part_o: [n_seqs, n_heads, n_blocks, hd] float32; part_ml: [n_seqs, n_heads, n_blocks, 2].
// With budget > 0 the work is dealt out by the sequences' lengths instead (see the kernel):
// n_blocks is not used, and the partials are [budget + n_seqs * n_kv, n_heads / n_kv, hd] and
// [..., 2].
extern "C" int llm_attention_decode_bf16(const void* q, int q_stride, const void* k_pages,
                                         const void* v_pages, const int* table, int table_stride,
                                         int page_size, const int* seq_slot, const int* seq_pos0,
                                         float* part_o, float* part_ml, void* out,
                                         int n_seqs, int n_heads, int n_kv, int hd, float scale,
                                         int window, int n_blocks, int budget, hipStream_t stream) {
  if (n_seqs <= 0) return LLM_OK;
  if (page_size != PAGE || !attn_args_ok(q, q_stride, k_pages, v_pages, n_heads, n_kv, hd, window) ||
      n_blocks <= 0 || n_blocks > 1024 || n_kv > 65535 || n_seqs > 65535 || n_heads > 65535 || hd > 256 ||
      budget < 0 || budget > (1 << 20))
    return LLM_ERR_ARG;
  if ((n_blocks > 1 || budget > 0) && (!part_o || !part_ml)) return LLM_ERR_ARG;
  const float scale_log2 = scale * 1.4426950408889634f;
  if (budget > 0) {
    const dim3 flat((unsigned)(budget + n_seqs * n_kv));
    const dim3 cgrid(n_heads, n_seqs);
    const int cthreads = ((hd + 63) / 64) * 64;
#define CASE(D)                                                                                   \
  if (hd == D) {                                                                                  \
    constexpr int WAVES = (D > 192) ? 2 : 4;                                                      \
    attn_decode_kernel<D, WAVES, false><<<flat, WAVES * 64, 0, stream>>>(                         \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,        \
        table_stride, seq_slot, seq_pos0, part_o, part_ml, (bf16_t*)out, n_heads, n_kv,           \
        scale_log2, window, budget, n_seqs);                                                      \
    if (hipGetLastError() != hipSuccess) return LLM_ERR_LAUNCH;                                   \
    if (cthreads <= 128)                                                                          \
      attn_decode_combine_by_length_kernel<8><<<cgrid, dim3(cthreads, 8), 0, stream>>>(           \
          part_o, part_ml, seq_pos0, (bf16_t*)out, n_heads, n_kv, hd, window, budget, WAVES,      \
          n_seqs);                                                                                \
    else                                                                                          \
      attn_decode_combine_by_length_kernel<4><<<cgrid, dim3(cthreads, 4), 0, stream>>>(           \
          part_o, part_ml, seq_pos0, (bf16_t*)out, n_heads, n_kv, hd, window, budget, WAVES,      \
          n_seqs);                                                                                \
    return llm_launch_status();                                                                   \
  }
    FOR_HEAD_DIMS(CASE)
#undef CASE
    return LLM_ERR_ARG;
  }
  dim3 grid(n_blocks, n_kv, n_seqs);
  // pages overlapped within a wave where all blocks are resident at two a compute unit
  const bool ahead = hd <= 128 && (long long)n_blocks * n_kv * n_seqs <= 2LL * llm_compute_units();
#define CASE(D)                                                                                   \
  if (hd == D) {                                                                                  \
    constexpr int WAVES = (D > 192) ? 2 : 4;                                                      \
    if (ahead)                                                                                    \
      attn_decode_kernel<D, WAVES, true><<<grid, WAVES * 64, 0, stream>>>(                        \
          (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,      \
          table_stride, seq_slot, seq_pos0, part_o, part_ml, (bf16_t*)out, n_heads, n_kv,         \
          scale_log2, window, 0, n_seqs);                                                         \
    else                                                                                          \
      attn_decode_kernel<D, WAVES, false><<<grid, WAVES * 64, 0, stream>>>(                       \
          (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,      \
          table_stride, seq_slot, seq_pos0, part_o, part_ml, (bf16_t*)out, n_heads, n_kv,         \
          scale_log2, window, 0, n_seqs);                                                         \
    if (n_blocks > 1) {                                                                           \
      if (hipGetLastError() != hipSuccess) return LLM_ERR_LAUNCH;                                 \
      const dim3 cgrid(n_heads, n_seqs);                                                          \
      const int cthreads = ((hd + 63) / 64) * 64;                                                 \
      if (n_blocks <= 8)                                                                          \
        attn_decode_combine_kernel<8><<<cgrid, cthreads, 0, stream>>>(part_o, part_ml,            \
                                                                     (bf16_t*)out, n_heads, hd,   \
                                                                     n_blocks);                   \
      else if (n_blocks <= 32)                                                                    \
        attn_decode_combine_kernel<32><<<cgrid, cthreads, 0, stream>>>(part_o, part_ml,           \
                                                                      (bf16_t*)out, n_heads, hd,  \
                                                                      n_blocks);                  \
      else if (cthreads <= 128)                                                                   \
        attn_decode_combine_loop_kernel<8><<<cgrid, dim3(cthreads, 8), 0, stream>>>(              \
            part_o, part_ml, (bf16_t*)out, n_heads, hd, n_blocks);                                \
      else                                                                                        \
        attn_decode_combine_loop_kernel<4><<<cgrid, dim3(cthreads, 4), 0, stream>>>(              \
            part_o, part_ml, (bf16_t*)out, n_heads, hd, n_blocks);                                \
    }                                                                                             \
    return llm_launch_status();                                                                   \
  }
  FOR_HEAD_DIMS(CASE)
#undef CASE
  return LLM_ERR_ARG;
}

// Waves per block of the decode kernel for a head size (the host sizes its grid with it): four
// while their partial results fit the 64 KiB of shared memory a block may declare (with two,
// head sizes 160 and 192 read 3.3 and 2.7 TB/s at batch 64 and 4,096 keys; with four 4.7 and 4.1;
// the kernel's launch bounds ask for three such blocks a compute unit, without which head size
// 176 took 170 registers, two too many for that, and read 2.7 TB/s instead of 4.3).
extern "C" int llm_attention_decode_waves(int hd) { return hd > 192 ? 2 : 4; }
