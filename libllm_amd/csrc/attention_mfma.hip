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

template <int HD>
struct AttnState {
  f32x4 o[HD / 16];   // O^T[d = 16*dt + 4*(lane/16) + e][query = lane % 16]
  float m;            // running maximum of the scaled scores, in log2 units
  float l;            // running sum of exp2(score - m)
};

// One page.  kpage: [64][HD] keys; vpage: [HD][64] values; q: B fragments of this lane's query;
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
    const bf16_t* krow = kpage + (size_t)key_row * HD;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g * 8;
      const Frag a = (d < HD) ? frag_load(krow + d) : frag_zero();
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
    const bf16_t* vrow = vpage + (size_t)(dt * 16 + r) * PAGE + 8 * g;
    o = mfma_bf16(frag_load(vrow), p[0], o);
    o = mfma_bf16(frag_load(vrow + 32), p[1], o);
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
// grid (ceil(max_new / 64), n_heads, sequences), 4 waves, 16 query rows per wave.
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, const int* __restrict__ table, int table_stride,
    const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_pos0, bf16_t* __restrict__ out, int n_heads, int n_kv,
    float scale_log2, int window) {
  const int b = blockIdx.z, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int start = seq_start[b];
  const int n = seq_start[b + 1] - start;
  const int q0 = blockIdx.x * 64 + wave * 16;
  if (q0 >= n) return;                                   // the whole wave leaves; no barriers below
  const int pos0 = seq_pos0[b], slot = seq_slot[b];
  const int kvh = h / (n_heads / n_kv);
  const int row = q0 + r;
  const bool valid = row < n;
  Frag qf[(HD + 31) / 32];
  load_query<HD>(q + (size_t)(start + (valid ? row : n - 1)) * q_stride + (size_t)h * HD, valid, qf);
  const int qpos = pos0 + row;
  const int kmax = valid ? qpos : -1;
  const int kmin = !valid ? 0x7fffffff : ((window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0);
  const int first_pos = pos0 + q0;
  const int last_pos = pos0 + ((q0 + 15 < n) ? q0 + 15 : n - 1);
  const int pg_first = (window > 0 && first_pos - window + 1 > 0) ? (first_pos - window + 1) / PAGE : 0;
  const int pg_last = last_pos / PAGE;

  AttnState<HD> st;
  attn_init<HD>(st);
  const int* trow = table + (size_t)slot * table_stride;
  for (int pg = pg_first; pg <= pg_last; ++pg) {
    const size_t base = ((size_t)trow[pg] * n_kv + kvh) * PAGE * HD;
    attn_page<HD>(k_pages + base, v_pages + base, qf, scale_log2, pg * PAGE, kmin, kmax, st);
  }
  if (valid) {
    const float inv = 1.0f / st.l;
    bf16_t* orow = out + (size_t)(start + row) * n_heads * HD + (size_t)h * HD;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      uint2 pk;
      pk.x = (uint32_t)f32_to_bf16(st.o[dt][0] * inv) | ((uint32_t)f32_to_bf16(st.o[dt][1] * inv) << 16);
      pk.y = (uint32_t)f32_to_bf16(st.o[dt][2] * inv) | ((uint32_t)f32_to_bf16(st.o[dt][3] * inv) << 16);
      *reinterpret_cast<uint2*>(orow + dt * 16 + 4 * g) = pk;
    }
  }
}

// ---------------------------------------------------------------------------------- decoding
// One new token per sequence at position seq_pos0[b]; it sees keys kmin..pos.  grid (blocks, n_kv,
// sequences); a wave's 16 query columns are the query heads of the kv head's group (in blocks of 16
// if the group is larger).  The pages of the sequence are dealt out evenly to all waves of all
// blocks of a (sequence, kv head); a wave loads a whole page (keys and values) into registers
// before it computes, and the next page meanwhile.  The waves of a block merge their (O, m, l)
// through shared memory; with several blocks each writes its merged partial to global memory and
// a second kernel merges the partials in block order.
template <int HD>
struct PageFrags {
  Frag k[4][(HD + 31) / 32];
  Frag v[HD / 16][2];
};

template <int HD>
__device__ __forceinline__ void load_page(const bf16_t* __restrict__ kpage,
                                          const bf16_t* __restrict__ vpage, PageFrags<HD>& f) {
  constexpr int KS = (HD + 31) / 32;
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4) {
    const int key_row = (t4 >> 1) * 32 + 8 * (r >> 2) + 4 * (t4 & 1) + (r & 3);
    const bf16_t* krow = kpage + (size_t)key_row * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g * 8;
      f.k[t4][ks] = (d < HD) ? frag_load(krow + d) : frag_zero();
    }
  }
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    const bf16_t* vrow = vpage + (size_t)(dt * 16 + r) * PAGE + 8 * g;
    f.v[dt][0] = frag_load(vrow);
    f.v[dt][1] = frag_load(vrow + 32);
  }
}

// Same arithmetic as attn_page, on fragments already loaded.
template <int HD>
__device__ __forceinline__ void compute_page(const PageFrags<HD>& f, const Frag (&q)[(HD + 31) / 32],
                                             float scale_log2, int key0, int kmin, int kmax,
                                             AttnState<HD>& st) {
  constexpr int KS = (HD + 31) / 32;
  const int lane = threadIdx.x & 63, g = lane >> 4;
  float s[4][4];
#pragma unroll
  for (int t4 = 0; t4 < 4; ++t4) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) acc = mfma_bf16(f.k[t4][ks], q[ks], acc);
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
    o = mfma_bf16(f.v[dt][0], p[0], o);
    o = mfma_bf16(f.v[dt][1], p[1], o);
    st.o[dt] = o;
  }
}

template <int HD, int WAVES, bool DOUBLE>
__global__ __launch_bounds__(WAVES * 64, (!DOUBLE && HD <= 128) ? 2 : 1) void attn_decode_kernel(
    const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, const int* __restrict__ table, int table_stride,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_pos0, float* __restrict__ part_o,
    float* __restrict__ part_ml, bf16_t* __restrict__ out, int n_heads, int n_kv, float scale_log2,
    int window) {
  __shared__ float s_o[WAVES][HD][16];
  __shared__ float s_m[WAVES][16], s_l[WAVES][16];
  const int blk = blockIdx.x, n_blk = gridDim.x, kvh = blockIdx.y, b = blockIdx.z;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
  const int group = n_heads / n_kv;
  const int pos = seq_pos0[b], slot = seq_slot[b];
  const int kmin = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int pg_first = kmin / PAGE, pg_last = pos / PAGE;
  const int n_waves = n_blk * WAVES;
  const int per = (pg_last - pg_first + 1 + n_waves - 1) / n_waves;
  const int p0 = pg_first + (blk * WAVES + wave) * per;
  const int p1 = (p0 + per < pg_last + 1) ? p0 + per : pg_last + 1;
  const int* trow = table + (size_t)slot * table_stride;

  for (int hb = 0; hb < group; hb += 16) {
    const bool valid = hb + r < group;
    const int h = kvh * group + (valid ? hb + r : 0);
    Frag qf[(HD + 31) / 32];
    load_query<HD>(q + (size_t)b * q_stride + (size_t)h * HD, valid, qf);
    AttnState<HD> st;
    attn_init<HD>(st);
    const int lo = valid ? kmin : 0x7fffffff, hi = valid ? pos : -1;
    if (DOUBLE) {
      PageFrags<HD> f0, f1;
      if (p0 < p1) {
        const size_t base = ((size_t)trow[p0] * n_kv + kvh) * PAGE * HD;
        load_page<HD>(k_pages + base, v_pages + base, f0);
      }
      for (int pg = p0; pg < p1; pg += 2) {
        if (pg + 1 < p1) {
          const size_t base = ((size_t)trow[pg + 1] * n_kv + kvh) * PAGE * HD;
          load_page<HD>(k_pages + base, v_pages + base, f1);
        }
        compute_page<HD>(f0, qf, scale_log2, pg * PAGE, lo, hi, st);
        if (pg + 1 >= p1) break;
        if (pg + 2 < p1) {
          const size_t base = ((size_t)trow[pg + 2] * n_kv + kvh) * PAGE * HD;
          load_page<HD>(k_pages + base, v_pages + base, f0);
        }
        compute_page<HD>(f1, qf, scale_log2, (pg + 1) * PAGE, lo, hi, st);
      }
    } else {
      for (int pg = p0; pg < p1; ++pg) {
        const size_t base = ((size_t)trow[pg] * n_kv + kvh) * PAGE * HD;
        if (HD <= 128) {
          PageFrags<HD> f;
          load_page<HD>(k_pages + base, v_pages + base, f);
          compute_page<HD>(f, qf, scale_log2, pg * PAGE, lo, hi, st);
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
        const size_t idx = ((size_t)b * n_heads + hh) * n_blk + blk;
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
// order; grid (n_heads, sequences), one thread per dimension.
__global__ void attn_decode_combine_kernel(const float* __restrict__ part_o,
                                           const float* __restrict__ part_ml,
                                           bf16_t* __restrict__ out, int n_heads, int hd, int n_blk) {
  __shared__ float s_w[1024];
  const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
  const size_t idx0 = ((size_t)b * n_heads + h) * n_blk;
  float m = -INFINITY;
  for (int s = 0; s < n_blk; ++s) m = fmaxf(m, part_ml[(idx0 + s) * 2]);
  for (int s = d; s < n_blk; s += blockDim.x) {
    const float ms = part_ml[(idx0 + s) * 2];
    s_w[s] = (ms > -INFINITY) ? exp2f(ms - m) : 0.f;
  }
  __syncthreads();
  float l = 0.f, o = 0.f;
  for (int s = 0; s < n_blk; ++s) {
    const float w = s_w[s];
    l += part_ml[(idx0 + s) * 2 + 1] * w;
    if (d < hd) o += part_o[(idx0 + s) * hd + d] * w;
  }
  if (d < hd) out[((size_t)b * n_heads + h) * hd + d] = f32_to_bf16(o / l);
}

// ---------------------------------------------------------------------------------- entry points
#define FOR_HEAD_DIMS(X) X(16) X(32) X(48) X(64) X(80) X(96) X(112) X(128) X(160) X(192) X(256)

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
                                          hipStream_t stream) {
  if (n_seqs <= 0 || max_new <= 0) return LLM_OK;
  if (page_size != PAGE || !attn_args_ok(q, q_stride, k_pages, v_pages, n_heads, n_kv, hd, window) ||
      n_heads > 65535 || n_seqs > 65535)
    return LLM_ERR_ARG;
  const float scale_log2 = scale * 1.4426950408889634f;
  dim3 grid((max_new + 63) / 64, n_heads, n_seqs);
#define CASE(D)                                                                                   \
  if (hd == D) {                                                                                  \
    attn_prefill_kernel<D><<<grid, 256, 0, stream>>>(                                             \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,        \
        table_stride, seq_start, seq_slot, seq_pos0, (bf16_t*)out, n_heads, n_kv, scale_log2,     \
        window);                                                                                  \
    return llm_launch_status();                                                                   \
  }
  FOR_HEAD_DIMS(CASE)
#undef CASE
  return LLM_ERR_ARG;
}

// part_o: [n_seqs, n_heads, n_blocks, hd] float32; part_ml: [n_seqs, n_heads, n_blocks, 2].
// pages_per_wave: the most pages a wave will get (a hint: above 1 the kernel that keeps a second
// page in flight is used).
extern "C" int llm_attention_decode_bf16(const void* q, int q_stride, const void* k_pages,
                                         const void* v_pages, const int* table, int table_stride,
                                         int page_size, const int* seq_slot, const int* seq_pos0,
                                         float* part_o, float* part_ml, void* out,
                                         int n_seqs, int n_heads, int n_kv, int hd, float scale,
                                         int window, int n_blocks, int pages_per_wave, hipStream_t stream) {
  if (n_seqs <= 0) return LLM_OK;
  if (page_size != PAGE || !attn_args_ok(q, q_stride, k_pages, v_pages, n_heads, n_kv, hd, window) ||
      n_blocks <= 0 || n_blocks > 1024 || n_kv > 65535 || n_seqs > 65535 || n_heads > 65535 || hd > 256)
    return LLM_ERR_ARG;
  if (n_blocks > 1 && (!part_o || !part_ml)) return LLM_ERR_ARG;
  const float scale_log2 = scale * 1.4426950408889634f;
  dim3 grid(n_blocks, n_kv, n_seqs);
#define CASE(D)                                                                                   \
  if (hd == D) {                                                                                  \
    constexpr int WAVES = (D > 128) ? 2 : 4;                                                      \
    if (pages_per_wave > 1 && D <= 64)                                                            \
      attn_decode_kernel<D, WAVES, true><<<grid, WAVES * 64, 0, stream>>>(                        \
          (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,      \
          table_stride, seq_slot, seq_pos0, part_o, part_ml, (bf16_t*)out, n_heads, n_kv,         \
          scale_log2, window);                                                                    \
    else                                                                                          \
      attn_decode_kernel<D, WAVES, false><<<grid, WAVES * 64, 0, stream>>>(                       \
          (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,      \
          table_stride, seq_slot, seq_pos0, part_o, part_ml, (bf16_t*)out, n_heads, n_kv,         \
          scale_log2, window);                                                                    \
    if (n_blocks > 1) {                                                                           \
      if (hipGetLastError() != hipSuccess) return LLM_ERR_LAUNCH;                                 \
      attn_decode_combine_kernel<<<dim3(n_heads, n_seqs), ((hd + 63) / 64) * 64, 0, stream>>>(    \
          part_o, part_ml, (bf16_t*)out, n_heads, hd, n_blocks);                                  \
    }                                                                                             \
    return llm_launch_status();                                                                   \
  }
  FOR_HEAD_DIMS(CASE)
#undef CASE
  return LLM_ERR_ARG;
}

// Waves per block of the decode kernel for a head size (the host sizes its grid with it).
extern "C" int llm_attention_decode_waves(int hd) { return hd > 128 ? 2 : 4; }
