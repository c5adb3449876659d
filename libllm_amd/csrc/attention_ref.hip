// Attention over the paged cache for any head size, in float32 arithmetic: the kernel of the
// 32-bit path, and the fallback for head sizes the matrix-core kernels do not take.
//
// One wave per (token, head).  Query row of sequence b at absolute position p sees the cached keys
// max(0, p - window + 1) .. p of its slot (window 0: from 0), i.e. the causal mask aligned at the
// bottom right (src/flint/operators.cc:119-124); query head h reads kv head h / (n_heads / n_kv)
// (src/flint/operators.cc:43-56).  Scores are q.k * scale, softmax is max-subtracted and running
// (one page of 64 keys at a time), all in float32.
#include "common.h"

template <typename T, int PAGE, int MAX_HD>
__global__ __launch_bounds__(64) void attention_ref_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, const int* __restrict__ table, int table_stride,
    const int* __restrict__ tok_pos, const int* __restrict__ tok_seq,
    const int* __restrict__ seq_slot, T* __restrict__ out, int n_heads, int n_kv, int hd,
    float scale, int window) {
  __shared__ float qs[MAX_HD];
  const int m = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (n_heads / n_kv);
  const int pos = tok_pos[m];
  const int slot = seq_slot[tok_seq[m]];
  const T* qrow = q + (size_t)m * q_stride + (size_t)h * hd;
  for (int d = lane; d < hd; d += 64) qs[d] = Conv<T>::load(qrow + d) * scale;
  __syncthreads();

  constexpr int ND = MAX_HD / 64;
  float acc[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acc[i] = 0.f;
  float run_max = -INFINITY, run_sum = 0.f;

  const int k_first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* trow = table + (size_t)slot * table_stride;
  for (int pg = k_first / PAGE; pg <= pos / PAGE; ++pg) {
    const int page = trow[pg];
    const size_t kbase = ((size_t)page * n_kv + kvh) * llm_key_block(hd);
    const size_t vbase = ((size_t)page * n_kv + kvh) * llm_value_block(hd);
    const int key = pg * PAGE + lane;
    const bool valid = key >= k_first && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const T* kr = k_pages + kbase;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], Conv<T>::load(kr + llm_key_offset(lane, d)), dot);
      s = dot;
    }
    const float new_max = fmaxf(run_max, wave_max(s));     // finite: the page holds a valid key
    const float p = valid ? expf(s - new_max) : 0.f;
    const float corr = expf(run_max - new_max);            // exp(-inf) = 0 on the first page
    run_sum = run_sum * corr + wave_sum(p);
#pragma unroll
    for (int i = 0; i < ND; ++i) acc[i] *= corr;
    run_max = new_max;
    for (int j = 0; j < PAGE; ++j) {
      const float pj = __shfl(p, j, 64);
      if (pj == 0.f) continue;                             // uniform across the wave
      const T* vr = v_pages + vbase;
#pragma unroll
      for (int i = 0; i < ND; ++i) {
        const int d = lane + i * 64;
        if (d < hd) acc[i] = fmaf(pj, Conv<T>::load(vr + llm_value_offset(hd, d, j)), acc[i]);
      }
    }
  }
  T* orow = out + (size_t)m * n_heads * hd + (size_t)h * hd;
  const float inv = 1.0f / run_sum;
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = lane + i * 64;
    if (d < hd) Conv<T>::store(orow + d, acc[i] * inv);
  }
}

extern "C" int llm_attention_ref(const void* q, int dtype, int q_stride, const void* k_pages,
                                 const void* v_pages, const int* table, int table_stride,
                                 int page_size, const int* tok_pos, const int* tok_seq,
                                 const int* seq_slot, void* out, int M, int n_heads, int n_kv,
                                 int hd, float scale, int window, hipStream_t stream) {
  if (M <= 0) return LLM_OK;
  if (page_size != 64 || hd <= 0 || hd > 256 || n_heads <= 0 || n_kv <= 0 || n_heads % n_kv ||
      n_heads > 65535 || window < 0 || q_stride < n_heads * hd)
    return LLM_ERR_ARG;
  dim3 grid(M, n_heads);
  if (dtype == LLM_DTYPE_F32)
    attention_ref_kernel<float, 64, 256><<<grid, 64, 0, stream>>>(
        (const float*)q, q_stride, (const float*)k_pages, (const float*)v_pages, table, table_stride,
        tok_pos, tok_seq, seq_slot, (float*)out, n_heads, n_kv, hd, scale, window);
  else if (dtype == LLM_DTYPE_BF16)
    attention_ref_kernel<bf16_t, 64, 256><<<grid, 64, 0, stream>>>(
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, table,
        table_stride, tok_pos, tok_seq, seq_slot, (bf16_t*)out, n_heads, n_kv, hd, scale, window);
  else
    return LLM_ERR_ARG;
  return llm_launch_status();
}
