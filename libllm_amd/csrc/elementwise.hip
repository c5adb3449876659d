// Row-wise kernels: embedding gather, residual add + RMS norm, SiLU-mul, bias add, and the fused
// rotary rotation + cache write.  All arithmetic is float32; storage is float32 or bfloat16.
#include "common.h"

// ---------------------------------------------------------------------------------- embedding
// out[m, :] = table[ids[m], :] * scale, written as the float32 residual stream
// (reference: src/flint/cuda/lookup.cu:30-43).
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int H, int V, float scale) {
  const int m = blockIdx.x;
  int id = ids[m];
  if (id < 0 || id >= V) id = 0;   // the host checks ids; never read outside the table
  const T* row = table + (size_t)id * H;
  float* dst = out + (size_t)m * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = Conv<T>::load(row + i) * scale;
}

extern "C" int llm_embed(const void* table, int table_dtype, const int* ids, float* out, int M,
                         int H, int V, float scale, hipStream_t stream) {
  if (M <= 0) return LLM_OK;
  if (H <= 0 || V <= 0) return LLM_ERR_ARG;
  if (table_dtype == LLM_DTYPE_F32)
    embed_kernel<float><<<M, 256, 0, stream>>>((const float*)table, ids, out, H, V, scale);
  else if (table_dtype == LLM_DTYPE_BF16)
    embed_kernel<bf16_t><<<M, 256, 0, stream>>>((const bf16_t*)table, ids, out, H, V, scale);
  else
    return LLM_ERR_ARG;
  return llm_launch_status();
}

// The same, and what the RMS norm that reads these rows next needs from them (see the head of
// gemm_skinny.hip): raw[m, :] = bfloat16(out[m, :] * norm_w) and ssq[m, t], the sum of squares of
// out[m, 16 t .. 16 t + 15].  H is a multiple of 16; four threads share a tile of 16 columns.
template <typename T>
__global__ __launch_bounds__(256) void embed_norm_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                                         float* __restrict__ out, int H, int V, float scale,
                                                         const float* __restrict__ norm_w,
                                                         bf16_t* __restrict__ raw, float* __restrict__ ssq) {
  const int m = blockIdx.x;
  int id = ids[m];
  if (id < 0 || id >= V) id = 0;
  const T* row = table + (size_t)id * H;
  for (int i4 = threadIdx.x; i4 < H / 4; i4 += 256) {       // H / 4 is a multiple of 4: a tile's threads go together
    float4 v = Conv4<T>::load(row + i4 * 4);
    v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
    *reinterpret_cast<float4*>(out + (size_t)m * H + i4 * 4) = v;
    const float4 w = *reinterpret_cast<const float4*>(norm_w + i4 * 4);
    Conv4<bf16_t>::store(raw + (size_t)m * H + i4 * 4, make_float4(v.x * w.x, v.y * w.y, v.z * w.z, v.w * w.w));
    float ss = v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    ss += __shfl_xor(ss, 1, 64);
    ss += __shfl_xor(ss, 2, 64);
    if ((threadIdx.x & 3) == 0) ssq[(size_t)m * (H / 16) + i4 / 4] = ss;
  }
}

extern "C" int llm_embed_norm(const void* table, int table_dtype, const int* ids, float* out, int M, int H,
                              int V, float scale, const float* norm_w, void* raw, float* ssq,
                              hipStream_t stream) {
  if (M <= 0) return LLM_OK;
  if (H <= 0 || (H & 15) || V <= 0 || !norm_w || !raw || !ssq ||
      ((((uintptr_t)table) | ((uintptr_t)out) | ((uintptr_t)norm_w) | ((uintptr_t)raw)) & 15))
    return LLM_ERR_ARG;
  if (table_dtype == LLM_DTYPE_F32)
    embed_norm_kernel<float><<<M, 256, 0, stream>>>((const float*)table, ids, out, H, V, scale, norm_w,
                                                     (bf16_t*)raw, ssq);
  else if (table_dtype == LLM_DTYPE_BF16)
    embed_norm_kernel<bf16_t><<<M, 256, 0, stream>>>((const bf16_t*)table, ids, out, H, V, scale, norm_w,
                                                      (bf16_t*)raw, ssq);
  else
    return LLM_ERR_ARG;
  return llm_launch_status();
}

// ---------------------------------------------------------------------------------- add + RMS norm
// For output row b (input row r = rows ? rows[b] : b):
//   x = res[r] + delta[r] (stored back into res when delta is given)
//   out[b] = x * w * 1/sqrt(mean(x^2) + eps)         (src/flint/cuda/rms_norm.cu:45-76)
template <typename TD, typename TO, int NT>
__global__ void add_rmsnorm_kernel(float* __restrict__ res, const TD* __restrict__ delta, int n_delta,
                                   size_t delta_stride, const float* __restrict__ w, float eps,
                                   TO* __restrict__ out, const int* __restrict__ rows, int H) {
  __shared__ float scratch[NT / 64];
  const int b = blockIdx.x;
  const int r = rows ? rows[b] : b;
  float* x = res + (size_t)r * H;
  const TD* d = delta ? delta + (size_t)r * H : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += NT) {
    float v = x[i];
    if (d) {
      for (int j = 0; j < n_delta; ++j) v += Conv<TD>::load(d + j * delta_stride + i);   // in this order
      x[i] = v;
    }
    ss += v * v;
  }
  ss = block_sum<NT>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)b * H;
  for (int i = threadIdx.x; i < H; i += NT) Conv<TO>::store(o + i, x[i] * w[i] * inv);
}

// The same for rows of up to NT * 4 * NV elements (a multiple of 4): a thread keeps its share of
// the row in registers, so the row, the delta and the weight are each read once and all loads are
// in flight together.
template <typename TD, typename TO, int NT, int NV>
__global__ __launch_bounds__(NT) void add_rmsnorm_reg_kernel(float* __restrict__ res,
                                                              const TD* __restrict__ delta, int n_delta,
                                                              size_t delta_stride,
                                                              const float* __restrict__ w, float eps,
                                                              TO* __restrict__ out,
                                                              const int* __restrict__ rows, int H) {
  __shared__ float scratch[NT / 64];
  const int b = blockIdx.x;
  const int r = rows ? rows[b] : b;
  float* x = res + (size_t)r * H;
  const TD* d = delta ? delta + (size_t)r * H : nullptr;
  float4 v[NV], wv[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * NT) * 4;
    const bool in = i < H;
    v[j] = in ? *reinterpret_cast<const float4*>(x + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    wv[j] = in ? *reinterpret_cast<const float4*>(w + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    if (d && in) {
      // several deltas are added in this order; eight are asked for before the first is added, so
      // that a row waits for memory once and not once a delta
      for (int q0 = 0; q0 < n_delta; q0 += 8) {
        float4 dv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (q0 + u < n_delta) dv[u] = Conv4<TD>::load(d + (size_t)(q0 + u) * delta_stride + i);
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (q0 + u < n_delta) {
            v[j].x += dv[u].x;
            v[j].y += dv[u].y;
            v[j].z += dv[u].z;
            v[j].w += dv[u].w;
          }
      }
      *reinterpret_cast<float4*>(x + i) = v[j];
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) ss += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
  ss = block_sum<NT>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)b * H;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = (threadIdx.x + j * NT) * 4;
    if (i < H)
      Conv4<TO>::store(o + i, make_float4(v[j].x * wv[j].x * inv, v[j].y * wv[j].y * inv,
                                          v[j].z * wv[j].z * inv, v[j].w * wv[j].w * inv));
  }
}

// delta: nothing, a matrix like res, or n_delta of them delta_stride elements apart, added in order.
extern "C" int llm_add_rmsnorm(float* res, const void* delta, int delta_dtype, int n_delta,
                               size_t delta_stride, const float* w, float eps, void* out, int out_dtype,
                               const int* rows, int n_out, int H, hipStream_t stream) {
  if (n_out <= 0) return LLM_OK;
  if (H <= 0 || (delta != nullptr && n_delta < 1)) return LLM_ERR_ARG;
  constexpr int NT = 256;
  // rows of up to 16,384 elements stay in registers: 8 or 16 elements a thread, and for rows
  // beyond 4,096 elements more threads rather than more registers, so that a row's loads are all
  // asked for at once (a block is all that reads a row, and a compute unit reads slowly alone)
  const bool reg = (H % 4 == 0) && H <= 1024 * 4 * 4 && delta_stride % 4 == 0 &&
                   ((((uintptr_t)res) | ((uintptr_t)w) | ((uintptr_t)delta) | ((uintptr_t)out)) & 15) == 0;
#define REG(TD, TO, THREADS, NV)                                                                            \
    add_rmsnorm_reg_kernel<TD, TO, THREADS, NV><<<n_out, THREADS, 0, stream>>>(                       \
        res, (const TD*)delta, n_delta, delta_stride, w, eps, (TO*)out, rows, H)
#define LAUNCH(TD, TO) do {                                                                         \
  if (reg && H <= NT * 4 * 2) REG(TD, TO, NT, 2);                                                           \
  else if (reg && H <= NT * 4 * 4) REG(TD, TO, NT, 4);                                                      \
  else if (reg && H <= 512 * 4 * 4) REG(TD, TO, 512, 4);                                                    \
  else if (reg) REG(TD, TO, 1024, 4);                                                                       \
  else                                                                                              \
    add_rmsnorm_kernel<TD, TO, NT><<<n_out, NT, 0, stream>>>(res, (const TD*)delta, n_delta, delta_stride, w, eps, (TO*)out, rows, H); \
  } while (0)
  if (delta == nullptr) delta_dtype = out_dtype;
  if (delta_dtype == LLM_DTYPE_F32 && out_dtype == LLM_DTYPE_F32) LAUNCH(float, float);
  else if (delta_dtype == LLM_DTYPE_BF16 && out_dtype == LLM_DTYPE_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == LLM_DTYPE_F32 && out_dtype == LLM_DTYPE_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == LLM_DTYPE_BF16 && out_dtype == LLM_DTYPE_F32) LAUNCH(bf16_t, float);
  else return LLM_ERR_ARG;
#undef LAUNCH
#undef REG
  return llm_launch_status();
}

// ---------------------------------------------------------------------------------- SiLU-mul
// out[m, i] = gu[m, i] / (1 + exp(-gu[m, i])) * gu[m, I + i]: the gate is the first half
// (src/flint/cuda/swiglu.cu:44-49); `act` chooses another activation for the gate (common.h).
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, int act) {
  const int m = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= I) return;
  const T* row = gu + (size_t)m * 2 * I;
  const float g = Conv<T>::load(row + i);
  const float u = Conv<T>::load(row + I + i);
  Conv<T>::store(out + (size_t)m * I + i, llm_gated(act, g, u));
}

// The same for bfloat16 rows whose half width is a multiple of 8: 16 bytes of gate and of up per
// thread, any number of rows through a grid-stride loop.
__device__ __forceinline__ uint4 silu_mul_8(const uint4 g4, const uint4 u4, int act) {
  const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
  uint32_t ow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
    const float r0 = llm_gated(act, g0, u0), r1 = llm_gated(act, g1, u1);
    ow[j] = (uint32_t)f32_to_bf16(r0) | ((uint32_t)f32_to_bf16(r1) << 16);
  }
  return make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

// Two vectors a thread and round (the second half a grid apart), all four loads asked for before
// the first is used.
__global__ void silu_mul_vec_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int I,
                                    size_t total_vec, int act) {
  const int per_row = I / 8;
  const size_t span = (size_t)gridDim.x * blockDim.x;
  for (size_t v = (size_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec; v += 2 * span) {
    const size_t v2 = v + span;
    const bool two = v2 < total_vec;
    const size_t m = v / per_row, m2 = two ? v2 / per_row : m;
    const int i = (int)(v % per_row) * 8, i2 = two ? (int)(v2 % per_row) * 8 : i;
    const uint4 ga = *reinterpret_cast<const uint4*>(gu + m * 2 * I + i);
    const uint4 ua = *reinterpret_cast<const uint4*>(gu + m * 2 * I + I + i);
    const uint4 gb = *reinterpret_cast<const uint4*>(gu + m2 * 2 * I + i2);
    const uint4 ub = *reinterpret_cast<const uint4*>(gu + m2 * 2 * I + I + i2);
    *reinterpret_cast<uint4*>(out + m * I + i) = silu_mul_8(ga, ua, act);
    if (two) *reinterpret_cast<uint4*>(out + m2 * I + i2) = silu_mul_8(gb, ub, act);
  }
}

extern "C" int llm_silu_mul(const void* gu, void* out, int dtype, int M, int I, int act, hipStream_t stream) {
  if (M <= 0) return LLM_OK;
  if (I <= 0 || M > 65535 * 32 || act < 0 || act >= LLM_ACT_COUNT) return LLM_ERR_ARG;
  if (dtype == LLM_DTYPE_BF16 && I % 8 == 0 && ((((uintptr_t)gu) | ((uintptr_t)out)) & 15) == 0) {
    const size_t total_vec = (size_t)M * (I / 8);
    size_t blocks = (total_vec + 511) / 512;                      // two vectors a thread and round
    // no more than three blocks a compute unit, each going round several times: what the grid
    // touches at one moment then lies closer together in memory, and a long array streams a
    // sixth faster than with a block for every 512 vectors (6.4 against 5.4 TB/s when only read)
    const size_t cap = (size_t)llm_compute_units() * 3;
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    silu_mul_vec_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total_vec, act);
    return llm_launch_status();
  }
  // grid.y is limited to 65535: fold larger M into several launches
  for (int m0 = 0; m0 < M; m0 += 65535) {
    const int mm = (M - m0 < 65535) ? (M - m0) : 65535;
    dim3 grid((I + 255) / 256, mm);
    if (dtype == LLM_DTYPE_F32)
      silu_mul_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu + (size_t)m0 * 2 * I,
                                                        (float*)out + (size_t)m0 * I, I, act);
    else if (dtype == LLM_DTYPE_BF16)
      silu_mul_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu + (size_t)m0 * 2 * I,
                                                         (bf16_t*)out + (size_t)m0 * I, I, act);
    else
      return LLM_ERR_ARG;
  }
  return llm_launch_status();
}

// ---------------------------------------------------------------------------------- bias add
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const float* __restrict__ b, size_t total, int N) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < total; i += stride) Conv<T>::store(x + i, Conv<T>::load(x + i) + b[i % N]);
}

extern "C" int llm_add_bias(void* x, int dtype, const float* b, int M, int N, hipStream_t stream) {
  if (M <= 0) return LLM_OK;
  if (N <= 0) return LLM_ERR_ARG;
  const size_t total = (size_t)M * N;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 8192) blocks = 8192;
  if (dtype == LLM_DTYPE_F32) add_bias_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, b, total, N);
  else if (dtype == LLM_DTYPE_BF16) add_bias_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, b, total, N);
  else return LLM_ERR_ARG;
  return llm_launch_status();
}

// ---------------------------------------------------------------------------------- rotary + cache write
// One block per token.  Row layout of qkv: [q heads | k heads | v heads], each head_dim wide.
//   q, k: o[j] = x[j] c - x[j+r/2] s,  o[j+r/2] = x[j+r/2] c + x[j] s  for j < r/2, r = rot_dim
//         (rotate-half pairing, src/libllm/llama.cc:151-176); dims >= r pass through.
//   With `adjacent` the pairs are (2j, 2j+1) instead, still with the angle of pair j: the layout of
//   a projection whose output rows were reordered so that the two dims of a pair lie side by side.
//   q is rotated in place; k (rotated) and v go to the sequence's page of the cache:
//   page = table[slot, pos / PAGE], laid out as common.h says (keys in blocks of 16 dims, values
//   in halves of 32 positions).
template <typename T, int PAGE>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int row_stride, const float* __restrict__ bias,
                                     int n_heads, int n_kv, int hd, const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t, int rot_dim,
                                     const int* __restrict__ tok_pos, const int* __restrict__ tok_seq,
                                     const int* __restrict__ seq_slot, const int* __restrict__ table,
                                     int table_stride, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     int write_kv, int adjacent) {
  const int m = blockIdx.x;
  const int pos = tok_pos[m];
  T* row = qkv + (size_t)m * row_stride;
  const int half = rot_dim / 2;
  const int pass = hd - rot_dim;                 // dims that do not rotate
  const int per_head = half + pass;              // work items per rotating head
  const int n_rot_heads = n_heads + (write_kv ? n_kv : 0);
  size_t page_heads = 0;                         // (page, kv head 0) counted in kv heads
  if (write_kv) {
    const int slot = seq_slot[tok_seq[m]];
    page_heads = (size_t)table[(size_t)slot * table_stride + pos / PAGE] * n_kv;
  }
  const int in_page = pos % PAGE;
  const float* c = cos_t + (size_t)pos * half;
  const float* s = sin_t + (size_t)pos * half;
  const int rot_items = n_rot_heads * per_head;
  for (int it = threadIdx.x; it < rot_items; it += blockDim.x) {
    const int h = it / per_head;
    const int j = it % per_head;
    T* x = row + (size_t)h * hd;
    const float* b = bias ? bias + (size_t)h * hd : nullptr;
    const bool is_k = h >= n_heads;
    T* kdst = k_pages + (page_heads + (size_t)(is_k ? h - n_heads : 0)) * llm_key_block(hd);
    if (j < half) {
      const int d1 = adjacent ? 2 * j : j, d2 = adjacent ? 2 * j + 1 : j + half;
      float x1 = Conv<T>::load(x + d1), x2 = Conv<T>::load(x + d2);
      if (b) { x1 += b[d1]; x2 += b[d2]; }
      const float cj = c[j], sj = s[j];
      Conv<T>::store(is_k ? kdst + llm_key_offset(in_page, d1) : x + d1, x1 * cj - x2 * sj);
      Conv<T>::store(is_k ? kdst + llm_key_offset(in_page, d2) : x + d2, x2 * cj + x1 * sj);
    } else {
      const int d = rot_dim + (j - half);
      float v = Conv<T>::load(x + d);
      if (b) v += b[d];
      Conv<T>::store(is_k ? kdst + llm_key_offset(in_page, d) : x + d, v);
    }
  }
  if (write_kv) {
    const T* vrow = row + (size_t)(n_heads + n_kv) * hd;
    const float* b = bias ? bias + (size_t)(n_heads + n_kv) * hd : nullptr;
    for (int it = threadIdx.x; it < n_kv * hd; it += blockDim.x) {
      const int h = it / hd, d = it % hd;
      float v = Conv<T>::load(vrow + it);
      if (b) v += b[it];
      Conv<T>::store(v_pages + (page_heads + h) * llm_value_block(hd) + llm_value_offset(hd, d, in_page), v);
    }
  }
}

// The same for bfloat16 with neighbouring pairs, a tile of 64 rows and one head per block
// (grid: row tiles x (q heads + k heads + v heads)).  q and k move as 16-byte vectors (four pairs
// and their four angles at a time).  v is transposed through LDS, so that consecutive lanes write
// consecutive positions of a page: rows of a prompt lie in order, and a wave's 64 stores of two
// bytes then fall into two half lines instead of 64 lines.  Needs hd and rot_dim in multiples of 8.
// Rows of a decode step lie in as many pages, so their values' stores are a line each whatever the
// order: for few rows a v head is dealt to v_split blocks, each with hd / v_split of its dims
// (grid: row tiles x (q heads + k heads + v heads * v_split)).
template <int PAGE>
__global__ __launch_bounds__(256) void rope_kv_write_tile_kernel(
    bf16_t* __restrict__ qkv, int row_stride, const float* __restrict__ bias, int n_heads, int n_kv, int hd,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot_dim,
    const int* __restrict__ tok_pos, const int* __restrict__ tok_seq, const int* __restrict__ seq_slot,
    const int* __restrict__ table, int table_stride, bf16_t* __restrict__ k_pages,
    bf16_t* __restrict__ v_pages, int M, int v_split) {
  extern __shared__ __attribute__((aligned(16))) unsigned char tile_raw[];
  __shared__ int s_pos[64], s_page[64];
  const int tid = threadIdx.x, m0 = blockIdx.x * 64;
  const bool is_q = (int)blockIdx.y < n_heads, is_k = !is_q && (int)blockIdx.y < n_heads + n_kv;
  // the head whose columns of a row this block takes, and for a v head which of its dims
  const int v_block = (int)blockIdx.y - n_heads - n_kv;
  const int h = (is_q || is_k) ? (int)blockIdx.y : n_heads + n_kv + v_block / v_split;
  const int dims = (is_q || is_k) ? hd : hd / v_split, d0 = (is_q || is_k) ? 0 : (v_block % v_split) * dims;
  if (tid < 64) {
    const int m = m0 + tid;
    int pos = 0, page = 0;
    if (m < M) {
      pos = tok_pos[m];
      if (!is_q) page = table[(size_t)seq_slot[tok_seq[m]] * table_stride + pos / PAGE];
    }
    s_pos[tid] = pos;
    s_page[tid] = page;
  }
  __syncthreads();
  const int vecs = hd / 8, half = rot_dim / 2;
  const float* b = bias ? bias + (size_t)h * hd : nullptr;
  if (is_q || is_k) {
    for (int it = tid; it < 64 * vecs; it += 256) {
      const int r = it / vecs, d = (it % vecs) * 8, m = m0 + r;
      if (m >= M) continue;
      bf16_t* src = qkv + (size_t)m * row_stride + (size_t)h * hd + d;
      const uint4 raw = *reinterpret_cast<const uint4*>(src);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
      float x[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[2 * e] = bf16_to_f32((bf16_t)(w[e] & 0xffffu));
        x[2 * e + 1] = bf16_to_f32((bf16_t)(w[e] >> 16));
      }
      if (b) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] += b[d + e];
      }
      const int pos = s_pos[r];
      if (d < rot_dim) {
        const float4 c4 = *reinterpret_cast<const float4*>(cos_t + (size_t)pos * half + d / 2);
        const float4 s4 = *reinterpret_cast<const float4*>(sin_t + (size_t)pos * half + d / 2);
        const float c[4] = {c4.x, c4.y, c4.z, c4.w}, sn[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float x1 = x[2 * e], x2 = x[2 * e + 1];
          x[2 * e] = x1 * c[e] - x2 * sn[e];
          x[2 * e + 1] = x2 * c[e] + x1 * sn[e];
        }
      }
      uint4 out;
      out.x = (uint32_t)f32_to_bf16(x[0]) | ((uint32_t)f32_to_bf16(x[1]) << 16);
      out.y = (uint32_t)f32_to_bf16(x[2]) | ((uint32_t)f32_to_bf16(x[3]) << 16);
      out.z = (uint32_t)f32_to_bf16(x[4]) | ((uint32_t)f32_to_bf16(x[5]) << 16);
      out.w = (uint32_t)f32_to_bf16(x[6]) | ((uint32_t)f32_to_bf16(x[7]) << 16);
      bf16_t* dst = is_q ? src
                         : k_pages + ((size_t)s_page[r] * n_kv + (h - n_heads)) * llm_key_block(hd) +
                               llm_key_offset(pos % PAGE, d);
      *reinterpret_cast<uint4*>(dst) = out;
    }
    return;
  }
  // a v head: rows of the tile into LDS (a row takes hd + 2 values, an odd number of words, so that
  // a column is read without bank conflicts), then one dim a wave at a time, a row a lane
  const int kvh = h - n_heads - n_kv;
  uint32_t* tile = reinterpret_cast<uint32_t*>(tile_raw);
  const int row_w = dims / 2 + 1;                                  // words per row of the tile
  const int vecs_v = dims / 8;
  for (int it = tid; it < 64 * vecs_v; it += 256) {
    const int r = it / vecs_v, d = (it % vecs_v) * 8, m = m0 + r;
    uint4 raw = make_uint4(0u, 0u, 0u, 0u);
    if (m < M) raw = *reinterpret_cast<const uint4*>(qkv + (size_t)m * row_stride + (size_t)h * hd + d0 + d);
    uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    if (b) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float lo = bf16_to_f32((bf16_t)(w[e] & 0xffffu)) + b[d0 + d + 2 * e];
        const float hi = bf16_to_f32((bf16_t)(w[e] >> 16)) + b[d0 + d + 2 * e + 1];
        w[e] = (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) tile[r * row_w + d / 2 + e] = w[e];
  }
  __syncthreads();
  const int lane = tid & 63, wave = tid >> 6;
  if (m0 + lane < M) {
    const int pos = s_pos[lane];
    bf16_t* dst = v_pages + ((size_t)s_page[lane] * n_kv + kvh) * llm_value_block(hd);
    for (int d = wave; d < dims; d += 4) {
      const uint32_t w = tile[lane * row_w + d / 2];
      dst[llm_value_offset(hd, d0 + d, pos % PAGE)] = (bf16_t)((d & 1) ? (w >> 16) : (w & 0xffffu));
    }
  }
}

extern "C" int llm_rope_kv_write(void* qkv, int dtype, int row_stride, const float* bias, int n_heads,
                                 int n_kv, int hd, const float* cos_t, const float* sin_t, int rot_dim,
                                 const int* tok_pos, const int* tok_seq, const int* seq_slot,
                                 const int* table, int table_stride, void* k_pages, void* v_pages,
                                 int page_size, int write_kv, int adjacent, int M,
                                 hipStream_t stream) {
  if (M <= 0) return LLM_OK;
  if (page_size != 64 || hd <= 0 || n_heads <= 0 || n_kv < 0 || rot_dim < 0 || rot_dim > hd ||
      (rot_dim & 1))
    return LLM_ERR_ARG;
  if (rot_dim > 0 && (cos_t == nullptr || sin_t == nullptr)) return LLM_ERR_ARG;
  const int width = (n_heads + (write_kv ? 2 * n_kv : 0)) * hd;
  if (row_stride < width) return LLM_ERR_ARG;
  if (write_kv && (!k_pages || !v_pages || !table || !seq_slot || !tok_seq)) return LLM_ERR_ARG;
  const bool vec_ok = dtype == LLM_DTYPE_BF16 && (adjacent || rot_dim == 0) && hd % 8 == 0 && hd <= 256 &&
                      rot_dim % 8 == 0 && row_stride % 8 == 0 && ((uintptr_t)qkv & 15) == 0 &&
                      ((uintptr_t)cos_t & 15) == 0 && ((uintptr_t)sin_t & 15) == 0 &&
                      (!write_kv || ((uintptr_t)k_pages & 15) == 0) && M >= 64;
  if (vec_ok) {
    // few rows (a decode step's, a short prompt's): more blocks for the values, see the kernel
    const int v_split = (M > 256) ? 1 : (hd % 32 == 0) ? 4 : (hd % 16 == 0) ? 2 : 1;
    const dim3 grid((M + 63) / 64, n_heads + (write_kv ? n_kv + n_kv * v_split : 0));
    const size_t lds = write_kv ? (size_t)64 * (hd / v_split / 2 + 1) * 4 : 0;
    rope_kv_write_tile_kernel<64><<<grid, 256, lds, stream>>>(
        (bf16_t*)qkv, row_stride, bias, n_heads, n_kv, hd, cos_t, sin_t, rot_dim, tok_pos, tok_seq, seq_slot,
        table, table_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, M, v_split);
    return llm_launch_status();
  }
  if (dtype == LLM_DTYPE_F32)
    rope_kv_write_kernel<float, 64><<<M, 256, 0, stream>>>(
        (float*)qkv, row_stride, bias, n_heads, n_kv, hd, cos_t, sin_t, rot_dim, tok_pos, tok_seq,
        seq_slot, table, table_stride, (float*)k_pages, (float*)v_pages, write_kv, adjacent);
  else if (dtype == LLM_DTYPE_BF16)
    rope_kv_write_kernel<bf16_t, 64><<<M, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, bias, n_heads, n_kv, hd, cos_t, sin_t, rot_dim, tok_pos, tok_seq,
        seq_slot, table, table_stride, (bf16_t*)k_pages, (bf16_t*)v_pages, write_kv, adjacent);
  else
    return LLM_ERR_ARG;
  return llm_launch_status();
}
