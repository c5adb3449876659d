// Arg-max and temperature / top-k / top-p sampling over float32 logits, one block per row.
//
// Order of operations as in the reference (src/libllm/generator.cc:197-214, 47-113):
// z = logits / temperature, p = softmax(z) over the whole vocabulary, the top_k largest sorted
// from the largest (ties: lower index first), the shortest prefix with sum(p) >= top_p, one draw
// r = u * sum(kept), first candidate whose running sum exceeds r.  With top_k == 0 nothing is cut
// and the draw walks the vocabulary in index order.  u comes from a counter hash of
// (seed, stream, counter).
#include "common.h"

__device__ __forceinline__ uint32_t order_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);     // larger float -> larger key
}

__device__ __forceinline__ float counter_uniform(uint64_t seed, uint64_t stream, uint64_t counter) {
  uint64_t x = seed * 0x9E3779B97F4A7C15ull + stream * 0xBF58476D1CE4E5B9ull +
               counter * 0x94D049BB133111EBull + 0x2545F4914F6CDD1Dull;
  x ^= x >> 30;
  x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27;
  x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  return (float)(x >> 40) * (1.0f / 16777216.0f);
}

// ---------------------------------------------------------------------------------- arg-max
// The largest logit of a row, the lowest index winning a tie (the reference's top_k == 1 case,
// src/flint/cuda/test.cc:385-392).  Two stages so that a few rows still fill the GPU: blocks
// (row, part) reduce a slice of the vocabulary to one (value, index) pair, then one block per row
// reduces the pairs.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
  return v > bv || (v == bv && i < bi);
}

template <int NT>
__device__ __forceinline__ void block_argmax(float& bv, int& bi, float* sv, int* si) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < NT / 64; ++w)
      if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
  }
}

template <int NT>
__global__ __launch_bounds__(NT) void argmax_part_kernel(const float* __restrict__ logits, int V,
                                                          int per_part, float* __restrict__ pv,
                                                          int* __restrict__ pi) {
  __shared__ float sv[NT / 64];
  __shared__ int si[NT / 64];
  const float* x = logits + (size_t)blockIdx.y * V;
  const int lo = blockIdx.x * per_part;
  const int hi = min(V, lo + per_part);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += NT) {
    const float v = x[i];
    if (v > bv || (bi == 0x7fffffff && v == bv)) { bv = v; bi = i; }   // a thread's indices only grow
  }
  block_argmax<NT>(bv, bi, sv, si);
  if (threadIdx.x == 0) {
    pv[blockIdx.y * gridDim.x + blockIdx.x] = bv;
    pi[blockIdx.y * gridDim.x + blockIdx.x] = bi;
  }
}

template <int NT>
__global__ __launch_bounds__(NT) void argmax_final_kernel(const float* __restrict__ pv,
                                                           const int* __restrict__ pi, int parts,
                                                           int* __restrict__ out) {
  __shared__ float sv[NT / 64];
  __shared__ int si[NT / 64];
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int p = threadIdx.x; p < parts; p += NT) {
    const float v = pv[blockIdx.x * parts + p];
    const int i = pi[blockIdx.x * parts + p];
    if (better(v, i, bv, bi)) { bv = v; bi = i; }
  }
  block_argmax<NT>(bv, bi, sv, si);
  if (threadIdx.x == 0) out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
}

// How many parts a row of V logits is cut into; the scratch arrays hold R * parts entries.
extern "C" int llm_argmax_parts(int V) {
  int parts = (V + 2047) / 2048;
  return parts < 1 ? 1 : (parts > 256 ? 256 : parts);
}

extern "C" int llm_argmax(const float* logits, int* out, float* part_val, int* part_idx, int R, int V,
                          hipStream_t stream) {
  if (R <= 0) return LLM_OK;
  if (V <= 0 || R > 65535 || !part_val || !part_idx) return LLM_ERR_ARG;
  const int parts = llm_argmax_parts(V);
  const int per_part = (V + parts - 1) / parts;
  argmax_part_kernel<256><<<dim3(parts, R), 256, 0, stream>>>(logits, V, per_part, part_val, part_idx);
  if (hipGetLastError() != hipSuccess) return LLM_ERR_LAUNCH;
  argmax_final_kernel<64><<<R, 64, 0, stream>>>(part_val, part_idx, parts, out);
  return llm_launch_status();
}

// ---------------------------------------------------------------------------------- sampling
// Inclusive scan over the block in thread order; returns this thread's inclusive value and, through
// `total`, the sum over the block.  `buf` needs NT/64 elements.
template <typename T, int NT>
__device__ __forceinline__ T block_inclusive_scan(T v, T* buf, T* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const T o = __shfl_up(v, off, 64);
    if (lane >= off) v += o;
  }
  __syncthreads();
  if (lane == 63) buf[wave] = v;
  __syncthreads();
  T before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) {
    const T t = buf[w];
    if (w < wave) before += t;
    all += t;
  }
  *total = all;
  return v + before;
}

template <int NT, int KMAX>
__global__ __launch_bounds__(NT) void sample_kernel(const float* __restrict__ logits, int V,
                                                     float inv_temp, int top_k, float top_p,
                                                     uint64_t seed, const long long* __restrict__ streams,
                                                     const long long* __restrict__ counters,
                                                     int* __restrict__ out) {
  __shared__ float fbuf[NT / 64];
  __shared__ int ibuf[NT / 64];
  __shared__ unsigned int hist[256];
  __shared__ unsigned long long cand[KMAX];
  __shared__ unsigned int sh_prefix, sh_need, sh_count;
  __shared__ int sh_result;

  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * V;
  const float u = counter_uniform(seed, (uint64_t)streams[row], (uint64_t)counters[row]);

  // max and normaliser of softmax(z), z = x * inv_temp
  float mx = -INFINITY;
  for (int i = tid; i < V; i += NT) mx = fmaxf(mx, x[i] * inv_temp);
  mx = block_max<NT>(mx, fbuf);

  const int chunk = (V + NT - 1) / NT;
  const int c0 = min(V, tid * chunk), c1 = min(V, c0 + chunk);
  float part = 0.f;
  for (int i = c0; i < c1; ++i) part += expf(x[i] * inv_temp - mx);
  float Z;
  const float inc = block_inclusive_scan<float, NT>(part, fbuf, &Z);

  if (tid == 0) sh_result = V - 1;
  __syncthreads();

  if (top_k <= 0) {
    // nothing is cut: walk the vocabulary in index order
    const float r = u * Z;
    const float lo = inc - part;          // running sum before this thread's chunk
    if (c1 > c0 && r >= lo && r < inc) {
      float run = lo;
      int pick = c1 - 1;
      for (int i = c0; i < c1; ++i) {
        run += expf(x[i] * inv_temp - mx);
        if (r < run) { pick = i; break; }
      }
      sh_result = pick;
    }
    __syncthreads();
    if (tid == 0) out[row] = sh_result;
    return;
  }

  // ---- the top_k-th largest key by radix selection, 8 bits a pass
  if (tid == 0) { sh_prefix = 0; sh_need = (unsigned)top_k; }
  __syncthreads();
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int b = tid; b < 256; b += NT) hist[b] = 0;
    __syncthreads();
    const unsigned prefix = sh_prefix;
    for (int i = tid; i < V; i += NT) {
      const uint32_t key = order_key(x[i]);
      if (pass == 0 || (key >> (shift + 8)) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      unsigned need = sh_need, cum = 0;
      int b = 255;
      for (; b > 0; --b) {
        if (cum + hist[b] >= need) break;
        cum += hist[b];
      }
      sh_need = need - cum;               // still to take inside bin b
      sh_prefix = (prefix << 8) | (unsigned)b;
    }
    __syncthreads();
  }
  const uint32_t kth = sh_prefix;         // key of the top_k-th largest logit
  const int need_eq = (int)sh_need;       // how many logits equal to it are taken (lowest indices)
  const int n_gt = top_k - need_eq;

  // ---- collect: everything above the threshold, then the first need_eq equal ones by index
  if (tid == 0) sh_count = 0;
  for (int i = tid; i < KMAX; i += NT) cand[i] = 0ull;
  __syncthreads();
  int eq_mine = 0;
  for (int i = c0; i < c1; ++i) {
    const uint32_t key = order_key(x[i]);
    if (key > kth) {
      const unsigned p = atomicAdd(&sh_count, 1u);
      if (p < (unsigned)KMAX) cand[p] = ((unsigned long long)key << 32) | (0xffffffffu - (uint32_t)i);
    } else if (key == kth) {
      ++eq_mine;
    }
  }
  int eq_total;
  const int eq_inc = block_inclusive_scan<int, NT>(eq_mine, ibuf, &eq_total);
  int rank = eq_inc - eq_mine;
  if (eq_mine > 0 && rank < need_eq) {
    for (int i = c0; i < c1 && rank < need_eq; ++i) {
      if (order_key(x[i]) == kth) {
        cand[n_gt + rank] = ((unsigned long long)kth << 32) | (0xffffffffu - (uint32_t)i);
        ++rank;
      }
    }
  }
  __syncthreads();

  // ---- sort the candidates, largest first (bitonic over the next power of two)
  int P = 1;
  while (P < top_k) P <<= 1;
  for (int k = 2; k <= P; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      if (tid < P) {
        const int other = tid ^ j;
        if (other > tid) {
          const unsigned long long a = cand[tid], b = cand[other];
          const bool desc = (tid & k) == 0;
          if (desc ? (a < b) : (a > b)) { cand[tid] = b; cand[other] = a; }
        }
      }
      __syncthreads();
    }
  }

  // ---- nucleus and draw, sequentially in candidate order
  if (tid == 0) {
    float kept = 0.f;
    int n = 0;
    for (int i = 0; i < top_k; ++i) {
      const int idx = (int)(0xffffffffu - (uint32_t)(cand[i] & 0xffffffffull));
      kept += expf(x[idx] * inv_temp - mx) / Z;
      ++n;
      if (kept >= top_p) break;
    }
    const float r = u * kept;
    float run = 0.f;
    int pick = (int)(0xffffffffu - (uint32_t)(cand[n - 1] & 0xffffffffull));
    for (int i = 0; i < n; ++i) {
      const int idx = (int)(0xffffffffu - (uint32_t)(cand[i] & 0xffffffffull));
      run += expf(x[idx] * inv_temp - mx) / Z;
      if (r < run) { pick = idx; break; }
    }
    out[row] = pick;
  }
}

extern "C" int llm_sample(const float* logits, int* out, int R, int V, float temperature, int top_k,
                          float top_p, unsigned long long seed, const long long* streams,
                          const long long* counters, hipStream_t stream) {
  if (R <= 0) return LLM_OK;
  if (V <= 0 || !(temperature > 0.f) || top_k < 0 || top_k > 1024 || top_k > V ||
      !(top_p > 0.f && top_p <= 1.f) || (top_k == 0 && top_p < 1.f))
    return LLM_ERR_ARG;
  sample_kernel<1024, 1024><<<R, 1024, 0, stream>>>(logits, V, 1.0f / temperature, top_k, top_p,
                                                    (uint64_t)seed, streams, counters, out);
  return llm_launch_status();
}
