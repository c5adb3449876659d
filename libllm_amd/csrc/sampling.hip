// Arg-max and temperature / top-k / top-p sampling over float32 logits.
//
// Order of operations as in the reference (src/libllm/generator.cc:197-214, 47-113):
// z = logits / temperature, p = softmax(z) over the whole vocabulary, the top_k largest sorted
// from the largest (ties: lower index first), the shortest prefix with sum(p) >= top_p, one draw
// r = u * sum(kept), first candidate whose running sum exceeds r.  With top_k == 0 nothing is cut
// and the draw walks the vocabulary in index order.  u comes from a counter hash of
// (seed, stream, counter).
#include <mutex>

#include "common.h"
#include "no_alloc.h"

__device__ __forceinline__ uint32_t order_key(float x) {
  uint32_t u = __float_as_uint(x);
  if (u == 0x80000000u) u = 0u;                          // -0 and +0 are one value: ties go by index
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

// The same without scratch arrays from the caller (see no_alloc.h): the partial results live in a
// file-scope device array.  In host code the array's name stands for the symbol, not for device
// memory: its address on a device comes from hipGetSymbolAddress, once per device, and only that
// pointer goes to kernels.
static __device__ __align__(256) unsigned char argmax_static_scratch[LLM_ARGMAX_STATIC_BYTES];

#define LLM_MAX_DEVICES 64
static void* argmax_static_ptr[LLM_MAX_DEVICES];      // per device: each GPU has its own copy of the array
static std::mutex argmax_static_lock;

// The array's address on the current device; null if the runtime refuses.
static void* argmax_static_address() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= LLM_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> guard(argmax_static_lock);
  if (argmax_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(argmax_static_scratch)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    argmax_static_ptr[dev] = p;
  }
  return argmax_static_ptr[dev];
}

extern "C" int llm_argmax_static_init(void) {
  return argmax_static_address() != nullptr ? LLM_OK : LLM_ERR_LAUNCH;
}

extern "C" int llm_argmax_static_max_rows(int V) {
  if (V <= 0) return 0;
  const int rows = LLM_ARGMAX_STATIC_ENTRIES / llm_argmax_parts(V);
  return rows > 65535 ? 65535 : rows;
}

extern "C" int llm_argmax_static(const float* logits, int* out, int R, int V, hipStream_t stream) {
  if (R <= 0) return LLM_OK;
  if (V <= 0 || !logits || !out) return LLM_ERR_ARG;
  if (R > llm_argmax_static_max_rows(V)) return LLM_ERR_TOO_LARGE;
  void* base = argmax_static_address();
  if (base == nullptr) return LLM_ERR_LAUNCH;
  float* part_val = (float*)base;
  int* part_idx = (int*)((unsigned char*)base + (size_t)LLM_ARGMAX_STATIC_ENTRIES * sizeof(float));
  return llm_argmax(logits, out, part_val, part_idx, R, V, stream);
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

// The radix-selection step over a histogram of 256 bins: the bin in which the `need`-th largest
// key lies, and how many keys of that bin are still needed.  Threads 0..255 take part (the block
// has at least 256); bins are scanned from 255 down by a parallel prefix sum.  `wsum` needs 4
// entries.  All threads of the block must call it; the results are in sh_bin / sh_rest after it.
__device__ __forceinline__ void select_bin(const unsigned int* hist, unsigned need, unsigned* wsum,
                                           unsigned* sh_bin, unsigned* sh_rest) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  unsigned v = 0, inc = 0;
  if (tid < 256) {
    v = hist[255 - tid];
    inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned o = __shfl_up(inc, off, 64);
      if (lane >= off) inc += o;
    }
    if (lane == 63) wsum[wave] = inc;
  }
  __syncthreads();
  if (tid < 256) {
    unsigned before = 0;
    for (int w = 0; w < wave; ++w) before += wsum[w];
    inc += before;
    // the first bin (from the top) at which the running count reaches `need`; if the counts never
    // reach it (cannot happen when need <= number of keys) the lowest bin takes the rest
    const bool here = (inc >= need && inc - v < need) || (tid == 255 && inc < need);
    if (here) {
      *sh_bin = 255u - (unsigned)tid;
      *sh_rest = need - (inc - v);
    }
  }
  __syncthreads();
}

// Sampling in two stages, so that one row still uses many compute units.
//
// Stage 1, grid (parts, rows): a block owns a contiguous slice of at most SP_PER logits.  It
// writes the slice's maximum of z and its sum of exp(z - maximum), and, with top_k > 0, the
// slice's min(top_k, size) largest logits as 64-bit keys (order key << 32 | ~index: a larger key
// is a larger logit or, between equal logits, a lower index), found by radix selection over the
// slice held in shared memory.
// Stage 2, one block a row: the normaliser from the parts; with top_k > 0 the top_k largest of all
// candidate keys by radix selection over the 64-bit keys (they are distinct, so no ties remain),
// sorted, then nucleus and draw sequentially; with top_k == 0 the part and then the element at
// which the running sum in index order passes u * Z.
#define SP_PER 4096          // most logits of a stage-1 slice
#define SP_NT 512            // threads of a stage-1 block
#define SP_KMAX 1024         // most candidates kept

struct SampleParts {
  float* part_max;            // [rows, parts]
  float* part_sum;            // [rows, parts]
  unsigned long long* cand;   // [rows, parts, k_part]
};

__global__ __launch_bounds__(SP_NT) void sample_part_kernel(const float* __restrict__ logits, int V,
                                                             int per, float inv_temp, int k_part,
                                                             SampleParts out) {
  __shared__ float vals[SP_PER];
  __shared__ float fbuf[SP_NT / 64];
  __shared__ int ibuf[SP_NT / 64];
  __shared__ unsigned int hist[256], wsum[4];
  __shared__ unsigned int sh_prefix, sh_need, sh_count, sh_bin, sh_rest, sh_all;
  const int part = blockIdx.x, row = blockIdx.y, parts = gridDim.x, tid = threadIdx.x;
  const int lo = part * per;
  const int n = min(per, V - lo);                       // >= 1 by the choice of parts
  const float* x = logits + (size_t)row * V + lo;
  float mx = -INFINITY;
  for (int i = tid; i < n; i += SP_NT) {
    const float v = x[i];
    vals[i] = v;
    mx = fmaxf(mx, v * inv_temp);
  }
  mx = block_max<SP_NT>(mx, fbuf);                      // also orders the writes to vals
  float sum = 0.f;
  for (int i = tid; i < n; i += SP_NT) sum += expf(vals[i] * inv_temp - mx);
  sum = block_sum<SP_NT>(sum, fbuf);
  if (tid == 0) {
    out.part_max[row * parts + part] = mx;
    out.part_sum[row * parts + part] = sum;
  }
  if (k_part <= 0) return;
  unsigned long long* cand = out.cand + ((size_t)row * parts + part) * k_part;
  const int k = min(k_part, n);
  for (int i = k + tid; i < k_part; i += SP_NT) cand[i] = 0ull;       // a short slice: empty places

  // ---- the k-th largest key of the slice by radix selection, 8 bits a pass
  if (tid == 0) { sh_prefix = 0; sh_need = (unsigned)k; }
  __syncthreads();
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int b = tid; b < 256; b += SP_NT) hist[b] = 0;
    __syncthreads();
    const unsigned prefix = sh_prefix;
    for (int i = tid; i < n; i += SP_NT) {
      const uint32_t key = order_key(vals[i]);
      if (pass == 0 || (key >> (shift + 8)) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    select_bin(hist, sh_need, wsum, &sh_bin, &sh_rest);
    if (tid == 0) {
      // every key of the chosen bin is wanted: the bins below need not be told apart.  All keys
      // from the bin's lowest on are taken then, none by its index.
      const unsigned low = ((prefix << 8) | sh_bin) << shift;
      sh_all = (sh_rest == hist[sh_bin] && low > 0u && pass < 3);
      sh_need = sh_all ? 0u : sh_rest;
      sh_prefix = sh_all ? low - 1u : ((prefix << 8) | sh_bin);
    }
    __syncthreads();
    if (sh_all) break;
  }
  const uint32_t kth = sh_prefix;
  const int need_eq = (int)sh_need;          // how many logits equal to the k-th are taken: the lowest indices
  const int n_gt = k - need_eq;
  if (tid == 0) sh_count = 0;
  __syncthreads();
  // contiguous chunks per thread, so that equal keys are ranked by index
  const int chunk = (n + SP_NT - 1) / SP_NT;
  const int c0 = min(n, tid * chunk), c1 = min(n, c0 + chunk);
  int eq_mine = 0;
  for (int i = c0; i < c1; ++i) {
    const uint32_t key = order_key(vals[i]);
    if (key > kth) {
      const unsigned p = atomicAdd(&sh_count, 1u);
      cand[p] = ((unsigned long long)key << 32) | (0xffffffffu - (uint32_t)(lo + i));
    } else if (key == kth) {
      ++eq_mine;
    }
  }
  int eq_total;
  const int eq_inc = block_inclusive_scan<int, SP_NT>(eq_mine, ibuf, &eq_total);
  int rank = eq_inc - eq_mine;
  if (eq_mine > 0 && rank < need_eq) {
    for (int i = c0; i < c1 && rank < need_eq; ++i) {
      if (order_key(vals[i]) == kth) {
        cand[n_gt + rank] = ((unsigned long long)kth << 32) | (0xffffffffu - (uint32_t)(lo + i));
        ++rank;
      }
    }
  }
}

template <int NT>
__global__ __launch_bounds__(NT) void sample_final_kernel(const float* __restrict__ logits, int V,
                                                           int per, int parts, float inv_temp,
                                                           int top_k, int k_part, float top_p,
                                                           uint64_t seed,
                                                           const long long* __restrict__ streams,
                                                           const long long* __restrict__ counters,
                                                           SampleParts in, int* __restrict__ out,
                                                           int open_ended) {
  __shared__ float fbuf[NT / 64];
  __shared__ unsigned int hist[256], wsum[4];
  __shared__ unsigned long long cand[SP_KMAX];
  __shared__ unsigned long long sh_prefix;
  __shared__ unsigned int sh_need, sh_count, sh_bin, sh_rest, sh_all;
  __shared__ int sh_result, sh_part;
  __shared__ float sh_before;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)row * V;
  const float u = counter_uniform(seed, (uint64_t)streams[row], (uint64_t)counters[row]);
  const float* pm = in.part_max + (size_t)row * parts;
  const float* ps = in.part_sum + (size_t)row * parts;

  // the row's maximum and normaliser from the parts, in part order
  float mx = -INFINITY;
  for (int p = 0; p < parts; ++p) mx = fmaxf(mx, pm[p]);
  float Z = 0.f;
  for (int p = 0; p < parts; ++p) Z += ps[p] * expf(pm[p] - mx);

  if (top_k <= 0) {
    // nothing is cut: the part, then the element, where the running sum passes r
    const float r = u * Z;
    if (tid == 0) {
      float run = 0.f;
      int p = 0;
      for (; p < parts - 1; ++p) {
        const float next = run + ps[p] * expf(pm[p] - mx);
        if (r < next) break;
        run = next;
      }
      sh_part = p;
      sh_before = run;
    }
    __syncthreads();
    const int lo = sh_part * per;
    const int n = min(per, V - lo);
    const int chunk = (n + NT - 1) / NT;
    const int c0 = min(n, tid * chunk), c1 = min(n, c0 + chunk);
    float part = 0.f;
    for (int i = c0; i < c1; ++i) part += expf(x[lo + i] * inv_temp - mx);
    float total;
    const float inc = sh_before + block_inclusive_scan<float, NT>(part, fbuf, &total);
    if (tid == 0) sh_result = lo + n - 1;               // rounding left r beyond the part's end
    __syncthreads();
    const float before = inc - part;
    if (c1 > c0 && r >= before && r < inc) {
      float run = before;
      int pick = lo + c1 - 1;
      for (int i = c0; i < c1; ++i) {
        run += expf(x[lo + i] * inv_temp - mx);
        if (r < run) { pick = lo + i; break; }
      }
      sh_result = pick;
    } else if (tid == 0 && r < sh_before) {
      sh_result = lo;
    }
    __syncthreads();
    if (tid == 0) out[row] = sh_result;
    return;
  }

  // ---- the top_k largest candidate keys: radix selection over 64 bits, 8 bits a pass
  const unsigned long long* all = in.cand + (size_t)row * parts * k_part;
  const int C = parts * k_part;
  if (tid == 0) { sh_prefix = 0ull; sh_need = (unsigned)top_k; }
  __syncthreads();
  for (int pass = 0; pass < 8; ++pass) {
    const int shift = 56 - 8 * pass;
    for (int b = tid; b < 256; b += NT) hist[b] = 0;
    __syncthreads();
    const unsigned long long prefix = sh_prefix;
    for (int i = tid; i < C; i += NT) {
      const unsigned long long key = all[i];
      if (pass == 0 || (key >> (shift + 8)) == prefix) atomicAdd(&hist[(unsigned)(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    select_bin(hist, sh_need, wsum, &sh_bin, &sh_rest);
    if (tid == 0) {
      // every key of the chosen bin is wanted: the bin's lowest possible key is the bound
      sh_all = (sh_rest == hist[sh_bin] && pass < 7);
      sh_need = sh_rest;
      sh_prefix = ((prefix << 8) | (unsigned long long)sh_bin) << (sh_all ? shift : 0);
    }
    __syncthreads();
    if (sh_all) break;
  }
  const unsigned long long kth = sh_prefix;             // the top_k-th largest key, or a bound just below it; keys are distinct
  if (tid == 0) sh_count = 0;
  for (int i = tid; i < SP_KMAX; i += NT) cand[i] = 0ull;
  __syncthreads();
  for (int i = tid; i < C; i += NT) {
    const unsigned long long key = all[i];
    if (key >= kth && key != 0ull) {
      const unsigned p = atomicAdd(&sh_count, 1u);
      if (p < (unsigned)SP_KMAX) cand[p] = key;
    }
  }
  __syncthreads();

  // ---- sort the candidates, largest first (bitonic over the next power of two)
  int P = 1;
  while (P < top_k) P <<= 1;
  for (int k = 2; k <= P; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < P; t += NT) {
        const int other = t ^ j;
        if (other > t) {
          const unsigned long long a = cand[t], b = cand[other];
          const bool desc = (t & k) == 0;
          if (desc ? (a < b) : (a > b)) { cand[t] = b; cand[other] = a; }
        }
      }
      __syncthreads();
    }
  }

  // ---- nucleus and draw, sequentially in candidate order; the probabilities are fetched by all
  // threads first, so that the walk waits for memory once
  __shared__ float prob[SP_KMAX];
  for (int i = tid; i < top_k; i += NT) {
    const int idx = (int)(0xffffffffu - (uint32_t)(cand[i] & 0xffffffffull));
    prob[i] = expf(x[idx] * inv_temp - mx) / Z;
  }
  __syncthreads();
  if (tid == 0) {
    float kept = 0.f;
    int n = 0;
    for (int i = 0; i < top_k; ++i) {
      kept += prob[i];
      ++n;
      if (kept >= top_p) break;
    }
    if (open_ended && kept < top_p) {
      // no limit on the candidates was asked for, and the most probable top_k of them do not
      // reach top_p: the row is left to sample_nucleus_kernel, which walks the whole vocabulary
      out[row] = -1;
      return;
    }
    const float r = u * kept;
    float run = 0.f;
    int pick = n - 1;
    for (int i = 0; i < n; ++i) {
      run += prob[i];
      if (r < run) { pick = i; break; }
    }
    out[row] = (int)(0xffffffffu - (uint32_t)(cand[pick] & 0xffffffffull));
  }
}


// Nucleus sampling without a limit on the candidates (top_k == 0, top_p < 1) for the rows that
// sample_final_kernel has left (out[row] < 0: the SP_KMAX most probable tokens do not reach
// top_p).  One block a row.  In the order of the draw (probability falling, the lower index first
// among equals) the kept tokens are the shortest prefix whose probabilities sum to top_p or more,
// and the drawn token is the first whose running sum exceeds r = u * (sum of the kept).  Both are
// places where a running sum in that order crosses a mark, and each is found without sorting: by
// a descent over the 32-bit order key of the logit, 8 bits a pass, over histograms of probability
// instead of counts, then among the tokens of the last key (equal logits) by index.  Probabilities
// are counted in units of 2^-40 as integers, so that the sums do not depend on the order in which
// the threads add them.
#define NUC_NT 1024
#define NUC_ONE 1099511627776.0   // 2^40

struct NucleusShared {
  unsigned long long hist[256];
  unsigned long long wsum[4];
  unsigned long long above, pe, kept;
  uint32_t prefix;
  int bin, last_bin, pick, n_eq;
  int ibuf[NUC_NT / 64];
};

__device__ __forceinline__ unsigned long long nucleus_mass(float x, float inv_temp, float mx, float inv_z) {
  const float p = expf(x * inv_temp - mx) * inv_z;
  return (unsigned long long)((double)p * NUC_ONE + 0.5);
}

// The token at which the running sum, in drawing order, first reaches `target` (strict: first
// exceeds it).  Leaves its index in sh.pick and the running sum up to and including it in sh.kept.
__device__ void nucleus_cross(const float* __restrict__ x, int V, float inv_temp, float mx, float inv_z,
                              unsigned long long target, bool strict, NucleusShared& sh) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) { sh.prefix = 0u; sh.above = 0ull; sh.pe = 0ull; }
  __syncthreads();
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int b = tid; b < 256; b += NUC_NT) sh.hist[b] = 0ull;
    if (tid == 0) { sh.bin = -1; sh.last_bin = -1; }
    __syncthreads();
    const uint32_t prefix = sh.prefix;
    const unsigned long long above = sh.above;
    // a thread adds up the tokens that follow one another into the same bin before it touches
    // the histogram: the first passes have few bins, which all threads would crowd
    int cur = -1;
    unsigned long long acc = 0ull;
    for (int i = tid; i < V; i += NUC_NT) {
      const float v = x[i];
      const uint32_t key = order_key(v);
      if (pass != 0 && (key >> (shift + 8)) != prefix) continue;
      const int b = (int)((key >> shift) & 255u);
      if (b != cur) {
        if (acc) atomicAdd(&sh.hist[cur], acc);
        cur = b;
        acc = 0ull;
      }
      acc += nucleus_mass(v, inv_temp, mx, inv_z);
    }
    if (acc) atomicAdd(&sh.hist[cur], acc);
    __syncthreads();
    // bins from the top: inclusive running sums by threads 0..255
    unsigned long long v = 0ull, inc = 0ull;
    if (tid < 256) {
      v = sh.hist[255 - tid];
      inc = v;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long o = __shfl_up(inc, off, 64);
        if (lane >= off) inc += o;
      }
      if (lane == 63) sh.wsum[wave] = inc;
    }
    __syncthreads();
    if (tid < 256) {
      for (int w = 0; w < wave; ++w) inc += sh.wsum[w];
      const unsigned long long run = above + inc, before = run - v;
      const bool crossed = strict ? run > target : run >= target;
      const bool crossed_before = strict ? before > target : before >= target;
      if (v != 0ull && crossed && !crossed_before) sh.bin = 255 - tid;
      if (v != 0ull) atomicMax(&sh.last_bin, tid);           // the lowest bin that holds anything
    }
    __syncthreads();
    if (tid == 0) {
      // rounding may leave the whole sum short of the mark: the last token that has any
      // probability then ends the walk
      const int bin = sh.bin >= 0 ? sh.bin : (sh.last_bin >= 0 ? 255 - sh.last_bin : 0);
      unsigned long long skipped = 0ull;
      for (int b = 255; b > bin; --b) skipped += sh.hist[b];
      sh.above = above + skipped;
      sh.prefix = (prefix << 8) | (uint32_t)bin;
    }
    __syncthreads();
  }
  // the tokens whose key is the one found have equal logits and so equal probabilities: the
  // c-th of them by index is the place
  const uint32_t kth = sh.prefix;
  const int chunk = (V + NUC_NT - 1) / NUC_NT;
  const int c0 = min(V, tid * chunk), c1 = min(V, c0 + chunk);
  int eq_mine = 0;
  float eq_val = 0.f;
  for (int i = c0; i < c1; ++i)
    if (order_key(x[i]) == kth) { ++eq_mine; eq_val = x[i]; }
  int eq_total;
  const int eq_inc = block_inclusive_scan<int, NUC_NT>(eq_mine, sh.ibuf, &eq_total);
  if (eq_mine > 0 && eq_inc == eq_mine) sh.pe = nucleus_mass(eq_val, inv_temp, mx, inv_z);   // the first thread that has one
  // (the descent may end on a key that no token has, when every probability rounds to nothing or
  // the logits are not finite: then nobody writes the place, and it is token 0 with nothing kept
  // beyond what lies above)
  if (tid == 0) { sh.n_eq = eq_total; sh.pick = 0; sh.kept = sh.above; }
  __syncthreads();
  const unsigned long long pe = sh.pe, above = sh.above;
  long long c = 1;
  if (pe > 0ull && target >= above) {
    const unsigned long long gap = target - above;
    c = strict ? (long long)(gap / pe) + 1 : (long long)((gap + pe - 1) / pe);
  }
  if (c < 1) c = 1;
  if (c > eq_total) c = eq_total;
  const int rank0 = eq_inc - eq_mine;                        // equals before this thread's chunk
  if (eq_mine > 0 && c > rank0 && c <= eq_inc) {
    int rank = rank0;
    for (int i = c0; i < c1; ++i)
      if (order_key(x[i]) == kth && ++rank == c) { sh.pick = i; break; }
    sh.kept = above + (unsigned long long)c * pe;
  }
  __syncthreads();
}

__global__ __launch_bounds__(NUC_NT) void sample_nucleus_kernel(const float* __restrict__ logits, int V,
                                                               int parts, float inv_temp, float top_p,
                                                               uint64_t seed,
                                                               const long long* __restrict__ streams,
                                                               const long long* __restrict__ counters,
                                                               SampleParts in, int* __restrict__ out) {
  __shared__ NucleusShared sh;
  const int row = blockIdx.x;
  if (out[row] >= 0) return;                                 // decided among the most probable tokens
  const float* x = logits + (size_t)row * V;
  const float* pm = in.part_max + (size_t)row * parts;
  const float* ps = in.part_sum + (size_t)row * parts;
  float mx = -INFINITY;
  for (int p = 0; p < parts; ++p) mx = fmaxf(mx, pm[p]);
  float Z = 0.f;
  for (int p = 0; p < parts; ++p) Z += ps[p] * expf(pm[p] - mx);
  const float inv_z = 1.0f / Z;
  const double u = (double)counter_uniform(seed, (uint64_t)streams[row], (uint64_t)counters[row]);
  nucleus_cross(x, V, inv_temp, mx, inv_z, (unsigned long long)((double)top_p * NUC_ONE), false, sh);
  const unsigned long long kept = sh.kept;
  __syncthreads();
  nucleus_cross(x, V, inv_temp, mx, inv_z, (unsigned long long)(u * (double)kept), true, sh);
  if (threadIdx.x == 0) out[row] = sh.pick;
}

// Parts a row of V logits is cut into, and candidates kept per part: the scratch arrays hold
// rows * parts floats each and rows * parts * k_part keys.
extern "C" int llm_sample_parts(int V) {
  const int parts = (V + SP_PER - 1) / SP_PER;
  return parts < 1 ? 1 : parts;
}

extern "C" int llm_sample_k_part(int V, int top_k) {
  if (top_k <= 0) return 0;
  const int parts = llm_sample_parts(V);
  const int per = (V + parts - 1) / parts;
  return top_k < per ? top_k : per;
}

extern "C" int llm_sample(const float* logits, int* out, int R, int V, float temperature, int top_k,
                          float top_p, unsigned long long seed, const long long* streams,
                          const long long* counters, float* part_max, float* part_sum,
                          unsigned long long* cand, hipStream_t stream) {
  if (R <= 0) return LLM_OK;
  if (V <= 0 || R > 65535 || !(temperature > 0.f) || top_k < 0 || top_k > SP_KMAX || top_k > V ||
      !(top_p > 0.f && top_p <= 1.f) || !part_max || !part_sum)
    return LLM_ERR_ARG;
  // top_k == 0 with top_p < 1: a nucleus with no limit on the candidates.  The SP_KMAX most
  // probable tokens are tried first (nearly always they hold the nucleus); a row in which they
  // do not reach top_p is then done by the kernel that walks the whole vocabulary.
  const bool open_ended = top_k == 0 && top_p < 1.f;
  if (open_ended) top_k = V < SP_KMAX ? V : SP_KMAX;
  if (top_k > 0 && !cand) return LLM_ERR_ARG;
  const int parts = llm_sample_parts(V);
  if (parts > 65535) return LLM_ERR_ARG;
  const int per = (V + parts - 1) / parts;
  const int k_part = llm_sample_k_part(V, top_k);
  SampleParts sp{part_max, part_sum, cand};
  const float inv_temp = 1.0f / temperature;
  sample_part_kernel<<<dim3(parts, R), SP_NT, 0, stream>>>(logits, V, per, inv_temp, k_part, sp);
  if (hipGetLastError() != hipSuccess) return LLM_ERR_LAUNCH;
  sample_final_kernel<1024><<<R, 1024, 0, stream>>>(logits, V, per, parts, inv_temp, top_k, k_part,
                                                    top_p, (uint64_t)seed, streams, counters, sp, out,
                                                    open_ended && top_k < V ? 1 : 0);
  if (open_ended && top_k < V) {
    if (hipGetLastError() != hipSuccess) return LLM_ERR_LAUNCH;
    sample_nucleus_kernel<<<R, NUC_NT, 0, stream>>>(logits, V, parts, inv_temp, top_p, (uint64_t)seed,
                                                    streams, counters, sp, out);
  }
  return llm_launch_status();
}
