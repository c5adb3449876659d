// Shared helpers for the gfx950 kernels: storage types, conversions, wave and block reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LLM_DTYPE_F32 0
#define LLM_DTYPE_BF16 1

#define LLM_OK 0
#define LLM_ERR_ARG 1        // an argument the kernel refuses (size, dtype, alignment)
#define LLM_ERR_LAUNCH 2     // the runtime refused the launch
#define LLM_ERR_TOO_LARGE 3  // the operands exceed a fixed buffer of an entry point that allocates nothing

typedef uint16_t bf16_t;     // bfloat16 as raw bits: the upper half of an IEEE float

// Activations of a gated feed-forward, out = act(gate) * up.  An entry point with a gated epilogue
// takes the code in the upper bits of its `epilogue` argument (epilogue | act << 4); 0 is SiLU
// (src/flint/cuda/swiglu.cu:44-49).
#define LLM_ACT_SILU 0
#define LLM_ACT_GELU_TANH 1      // 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3)))
#define LLM_ACT_RELU 2
#define LLM_ACT_COUNT 3
__device__ __forceinline__ float llm_gated(int act, float g, float u) {
  if (act == LLM_ACT_GELU_TANH)
    return u * (0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))));
  if (act == LLM_ACT_RELU) return g > 0.f ? u * g : 0.f;
  return u * g / (1.0f + expf(-g));
}

// Layout of the cache's pages.  A page holds 64 positions of every kv head; per (page, kv head):
//   keys   [ceil(hd / 16)][64 positions][16 dims]   (blocks of 16 dims; a head size that is no
//                                                    multiple of 16 pads its last block)
//   values [2][hd][32 positions]                    (halves of 32 positions)
// so that the 16-byte pieces which one load instruction of the attention kernels takes (8 dims of
// each of 4 consecutive keys and their neighbours in the same block; 8 positions of each of 16
// consecutive dims) fill whole 128-byte lines: a line is then fetched by one instruction and not by
// two, and streams a seventh faster (6.9 against 6.1 TB/s for the pages of a decode step).
#define LLM_PAGE 64
__host__ __device__ inline int llm_key_block(int hd) { return ((hd + 15) / 16) * 16 * LLM_PAGE; }    // elements per (page, kv head)
__host__ __device__ inline int llm_value_block(int hd) { return hd * LLM_PAGE; }
__host__ __device__ inline size_t llm_key_offset(int pos, int d) { return (size_t)(d >> 4) * (16 * LLM_PAGE) + pos * 16 + (d & 15); }
__host__ __device__ inline size_t llm_value_offset(int hd, int d, int pos) { return (size_t)(pos >> 5) * hd * 32 + (size_t)d * 32 + (pos & 31); }

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

template <typename T> struct Conv;
template <> struct Conv<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Conv<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
};

// Four consecutive elements in one memory instruction (p aligned to four elements).
template <typename T> struct Conv4;
template <> struct Conv4<float> {
  static __device__ __forceinline__ float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ __forceinline__ void store(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Conv4<bf16_t> {
  static __device__ __forceinline__ float4 load(const bf16_t* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
  }
  static __device__ __forceinline__ void store(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
    u.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024); every thread gets the result.
// `scratch` needs NT/64 floats of shared memory; the order of additions is fixed.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) total += scratch[w];
  return total;
}

template <int NT>
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
#pragma unroll
  for (int w = 1; w < NT / 64; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

static inline int llm_launch_status() {
  return hipGetLastError() == hipSuccess ? LLM_OK : LLM_ERR_LAUNCH;
}

// Compute units of the current device, asked once (launchers weigh their grids against it).
static inline int llm_compute_units() {
  static int units = 0;
  if (units == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      units = n;
    else
      units = 256;
  }
  return units;
}
