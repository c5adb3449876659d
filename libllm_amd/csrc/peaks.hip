// What this GPU reaches at most, measured: the denominators of the rooflines that the benchmark
// prints beside the published peaks.  A read of a long array, a copy of it, a loop of matrix-core
// instructions on registers and a loop of float32 multiply-adds.  (The reference times single
// operators with events over warm-up and timed runs, src/flint/cuda/benchmark.cc:38-53.)
#include "common.h"
#include "mfma.h"

// Every thread reads 16 bytes at a time, four loads in flight, a grid stride apart; the values are
// folded into one word a thread and written out, so that no load can be dropped.
__global__ __launch_bounds__(256) void peak_read_kernel(const uint4* __restrict__ src, size_t n16,
                                                        uint32_t* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t acc = 0;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n16; i += stride) {
    const uint4 a = src[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

// The same with the non-temporal hint on every load, as the products stream their weights.
typedef uint32_t peak_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void peak_read_stream_kernel(const peak_u32x4* __restrict__ src, size_t n16,
                                                               uint32_t* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  peak_u32x4 acc = {0u, 0u, 0u, 0u};
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const peak_u32x4 a = __builtin_nontemporal_load(src + i), b = __builtin_nontemporal_load(src + i + stride),
                     c = __builtin_nontemporal_load(src + i + 2 * stride),
                     d = __builtin_nontemporal_load(src + i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc.x ^ acc.y ^ acc.z ^ acc.w;
}

__global__ __launch_bounds__(256) void peak_copy_kernel(const uint4* __restrict__ src,
                                                        uint4* __restrict__ dst, size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    dst[i] = a;
    dst[i + stride] = b;
    dst[i + 2 * stride] = c;
    dst[i + 3 * stride] = d;
  }
  for (; i < n16; i += stride) dst[i] = src[i];
}

// Eight independent accumulators a wave, so that a matrix instruction never waits for the one
// before it; the operands are made from the thread's index and stay in registers.
__global__ __launch_bounds__(256) void peak_mfma_bf16_kernel(float* __restrict__ out, int iters) {
  Frag a, b;
  const uint32_t seed = 0x3f803f80u + (threadIdx.x & 3);          // bfloat16 values near 1
  a.u = make_uint4(seed, seed, seed, seed);
  b.u = make_uint4(seed ^ 0x00010000u, seed, seed, seed);
  f32x4 acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = mfma_bf16(a, b, acc[j]);
  }
  f32x4 s = acc[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) s += acc[j];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s[0] + s[1] + s[2] + s[3];
}

// Sixteen independent chains of float32 multiply-adds a thread.
__global__ __launch_bounds__(256) void peak_fma_f32_kernel(float* __restrict__ out, int iters) {
  float acc[16];
  const float x = 1.0f + 1e-7f * threadIdx.x, y = 1e-9f * (blockIdx.x + 1);
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = (float)j;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = fmaf(acc[j], x, y);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) s += acc[j];
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

static int peak_blocks(int per_unit) { return llm_compute_units() * per_unit; }

// sink: at least llm_peak_sink_words() 32-bit words.
extern "C" int llm_peak_sink_words() { return peak_blocks(8) * 256; }

// half_blocks_per_unit: blocks of 256 threads for every two compute units (1 to 16).  The grid's
// size decides how far apart in memory the loads of one moment lie, and with it the bandwidth: a
// block or two a unit reads a sixth faster than eight (6.4 against 5.4 TB/s on an MI355X).
// streaming: the loads carry the non-temporal hint.
extern "C" int llm_peak_read(const void* src, size_t bytes, void* sink, int half_blocks_per_unit,
                             int streaming, hipStream_t stream) {
  if (!src || !sink || bytes < 16 || (((uintptr_t)src) & 15) || half_blocks_per_unit < 1 || half_blocks_per_unit > 16)
    return LLM_ERR_ARG;
  const int blocks = (peak_blocks(half_blocks_per_unit) + 1) / 2;
  if (streaming)
    peak_read_stream_kernel<<<blocks, 256, 0, stream>>>((const peak_u32x4*)src, bytes / 16, (uint32_t*)sink);
  else
    peak_read_kernel<<<blocks, 256, 0, stream>>>((const uint4*)src, bytes / 16, (uint32_t*)sink);
  return llm_launch_status();
}

extern "C" int llm_peak_copy(const void* src, void* dst, size_t bytes, int half_blocks_per_unit,
                             hipStream_t stream) {
  if (!src || !dst || bytes < 16 || ((((uintptr_t)src) | ((uintptr_t)dst)) & 15) || half_blocks_per_unit < 1 ||
      half_blocks_per_unit > 16)
    return LLM_ERR_ARG;
  const int blocks = (peak_blocks(half_blocks_per_unit) + 1) / 2;
  peak_copy_kernel<<<blocks, 256, 0, stream>>>((const uint4*)src, (uint4*)dst, bytes / 16);
  return llm_launch_status();
}

// Runs the loop on two blocks of four waves a compute unit; returns in *flops what the launch
// computes (2 * 16 * 16 * 32 a matrix instruction), so that the caller divides by its own time.
extern "C" int llm_peak_mfma_bf16(void* sink, int iters, double* flops, hipStream_t stream) {
  if (!sink || iters <= 0 || !flops) return LLM_ERR_ARG;
  const int blocks = peak_blocks(2);
  peak_mfma_bf16_kernel<<<blocks, 256, 0, stream>>>((float*)sink, iters);
  *flops = (double)blocks * 4.0 * iters * 8.0 * (2.0 * 16 * 16 * 32);
  return llm_launch_status();
}

extern "C" int llm_peak_fma_f32(void* sink, int iters, double* flops, hipStream_t stream) {
  if (!sink || iters <= 0 || !flops) return LLM_ERR_ARG;
  const int blocks = peak_blocks(8);
  peak_fma_f32_kernel<<<blocks, 256, 0, stream>>>((float*)sink, iters);
  *flops = (double)blocks * 256.0 * iters * 16.0 * 2.0;
  return llm_launch_status();
}
