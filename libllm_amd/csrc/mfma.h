// Matrix-core (MFMA) fragments for gfx950, bfloat16 inputs with float32 accumulation.
//
// v_mfma_f32_16x16x32_bf16 computes C[16x16] += A[16x32] * B[32x16] per wave.  Lane l holds
//   A[i = l % 16][k = 8 * (l / 16) .. + 7]     (8 consecutive k of one row)
//   B[k = 8 * (l / 16) .. + 7][j = l % 16]     (8 consecutive k of one column)
//   C[i = 4 * (l / 16) + e][j = l % 16], e = 0..3
// Which real index a k slot stands for is free as long as A and B agree.
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

union Frag {
  uint4 u;
  bf16x8 v;
  bf16_t h[8];
};

__device__ __forceinline__ Frag frag_zero() {
  Frag f;
  f.u = make_uint4(0u, 0u, 0u, 0u);
  return f;
}

// 16 bytes from global memory (the address must be 16-byte aligned)
__device__ __forceinline__ Frag frag_load(const bf16_t* p) {
  Frag f;
  f.u = *reinterpret_cast<const uint4*>(p);
  return f;
}

// The same for data that is read once and not again soon (a weight matrix streamed through a
// product): the load carries the non-temporal hint, so the lines do not push what the other waves
// read again and again (the rows of X, tables) out of the chiplet's cache.  Whole engines compared
// in one process, the weights of the skinny product so: 0.856 against 0.900 ms a decode step at
// batch 1, 1.010 against 1.037 at batch 8, 2.65 against 2.67 at batch 64 (1B shape).  The hint
// pays only where every load instruction of a wave takes whole 128-byte lines: a wave that takes
// half a line now and the other half a few instructions later needs the near cache for the second
// half, and the hint gives that up (pages of keys and values read so were 1 to 3 % slower until
// the pages were laid out for whole-line loads; since then decode attention streams them too).
typedef uint32_t u32x4_raw __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Frag frag_load_stream(const bf16_t* p) {
  Frag f;
  const u32x4_raw v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_raw*>(p));
  f.u = make_uint4(v.x, v.y, v.z, v.w);
  return f;
}

__device__ __forceinline__ f32x4 mfma_bf16(const Frag& a, const Frag& b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
}

// Two floats rounded to bfloat16 (nearest even) by the hardware convert, packed low | high << 16.
typedef __bf16 bf16x2_hw __attribute__((ext_vector_type(2)));
typedef float f32x2_hw __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
  const f32x2_hw v = {lo, hi};
  const bf16x2_hw b = __builtin_convertvector(v, bf16x2_hw);
  return *reinterpret_cast<const uint32_t*>(&b);
}

// 2^x by the hardware instruction: results below the normal range become zero.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
