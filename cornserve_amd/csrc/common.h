// Shared device/host helpers for the gfx950 (CDNA4) kernels of the Eric encoder forward pass.
// Everything here is wave64-only and assumes MI355X: 64-wide wavefronts, 160 KB LDS per CU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cornserve_amd.h"  // the public C ABI (status codes, argument structs, prototypes)

typedef __bf16 bf16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(int)))) int i32x2_t;

#define CS_DEVICE __device__ __forceinline__

// bf16 <-> fp32. The cast is round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950).
CS_DEVICE float bf2f(bf16_t x) { return (float)x; }
CS_DEVICE bf16_t f2bf(float x) { return (bf16_t)x; }
// Round an fp32 value to bf16 precision and return it as fp32 (a "rounding point").
CS_DEVICE float rbf(float x) { return (float)(bf16_t)x; }

// One rotary pair in fp32 with every product and sum rounded on its own (no fused multiply-add), as the
// reference's tensor program computes it (x1*cos - x2*sin, x1*sin + x2*cos): every kernel that rotates gives
// the same bits, whichever of them a launch selects.
CS_DEVICE float rot_first(float x1, float x2, float co, float si) {
#pragma clang fp contract(off)
  const float p = x1 * co, q = x2 * si;
  return p - q;
}
CS_DEVICE float rot_second(float x1, float x2, float co, float si) {
#pragma clang fp contract(off)
  const float p = x1 * si, q = x2 * co;
  return p + q;
}

CS_DEVICE float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
CS_DEVICE float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// Last launch error -> status code. Never aborts the process.
static inline int cs_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? CS_OK : CS_ERR_LAUNCH;
}
