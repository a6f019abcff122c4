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
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int i32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(int)))) int i32x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4_t;

#define CS_DEVICE __device__ __forceinline__

// bf16 <-> fp32. The cast is round-to-nearest-even (v_cvt_pk_bf16_f32 on gfx950).
CS_DEVICE float bf2f(bf16_t x) { return (float)x; }
CS_DEVICE bf16_t f2bf(float x) { return (bf16_t)x; }
// Round an fp32 value to bf16 precision and return it as fp32 (a "rounding point").
CS_DEVICE float rbf(float x) { return (float)(bf16_t)x; }

// Residual stream with 16 significant bits: a value is kept as a bf16 "hi" plane, which is what the next GEMM reads
// as its operand, and a byte "lo" plane holding the next 8 mantissa bits as a signed correction:
//   value = bits(hi) << 16  +  (int8)lo << 8     (as an fp32 bit pattern: sign-magnitude, so the sum is monotone)
// split24 rounds an fp32 value to 24 bits (nearest, at bit 8), then rounds those 24 bits half-up in magnitude to hi;
// lo is what is left.  A zero lo plane means "the value is hi exactly", so a plain bf16 tensor next to a zero-filled
// byte plane is a valid pair.  The residual additions of an encoder then lose 2^-17 per addition instead of the 2^-9
// of a bf16 stream, for 3 bytes per element instead of the 6 of an fp32 stream plus its bf16 copy.
CS_DEVICE float join24(uint32_t hi_bits, uint32_t lo_byte) {
  const int32_t corr = (int32_t)(int8_t)lo_byte;
  return __builtin_bit_cast(float, (uint32_t)((int32_t)(hi_bits << 16) + (corr << 8)));
}
CS_DEVICE void split24(float v, uint32_t& hi_bits, uint32_t& lo_byte) {
  const uint32_t b = __builtin_bit_cast(uint32_t, v) + 0x80u;
  lo_byte = (b >> 8) & 0xFFu;
  hi_bits = (b + 0x8000u) >> 16;
}

// Four values at once: the addend's planes as raw words (two bf16 per word, four bytes in one word) joined with four
// fp32 increments, and the sums split again.  Same results as join24 / split24 element by element, in byte-select form
// (seven vector instructions per value instead of eleven): with the correction byte's top bit flipped (lo' = lo ^ 0x80,
// all four bytes of a word at once) the pair is an unsigned 24-bit word offset by half a bf16 unit,
//   bits(value) = ((hi << 16) | (lo' << 8)) - 0x8000        and        (hi << 16) | (lo' << 8) = (bits(sum) + 0x8080) & ~0xFF
// (adding 0x80 rounds to 24 bits, adding 0x8000 more rounds those half-up to hi and flips the top bit of the byte below).
CS_DEVICE void add_split24(const float (&delta)[4], u32x2_t hi_in, uint32_t lo_in, u32x2_t& hi_out, uint32_t& lo_out) {
  const uint32_t lo_f = lo_in ^ 0x80808080u;
  // v_perm_b32: selector byte 0..3 picks that byte of the second source, 4..7 of the first, 0x0c a zero byte
  const uint32_t w0 = __builtin_amdgcn_perm(hi_in[0], lo_f, 0x0504000cu);   // [hi0.b1 hi0.b0 lo'.b0 0]
  const uint32_t w1 = __builtin_amdgcn_perm(hi_in[0], lo_f, 0x0706010cu);
  const uint32_t w2 = __builtin_amdgcn_perm(hi_in[1], lo_f, 0x0504020cu);
  const uint32_t w3 = __builtin_amdgcn_perm(hi_in[1], lo_f, 0x0706030cu);
  const uint32_t c0 = __builtin_bit_cast(uint32_t, delta[0] + __builtin_bit_cast(float, w0 - 0x8000u)) + 0x8080u;
  const uint32_t c1 = __builtin_bit_cast(uint32_t, delta[1] + __builtin_bit_cast(float, w1 - 0x8000u)) + 0x8080u;
  const uint32_t c2 = __builtin_bit_cast(uint32_t, delta[2] + __builtin_bit_cast(float, w2 - 0x8000u)) + 0x8080u;
  const uint32_t c3 = __builtin_bit_cast(uint32_t, delta[3] + __builtin_bit_cast(float, w3 - 0x8000u)) + 0x8080u;
  hi_out = u32x2_t{__builtin_amdgcn_perm(c1, c0, 0x07060302u), __builtin_amdgcn_perm(c3, c2, 0x07060302u)};
  lo_out = (__builtin_amdgcn_perm(c1, c0, 0x0c0c0501u) | __builtin_amdgcn_perm(c3, c2, 0x05010c0cu)) ^ 0x80808080u;
}

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

// Workgroup b of a launch runs on XCD b mod 8, and every XCD has an L2 of its own.  This maps the launch index to a work
// index (a bijection on 0..n-1) that gives every XCD one contiguous eighth of the work, so that work items that read
// the same cache lines (neighbouring rows, neighbouring patches) meet in one L2 instead of fetching the lines eight times.
CS_DEVICE unsigned xcd_contiguous(unsigned b, unsigned n) {
  const unsigned k = b & 7u, q = n >> 3, r = n & 7u;
  return k * q + min(k, r) + (b >> 3);
}

// Last launch error -> status code. Never aborts the process.
static inline int cs_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? CS_OK : CS_ERR_LAUNCH;
}
