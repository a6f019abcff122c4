// Shared pieces of the gfx950 GEMM kernels: LDS swizzle, activation functions and the fused epilogue.
#pragma once
#include "common.h"

namespace csgemm {

constexpr int BK = 64;  // K step (bf16 elements): 128 bytes per tile row = 8 chunks of 16 B

// Byte offset of 16-byte chunk `chunk` of row `row` in a [rows][64] bf16 LDS tile (128-byte rows).
// The LDS has 64 banks of 4 bytes, so a 16-byte-per-lane access is served 16 lanes at a time and is
// conflict-free only if those 16 lanes fall into 16 different 16-byte groups of a 256-byte span.  The MFMA
// fragment reads have 16 consecutive lanes on 16 consecutive rows of ONE logical chunk; XOR-ing the chunk
// with (row ^ row/8) & 7 spreads them over all 8 chunk slots of both row parities.
CS_DEVICE int swz_key(int row) { return (row ^ (row >> 3)) & 7; }
CS_DEVICE int swz(int row, int chunk) { return row * 128 + ((chunk ^ swz_key(row)) << 4); }

CS_DEVICE float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }
// 0.5 x (1 + tanh(u)) == x * sigmoid(2u): one exponential and one hardware reciprocal instead of tanhf.
CS_DEVICE float gelu_tanh(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  const float u = k0 * (x + k1 * x * x * x);
  return x * __builtin_amdgcn_rcpf(1.0f + __expf(-2.0f * u));
}
// x * sigmoid(1.702 x)
CS_DEVICE float quick_gelu(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-1.702f * x)); }
// x * sigmoid(x) with the hardware reciprocal (1 ulp) instead of an IEEE division sequence.
CS_DEVICE float silu(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }


// Fused epilogue for one wave's accumulators.  acc[i][j][4g+q] = C[m][n] with
//   m = m_base + i*32 + lane%32,   n = n_base + j*32 + 8g + 4*(lane/32) + q
// (W was the MFMA "A" operand, so a lane owns one output row and groups of 4 consecutive columns).
template <int EPI, int MT, int NT>
CS_DEVICE void epilogue(const CsGemmArgs& p, const f32x16_t (&acc)[MT][NT], int m_base, int n_base, int lane) {
  const bf16_t* const pBias = (const bf16_t*)p.bias;
  const bf16_t* const pRes = (const bf16_t*)p.residual;
  const bf16_t* const pPos = (const bf16_t*)p.pos;
  bf16_t* const pC = (bf16_t*)p.C;
  const int frag_row = lane & 31, frag_half = lane >> 5;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m_base + i * 32 + frag_row;
    if (m >= p.M) continue;
    const int64_t crow = p.c_rows ? (int64_t)p.c_rows[m] : (int64_t)m;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n_base + j * 32 + 8 * g + 4 * frag_half;
        if (n >= p.N) continue;
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = acc[i][j][4 * g + q];
        if (p.w_scale) {
          const f32x4_t s = *(const f32x4_t*)(p.w_scale + n);
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] *= s[q];
        }
        if (p.bias) {
          const bf16x4_t b = *(const bf16x4_t*)(pBias + n);
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] += bf2f(b[q]);
        }
        if (EPI == CS_EPI_SWIGLU) {
          // SiLU(gate) * up on the fp32 sums with one rounding of the product (the same as the direct-to-LDS kernel)
          const float gate0 = silu(v[0]), up0 = v[1];
          const float gate1 = silu(v[2]), up1 = v[3];
          bf16x2_t o;
          o[0] = f2bf(gate0 * up0);
          o[1] = f2bf(gate1 * up1);
          *(bf16x2_t*)(pC + crow * p.ldc + (n >> 1)) = o;
        } else {
          if (EPI == CS_EPI_GELU_ERF) {
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = gelu_erf(v[q]);
          } else if (EPI == CS_EPI_GELU_TANH) {
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = gelu_tanh(v[q]);
          } else if (EPI == CS_EPI_QUICK_GELU) {
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = quick_gelu(v[q]);
          } else if (EPI == CS_EPI_RESIDUAL) {
            const bf16x4_t r = *(const bf16x4_t*)(pRes + (int64_t)m * p.ldr + n);
            if (p.c_lo) {  // residual stream with 16 significant bits: join, add unrounded, split
              const uint32_t lo4 = p.residual_lo ? *(const uint32_t*)(p.residual_lo + (int64_t)m * p.ldr + n) : 0u;
              u32x2_t hi_words;
              uint32_t packed_lo;
              add_split24(v, __builtin_bit_cast(u32x2_t, r), lo4, hi_words, packed_lo);
              const bf16x4_t o = __builtin_bit_cast(bf16x4_t, hi_words);
              *(bf16x4_t*)(pC + crow * p.ldc + n) = o;
              *(uint32_t*)(p.c_lo + crow * p.ldc + n) = packed_lo;
              continue;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = rbf(v[q]) + bf2f(r[q]);
          }
          if (p.pos) {
            const bf16x4_t r = *(const bf16x4_t*)(pPos + (int64_t)(m % p.pos_period) * p.ldpos + n);
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = rbf(v[q]) + bf2f(r[q]);
          }
          bf16x4_t o;
#pragma unroll
          for (int q = 0; q < 4; ++q) o[q] = f2bf(v[q]);
          *(bf16x4_t*)(pC + crow * p.ldc + n) = o;
        }
      }
    }
  }
}

}  // namespace csgemm
