// HBM-bound row kernels for gfx950: RMSNorm, GemmaRMSNorm, LayerNorm, AvgPool+GemmaRMSNorm, casts.
//
// One 64-wide wavefront owns one row.  A row of H bf16 values is read as 16-byte chunks (8 values),
// lane i takes chunks i, i+64, i+128, ... so every load instruction of the wave covers 1 KB of
// consecutive bytes; the row stays in registers between the reduction and the scaling pass, so each
// element is read from HBM once and written once (algorithmic traffic: 4 bytes per element).
// Reductions are butterfly shuffles inside the wave; no LDS, no atomics.
//
// Reference semantics:
//   RMSNorm      eric/models/layers/norm.py:35-70   (fp32 stats, cast to bf16, THEN multiply by w)
//   GemmaRMSNorm eric/models/layers/norm.py:90-113  (fp32 x*rsqrt*(1+w), single cast)
//   LayerNorm    torch.nn.LayerNorm as used at eric/models/layers/siglip.py:173-175,333
//   AvgPool2d    eric/models/gemma3.py:36-44 (bf16 result) followed by GemmaRMSNorm (:46)
#include "common.h"

namespace {

constexpr int ROWS_PER_BLOCK = 4;  // 256 threads

template <int NC>
CS_DEVICE void load_row(const bf16_t* row, int nchunks, int lane, float (&v)[NC][8]) {
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int c = lane + 64 * j;
    if (c < nchunks) {
      const bf16x8_t x = *(const bf16x8_t*)(row + c * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[j][e] = bf2f(x[e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[j][e] = 0.f;
    }
  }
}

template <int NC, bool GEMMA>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const bf16_t* __restrict__ x, int64_t ldx,
                                                      const bf16_t* __restrict__ w, bf16_t* __restrict__ y,
                                                      int64_t ldy, int rows, int H, float eps) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nchunks = H >> 3;
  float v[NC][8];
  load_row<NC>(x + (int64_t)row * ldx, nchunks, lane, v);
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NC; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[j][e] * v[j][e];
  ss = wave_sum(ss);
  const float rs = rsqrtf(ss / (float)H + eps);
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int c = lane + 64 * j;
    if (c < nchunks) {
      const bf16x8_t wv = *(const bf16x8_t*)(w + c * 8);
      bf16x8_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (GEMMA)
          o[e] = f2bf(v[j][e] * rs * (1.0f + bf2f(wv[e])));
        else
          o[e] = f2bf(rbf(v[j][e] * rs) * bf2f(wv[e]));
      }
      *(bf16x8_t*)(y + (int64_t)row * ldy + c * 8) = o;
    }
  }
}

template <int NC>
__global__ __launch_bounds__(256) void layernorm_kernel(const bf16_t* __restrict__ x, int64_t ldx,
                                                        const bf16_t* __restrict__ w,
                                                        const bf16_t* __restrict__ b, bf16_t* __restrict__ y,
                                                        int64_t ldy, int rows, int H, float eps) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nchunks = H >> 3;
  float v[NC][8];
  load_row<NC>(x + (int64_t)row * ldx, nchunks, lane, v);
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < NC; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) s += v[j][e];
  const float mean = wave_sum(s) / (float)H;
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    if (lane + 64 * j < nchunks) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = v[j][e] - mean;
        ss += d * d;
      }
    }
  }
  const float rstd = rsqrtf(wave_sum(ss) / (float)H + eps);
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int c = lane + 64 * j;
    if (c < nchunks) {
      const bf16x8_t wv = *(const bf16x8_t*)(w + c * 8);
      const bf16x8_t bv = *(const bf16x8_t*)(b + c * 8);
      bf16x8_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = f2bf((v[j][e] - mean) * rstd * bf2f(wv[e]) + bf2f(bv[e]));
      *(bf16x8_t*)(y + (int64_t)row * ldy + c * 8) = o;
    }
  }
}

// Eight per-lane partial sums -> their eight totals over the wave, with 10 lane exchanges instead of 48: each of
// the first three exchanges (lane ^ 32, ^ 16, ^ 8) hands the partner the half of the values it keeps, so the number
// of live values halves; three more exchanges finish the one value left.  Lane l returns the total of part l >> 3.
static_assert(CS_SUMSQ_PARTS == 8, "wave_sum_parts halves eight values three times");
CS_DEVICE float wave_sum_parts(const float (&part)[8], int lane) {
  const bool b5 = lane & 32, b4 = lane & 16, b3 = lane & 8;
  float a[4], b[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float keep = b5 ? part[4 + i] : part[i], give = b5 ? part[i] : part[4 + i];
    a[i] = keep + __shfl_xor(give, 32, 64);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float keep = b4 ? a[2 + i] : a[i], give = b4 ? a[i] : a[2 + i];
    b[i] = keep + __shfl_xor(give, 16, 64);
  }
  float c = (b3 ? b[1] : b[0]) + __shfl_xor(b3 ? b[0] : b[1], 8, 64);
  c += __shfl_xor(c, 4, 64);
  c += __shfl_xor(c, 2, 64);
  c += __shfl_xor(c, 1, 64);
  return c;
}

// Sums of squares of a row in parts of 160 columns (20 chunks): the variance term of RMSNorm in the form
// that a GEMM with CsGemmArgs.a_row_sumsq consumes.  out is [rows][CS_SUMSQ_PARTS].
template <bool WITH_SUM>
__global__ __launch_bounds__(256) void row_sumsq_kernel(const bf16_t* __restrict__ x, int64_t ldx, int rows, int H,
                                                        float* __restrict__ out, float* __restrict__ sum_out) {
  constexpr int NC = (160 * CS_SUMSQ_PARTS / 8 + 63) / 64;
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nchunks = H >> 3;
  float v[NC][8];
  load_row<NC>(x + (int64_t)row * ldx, nchunks, lane, v);
  float part[CS_SUMSQ_PARTS], spart[WITH_SUM ? CS_SUMSQ_PARTS : 1];
#pragma unroll
  for (int q = 0; q < CS_SUMSQ_PARTS; ++q) {
    part[q] = 0.f;
    if (WITH_SUM) spart[WITH_SUM ? q : 0] = 0.f;
  }
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    float ss = 0.f, sm = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      ss += v[j][e] * v[j][e];
      sm += v[j][e];
    }
    const int q_of_chunk = (lane + 64 * j) / 20;
#pragma unroll
    for (int q = 0; q < CS_SUMSQ_PARTS; ++q) {
      part[q] += (q == q_of_chunk) ? ss : 0.f;
      if (WITH_SUM) spart[WITH_SUM ? q : 0] += (q == q_of_chunk) ? sm : 0.f;
    }
  }
  // lane l ends up with the total of part l / 8: eight lanes each store one value
  const float tot = wave_sum_parts(part, lane);
  if ((lane & 7) == 0) out[(int64_t)row * CS_SUMSQ_PARTS + (lane >> 3)] = tot;
  if constexpr (WITH_SUM) {
    const float stot = wave_sum_parts(spart, lane);
    if ((lane & 7) == 0) sum_out[(int64_t)row * CS_SUMSQ_PARTS + (lane >> 3)] = stot;
  }
}

// One wave per pooled token: mean over a k x k neighbourhood of the side x side token grid, rounded to
// bf16 (AvgPool2d output dtype), then GemmaRMSNorm over the channel axis.
template <int NC>
__global__ __launch_bounds__(256) void avgpool_gemma_kernel(const bf16_t* __restrict__ x,
                                                            const bf16_t* __restrict__ w,
                                                            bf16_t* __restrict__ y, int B, int side, int k,
                                                            int H, float eps) {
  const int lane = threadIdx.x & 63;
  const int oside = side / k;
  const int tok = blockIdx.x * ROWS_PER_BLOCK + (threadIdx.x >> 6);
  if (tok >= B * oside * oside) return;
  const int b = tok / (oside * oside);
  const int oy = (tok / oside) % oside, ox = tok % oside;
  const int nchunks = H >> 3;
  float acc[NC][8];
#pragma unroll
  for (int j = 0; j < NC; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
  for (int dy = 0; dy < k; ++dy) {
    for (int dx = 0; dx < k; ++dx) {
      const int64_t src = ((int64_t)b * side + (oy * k + dy)) * side + (ox * k + dx);
      float v[NC][8];
      load_row<NC>(x + src * H, nchunks, lane, v);
#pragma unroll
      for (int j = 0; j < NC; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j][e] += v[j][e];
    }
  }
  const float inv = 1.0f / (float)(k * k);
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NC; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      acc[j][e] = rbf(acc[j][e] * inv);
      ss += acc[j][e] * acc[j][e];
    }
  const float rs = rsqrtf(wave_sum(ss) / (float)H + eps);
#pragma unroll
  for (int j = 0; j < NC; ++j) {
    const int c = lane + 64 * j;
    if (c < nchunks) {
      const bf16x8_t wv = *(const bf16x8_t*)(w + c * 8);
      bf16x8_t o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = f2bf(acc[j][e] * rs * (1.0f + bf2f(wv[e])));
      *(bf16x8_t*)(y + (int64_t)tok * H + c * 8) = o;
    }
  }
}

__global__ __launch_bounds__(256) void cast_f32_bf16_kernel(const float* __restrict__ in,
                                                            bf16_t* __restrict__ out, int64_t n8) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n8; i += stride) {
    const f32x4_t a = *(const f32x4_t*)(in + i * 8);
    const f32x4_t b = *(const f32x4_t*)(in + i * 8 + 4);
    bf16x8_t o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[e] = f2bf(a[e]);
      o[4 + e] = f2bf(b[e]);
    }
    *(bf16x8_t*)(out + i * 8) = o;
  }
}
__global__ void cast_f32_bf16_tail(const float* in, bf16_t* out, int64_t start, int64_t n) {
  int64_t i = start + threadIdx.x;
  if (i < n) out[i] = f2bf(in[i]);
}

inline bool row_args_ok(const void* x, int64_t ldx, const void* y, int64_t ldy, int rows, int H) {
  return x && y && rows >= 0 && H > 0 && H % 8 == 0 && ldx % 8 == 0 && ldy % 8 == 0 && ldx >= H && ldy >= H &&
         !(((uintptr_t)x | (uintptr_t)y) & 15);
}

}  // namespace

#define CS_DISPATCH_NC(H, CALL)        \
  do {                                 \
    const int nc_ = ((H) / 8 + 63) / 64; \
    if (nc_ <= 1) { CALL(1); }         \
    else if (nc_ == 2) { CALL(2); }    \
    else if (nc_ == 3) { CALL(3); }    \
    else if (nc_ == 4) { CALL(4); }    \
    else if (nc_ <= 8) { CALL(8); }    \
    else if (nc_ <= 16) { CALL(16); }  \
    else return CS_ERR_UNSUPPORTED;    \
  } while (0)

extern "C" int cs_rmsnorm(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int32_t rows,
                          int32_t H, float eps, int32_t gemma, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!row_args_ok(x, ldx, y, ldy, rows, H) || !w || ((uintptr_t)w & 15)) return CS_ERR_INVALID_ARG;
  if (rows == 0) return CS_OK;
  const dim3 grid((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK), block(256);
#define CALL(NC)                                                                                         \
  if (gemma)                                                                                             \
    hipLaunchKernelGGL((rmsnorm_kernel<NC, true>), grid, block, 0, stream, (const bf16_t*)x, ldx,        \
                       (const bf16_t*)w, (bf16_t*)y, ldy, rows, H, eps);                                 \
  else                                                                                                   \
    hipLaunchKernelGGL((rmsnorm_kernel<NC, false>), grid, block, 0, stream, (const bf16_t*)x, ldx,       \
                       (const bf16_t*)w, (bf16_t*)y, ldy, rows, H, eps)
  CS_DISPATCH_NC(H, CALL);
#undef CALL
  return cs_launch_status();
}

extern "C" int cs_row_stats(const void* x, int64_t ldx, int32_t rows, int32_t H, float* out, float* sum_out, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!x || !out || rows < 0 || H <= 0 || H % 8 || ldx % 8 || ldx < H ||
      (((uintptr_t)x | (uintptr_t)out | (uintptr_t)sum_out) & 15))
    return CS_ERR_INVALID_ARG;
  if (H > 160 * CS_SUMSQ_PARTS) return CS_ERR_UNSUPPORTED;
  if (rows == 0) return CS_OK;
  const dim3 grid((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK), block(256);
  if (sum_out)
    hipLaunchKernelGGL(row_sumsq_kernel<true>, grid, block, 0, stream, (const bf16_t*)x, ldx, rows, H, out, sum_out);
  else
    hipLaunchKernelGGL(row_sumsq_kernel<false>, grid, block, 0, stream, (const bf16_t*)x, ldx, rows, H, out, sum_out);
  return cs_launch_status();
}

extern "C" int cs_row_sumsq(const void* x, int64_t ldx, int32_t rows, int32_t H, float* out, void* stream_) {
  return cs_row_stats(x, ldx, rows, H, out, nullptr, stream_);
}

extern "C" int cs_layernorm(const void* x, int64_t ldx, const void* w, const void* b, void* y, int64_t ldy,
                            int32_t rows, int32_t H, float eps, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!row_args_ok(x, ldx, y, ldy, rows, H) || !w || !b || (((uintptr_t)w | (uintptr_t)b) & 15))
    return CS_ERR_INVALID_ARG;
  if (rows == 0) return CS_OK;
  const dim3 grid((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK), block(256);
#define CALL(NC)                                                                                   \
  hipLaunchKernelGGL((layernorm_kernel<NC>), grid, block, 0, stream, (const bf16_t*)x, ldx,        \
                     (const bf16_t*)w, (const bf16_t*)b, (bf16_t*)y, ldy, rows, H, eps)
  CS_DISPATCH_NC(H, CALL);
#undef CALL
  return cs_launch_status();
}

extern "C" int cs_avgpool_gemma_rmsnorm(const void* x, const void* w, void* y, int32_t B, int32_t side,
                                        int32_t k, int32_t H, float eps, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!x || !w || !y || B < 0 || side <= 0 || k <= 0 || side % k || H <= 0 || H % 8) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) return CS_ERR_INVALID_ARG;
  if (B == 0) return CS_OK;
  const int toks = B * (side / k) * (side / k);
  const dim3 grid((toks + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK), block(256);
#define CALL(NC)                                                                                  \
  hipLaunchKernelGGL((avgpool_gemma_kernel<NC>), grid, block, 0, stream, (const bf16_t*)x,        \
                     (const bf16_t*)w, (bf16_t*)y, B, side, k, H, eps)
  CS_DISPATCH_NC(H, CALL);
#undef CALL
  return cs_launch_status();
}

extern "C" int cs_cast_f32_bf16(const float* in, void* out, int64_t n, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n < 0 || (n > 0 && (!in || !out))) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)in | (uintptr_t)out) & 15) return CS_ERR_INVALID_ARG;
  if (n == 0) return CS_OK;
  const int64_t n8 = n / 8;
  if (n8 > 0) {
    const int blocks = (int)((n8 + 255) / 256 < 8192 ? (n8 + 255) / 256 : 8192);
    hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3(blocks), dim3(256), 0, stream, in, (bf16_t*)out, n8);
  }
  if (n8 * 8 < n) hipLaunchKernelGGL(cast_f32_bf16_tail, dim3(1), dim3(8), 0, stream, in, (bf16_t*)out, n8 * 8, n);
  return cs_launch_status();
}
