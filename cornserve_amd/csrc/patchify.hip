// Strided patch gather for the SigLIP patch embedding (gfx950).
//
// nn.Conv2d(C, E, kernel=stride=p, padding="valid") (eric/models/layers/siglip.py:30-36,94-95) over
// NCHW pixels equals a GEMM between the flattened non-overlapping patches and the [E, C*p*p] weight.
// This kernel lays the patches out as the GEMM's A operand: row m = (b, py, px), column (c, ky, kx),
// zero-padded to the leading dimension so the GEMM's 16-byte loads stay aligned (C*p*p = 588 is not a
// multiple of 8).  Consecutive threads take consecutive px of one image row, so the reads of a wave
// cover one contiguous 64*p*2-byte span of the source image.
#include "common.h"

namespace {

__global__ __launch_bounds__(256) void patchify_kernel(const bf16_t* __restrict__ px, int B, int C, int H, int W,
                                                       int p, bf16_t* __restrict__ out, int64_t ldo) {
  const int gw = W / p, gh = H / p;
  const int64_t total = (int64_t)B * gh * C * p * gw;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int x = i % gw;
  i /= gw;
  const int ky = i % p;
  i /= p;
  const int c = i % C;
  i /= C;
  const int y = i % gh;
  const int b = (int)(i / gh);
  const bf16_t* src = px + (((int64_t)b * C + c) * H + (y * p + ky)) * W + x * p;
  bf16_t* dst = out + ((int64_t)(b * gh + y) * gw + x) * ldo + (c * p + ky) * p;
  for (int kx = 0; kx < p; kx += 2) *(bf16x2_t*)(dst + kx) = *(const bf16x2_t*)(src + kx);
  // the thread that owns the last (c, ky) slice of a patch also clears the row's padding
  if (c == C - 1 && ky == p - 1) {
    bf16_t* row = out + ((int64_t)(b * gh + y) * gw + x) * ldo;
    for (int k = C * p * p; k < ldo; ++k) row[k] = f2bf(0.f);
  }
}

}  // namespace

extern "C" int cs_patchify_nchw(const void* pixels, int32_t B, int32_t C, int32_t H, int32_t W, int32_t patch,
                                void* out, int64_t ldo, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!pixels || !out || B < 0 || C <= 0 || H <= 0 || W <= 0 || patch <= 0 || patch % 2 || H % patch ||
      W % patch || ldo < (int64_t)C * patch * patch || ldo % 2 || (((uintptr_t)pixels | (uintptr_t)out) & 3))
    return CS_ERR_INVALID_ARG;
  if (B == 0) return CS_OK;
  const int64_t total = (int64_t)B * (H / patch) * C * patch * (W / patch);
  hipLaunchKernelGGL(patchify_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                     (const bf16_t*)pixels, B, C, H, W, patch, (bf16_t*)out, ldo);
  return cs_launch_status();
}
