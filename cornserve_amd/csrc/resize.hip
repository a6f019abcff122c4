// Bicubic resampling of uint8 frames (gfx950), bit for bit what Pillow's `Image.resize(..., BICUBIC)` returns: the
// resampling the Hugging Face Qwen2-VL image processor's PIL backend applies before rescale + normalise (the
// reference runs that processor on the router's CPU: ModalityProcessor, eric/models/qwen2_5_vl.py:488-512, called
// from eric/router/processor.py:46-131).  Pillow (libImaging/Resample.c) resamples in two passes, along x and then
// along y, each a convolution with per-output-position integer taps:
//   taps      for output position i: centre = (i + 0.5) * in/out, support = 2 * max(in/out, 1); the cubic
//             (a = -0.5) kernel sampled at the input positions inside [centre - support, centre + support), in
//             double precision, normalised to sum 1, then rounded to 22 fractional bits (half away from zero);
//   one pass  out = clamp((2^21 + sum(pixel * tap)) >> 22, 0, 255) in 32-bit integers, stored as uint8 between
//             the passes.
// The taps are computed on the host in the same double-precision operation order (cs_resize_bicubic_taps_host),
// the passes run here; both are byte work bound by HBM.
#include <math.h>
#include <stdlib.h>

#include "common.h"

namespace {

constexpr int PRECISION_BITS = 32 - 8 - 2;

double cubic(double x) {
#pragma clang fp contract(off)
  const double a = -0.5;
  if (x < 0.0) x = -x;
  if (x < 1.0) return ((a + 2.0) * x - (a + 3.0)) * x * x + 1;
  if (x < 2.0) return (((x - 5) * x + 8) * x - 4) * a;
  return 0.0;
}

// One pass along the middle axis of src [outer, in_size, inner] -> dst [outer, out_size, inner]; a thread makes V
// neighbouring bytes of the inner axis (they share their taps).  Along x: outer = frames * rows, inner = channels;
// along y: outer = frames, inner = row bytes.
template <int V>
__global__ __launch_bounds__(256) void resample_pass_kernel(const uint8_t* __restrict__ src, int64_t n_out, int in_size,
                                                            int out_size, int inner_v, const int32_t* __restrict__ bounds,
                                                            const int32_t* __restrict__ taps, int ksize,
                                                            uint8_t* __restrict__ dst) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;   // output piece (outer, position, piece of inner)
  if (o >= n_out) return;
  const int iv = (int)(o % inner_v);
  const int64_t rest = o / inner_v;
  const int pos = (int)(rest % out_size);
  const int64_t outer = rest / out_size;
  const int first = bounds[2 * pos], n = bounds[2 * pos + 1];
  const int32_t* k = taps + (int64_t)pos * ksize;
  const int64_t inner = (int64_t)inner_v * V;
  const uint8_t* s = src + (outer * in_size + first) * inner + (int64_t)iv * V;
  int32_t acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = 1 << (PRECISION_BITS - 1);
  for (int x = 0; x < n; ++x, s += inner) {
    const int32_t kx = k[x];
    if constexpr (V == 4) {
      const uint32_t w = *(const uint32_t*)s;
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] += (int32_t)((w >> (8 * e)) & 0xFFu) * kx;
    } else {
      acc[0] += (int32_t)s[0] * kx;
    }
  }
  uint8_t* d = dst + (outer * out_size + pos) * inner + (int64_t)iv * V;
  if constexpr (V == 4) {
    uint32_t w = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) w |= (uint32_t)min(max(acc[e] >> PRECISION_BITS, 0), 255) << (8 * e);
    *(uint32_t*)d = w;
  } else {
    d[0] = (uint8_t)min(max(acc[0] >> PRECISION_BITS, 0), 255);
  }
}

}  // namespace

extern "C" int cs_resize_bicubic_taps_host(int32_t in_size, int32_t out_size, int32_t* bounds, int32_t* taps,
                                           int32_t cap_ksize, int32_t* ksize_out) {
#pragma clang fp contract(off)
  if (in_size <= 0 || out_size <= 0 || !ksize_out) return CS_ERR_INVALID_ARG;
  // Pillow keeps the box as floats: the whole image is [0, (float)in_size)
  double scale = (double)((float)in_size - 0.0f) / out_size;
  double filterscale = scale;
  if (filterscale < 1.0) filterscale = 1.0;
  const double support = 2.0 * filterscale;
  const int ksize = (int)ceil(support) * 2 + 1;
  *ksize_out = ksize;
  if (!bounds && !taps) return CS_OK;   // size query
  if (!bounds || !taps || cap_ksize < ksize) return CS_ERR_INVALID_ARG;
  const double ss = 1.0 / filterscale;
  for (int i = 0; i < out_size; ++i) {
    const double center = 0.0 + (i + 0.5) * scale;
    int first = (int)(center - support + 0.5);
    if (first < 0) first = 0;
    int last = (int)(center + support + 0.5);
    if (last > in_size) last = in_size;
    const int n = last - first;
    int32_t* k = taps + (int64_t)i * cap_ksize;
    double w[64];
    double* ws = w;
    double* heap = nullptr;
    if (n > 64) ws = heap = (double*)malloc(sizeof(double) * n);
    if (!ws) return CS_ERR_INVALID_ARG;
    double ww = 0.0;
    for (int x = 0; x < n; ++x) {
      ws[x] = cubic((x + first - center + 0.5) * ss);
      ww += ws[x];
    }
    for (int x = 0; x < n; ++x) {
      const double v = ww != 0.0 ? ws[x] / ww : ws[x];
      k[x] = v < 0 ? (int)(-0.5 + v * (1 << PRECISION_BITS)) : (int)(0.5 + v * (1 << PRECISION_BITS));
    }
    for (int x = n > 0 ? n : 0; x < cap_ksize; ++x) k[x] = 0;
    free(heap);
    bounds[2 * i] = first;
    bounds[2 * i + 1] = n > 0 ? n : 0;
  }
  return CS_OK;
}

extern "C" int cs_resize_u8_pass(const void* src, int64_t outer, int32_t in_size, int32_t out_size, int64_t inner,
                                 const int32_t* bounds, const int32_t* taps, int32_t ksize, void* dst, void* stream) {
  if (!src || !dst || !bounds || !taps) return CS_ERR_INVALID_ARG;
  if (outer <= 0 || in_size <= 0 || out_size <= 0 || inner <= 0 || ksize <= 0) return CS_ERR_INVALID_ARG;
  if (inner > 0x7fffffff) return CS_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const bool words = inner % 4 == 0 && (uintptr_t)src % 4 == 0 && (uintptr_t)dst % 4 == 0;
  const int v = words ? 4 : 1;
  const int64_t n_out = outer * out_size * (inner / v);
  const int64_t grid = (n_out + 255) / 256;
  if (grid > 0x7fffffff) return CS_ERR_UNSUPPORTED;
  if (words)
    hipLaunchKernelGGL(resample_pass_kernel<4>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t*)src, n_out, in_size,
                       out_size, (int)(inner / 4), bounds, taps, ksize, (uint8_t*)dst);
  else
    hipLaunchKernelGGL(resample_pass_kernel<1>, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t*)src, n_out, in_size,
                       out_size, (int)inner, bounds, taps, ksize, (uint8_t*)dst);
  return cs_launch_status();
}
