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

// 24-bit multiply: a byte times a tap.  Taps of a normalised filter stay below 2^23 in magnitude (a weight is at most
// a few percent above 1.0 = 2^22), and the low 32 bits of the product are what the 32-bit accumulation keeps anyway.
CS_DEVICE int32_t mad24(int32_t px, int32_t tap, int32_t acc) { return __mul24(px, tap) + acc; }
// The empty statement keeps each clamped value a 32-bit value of its own: without it the compiler packs two of them with
// v_ashr_pk_u8_i32, which leaves the upper half of its destination register as it was, and then ORs the other bytes
// into that register as if the upper half were zero.
CS_DEVICE uint32_t clamp8(int32_t acc) {
  uint32_t c = (uint32_t)min(max(acc >> PRECISION_BITS, 0), 255);
  asm volatile("" : "+v"(c));
  return c;
}

// One pass along the middle axis of src [outer, in_size, inner] -> dst [outer, out_size, inner]; a thread makes V
// neighbouring bytes of the inner axis (they share their taps).  Any shape; the two kernels below serve the usual ones.
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
      for (int e = 0; e < 4; ++e) acc[e] = mad24((int32_t)((w >> (8 * e)) & 0xFFu), kx, acc[e]);
    } else {
      acc[0] = mad24((int32_t)s[0], kx, acc[0]);
    }
  }
  uint8_t* d = dst + (outer * out_size + pos) * inner + (int64_t)iv * V;
  if constexpr (V == 4) {
    uint32_t w = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) w |= clamp8(acc[e]) << (8 * e);
    *(uint32_t*)d = w;
  } else {
    d[0] = (uint8_t)clamp8(acc[0]);
  }
}

// The pass along y (a long inner axis: whole image rows of W*C bytes): a workgroup makes 1024 bytes of ONE output row,
// so the window and the taps are the same for all its lanes and come through scalar loads; a lane makes four
// neighbouring bytes from one coalesced 4-byte load per tap.
__global__ __launch_bounds__(256) void resample_rows_kernel(const uint8_t* __restrict__ src, int in_size, int out_size,
                                                            int inner_w, int chunks, const int32_t* __restrict__ bounds,
                                                            const int32_t* __restrict__ taps, int ksize,
                                                            uint8_t* __restrict__ dst) {
  // work index -> (1024-byte column of the image, output row), rows fastest, a contiguous eighth of it per XCD: the
  // workgroups that read the same input rows (neighbouring output rows of one column) share an L2
  const unsigned v = xcd_contiguous(blockIdx.x, gridDim.x);
  const unsigned n_rows = gridDim.x / (unsigned)chunks;   // outer * out_size
  const unsigned chunk = v / n_rows, row = v % n_rows;
  const unsigned pos = row % (unsigned)out_size, outer = row / (unsigned)out_size;
  const int iw = (int)chunk * 256 + threadIdx.x;   // word of the row
  if (iw >= inner_w) return;
  const int first = bounds[2 * pos], n = bounds[2 * pos + 1];
  const int32_t* k = taps + (int64_t)pos * ksize;
  const uint32_t* s = (const uint32_t*)src + ((int64_t)outer * in_size + first) * inner_w + iw;
  int32_t acc[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) acc[e] = 1 << (PRECISION_BITS - 1);
  int x = 0;
  for (; x + 4 <= n; x += 4) {   // four loads in flight (eight were slower)
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = s[(int64_t)(x + j) * inner_w];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int32_t kx = k[x + j];
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = mad24((int32_t)((w[j] >> (8 * e)) & 0xFFu), kx, acc[e]);
    }
  }
  for (; x < n; ++x) {
    const uint32_t w = s[(int64_t)x * inner_w];
    const int32_t kx = k[x];
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = mad24((int32_t)((w >> (8 * e)) & 0xFFu), kx, acc[e]);
  }
  uint32_t o = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) o |= clamp8(acc[e]) << (8 * e);
  ((uint32_t*)dst)[(int64_t)row * inner_w + iw] = o;
}

// The pass along x of three interleaved channels (RGB rows).  A workgroup makes 256 neighbouring output positions of
// XR_ROWS image rows; lane p keeps the KS taps of its position in registers for all of them.  The bytes of a row that the
// 256 windows cover (one contiguous span) are staged in LDS with aligned 16-byte loads (every piece loaded holds at least
// one byte of the span, so no load leaves the allocation), `batch` rows at a time (as many as fit 1024 pieces: the loads
// of a whole batch are in flight together, and the next batch is fetched while this one is computed); a lane then reads
// its window from LDS at constant offsets from its first byte.  Taps past a window's count are zero, so every lane reads
// KS pixels (reads past the staged span see stale LDS bytes times zero).  This removes the one byte load and one tap load
// per tap and output byte that bound the general kernel above.
constexpr int XR_ROWS = 32;
constexpr int XR_PIECES = 4;   // 16-byte pieces per lane and batch: 16 KB per batch
template <int KS>
__global__ __launch_bounds__(256) void resample_x_rgb_kernel(const uint8_t* __restrict__ src, int rows, int in_size,
                                                             int out_size, const int32_t* __restrict__ bounds,
                                                             const int32_t* __restrict__ taps, int ksize,
                                                             uint8_t* __restrict__ dst, int buf_bytes, int batch) {
  extern __shared__ __attribute__((aligned(16))) uint8_t stage[];   // two batches of `batch` row buffers of buf_bytes
  const int tiles = (out_size + 255) / 256;
  const unsigned tile = blockIdx.x % (unsigned)tiles, group = blockIdx.x / (unsigned)tiles;
  const int p0 = (int)tile * 256;
  const int n_pos = min(256, out_size - p0);
  const int p = p0 + min((int)threadIdx.x, n_pos - 1);   // lanes past the last position repeat it and store nothing
  const int first = bounds[2 * p];
  int32_t k[KS];
#pragma unroll
  for (int x = 0; x < KS; ++x) k[x] = x < ksize ? taps[(int64_t)p * ksize + x] : 0;
  const int span_lo = bounds[2 * p0];
  const int last = p0 + n_pos - 1;
  const int span_bytes = (bounds[2 * last] + bounds[2 * last + 1] - span_lo) * 3;
  const int row0 = (int)group * XR_ROWS;
  const int n_rows = min(XR_ROWS, rows - row0);
  const int ppr = buf_bytes >> 4;   // pieces per row buffer
  const int batch_bytes = batch * buf_bytes;
  // where this lane's pieces of a batch sit: (row of the batch, piece of the row), the same for every batch
  int piece_row[XR_PIECES], piece_q[XR_PIECES];
#pragma unroll
  for (int j = 0; j < XR_PIECES; ++j) {
    const int i = (int)threadIdx.x + 256 * j;
    piece_row[j] = i / ppr;
    piece_q[j] = i - piece_row[j] * ppr;
  }
  u32x4_t held[XR_PIECES];
  uint32_t have = 0;
  auto row_begin = [&](int r) { return (uintptr_t)src + ((int64_t)(row0 + r) * in_size + span_lo) * 3; };
  // this lane's pieces of the batch that starts at row r0 (kept in registers until the buffer is free)
  auto fetch = [&](int r0) {
    have = 0;
#pragma unroll
    for (int j = 0; j < XR_PIECES; ++j) {
      const int r = r0 + piece_row[j];
      if (piece_row[j] < batch && r < n_rows) {
        const uintptr_t begin = row_begin(r);
        const uintptr_t a0 = begin & ~(uintptr_t)15;
        const int pieces = min((int)((begin + span_bytes - a0 + 15) >> 4), ppr);   // never past the buffer, whatever the bounds say
        if (piece_q[j] < pieces) {
          held[j] = *(const u32x4_t*)(a0 + 16 * (uintptr_t)piece_q[j]);
          have |= 1u << j;
        }
      }
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int j = 0; j < XR_PIECES; ++j)
      if (have >> j & 1) *(u32x4_t*)(stage + buf * batch_bytes + piece_row[j] * buf_bytes + 16 * piece_q[j]) = held[j];
  };
  fetch(0);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int r0 = 0; r0 < n_rows; r0 += batch, buf ^= 1) {
    if (r0 + batch < n_rows) fetch(r0 + batch);
    const int nb = min(batch, n_rows - r0);
    for (int rr = 0; rr < nb; ++rr) {
      const int shift = (int)(row_begin(r0 + rr) & 15);
      const uint8_t* win = stage + buf * batch_bytes + rr * buf_bytes + shift + (first - span_lo) * 3;
      int32_t a0 = 1 << (PRECISION_BITS - 1), a1 = a0, a2 = a0;
#pragma unroll
      for (int x = 0; x < KS; ++x) {
        a0 = mad24((int32_t)win[3 * x + 0], k[x], a0);
        a1 = mad24((int32_t)win[3 * x + 1], k[x], a1);
        a2 = mad24((int32_t)win[3 * x + 2], k[x], a2);
      }
      if ((int)threadIdx.x < n_pos) {
        uint8_t* d = dst + ((int64_t)(row0 + r0 + rr) * out_size + p) * 3;
        d[0] = (uint8_t)clamp8(a0);
        d[1] = (uint8_t)clamp8(a1);
        d[2] = (uint8_t)clamp8(a2);
      }
    }
    if (r0 + batch < n_rows) put(buf ^ 1);
    __syncthreads();
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

namespace {

template <int KS>
void launch_x_rgb(hipStream_t st, unsigned grid, size_t lds, const uint8_t* src, int rows, int in_size, int out_size,
                  const int32_t* bounds, const int32_t* taps, int ksize, uint8_t* dst, int buf_bytes, int batch) {
  hipLaunchKernelGGL(resample_x_rgb_kernel<KS>, dim3(grid), dim3(256), lds, st, src, rows, in_size, out_size, bounds, taps,
                     ksize, dst, buf_bytes, batch);
}

}  // namespace

extern "C" int cs_resize_u8_pass(const void* src, int64_t outer, int32_t in_size, int32_t out_size, int64_t inner,
                                 const int32_t* bounds, const int32_t* taps, int32_t ksize, void* dst, void* stream) {
  if (!src || !dst || !bounds || !taps) return CS_ERR_INVALID_ARG;
  if (outer <= 0 || in_size <= 0 || out_size <= 0 || inner <= 0 || ksize <= 0) return CS_ERR_INVALID_ARG;
  if (inner > 0x7fffffff) return CS_ERR_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const bool words = inner % 4 == 0 && (uintptr_t)src % 4 == 0 && (uintptr_t)dst % 4 == 0;
  // RGB rows along x: windows of neighbouring positions advance by in/out, so 256 of them span at most this many pixels
  const int64_t span_cap = (255 * (int64_t)in_size + out_size - 1) / out_size + ksize + 2;
  const int ks = ksize <= 5 ? 5 : ksize <= 7 ? 7 : ksize <= 9 ? 9 : ksize <= 11 ? 11 : ksize <= 13 ? 13 : ksize <= 15 ? 15
               : ksize <= 17 ? 17 : ksize <= 21 ? 21 : ksize <= 25 ? 25 : 32;
  const int64_t row_buf = (15 + (span_cap + ks) * 3 + 16 + 15) / 16 * 16;   // alignment shift + span + the last window's zero taps
  if (inner == 3 && ksize <= 32 && row_buf <= (int64_t)XR_PIECES * 256 * 16 && outer <= 0x7fffffff) {
    const int buf_bytes = (int)row_buf;
    const int64_t tiles = (out_size + 255) / 256, groups = (outer + XR_ROWS - 1) / XR_ROWS;
    if (tiles * groups <= 0x7fffffff) {
      const unsigned grid = (unsigned)(tiles * groups);
      const int batch = (int)(XR_PIECES * 256 / (buf_bytes / 16) < 8 ? XR_PIECES * 256 / (buf_bytes / 16) : 8);
      const size_t lds = 2 * (size_t)batch * buf_bytes;
      const uint8_t* s = (const uint8_t*)src;
      uint8_t* d = (uint8_t*)dst;
      const int rows = (int)outer;
      switch (ks) {
        case 5: launch_x_rgb<5>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 7: launch_x_rgb<7>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 9: launch_x_rgb<9>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 11: launch_x_rgb<11>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 13: launch_x_rgb<13>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 15: launch_x_rgb<15>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 17: launch_x_rgb<17>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 21: launch_x_rgb<21>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        case 25: launch_x_rgb<25>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
        default: launch_x_rgb<32>(st, grid, lds, s, rows, in_size, out_size, bounds, taps, ksize, d, buf_bytes, batch); break;
      }
      return cs_launch_status();
    }
  }
  if (words && inner >= 256) {   // whole rows: one output row per workgroup column, taps through scalar loads
    const int inner_w = (int)(inner / 4);
    const int64_t chunks = (inner_w + 255) / 256;
    const int64_t grid = chunks * outer * out_size;
    if (grid <= 0x7fffffff && outer * out_size <= 0x7fffffff) {
      hipLaunchKernelGGL(resample_rows_kernel, dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t*)src, in_size, out_size,
                         inner_w, (int)chunks, bounds, taps, ksize, (uint8_t*)dst);
      return cs_launch_status();
    }
  }
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
