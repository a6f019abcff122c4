// Integer index routines, row gather and rotary embedding of the Qwen2.5-VL vision encoder (gfx950).
//
// The reference builds the window permutation with a Python loop per image, boolean masks and a
// .tolist() host sync (eric/models/qwen2_5_vl.py:357-386), the position ids with another per-image
// loop (:325-355), and then gathers hidden states and the rotary table (:438-443).  Here the
// per-item scalars are computed once on the host (a few integers per image), and one device kernel
// fills every per-patch array from a closed form, one thread per patch:
//
//   a merged unit (frame f, row r, col c) of an item with merged grid gh x gw sits in window
//   (wr, wc) = (r / win, c / win) of height rh = min(win, gh - wr*win) and width cw = min(win, gw - wc*win);
//   its position in window order is
//       base + f*gh*gw + wr*win*gw + rh*wc*win + (r - wr*win)*cw + (c - wc*win)
//   because the windows of one frame are emitted row-major and each window row-major inside
//   (permute(0,1,3,2,4) then boolean compaction, :372-379).  Empty pad windows contribute nothing.
#include <math.h>

#include "common.h"

namespace {

struct ItemMeta {  // matches the int32[8] record documented in cornserve_amd.h
  int t, gh, gw, unit_base, nwr, nwc, patch_base, src_unit_base;
};

__global__ __launch_bounds__(256) void vit_index_kernel(const ItemMeta* __restrict__ meta, int merge, int win,
                                                        const float* __restrict__ inv_freq, int rot_dim,
                                                        int32_t* __restrict__ window_index,
                                                        int32_t* __restrict__ reverse_index,
                                                        int32_t* __restrict__ src_rows,
                                                        int32_t* __restrict__ pos_ids,
                                                        float* __restrict__ cos_sin) {
  const ItemMeta it = meta[blockIdx.y];
  const int mm = merge * merge;
  const int frame_units = it.gh * it.gw;
  const int n_patches = it.t * frame_units * mm;
  const int pl = blockIdx.x * blockDim.x + threadIdx.x;  // patch within the item, ORIGINAL order
  if (pl >= n_patches) return;
  const int ul = pl / mm, s = pl - ul * mm;
  const int f = ul / frame_units;
  const int rem = ul - f * frame_units;
  const int r = rem / it.gw, c = rem - r * it.gw;
  const int wr = r / win, wc = c / win;
  const int rh = min(win, it.gh - wr * win);
  const int cw = min(win, it.gw - wc * win);
  const int pos = wr * win * it.gw + rh * wc * win + (r - wr * win) * cw + (c - wc * win);
  const int u = it.unit_base + ul;                     // original unit id
  const int up = it.unit_base + f * frame_units + pos;  // window-order unit id
  if (s == 0) {
    if (window_index) window_index[up] = u;
    if (reverse_index) reverse_index[u] = up;
  }
  const int h = r * merge + s / merge;
  const int w = c * merge + s % merge;
  const int64_t row_orig = (int64_t)u * mm + s;
  const int64_t row_win = (int64_t)up * mm + s;
  // (the caller's patch matrix may hold the items in another order than they are processed in)
  if (src_rows) src_rows[row_win] = (int32_t)((int64_t)(it.src_unit_base + ul) * mm + s);
  if (pos_ids) {
    pos_ids[row_orig * 2 + 0] = h;
    pos_ids[row_orig * 2 + 1] = w;
  }
  if (cos_sin) {
    const int half = rot_dim / 2;
    float* out = cos_sin + row_win * (2 * rot_dim);
    for (int j = 0; j < half; ++j) {
      const float fr = inv_freq[j];
      const float ah = (float)h * fr, aw = (float)w * fr;
      out[j] = cosf(ah);
      out[half + j] = cosf(aw);
      out[rot_dim + j] = sinf(ah);
      out[rot_dim + half + j] = sinf(aw);
    }
  }
}

// Qwen3-VL learned position embedding, bilinearly interpolated from its side x side table to an item's h x w patch
// grid (eric/models/qwen3_vl.py:364-420), written in patch order (2x2-block-major rows, repeated per frame).  The
// arithmetic follows the reference's tensor program step by step: fp32 linspace positions (torch's two-sided
// formula), fp32 corner weights, weights and table rows in bf16, each product rounded to bf16, the four products
// summed in fp32 and rounded once.  One thread per 8 channels of one patch.
__global__ __launch_bounds__(256) void pos_embed_interp_kernel(const bf16_t* __restrict__ table, int side, int E,
                                                               const ItemMeta* __restrict__ meta, int merge,
                                                               bf16_t* __restrict__ out, int64_t ldo) {
  const ItemMeta it = meta[blockIdx.y];
  const int chunks = E >> 3;
  const int mm = merge * merge;
  const int h = it.gh * merge, w = it.gw * merge;
  const int64_t n = (int64_t)it.t * h * w * chunks;
  const unsigned idx = blockIdx.x * blockDim.x + threadIdx.x;   // (below 2^31: checked on the host)
  if (idx >= n) return;
  const int pl = (int)(idx / (unsigned)chunks);   // patch within the item, in patch (block-major) order
  const int c = (int)(idx - (unsigned)pl * chunks);
  const int ul = pl / mm, s = pl - ul * mm;
  const int rem = ul % (it.gh * it.gw);
  const int y = (rem / it.gw) * merge + s / merge, x = (rem % it.gw) * merge + s % merge;
  auto position = [&](int i, int steps) -> float {   // torch.linspace(0, side - 1, steps)[i] in fp32
    if (steps == 1) return 0.f;
    const float end = (float)(side - 1);
    const float step = end / (float)(steps - 1);
    return i < steps / 2 ? step * (float)i : __fmaf_rn(-step, (float)(steps - i - 1), end);
  };
  const float hy = position(y, h), wx = position(x, w);
  const int y0 = (int)hy, x0 = (int)wx;
  const int y1 = min(y0 + 1, side - 1), x1 = min(x0 + 1, side - 1);
  const float dh = hy - (float)y0, dw = wx - (float)x0;
  const float w11 = dh * dw, w10 = dh - w11, w01 = dw - w11, w00 = 1.f - dh - dw + w11;
  const float wq[4] = {rbf(w00), rbf(w01), rbf(w10), rbf(w11)};
  const bf16_t* rows[4] = {table + (int64_t)(y0 * side + x0) * E, table + (int64_t)(y0 * side + x1) * E,
                           table + (int64_t)(y1 * side + x0) * E, table + (int64_t)(y1 * side + x1) * E};
  float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const bf16x8_t e = *(const bf16x8_t*)(rows[k] + c * 8);
#pragma unroll
    for (int q = 0; q < 8; ++q) acc[q] += rbf(bf2f(e[q]) * wq[k]);
  }
  bf16x8_t o;
#pragma unroll
  for (int q = 0; q < 8; ++q) o[q] = f2bf(acc[q]);
  *(bf16x8_t*)(out + (int64_t)(it.patch_base + pl) * ldo + c * 8) = o;
}

// Rows mixed from up to four source rows: LLaVA-OneVision's merge of per-tile features into one sequence
// (eric/models/llava_onevision.py:78-153: tiles laid out as one grid, the padding cropped, large grids shrunk with
// torch.nn.functional.interpolate(mode="bilinear"), a newline row behind every grid row) and its 2x pooling of video
// frames (:169-183).  The caller turns that tensor program into, per output row, four source rows (y0x0, y0x1, y1x0,
// y1x1) and the two fractions (ly, lx) of the interpolation; the value is
//   (1-ly) * ((1-lx)*a00 + lx*a01) + ly * ((1-lx)*a10 + lx*a11)
// in fp32 with no contraction, rounded once to bf16 (the form of torch's bilinear kernel on a GPU, which accumulates
// bf16 inputs in fp32).  ly == lx == 0 copies row y0x0 bit for bit (crop, reorder, newline).  A tap outside
// [0, n_src) gives a zero row instead of a stray read.  One thread per 8 channels of one output row.
__global__ __launch_bounds__(256) void rows_bilinear_kernel(const bf16_t* __restrict__ src, int64_t lds, int n_src,
                                                            const int32_t* __restrict__ taps,
                                                            const float* __restrict__ frac, int n_rows, int E,
                                                            bf16_t* __restrict__ out, int64_t ldo) {
#pragma clang fp contract(off)
  const int chunks = E >> 3;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)n_rows * chunks) return;
  const int r = (int)(idx / chunks), c = (int)(idx - (int64_t)r * chunks);
  const i32x4_t t = *(const i32x4_t*)(taps + 4 * (int64_t)r);
  const float ly = frac[2 * (int64_t)r], lx = frac[2 * (int64_t)r + 1];
  bf16_t* dst = out + (int64_t)r * ldo + c * 8;
  bool ok = true;
#pragma unroll
  for (int k = 0; k < 4; ++k) ok = ok && t[k] >= 0 && t[k] < n_src;
  bf16x8_t o;
  if (!ok) {
#pragma unroll
    for (int q = 0; q < 8; ++q) o[q] = f2bf(0.f);
  } else if (ly == 0.f && lx == 0.f) {
    o = *(const bf16x8_t*)(src + (int64_t)t[0] * lds + c * 8);
  } else {
    const bf16x8_t a00 = *(const bf16x8_t*)(src + (int64_t)t[0] * lds + c * 8);
    const bf16x8_t a01 = *(const bf16x8_t*)(src + (int64_t)t[1] * lds + c * 8);
    const bf16x8_t a10 = *(const bf16x8_t*)(src + (int64_t)t[2] * lds + c * 8);
    const bf16x8_t a11 = *(const bf16x8_t*)(src + (int64_t)t[3] * lds + c * 8);
    const float hy = 1.f - ly, hx = 1.f - lx;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const float top = hx * bf2f(a00[q]) + lx * bf2f(a01[q]);
      const float bot = hx * bf2f(a10[q]) + lx * bf2f(a11[q]);
      o[q] = f2bf(hy * top + ly * bot);
    }
  }
  *(bf16x8_t*)dst = o;
}

template <typename V>
__global__ __launch_bounds__(256) void row_gather_kernel(const char* __restrict__ in, int64_t in_stride,
                                                         const int32_t* __restrict__ rows,
                                                         char* __restrict__ out, int64_t out_stride, int n_rows,
                                                         int n_vec) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n_rows) return;
  const V* src = (const V*)(in + (int64_t)rows[row] * in_stride);
  V* dst = (V*)(out + (int64_t)row * out_stride);
  for (int i = lane; i < n_vec; i += 64) dst[i] = src[i];
}

// In-place rotary on the q and k column blocks of a packed [L, 3*heads*d] buffer.  One thread owns
// VEC (8, or 4 when d/2 is not a multiple of 8) consecutive j of one (row, head) in BOTH q and k: it fetches the
// cosines and sines once, reads x[j..j+VEC) and x[d/2+j..) of q and of k, rotates in fp32 and writes the halves back
// with a single bf16 rounding.  Work items are numbered with 32 bits (checked on the host).
template <int VEC>
__global__ __launch_bounds__(256) void rope_qk_kernel(bf16_t* __restrict__ qkv, int64_t ld,
                                                      const float* __restrict__ cos_sin, int L, int heads, int d) {
  typedef __attribute__((__vector_size__(VEC * sizeof(__bf16)))) __bf16 vec_t;
  const int half = d >> 1;
  const unsigned cpr = (unsigned)half / VEC;  // chunks per (row, head)
  const unsigned per_row = (unsigned)heads * cpr;
  const unsigned total = (unsigned)L * per_row;
  const unsigned idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const unsigned l = idx / per_row, rem = idx - l * per_row;
  const unsigned h = rem / cpr, jc = rem - h * cpr;
  bf16_t* qb = qkv + (int64_t)l * ld + h * d + jc * VEC;
  bf16_t* kb = qb + heads * d;
  const float* cs = cos_sin + (int64_t)l * d + jc * VEC;
  const vec_t q1 = *(const vec_t*)qb, q2 = *(const vec_t*)(qb + half);
  const vec_t k1 = *(const vec_t*)kb, k2 = *(const vec_t*)(kb + half);
  float co[VEC], si[VEC];
#pragma unroll
  for (int e = 0; e < VEC; e += 4) {
    const f32x4_t c = *(const f32x4_t*)(cs + e), s = *(const f32x4_t*)(cs + half + e);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      co[e + q] = c[q];
      si[e + q] = s[q];
    }
  }
  vec_t o1, o2, p1, p2;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const float a = bf2f(q1[e]), b = bf2f(q2[e]);
    o1[e] = f2bf(rot_first(a, b, co[e], si[e]));
    o2[e] = f2bf(rot_second(a, b, co[e], si[e]));
    const float c = bf2f(k1[e]), g = bf2f(k2[e]);
    p1[e] = f2bf(rot_first(c, g, co[e], si[e]));
    p2[e] = f2bf(rot_second(c, g, co[e], si[e]));
  }
  *(vec_t*)qb = o1;
  *(vec_t*)(qb + half) = o2;
  *(vec_t*)kb = p1;
  *(vec_t*)(kb + half) = p2;
}

}  // namespace

extern "C" int cs_abi_version(void) { return CS_ABI_VERSION; }

extern "C" int cs_vit_seqlens_host(const int64_t* grid_thw_host, int32_t n_items, int32_t merge, int32_t win,
                                   int32_t* cu_window_host, int32_t cap_window, int32_t* n_cu_window,
                                   int32_t* cu_full_host, int32_t cap_full, int32_t* n_cu_full,
                                   int32_t* item_meta_host, int64_t* total_patches) {
  if (!grid_thw_host || n_items < 0 || merge <= 0 || win <= 0 || !cu_window_host || !cu_full_host ||
      !n_cu_window || !n_cu_full || !item_meta_host || !total_patches || cap_window < 1 || cap_full < 1)
    return CS_ERR_INVALID_ARG;
  const int64_t mm = (int64_t)merge * merge;
  int nw = 0, nf = 0;
  cu_window_host[nw++] = 0;
  cu_full_host[nf++] = 0;
  int64_t unit_base = 0, cu_w = 0, cu_f = 0;
  for (int i = 0; i < n_items; ++i) {
    const int64_t t = grid_thw_host[3 * i], h = grid_thw_host[3 * i + 1], w = grid_thw_host[3 * i + 2];
    if (t <= 0 || h <= 0 || w <= 0 || h % merge || w % merge) return CS_ERR_INVALID_ARG;
    const int64_t gh = h / merge, gw = w / merge;
    if ((unit_base + t * gh * gw) * mm > INT32_MAX) return CS_ERR_TOO_LARGE;
    // The reference pads by win - n % win, i.e. a full extra (empty) window when n divides evenly
    // (qwen2_5_vl.py:367-370); empty windows repeat the running total and unique_consecutive (:436)
    // drops the repeats.  Walk the padded window grid literally and drop repeats the same way.
    const int64_t nwh = (gh + (win - gh % win)) / win, nww = (gw + (win - gw % win)) / win;
    for (int64_t f = 0; f < t; ++f) {
      for (int64_t wr = 0; wr < nwh; ++wr) {
        const int64_t rh = gh - wr * win < 0 ? 0 : (gh - wr * win < win ? gh - wr * win : win);
        for (int64_t wc = 0; wc < nww; ++wc) {
          const int64_t cw = gw - wc * win < 0 ? 0 : (gw - wc * win < win ? gw - wc * win : win);
          cu_w += rh * cw * mm;
          if ((int64_t)cu_window_host[nw - 1] != cu_w) {
            if (nw >= cap_window) return CS_ERR_TOO_LARGE;
            cu_window_host[nw++] = (int32_t)cu_w;
          }
        }
      }
      // one full-attention segment per frame (qwen2_5_vl.py:445-448)
      cu_f += h * w;
      if (nf >= cap_full) return CS_ERR_TOO_LARGE;
      cu_full_host[nf++] = (int32_t)cu_f;
    }
    int32_t* m = item_meta_host + 8 * i;
    m[0] = (int32_t)t;
    m[1] = (int32_t)gh;
    m[2] = (int32_t)gw;
    m[3] = (int32_t)unit_base;
    m[4] = (int32_t)((gh + win - 1) / win);
    m[5] = (int32_t)((gw + win - 1) / win);
    m[6] = (int32_t)(unit_base * mm);
    m[7] = (int32_t)unit_base;
    unit_base += t * gh * gw;
  }
  *n_cu_window = nw;
  *n_cu_full = nf;
  *total_patches = unit_base * mm;
  return CS_OK;
}

extern "C" int cs_vit_index(const int32_t* item_meta, int32_t n_items, int32_t max_units_per_item,
                            int32_t merge, int32_t win, const float* inv_freq, int32_t rot_dim,
                            int32_t* window_index, int32_t* reverse_index, int32_t* src_rows, int32_t* pos_ids,
                            float* cos_sin, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!item_meta || n_items < 0 || max_units_per_item < 0 || merge <= 0 || win <= 0) return CS_ERR_INVALID_ARG;
  if (cos_sin && (!inv_freq || rot_dim <= 0 || rot_dim % 2)) return CS_ERR_INVALID_ARG;
  if (n_items == 0 || max_units_per_item == 0) return CS_OK;
  if (n_items > 65535) return CS_ERR_TOO_LARGE;
  const int64_t max_patches = (int64_t)max_units_per_item * merge * merge;
  const dim3 grid((unsigned)((max_patches + 255) / 256), n_items), block(256);
  hipLaunchKernelGGL(vit_index_kernel, grid, block, 0, stream, (const ItemMeta*)item_meta, merge, win, inv_freq,
                     rot_dim, window_index, reverse_index, src_rows, pos_ids, cos_sin);
  return cs_launch_status();
}

extern "C" int cs_pos_embed_interp(const void* table, int32_t side, int32_t E, const int32_t* item_meta, int32_t n_items,
                                   int32_t max_units_per_item, int32_t merge, void* out, int64_t ldo, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!table || !item_meta || !out || side <= 0 || E <= 0 || E % 8 || n_items < 0 || max_units_per_item < 0 || merge <= 0 ||
      ldo < E || ldo % 8 || (((uintptr_t)table | (uintptr_t)out) & 15))
    return CS_ERR_INVALID_ARG;
  if (n_items == 0 || max_units_per_item == 0) return CS_OK;
  if (n_items > 65535) return CS_ERR_TOO_LARGE;
  const int64_t work = (int64_t)max_units_per_item * merge * merge * (E / 8);
  if (work > 0x7fffff00) return CS_ERR_TOO_LARGE;   // the kernel indexes its work with 32 bits
  const dim3 grid((unsigned)((work + 255) / 256), n_items), block(256);
  hipLaunchKernelGGL(pos_embed_interp_kernel, grid, block, 0, stream, (const bf16_t*)table, side, E,
                     (const ItemMeta*)item_meta, merge, (bf16_t*)out, ldo);
  return cs_launch_status();
}

extern "C" int cs_rows_bilinear(const void* src, int64_t lds, int32_t n_src_rows, const int32_t* taps, const float* frac,
                                int32_t n_rows, int32_t E, void* out, int64_t ldo, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n_rows < 0 || n_src_rows < 0 || E <= 0 || E % 8 || lds < E || lds % 8 || ldo < E || ldo % 8) return CS_ERR_INVALID_ARG;
  if (n_rows == 0) return CS_OK;
  if (!src || !taps || !frac || !out || (((uintptr_t)src | (uintptr_t)out | (uintptr_t)taps) & 15) || ((uintptr_t)frac & 3))
    return CS_ERR_INVALID_ARG;
  const int64_t work = (int64_t)n_rows * (E / 8);
  if ((work + 255) / 256 > 0x7fffffff) return CS_ERR_TOO_LARGE;
  hipLaunchKernelGGL(rows_bilinear_kernel, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, stream, (const bf16_t*)src,
                     lds, n_src_rows, taps, frac, n_rows, E, (bf16_t*)out, ldo);
  return cs_launch_status();
}

extern "C" int cs_row_gather(const void* in, int64_t in_stride_bytes, const int32_t* rows, void* out,
                             int64_t out_stride_bytes, int32_t n_rows, int32_t row_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (n_rows < 0 || row_bytes <= 0 || row_bytes % 4 || in_stride_bytes % 4 || out_stride_bytes % 4)
    return CS_ERR_INVALID_ARG;
  if (n_rows == 0) return CS_OK;  // an empty gather may come with null buffers
  if (!in || !rows || !out) return CS_ERR_INVALID_ARG;
  const dim3 grid((n_rows + 3) / 4), block(256);
  const bool v16 = !(row_bytes % 16) && !(in_stride_bytes % 16) && !(out_stride_bytes % 16) &&
                   !(((uintptr_t)in | (uintptr_t)out) & 15);
  if (v16)
    hipLaunchKernelGGL(row_gather_kernel<i32x4_t>, grid, block, 0, stream, (const char*)in, in_stride_bytes, rows,
                       (char*)out, out_stride_bytes, n_rows, row_bytes / 16);
  else
    hipLaunchKernelGGL(row_gather_kernel<int>, grid, block, 0, stream, (const char*)in, in_stride_bytes, rows,
                       (char*)out, out_stride_bytes, n_rows, row_bytes / 4);
  return cs_launch_status();
}

extern "C" int cs_rope_qk(void* qkv, int64_t ld, const float* cos_sin, int32_t L, int32_t heads, int32_t head_dim,
                          void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!qkv || !cos_sin || L < 0 || heads <= 0 || head_dim <= 0 || head_dim % 8 || ld % 8 ||
      ld < (int64_t)3 * heads * head_dim || (((uintptr_t)qkv | (uintptr_t)cos_sin) & 15))
    return CS_ERR_INVALID_ARG;
  if (L == 0) return CS_OK;
  const int vec = head_dim % 16 == 0 ? 8 : 4;   // d/2 is a multiple of 4 only for head dim 72: 8-byte vectors
  const int64_t total = (int64_t)L * heads * (head_dim / 2 / vec);
  if (total > 0x7fffff00) return CS_ERR_TOO_LARGE;   // the kernel numbers its work items with 32 bits
  const dim3 grid((unsigned)((total + 255) / 256)), block(256);
  if (vec == 8)
    hipLaunchKernelGGL(rope_qk_kernel<8>, grid, block, 0, stream, (bf16_t*)qkv, ld, cos_sin, L, heads, head_dim);
  else
    hipLaunchKernelGGL(rope_qk_kernel<4>, grid, block, 0, stream, (bf16_t*)qkv, ld, cos_sin, L, heads, head_dim);
  return cs_launch_status();
}
