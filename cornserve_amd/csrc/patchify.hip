// Patch layout kernels (gfx950): strided patch gather for the SigLIP patch embedding, and uint8 frames ->
// normalised patch rows for the Qwen2-VL family.
//
// nn.Conv2d(C, E, kernel=stride=p, padding="valid") (eric/models/layers/siglip.py:30-36,94-95) over
// NCHW pixels equals a GEMM between the flattened non-overlapping patches and the [E, C*p*p] weight.
// This kernel lays the patches out as the GEMM's A operand: row m = (b, py, px), column (c, ky, kx),
// zero-padded to the leading dimension so the GEMM's 16-byte loads stay aligned (C*p*p = 588 is not a
// multiple of 8).  A workgroup takes a run of up to npx neighbouring patches of one patch row: it copies
// their C*p image-row segments (contiguous npx*p pixels each) into LDS with coalesced loads, then writes the
// npx output rows (one contiguous span of npx*ldo elements) with coalesced stores of V elements per lane,
// gathering the pairs from LDS.
#include "common.h"

namespace {

// P is the patch size as a constant (divisions by constants), or 0 for any even value; V = elements per store.
template <int P, int V>
__global__ __launch_bounds__(256) void patchify_kernel(const bf16_t* __restrict__ px, int C, int H, int W, int p_any,
                                                       int gh, int gw, int npx, int chunks,
                                                       bf16_t* __restrict__ out, int ldo) {
  extern __shared__ bf16x2_t band[];   // [C*p][n*p/2] pixel pairs
  const int p = P ? P : p_any;
  const int hp = p >> 1;
  unsigned wg = xcd_contiguous(blockIdx.x, gridDim.x);   // -> (image, patch row, run of patches); neighbours share an L2
  const int ch = wg % (unsigned)chunks;
  wg /= (unsigned)chunks;
  const int y = wg % (unsigned)gh, b = wg / (unsigned)gh;
  const int x0 = ch * npx;
  const int n = min(npx, gw - x0);
  const int hw = n * hp;               // pairs per image-row segment
  const int rows = C * p;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int r = wave; r < rows; r += 4) {   // one wave per image-row segment
    const int c = r / p, ky = r - c * p;
    const bf16_t* src = px + (((int64_t)b * C + c) * H + (y * p + ky)) * W + x0 * p;
    for (int xx = lane; xx < hw; xx += 64) band[r * hw + xx] = *(const bf16x2_t*)(src + 2 * xx);
  }
  __syncthreads();
  const int K = rows * p;
  const unsigned upr = (unsigned)ldo / V;   // stores per output row
  bf16_t* span = out + ((int64_t)(b * gh + y) * gw + x0) * ldo;
  for (unsigned i = threadIdx.x; i < (unsigned)n * upr; i += 256) {
    const int kp = i / upr;
    const int k0 = (int)(i - kp * upr) * V;
    int v[V / 2];
#pragma unroll
    for (int e = 0; e < V / 2; ++e) {
      const int k = k0 + 2 * e;   // output column -> (image-row segment c*p + ky, kx); a pair never straddles segments (p even)
      const int r = k / p, kx = k - r * p;
      v[e] = k < K ? __builtin_bit_cast(int, band[r * hw + kp * hp + (kx >> 1)]) : 0;   // bf16 zero is all-zero bits
    }
    bf16_t* dst = span + (int64_t)i * V;
    if constexpr (V == 8) {
      i32x4_t o = {v[0], v[1], v[2], v[3]};
      *(i32x4_t*)dst = o;
    } else {
      *(int*)dst = v[0];
    }
  }
}

// Qwen2-VL family: resized uint8 frames [T,H,W,3] -> the flat patch rows the encoder consumes, with the
// rescale + normalise step applied through a per-channel table of the 256 byte values (so the arithmetic of
// the caller's image processor is reproduced bit for bit whatever its operation order: the caller computes
// the table with it).  Rows are ordered (t, block row, block col, row in block, col in block) with blocks of
// merge x merge patches, columns (channel, temporal, y, x); temporal slot tt of row group t shows frame
// min(t*temporal + tt, T-1): an image is one frame repeated, a video's last frame is repeated to fill a group.
// One workgroup writes QP_ROWS output rows (a row's place in the frame is worked out once and kept in LDS, as is
// the table); a thread writes two neighbouring x at a time.
// This form takes any even patch size and any temporal size; the segment kernel below serves the usual ones.
constexpr int QP_ROWS = 8;
template <typename OUT>
__global__ __launch_bounds__(256) void qwen_patchify_u8_kernel(const uint8_t* __restrict__ frames, int T, int H, int W,
                                                               int p, int m, int tps, const float* __restrict__ table,
                                                               OUT* __restrict__ out, int64_t ldo, int rows) {
  __shared__ float lut[3 * 256];
  for (int i = threadIdx.x; i < 3 * 256; i += 256) lut[i] = table[i];
  __syncthreads();
  const int hp = p >> 1;
  const int pairs = 3 * tps * p * hp;
  // where each of this workgroup's rows sits in the frame: (first frame of the group, top pixel row, left pixel column)
  __shared__ int where[QP_ROWS][3];
  const int row0 = (int)xcd_contiguous(blockIdx.x, gridDim.x) * QP_ROWS;   // neighbouring rows share an L2
  const int n_rows = min(rows - row0, QP_ROWS);
  if (threadIdx.x < n_rows) {
    const int bw = W / (p * m), bh = H / (p * m);
    int r = row0 + threadIdx.x;   // output row -> (t, block row, block column, row in block, column in block)
    const int mx = r % m;
    r /= m;
    const int my = r % m;
    r /= m;
    const int bx = r % bw;
    r /= bw;
    const int by = r % bh;
    where[threadIdx.x][0] = (r / bh) * tps;
    where[threadIdx.x][1] = (by * m + my) * p;
    where[threadIdx.x][2] = (bx * m + mx) * p;
  }
  __syncthreads();
  // work item -> (row of the workgroup, channel, temporal slot, y, x pair), x fastest: 2*q is the output column
  for (int i = threadIdx.x; i < n_rows * pairs; i += 256) {
    const int k = i / pairs, q = i - k * pairs;
    const int xp = q % hp, q1 = q / hp;
    const int py = q1 % p, q2 = q1 / p;
    const int tt = q2 % tps, c = q2 / tps;
    const int f = min(where[k][0] + tt, T - 1);
    const uint8_t* src = frames + (((int64_t)f * H + (where[k][1] + py)) * W + (where[k][2] + 2 * xp)) * 3 + c;
    const float v0 = lut[c * 256 + src[0]], v1 = lut[c * 256 + src[3]];
    OUT* dst = out + (int64_t)(row0 + k) * ldo + 2 * q;
    if constexpr (sizeof(OUT) == 2) {
      bf16x2_t o;
      o[0] = f2bf(v0);
      o[1] = f2bf(v1);
      *(bf16x2_t*)dst = o;
    } else {
      dst[0] = v0;
      dst[1] = v1;
    }
  }
}

typedef uint32_t u32x4a_t __attribute__((ext_vector_type(4), aligned(4)));   // four words at 4-byte alignment

// The same operation for the usual patch sizes (P = 14, 16), organised by source segments: the 3*P bytes of one
// image row of one patch hold the P pixels of all three channels, i.e. three runs of P output values.  A workgroup
// takes a few output rows (seg_rows_per_workgroup) = rows * tps * P segments; it copies the aligned 4-byte words that cover every segment
// into LDS with coalesced loads (consecutive lanes take consecutive 16-byte pieces of a segment; every word loaded holds at
// least one byte of the frames, so no load leaves the allocation), then one lane per segment shifts its words into
// place, looks the 3*P bytes up in the table and stores the three runs.  About a fifth of the instructions per output
// value of the per-value kernel above.
// Output rows per workgroup of the segment kernel: with the usual temporal size 2 a row has 2 * P segments, and the
// workgroup has one lane per segment (P = 14: 9 rows = 252 segments, P = 16: 8 rows = 256).
constexpr int seg_rows_per_workgroup(int p) { return 256 / (2 * p); }

template <typename OUT, int P>
__global__ __launch_bounds__(256) void qwen_patchify_u8_seg_kernel(const uint8_t* __restrict__ frames, int T, int H, int W,
                                                                   int m, int tps, const float* __restrict__ table,
                                                                   OUT* __restrict__ out, int64_t ldo, int rows) {
  constexpr int ROWS = seg_rows_per_workgroup(P);
  constexpr int SEG = 3 * P;               // bytes per segment
  constexpr int NDW = (SEG + 3 + 3) / 4;   // words that cover a segment starting at byte 0..3 of a word
  constexpr int ND = (SEG + 3) / 4;        // words of a segment once shifted into place
  __shared__ float lut[3 * 256];
  __shared__ int where[ROWS][3];
  extern __shared__ __attribute__((aligned(16))) char dyn[];   // int64 segment offsets, then NDW words per segment
  for (int i = threadIdx.x; i < 3 * 256; i += 256) lut[i] = table[i];
  const int row0 = (int)xcd_contiguous(blockIdx.x, gridDim.x) * ROWS;   // neighbouring rows (patches of one image row) share an L2
  const int n_rows = min(rows - row0, ROWS);
  if (threadIdx.x < n_rows) {
    const int bw = W / (P * m), bh = H / (P * m);
    int r = row0 + threadIdx.x;   // output row -> (t, block row, block column, row in block, column in block)
    const int mx = r % m;
    r /= m;
    const int my = r % m;
    r /= m;
    const int bx = r % bw;
    r /= bw;
    const int by = r % bh;
    where[threadIdx.x][0] = (r / bh) * tps;
    where[threadIdx.x][1] = (by * m + my) * P;
    where[threadIdx.x][2] = (bx * m + mx) * P;
  }
  __syncthreads();
  const int spr = tps * P;              // segments per output row
  const int nseg = n_rows * spr;
  const int max_seg = (ROWS * spr + 1) & ~1;   // even: the words behind the offsets stay 16-byte aligned
  int64_t* segoff = (int64_t*)dyn;      // byte offset of each segment in frames
  uint32_t* words = (uint32_t*)(dyn + (size_t)max_seg * 8);
  for (int s = threadIdx.x; s < nseg; s += 256) {
    const int k = s / spr, rem = s - k * spr;
    const int tt = rem / P, py = rem - tt * P;
    const int f = min(where[k][0] + tt, T - 1);
    segoff[s] = (((int64_t)f * H + (where[k][1] + py)) * W + where[k][2]) * 3;
  }
  __syncthreads();
  // four words per lane and load (words need 4-byte alignment only); a chunk's tail is left out word by word where it
  // would lie past the segment's last byte
  constexpr int NCH = (NDW + 3) / 4;
  for (int i = threadIdx.x; i < nseg * NCH; i += 256) {
    const int s = i / NCH, q = i - s * NCH;
    const uintptr_t addr = (uintptr_t)frames + segoff[s];
    const int last = ((int)(addr & 3) + SEG - 1) >> 2;   // index of the last word that holds a byte of the segment
    const uint32_t* src = (const uint32_t*)(addr & ~(uintptr_t)3) + 4 * q;
    uint32_t* dst = words + s * NDW + 4 * q;
    const int n = min(last - 4 * q + 1, min(4, NDW - 4 * q));   // words of this chunk to fetch (>= 1 for the chunks of P = 14, 16)
    uint32_t w[4] = {0, 0, 0, 0};
    if (n >= 4) {
      const u32x4a_t v = *(const u32x4a_t*)src;
      w[0] = v[0], w[1] = v[1], w[2] = v[2], w[3] = v[3];
    } else {
      if (n > 0) w[0] = src[0];
      if (n > 1) w[1] = src[1];
      if (n > 2) w[2] = src[2];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (4 * q + j < NDW) dst[j] = w[j];
  }
  __syncthreads();
  for (int s = threadIdx.x; s < nseg; s += 256) {
    const int lead = (int)(((uintptr_t)frames + segoff[s]) & 3);
    uint32_t raw[NDW + 1], d[ND];
#pragma unroll
    for (int j = 0; j < NDW; ++j) raw[j] = words[s * NDW + j];
    raw[NDW] = 0;
#pragma unroll
    for (int j = 0; j < ND; ++j) d[j] = __builtin_amdgcn_alignbyte(raw[j + 1], raw[j], lead);   // bytes lead.. of (raw[j+1]:raw[j])
    const int k = s / spr, rem = s - k * spr;   // rem = tt * P + py: the run's place inside a channel's columns
    OUT* dst = out + (int64_t)(row0 + k) * ldo + rem * P;
#pragma unroll
    for (int c = 0; c < 3; ++c) {
      OUT* o = dst + c * spr * P;
#pragma unroll
      for (int x = 0; x < P; x += 2) {
        const int b0 = 3 * x + c, b1 = 3 * (x + 1) + c;
        const float v0 = lut[c * 256 + ((d[b0 >> 2] >> (8 * (b0 & 3))) & 255)];
        const float v1 = lut[c * 256 + ((d[b1 >> 2] >> (8 * (b1 & 3))) & 255)];
        if constexpr (sizeof(OUT) == 2) {
          bf16x2_t q;
          q[0] = f2bf(v0);
          q[1] = f2bf(v1);
          *(bf16x2_t*)(o + x) = q;
        } else {
          o[x] = v0;
          o[x + 1] = v1;
        }
      }
    }
  }
}

template <typename OUT>
void launch_qwen_patchify_u8(int rows, hipStream_t stream, const uint8_t* frames, int T, int H, int W, int p, int m,
                             int tps, const float* table, OUT* out, int64_t ldo) {
  const dim3 grid((unsigned)((rows + QP_ROWS - 1) / QP_ROWS)), block(256);
  // segment form: LDS for the offsets and words of the segments of a workgroup's rows
  const int seg_rows = (p == 14 || p == 16) ? seg_rows_per_workgroup(p) : 1;
  const size_t seg_lds = (size_t)((seg_rows * tps * p + 1) & ~1) * (8 + 4 * ((3 * p + 6) / 4));
  const dim3 seg_grid((unsigned)((rows + seg_rows - 1) / seg_rows));
  if (p == 14 && seg_lds <= 48 * 1024)
    hipLaunchKernelGGL((qwen_patchify_u8_seg_kernel<OUT, 14>), seg_grid, block, seg_lds, stream, frames, T, H, W, m, tps, table, out, ldo, rows);
  else if (p == 16 && seg_lds <= 48 * 1024)
    hipLaunchKernelGGL((qwen_patchify_u8_seg_kernel<OUT, 16>), seg_grid, block, seg_lds, stream, frames, T, H, W, m, tps, table, out, ldo, rows);
  else
    hipLaunchKernelGGL((qwen_patchify_u8_kernel<OUT>), grid, block, 0, stream, frames, T, H, W, p, m, tps, table, out, ldo, rows);
}

}  // namespace

extern "C" int cs_qwen_patchify_u8(const void* frames, int32_t T, int32_t H, int32_t W, int32_t patch, int32_t merge,
                                   int32_t temporal, const float* table, void* out, int64_t ldo, int32_t out_fp32,
                                   void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!frames || !table || !out || T < 0 || H <= 0 || W <= 0 || patch <= 0 || patch % 2 || merge <= 0 || temporal <= 0)
    return CS_ERR_INVALID_ARG;
  if (H % (patch * merge) || W % (patch * merge)) return CS_ERR_INVALID_ARG;
  const int64_t cols = (int64_t)3 * temporal * patch * patch;
  if (ldo < cols || ldo % 2 || ((uintptr_t)out & (out_fp32 ? 7 : 3)) || ((uintptr_t)table & 3)) return CS_ERR_INVALID_ARG;
  if (T == 0) return CS_OK;
  const int64_t rows = (int64_t)((T + temporal - 1) / temporal) * (H / patch) * (W / patch);
  if (rows > 0x7fffffff) return CS_ERR_TOO_LARGE;
  if (out_fp32)
    launch_qwen_patchify_u8<float>((int)rows, stream, (const uint8_t*)frames, T, H, W, patch, merge, temporal, table, (float*)out, ldo);
  else
    launch_qwen_patchify_u8<bf16_t>((int)rows, stream, (const uint8_t*)frames, T, H, W, patch, merge, temporal, table, (bf16_t*)out, ldo);
  return cs_launch_status();
}

extern "C" int cs_patchify_nchw(const void* pixels, int32_t B, int32_t C, int32_t H, int32_t W, int32_t patch,
                                void* out, int64_t ldo, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!pixels || !out || B < 0 || C <= 0 || H <= 0 || W <= 0 || patch <= 0 || patch % 2 || H < patch ||
      W < patch || W % 2 || ldo < (int64_t)C * patch * patch || ldo % 2 || (((uintptr_t)pixels | (uintptr_t)out) & 3))
    return CS_ERR_INVALID_ARG;
  if (B == 0) return CS_OK;
  const int gh = H / patch, gw = W / patch;
  if (ldo > 0x7fffffff / 16 || (int64_t)C * patch * patch > 0x7fffffff / 16) return CS_ERR_TOO_LARGE;
  // patches per workgroup: eight, fewer when the image-row segments of eight would not fit 64 KB of LDS
  int npx = 8;
  while (npx > 1 && (int64_t)C * patch * npx * patch * 2 > 65536) npx >>= 1;
  const int64_t lds = (int64_t)C * patch * npx * patch * 2;
  if (lds > 65536) return CS_ERR_TOO_LARGE;
  const int chunks = (gw + npx - 1) / npx;
  const int64_t wgs = (int64_t)B * gh * chunks;
  if (wgs > 0x7fffffff) return CS_ERR_TOO_LARGE;
  const bool wide = ldo % 8 == 0 && ((uintptr_t)out & 15) == 0;
  const dim3 grid((unsigned)wgs), block(256);
#define CS_PATCHIFY(P, V)                                                                                       \
  hipLaunchKernelGGL((patchify_kernel<P, V>), grid, block, (size_t)lds, stream, (const bf16_t*)pixels, C, H, W, \
                     patch, gh, gw, npx, chunks, (bf16_t*)out, (int)ldo)
  if (patch == 14) {
    if (wide) CS_PATCHIFY(14, 8); else CS_PATCHIFY(14, 2);
  } else if (patch == 16) {
    if (wide) CS_PATCHIFY(16, 8); else CS_PATCHIFY(16, 2);
  } else {
    if (wide) CS_PATCHIFY(0, 8); else CS_PATCHIFY(0, 2);
  }
#undef CS_PATCHIFY
  return cs_launch_status();
}
