// Fast-path bf16 MFMA GEMM for gfx950: choice of the tile form.  The kernel itself is in gemm_fast_impl.h; each tile
// form is built in its own translation unit (gemm_fast_t*.hip).
#include <stdlib.h>

#include "gemm_common.h"

// Epilogue / folded-norm dispatch of one tile form each (gemm_fast_t<rows>x<cols>.hip).
int cs_gemm_fast_tile_256x256(const CsGemmArgs& a, hipStream_t stream);
int cs_gemm_fast_tile_256x160(const CsGemmArgs& a, hipStream_t stream);
int cs_gemm_fast_tile_128x160(const CsGemmArgs& a, hipStream_t stream);
int cs_gemm_fast_tile_128x192(const CsGemmArgs& a, hipStream_t stream);
int cs_gemm_fast_tile_256x128(const CsGemmArgs& a, hipStream_t stream);

namespace {

using csgemm::BK;

// Time of a launch in units of "one 256x256 tile on every CU": rounds of 256 workgroups times tile area.
double rounds_cost(int M, int N, int bm, int bn) {
  const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  const int64_t rounds = (tiles + 255) / 256;
  return (double)rounds * bm * bn / (256.0 * 256.0);
}

}  // namespace

// Called by cs_gemm after argument validation.  Sets *handled when this path took the problem.
int cs_gemm_fast(const CsGemmArgs& a, hipStream_t stream, bool* handled) {
  *handled = false;
  if (a.M < 1 || a.N < 8) return CS_OK;
  if (a.w_fp8 ? (!a.w_scale || a.pos) : (a.w_scale != nullptr)) return CS_OK;
  if (a.K % BK || a.K < 3 * BK) return CS_OK;  // the ring pipeline is written for at least three K tiles
  if (a.N % 8 || a.ldc % 8 || ((uintptr_t)a.C & 15)) return CS_OK;  // 16-byte output stores
  if (a.pos && a.epilogue != CS_EPI_BIAS) return CS_OK;  // the position addend only pairs with the plain epilogue here
  if (a.a_rows) return CS_OK;  // gathered A rows can lie anywhere: the general kernel keeps 64-bit pointers
  // per-lane source offsets are 32-bit byte offsets from the matrix bases
  if ((int64_t)a.M * a.lda * 2 >= (int64_t)UINT32_MAX || (int64_t)a.N * a.ldw * (a.w_fp8 ? 1 : 2) >= (int64_t)UINT32_MAX)
    return CS_OK;
  *handled = true;
  // Tile shape: the one that needs the least chip time (tile quantisation over the 256 CUs).  The narrow
  // 256x160 tile exists for N = 1280 (8 column tiles: 8192 rows give exactly 256 workgroups).
  const double c256 = rounds_cost(a.M, a.N, 256, 256);
  const double c160 = rounds_cost(a.M, a.N, 256, 160) * 1.15;  // narrower tiles: more LDS and L2 traffic per FLOP
  // Few rows: 160-column tiles of 256 rows would leave half of the compute units or more without a tile (N = 1280
  // gives 8 column tiles, so 1024 rows are 32 workgroups).  The 128x160 form has the same waves-by-columns layout,
  // so every output element and every row-sum part is computed by the same sequence of operations: results do not
  // depend on which of the two a batch size selects.
  const bool few_rows = !a.w_fp8 && (int64_t)((a.M + 255) / 256) * ((a.N + 159) / 160) <= 128;
  auto narrow = [&]() { return few_rows ? cs_gemm_fast_tile_128x160(a, stream) : cs_gemm_fast_tile_256x160(a, stream); };
  // Row sums of squares come in CS_SUMSQ_PARTS parts, one per column tile of the 160-column forms.
  if (a.c_row_sumsq) {
    if (a.N > CS_SUMSQ_PARTS * 160 || a.w_fp8) return CS_ERR_UNSUPPORTED;
    return narrow();
  }
  if (a.a_row_sum) return narrow();   // see dispatch_epi_w
  // Few rows and many columns: when 256x128 tiles fit in one round they put more compute units to work than the
  // forms above (1024 rows x 6912 columns: 216 workgroups against 176 of 256x160 or 108 of 256x256), and a launch
  // of one round is bound by what a single compute unit pulls in per K tile, not by the chip's throughput.  The
  // accumulation order of an output element is the same in every tile form, so the choice changes no bit.  Taken
  // for the SwiGLU epilogue only, where it measures faster inside the model (gate|up of one image); the QKV
  // projection of two images (240 workgroups against 192) is faster alone and slower in the model.
  if (a.epilogue == CS_EPI_SWIGLU) {
    const int64_t t128 = (int64_t)((a.M + 255) / 256) * ((a.N + 127) / 128);
    const double c128 = rounds_cost(a.M, a.N, 256, 128) * 1.10;
    if (t128 <= 256 && !few_rows && c128 < c160 - 0.05 && c128 < c256 - 0.05) return cs_gemm_fast_tile_256x128(a, stream);
  }
  if (c160 < c256) return narrow();
  // Column split.  When the last round of 256x256 tiles would leave most CUs idle, the leading columns
  // that fill whole rounds go to one launch and the remaining columns to a second launch with smaller
  // tiles (256x128 or 128x192: more workgroups, each shorter).  The two launches write disjoint column
  // ranges of C.
  {
    const int tn = (a.N + 255) / 256;
    double best = c256;
    int best_cols = 0;
    bool best_192 = false;
    for (int c = tn - 1; c >= 1 && c >= tn - 12; --c) {
      const int rest = a.N - c * 256;
      const double lead = rounds_cost(a.M, c * 256, 256, 256);
      const double c128 = lead + rounds_cost(a.M, rest, 256, 128) * 1.10 + 0.15;  // + per-tile fixed cost of a round
      const double c192 = lead + rounds_cost(a.M, rest, 128, 192) * 1.20 + 0.15;
      if (c128 < best - 0.05) {
        best = c128;
        best_cols = c;
        best_192 = false;
      }
      if (c192 < best - 0.02) {
        best = c192;
        best_cols = c;
        best_192 = true;
      }
    }
    if (best_cols > 0) {
      const int n1 = best_cols * 256;
      CsGemmArgs lo = a, hi = a;
      lo.N = n1;
      lo.prefetch = nullptr;  // the tail launch is the one with idle compute units
      hi.N = a.N - n1;
      hi.W = (const char*)a.W + (int64_t)n1 * a.ldw * (a.w_fp8 ? 1 : 2);
      if (a.w_scale) hi.w_scale = a.w_scale + n1;
      if (a.bias) hi.bias = (const char*)a.bias + (int64_t)n1 * 2;
      if (a.residual) hi.residual = (const char*)a.residual + (int64_t)n1 * 2;
      if (a.residual_lo) hi.residual_lo = a.residual_lo + n1;
      if (a.c_lo) hi.c_lo = a.c_lo + n1;
      if (a.pos) hi.pos = (const char*)a.pos + (int64_t)n1 * 2;
      hi.C = (char*)a.C + (int64_t)(a.epilogue == CS_EPI_SWIGLU ? n1 / 2 : n1) * 2;
      const int st = cs_gemm_fast_tile_256x256(lo, stream);
      if (st != CS_OK) return st;
      if (best_192) return cs_gemm_fast_tile_128x192(hi, stream);
      return cs_gemm_fast_tile_256x128(hi, stream);
    }
  }
  return cs_gemm_fast_tile_256x256(a, stream);
}
