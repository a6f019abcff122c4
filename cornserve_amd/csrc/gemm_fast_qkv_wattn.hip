// QKV projection with rotary and window attention as its epilogue: the 256x256 tile with one window of up to 64 rows per
// wavefront (waves 4 x 1) and one head per column tile.  The kernel is gemm_fast_kernel (gemm_fast_impl.h).  The
// accumulators live in accumulation registers that only inline assembly touches (CS_ALL_ACC_REGS: the build checks this
// file's compiler output for stray uses of them).
#include "gemm_fast_impl.h"

extern "C" int cs_qkv_window_attn(const CsGemmArgs* gemm, const float* cos_sin, float scale, int32_t heads,
                                  int32_t head_dim, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!gemm || !cos_sin || heads <= 0) return CS_ERR_INVALID_ARG;
  CsGemmArgs a = *gemm;
  if (!a.A || !a.W || !a.C || !a.bias || a.M < 0 || a.K <= 0) return CS_ERR_INVALID_ARG;
  const bool ragged = a.attn_win_start != nullptr;
  if (ragged ? (a.attn_n_win < 1 || a.M < 4 * a.attn_n_win || a.M > 64 * (int64_t)a.attn_n_win || a.M % 4) : a.attn_n_win != 0)
    return CS_ERR_INVALID_ARG;
  if (head_dim != 80 || a.N != heads * 256 || (!ragged && a.M % 64) || a.K % csgemm::BK || a.K < 3 * csgemm::BK) return CS_ERR_UNSUPPORTED;
  if (a.residual || a.pos || a.a_rows || a.c_rows || a.c_row_sumsq || a.a_row_sum || a.c_row_sum || a.c_lo || a.residual_lo ||
      a.conv_patch)
    return CS_ERR_INVALID_ARG;
  // fp8 weights: e4m3 bytes packed like the bf16 rows, with their per-output-channel scales packed like the bias; no
  // folded norm with them (as for cs_gemm)
  if (a.w_fp8 ? (!a.w_scale || ((uintptr_t)a.w_scale & 15)) : (a.w_scale != nullptr)) return CS_ERR_INVALID_ARG;
  if (a.w_fp8 && a.a_row_sumsq) return CS_ERR_UNSUPPORTED;
  if (a.lda % 8 || a.ldw % (a.w_fp8 ? 16 : 8) || a.ldc % 4 || a.ldc < heads * 80) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)a.A | (uintptr_t)a.W | (uintptr_t)cos_sin | (uintptr_t)a.a_row_sumsq) & 15) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)a.C | (uintptr_t)a.bias) & 7) return CS_ERR_INVALID_ARG;
  if (a.prefetch ? (((uintptr_t)a.prefetch & 15) || a.prefetch_bytes < 0) : a.prefetch_bytes != 0) return CS_ERR_INVALID_ARG;
  // per-lane source offsets of the direct loads are 32-bit byte offsets from the matrix bases
  if ((int64_t)a.M * a.lda * 2 >= (int64_t)UINT32_MAX || (int64_t)a.N * a.ldw * (a.w_fp8 ? 1 : 2) >= (int64_t)UINT32_MAX)
    return CS_ERR_UNSUPPORTED;
  if (a.M == 0) return CS_OK;
  a.attn_cos_sin = cos_sin;
  a.attn_scale_log2e = scale * 1.4426950408889634f;
  a.epilogue = CS_EPI_BIAS;
  if (ragged) {
    if ((uintptr_t)a.attn_win_start & 3 || (int64_t)a.attn_n_win * 64 > INT32_MAX) return CS_ERR_INVALID_ARG;
    a.M = a.attn_n_win * 64;   // virtual rows: one 64-row slot per window
    if (a.w_fp8) return launch<256, 256, 4, 1, CS_EPI_QKV_WATTN_RAGGED, true, 0>(a, stream);
    if (a.a_row_sumsq) return launch<256, 256, 4, 1, CS_EPI_QKV_WATTN_RAGGED, false, FUSE_NORM_A>(a, stream);
    return launch<256, 256, 4, 1, CS_EPI_QKV_WATTN_RAGGED, false, 0>(a, stream);
  }
  if (a.w_fp8) return launch<256, 256, 4, 1, CS_EPI_QKV_WATTN, true, 0>(a, stream);
  if (a.a_row_sumsq) return launch<256, 256, 4, 1, CS_EPI_QKV_WATTN, false, FUSE_NORM_A>(a, stream);
  return launch<256, 256, 4, 1, CS_EPI_QKV_WATTN, false, 0>(a, stream);
}
