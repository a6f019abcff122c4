// RMSNorm-folded GEMM for callers that cannot allocate: the per-row sums of squares that cs_gemm takes as a
// workspace argument (CsGemmArgs.a_row_sumsq, filled by cs_row_sumsq) live in a static device array of this library
// instead.  Same kernels, same arguments otherwise; nothing is allocated or freed here.
#include <mutex>

#include "common.h"

namespace {

// Partial results passed from the row-sums launch to the GEMM launch: fp32 [CS_NOALLOC_MAX_ROWS][CS_SUMSQ_PARTS].
// Every GPU the library runs on holds its own copy of this array (at its own address) until the process ends.
static __device__ __align__(256) float scratch[(size_t)CS_NOALLOC_MAX_ROWS * CS_SUMSQ_PARTS];

// `scratch` in host code is only a handle of the symbol, not a device address: the address on each device is
// looked up once, with that device current, and every launch gets the looked-up pointer.
constexpr int MAX_DEVICES = 64;
float* scratch_ptr[MAX_DEVICES];
std::once_flag scratch_once[MAX_DEVICES];
hipError_t scratch_err[MAX_DEVICES];

float* scratch_on_current_device(int* status) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    *status = CS_ERR_LAUNCH;
    return nullptr;
  }
  std::call_once(scratch_once[dev], [dev]() {
    void* p = nullptr;
    scratch_err[dev] = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    scratch_ptr[dev] = scratch_err[dev] == hipSuccess ? (float*)p : nullptr;
  });
  if (scratch_err[dev] != hipSuccess || !scratch_ptr[dev]) {
    *status = CS_ERR_LAUNCH;
    return nullptr;
  }
  *status = CS_OK;
  return scratch_ptr[dev];
}

}  // namespace

extern "C" int cs_gemm_rmsnorm_noalloc(const CsGemmArgs* args, void* stream) {
  if (!args) return CS_ERR_INVALID_ARG;
  // The library supplies the row sums: the caller must not, and A must be a plain matrix whose K columns are the
  // normalised width (no row gather: the sums are taken over A's own rows 0..M-1).
  if (args->a_row_sumsq || args->a_row_sum || args->a_rows || args->w_fp8) return CS_ERR_INVALID_ARG;
  if (args->M < 0 || args->K <= 0 || args->N <= 0) return CS_ERR_INVALID_ARG;
  if (args->M > CS_NOALLOC_MAX_ROWS) return CS_ERR_TOO_LARGE;
  if (args->K > 160 * CS_SUMSQ_PARTS) return CS_ERR_TOO_LARGE;
  // Everything cs_gemm would refuse for a folded-norm launch is refused HERE, before the row-sums launch is
  // enqueued: the folded form exists in the direct-to-LDS kernel only (K a multiple of 64 and at least 192, N a
  // multiple of 8, 16-byte aligned rows of C), with the plain-bias and the SiLU-gate epilogues, and without the
  // position addend or output row sums.
  if (!args->A || !args->W || !args->C) return CS_ERR_INVALID_ARG;
  if (args->K % 64 || args->K < 192) return CS_ERR_UNSUPPORTED;
  if (args->epilogue != CS_EPI_BIAS && args->epilogue != CS_EPI_SWIGLU) return CS_ERR_UNSUPPORTED;
  if (args->pos || args->c_row_sumsq || args->c_row_sum || args->w_col_sum || args->w_scale || args->conv_patch ||
      args->c_lo || args->residual_lo)
    return CS_ERR_UNSUPPORTED;
  if (args->N < 8 || args->N % 8 || args->ldc % 8 || args->lda % 8 || args->ldw % 8) return CS_ERR_UNSUPPORTED;
  if ((((uintptr_t)args->A | (uintptr_t)args->W | (uintptr_t)args->C) & 15) || ((uintptr_t)args->bias & 7))
    return CS_ERR_INVALID_ARG;
  if ((int64_t)args->M * args->lda * 2 >= (int64_t)UINT32_MAX || (int64_t)args->N * args->ldw * 2 >= (int64_t)UINT32_MAX)
    return CS_ERR_UNSUPPORTED;
  int st = CS_OK;
  float* sums = scratch_on_current_device(&st);
  if (!sums) return st;
  // cs_row_sumsq writes all CS_SUMSQ_PARTS parts of rows 0..M-1 (zeros beyond K), so nothing of an earlier call's
  // contents is read: no clearing is needed.
  st = cs_row_sumsq(args->A, args->lda, args->M, args->K, sums, stream);
  if (st != CS_OK) return st;
  CsGemmArgs a = *args;
  a.a_row_sumsq = sums;
  return cs_gemm(&a, stream);
}
