// The 256x128 tile form (2x2 waves) of the fast bf16 / fp8-weight MFMA GEMM: every epilogue and folded-norm
// variant of this tile shape.  The accumulators live in accumulation registers that only inline assembly touches
// (CS_ALL_ACC_REGS: the build checks this file's compiler output for stray uses of them).
#include "gemm_fast_impl.h"

int cs_gemm_fast_tile_256x128(const CsGemmArgs& a, hipStream_t stream) { return dispatch_epi<256, 128, 2, 2>(a, stream); }
