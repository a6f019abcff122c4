// The 256x160 tile form (4x1 waves) of the fast bf16 / fp8-weight MFMA GEMM: every epilogue and folded-norm
// variant of this tile shape.  The accumulators live in accumulation registers that only inline assembly touches
// (CS_ALL_ACC_REGS: the build checks this file's compiler output for stray uses of them).
#include "gemm_fast_impl.h"

int cs_gemm_fast_tile_256x160(const CsGemmArgs& a, hipStream_t stream) { return dispatch_epi<256, 160, 4, 1>(a, stream); }
