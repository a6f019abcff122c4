// bf16 MFMA GEMM for gfx950:  C[M,N] = epilogue( A[M,K] . W[N,K]^T )
//
// This is the F.linear of the Eric encoders (reference: eric/models/layers/linear.py:179-188 and
// :537-554 at TP=1 are plain F.linear(x, W, b)).  Both operands are K-contiguous, which is the native
// operand form of v_mfma_f32_32x32x16_bf16 (8 consecutive k per lane), so no transposes are needed.
//
// Work decomposition: one 512-thread workgroup (8 waves, 2 per SIMD) owns a BM x BN tile of C and
// walks K in steps of 64.  Tiles are staged global -> registers -> LDS (XOR-swizzled 16-byte chunks,
// conflict-free for both the 16 B writes and the MFMA fragment reads), double buffered so the global
// loads of step k+1 are in flight while step k is on the matrix cores.  W is fed as the MFMA "A"
// operand and the activations as "B", so that each lane ends up owning one row m of C and groups of 4
// consecutive columns n: epilogues that pair adjacent columns (SwiGLU on interleaved gate|up) and
// 8-byte packed stores fall out of that.
//
// Epilogues (all optional-bias, fp32 accumulate; an activation takes the fp32 sum and the result is rounded once,
// where the reference, computing in bf16, also rounds the linear layer's output in between):
//   EPI_BIAS       y = bf16(acc + b)
//   EPI_RESIDUAL   y = bf16( bf16(acc + b) + r )                     (qwen2_5_vl.py:175,177)
//   EPI_SWIGLU     y[j] = bf16( silu(acc[2j]+b[2j]) * (acc[2j+1]+b[2j+1]) )   (qwen2_5_vl.py:143-148)
//   EPI_GELU_ERF   y = bf16(gelu_erf(acc + b))                       (qwen2_5_vl.py:218-222)
//   EPI_GELU_TANH  y = bf16(gelu_tanh(acc + b))                      (siglip.py:155-163)
// plus an optional fp32 per-output-channel scale applied to acc (fp8-e4m3 weights, W_FP8 = true), an
// optional gather of A rows (a_rows) and scatter of C rows (c_rows) used to fuse the window permutation
// (qwen2_5_vl.py:438-440) and its inverse (:478-479) into the neighbouring GEMMs, and an optional second
// residual-like addend indexed by (row % pos_period) for the SigLIP position embedding (siglip.py:100).
#include "gemm_common.h"

int cs_gemm_fast(const CsGemmArgs& a, hipStream_t stream, bool* handled);

namespace {

using namespace csgemm;
constexpr int NTHREADS = 512;    // 8 waves
constexpr int WAVES_M = 2;
constexpr int WAVES_N = 4;

// 16 fp8-e4m3 (OCP) values -> 16 bf16.  Conversion is exact: every e4m3 value is representable in bf16.
CS_DEVICE void fp8x16_to_bf16(const i32x4_t& in, bf16x8_t& lo, bf16x8_t& hi) {
  float f[16];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    auto p0 = __builtin_amdgcn_cvt_pk_f32_fp8(in[i], false);
    auto p1 = __builtin_amdgcn_cvt_pk_f32_fp8(in[i], true);
    f[4 * i + 0] = p0[0];
    f[4 * i + 1] = p0[1];
    f[4 * i + 2] = p1[0];
    f[4 * i + 3] = p1[1];
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    lo[i] = (bf16_t)f[i];
    hi[i] = (bf16_t)f[8 + i];
  }
}

// CONV: the activation operand is gathered from NCHW pixels (a convolution with stride = kernel; see CsGemmArgs.conv_patch):
// row m is a patch, its K elements are the patch's pixels in (c, ky, kx) order, fetched as 4-byte pixel pairs.
template <int BM, int BN, int EPI, bool W_FP8, bool CONV = false>
__global__ __launch_bounds__(NTHREADS) void gemm_kernel(const CsGemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const bf16_t* const pA = (const bf16_t*)p.A;
  constexpr int A_BYTES = BM * BK * 2;
  constexpr int W_BYTES = BN * BK * 2;
  constexpr int STAGE = A_BYTES + W_BYTES;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int MT = WTM / 32, NT = WTN / 32;
  constexpr int A_ITERS = BM / 64;                    // 16 B chunks per thread per stage (A)
  constexpr int W_ITERS = W_FP8 ? BN / 128 : BN / 64; // fp8: one 16 B load carries two bf16 chunks

  // ---- tile coordinates: XCD-aware remap, then bands of 8 tile-rows walked column-major so the 32
  //      workgroups resident on one XCD share 8 A panels and 4 W panels through that XCD's L2.
  const int nb = gridDim.x;
  int bid = blockIdx.x;
  {
    const int per = nb >> 3;
    if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  }
  constexpr int GM = 8;
  const int band_sz = GM * p.tiles_n;
  const int band = bid / band_sz;
  const int within = bid - band * band_sz;
  const int rows_in_band = min(GM, p.tiles_m - band * GM);
  const int tm = band * GM + within % rows_in_band;
  const int tn = within / rows_in_band;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;

  // ---- global -> LDS staging assignment: thread -> (row r0 + 64*i, chunk c)
  const int ld_c = tid & 7;
  const int ld_r = tid >> 3;
  const bf16_t* a_ptr[A_ITERS];
  const int conv_pw = CONV ? p.conv_w / p.conv_patch : 1;                   // patches per image row
  const int conv_pi = CONV ? (p.conv_h / p.conv_patch) * conv_pw : 1;       // patches per image
  const int conv_kreal = CONV ? p.conv_c * p.conv_patch * p.conv_patch : 0;
#pragma unroll
  for (int i = 0; i < A_ITERS; ++i) {
    int r = min(m0 + ld_r + 64 * i, p.M - 1);
    if constexpr (CONV) {   // first pixel of patch r: image b, patch row py, patch column px, channel 0
      const int b = r / conv_pi, q = r - b * conv_pi, py = q / conv_pw, px = q - py * conv_pw;
      a_ptr[i] = pA + ((int64_t)b * p.conv_c * p.conv_h + (int64_t)py * p.conv_patch) * p.conv_w + px * p.conv_patch;
    } else {
      if (p.a_rows) r = p.a_rows[r];
      a_ptr[i] = pA + (int64_t)r * p.lda + ld_c * 8;
    }
  }
  const char* w_ptr[W_ITERS];
  int w_lr[W_ITERS], w_lc[W_ITERS];
#pragma unroll
  for (int i = 0; i < W_ITERS; ++i) {
    if (W_FP8) {
      // 64 fp8 per row = 4 chunks of 16 B; thread -> row tid/4 + 128*i, 16-element group tid%4
      w_lr[i] = (tid >> 2) + 128 * i;
      w_lc[i] = (tid & 3) * 2;
      int r = min(n0 + w_lr[i], p.N - 1);
      w_ptr[i] = (const char*)p.W + (int64_t)r * p.ldw + (tid & 3) * 16;
    } else {
      w_lr[i] = ld_r + 64 * i;
      w_lc[i] = ld_c;
      int r = min(n0 + w_lr[i], p.N - 1);
      w_ptr[i] = (const char*)p.W + ((int64_t)r * p.ldw + ld_c * 8) * 2;
    }
  }

  i32x4_t ga[A_ITERS], gw[W_ITERS];
  const i32x4_t zero4 = {0, 0, 0, 0};

  auto load_global = [&](int kt) {
    const int k0 = kt * BK;
    if constexpr (CONV) {
      // The thread's 8 consecutive k = four pixel pairs.  k is even and so is the patch size, so a pair never
      // straddles a patch row; its offset from the patch's first pixel is (c*H + ky)*W + kx.
      const int kk = k0 + ld_c * 8;
      int off[4];
      bool ok[4];
      int c = kk / (p.conv_patch * p.conv_patch), rem = kk - c * p.conv_patch * p.conv_patch;
      int ky = rem / p.conv_patch, kx = rem - ky * p.conv_patch;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        off[j] = (c * p.conv_h + ky) * p.conv_w + kx;
        ok[j] = kk + 2 * j < conv_kreal;
        kx += 2;
        if (kx >= p.conv_patch) {
          kx = 0;
          if (++ky == p.conv_patch) {
            ky = 0;
            ++c;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < A_ITERS; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) ga[i][j] = ok[j] ? *(const int*)(a_ptr[i] + off[j]) : 0;
    } else {
#pragma unroll
      for (int i = 0; i < A_ITERS; ++i) {
        ga[i] = (k0 + ld_c * 8 < p.K) ? *(const i32x4_t*)(a_ptr[i] + k0) : zero4;
      }
    }
#pragma unroll
    for (int i = 0; i < W_ITERS; ++i) {
      if (W_FP8)
        gw[i] = (k0 + (tid & 3) * 16 < p.K) ? *(const i32x4_t*)(w_ptr[i] + k0) : zero4;
      else
        gw[i] = (k0 + ld_c * 8 < p.K) ? *(const i32x4_t*)(w_ptr[i] + (int64_t)k0 * 2) : zero4;
    }
  };
  auto store_lds = [&](int stage) {
    char* As = smem + stage * STAGE;
    char* Ws = As + A_BYTES;
#pragma unroll
    for (int i = 0; i < A_ITERS; ++i) *(i32x4_t*)(As + swz(ld_r + 64 * i, ld_c)) = ga[i];
#pragma unroll
    for (int i = 0; i < W_ITERS; ++i) {
      if (W_FP8) {
        bf16x8_t lo, hi;
        fp8x16_to_bf16(gw[i], lo, hi);
        *(bf16x8_t*)(Ws + swz(w_lr[i], w_lc[i])) = lo;
        *(bf16x8_t*)(Ws + swz(w_lr[i], w_lc[i] + 1)) = hi;
      } else {
        *(i32x4_t*)(Ws + swz(w_lr[i], w_lc[i])) = gw[i];
      }
    }
  };

  f32x16_t acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;

  auto compute = [&](int stage) {
    const char* As = smem + stage * STAGE;
    const char* Ws = As + A_BYTES;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8_t wf[NT], xf[MT];
#pragma unroll
      for (int j = 0; j < NT; ++j)
        wf[j] = *(const bf16x8_t*)(Ws + swz(wn * WTN + j * 32 + frag_row, ks * 2 + frag_half));
#pragma unroll
      for (int i = 0; i < MT; ++i)
        xf[i] = *(const bf16x8_t*)(As + swz(wm * WTM + i * 32 + frag_row, ks * 2 + frag_half));
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[j], xf[i], acc[i][j], 0, 0, 0);
    }
  };

  const int nk = (p.K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) load_global(kt + 1);
    compute(cur);
    if (kt + 1 < nk) store_lds(cur ^ 1);
    __syncthreads();
  }

  csgemm::epilogue<EPI, MT, NT>(p, acc, m0 + wm * WTM, n0 + wn * WTN, lane);
}

template <int BM, int BN, int EPI, bool W_FP8, bool CONV = false>
int launch(const CsGemmArgs& a, hipStream_t stream) {
  CsGemmArgs p = a;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  constexpr int lds = 2 * (BM + BN) * BK * 2;
  static bool attr_set = false;
  auto kern = gemm_kernel<BM, BN, EPI, W_FP8, CONV>;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return CS_ERR_LAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(NTHREADS), lds, stream, p);
  return cs_launch_status();
}

template <int BM, int BN, bool W_FP8>
int dispatch_epi(const CsGemmArgs& a, hipStream_t s) {
  switch (a.epilogue) {
    case CS_EPI_BIAS: return launch<BM, BN, CS_EPI_BIAS, W_FP8>(a, s);
    case CS_EPI_RESIDUAL: return launch<BM, BN, CS_EPI_RESIDUAL, W_FP8>(a, s);
    case CS_EPI_SWIGLU: return launch<BM, BN, CS_EPI_SWIGLU, W_FP8>(a, s);
    case CS_EPI_GELU_ERF: return launch<BM, BN, CS_EPI_GELU_ERF, W_FP8>(a, s);
    case CS_EPI_GELU_TANH: return launch<BM, BN, CS_EPI_GELU_TANH, W_FP8>(a, s);
    case CS_EPI_QUICK_GELU: return launch<BM, BN, CS_EPI_QUICK_GELU, W_FP8>(a, s);
    default: return CS_ERR_INVALID_ARG;
  }
}

}  // namespace

extern "C" int cs_gemm(const CsGemmArgs* args, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!args) return CS_ERR_INVALID_ARG;
  const CsGemmArgs& a = *args;
  if (a.M < 0 || a.N <= 0 || a.K <= 0) return CS_ERR_INVALID_ARG;
  if (a.M == 0 && a.W) return CS_OK;  // an empty batch may come with null activation buffers
  if (!a.A || !a.W || !a.C) return CS_ERR_INVALID_ARG;
  // 16-byte vector loads along K and 8-byte packed stores along N.
  if (a.K % 8 || (a.lda % 8 && !a.conv_patch) || a.N % 4 || a.ldc % 2) return CS_ERR_INVALID_ARG;
  if (a.w_fp8 ? (a.ldw % 16 || a.K % 16 || !a.w_scale) : (a.ldw % 8)) return CS_ERR_INVALID_ARG;
  if (a.epilogue == CS_EPI_RESIDUAL && (!a.residual || a.ldr % 4)) return CS_ERR_INVALID_ARG;
  if (a.epilogue != CS_EPI_SWIGLU && a.ldc % 4) return CS_ERR_INVALID_ARG;
  // the byte planes of a 16-bit residual stream: only with the residual epilogue, 4-byte accesses along N
  if ((a.c_lo || a.residual_lo) && (a.epilogue != CS_EPI_RESIDUAL || a.pos || !a.c_lo)) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)a.c_lo | (uintptr_t)a.residual_lo) & 7) return CS_ERR_INVALID_ARG;
  if (a.pos && (a.pos_period <= 0 || a.ldpos % 4 || a.epilogue == CS_EPI_SWIGLU)) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)a.A | (uintptr_t)a.W) & 15) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)a.C | (uintptr_t)a.bias | (uintptr_t)a.residual | (uintptr_t)a.pos) & 7) return CS_ERR_INVALID_ARG;
  if ((uintptr_t)a.w_scale & 15) return CS_ERR_INVALID_ARG;
  if (a.prefetch ? (((uintptr_t)a.prefetch & 15) || a.prefetch_bytes < 0) : a.prefetch_bytes != 0) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)a.a_row_sumsq | (uintptr_t)a.c_row_sumsq | (uintptr_t)a.a_row_sum | (uintptr_t)a.c_row_sum |
       (uintptr_t)a.w_col_sum) & 15)
    return CS_ERR_INVALID_ARG;

  if (a.conv_patch) {   // strided-gather form of the activation operand: general kernel only
    if (a.conv_patch < 2 || a.conv_patch % 2 || a.conv_w % 2 || a.conv_c < 1 || a.conv_h < a.conv_patch ||
        a.conv_w < a.conv_patch || a.epilogue != CS_EPI_BIAS || a.w_fp8 || a.a_rows || a.a_row_sumsq || a.c_row_sumsq ||
        a.a_row_sum || a.c_row_sum)
      return CS_ERR_INVALID_ARG;
    const int64_t per_image = (int64_t)(a.conv_h / a.conv_patch) * (a.conv_w / a.conv_patch);
    if (a.M % per_image || a.K < a.conv_c * a.conv_patch * a.conv_patch || a.K >= a.conv_c * a.conv_patch * a.conv_patch + 8 ||
        (int64_t)a.conv_c * a.conv_h * a.conv_w >= ((int64_t)1 << 31))
      return CS_ERR_INVALID_ARG;
    const int64_t t256 = (int64_t)((a.M + 255) / 256) * ((a.N + 255) / 256);
    return t256 < 192 ? launch<128, 128, CS_EPI_BIAS, false, true>(a, stream) : launch<256, 256, CS_EPI_BIAS, false, true>(a, stream);
  }
  // Fast path (direct-to-LDS pipeline) when the shape allows it; otherwise the general kernel below.
  {
    bool handled = false;
    const int st = cs_gemm_fast(a, stream, &handled);
    if (handled) return st;
  }
  if (a.a_row_sumsq || a.c_row_sumsq || a.a_row_sum || a.c_row_sum) return CS_ERR_UNSUPPORTED;  // the folded norms exist in the fast kernel only
  // Tile choice: 256x256 when that fills the chip's 256 CUs reasonably, else smaller tiles for more workgroups.
  const int64_t t256 = (int64_t)((a.M + 255) / 256) * ((a.N + 255) / 256);
  const bool small = t256 < 192;
  if (a.w_fp8) {
    return small ? dispatch_epi<128, 128, true>(a, stream) : dispatch_epi<256, 256, true>(a, stream);
  }
  return small ? dispatch_epi<128, 128, false>(a, stream) : dispatch_epi<256, 256, false>(a, stream);
}
