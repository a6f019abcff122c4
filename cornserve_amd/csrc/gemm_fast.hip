// Fast-path bf16 MFMA GEMM for gfx950:  C[M,N] = epilogue(A[M,K] . W[N,K]^T),  K % 64 == 0, bf16 weights.
//
// Pipeline.  One 512-thread workgroup (8 waves, 2 per SIMD) owns a BM x BN tile of C and walks K in steps
// of 64.  Tiles go global -> LDS directly (global_load_lds_dwordx4: each lane fetches 16 bytes and the
// hardware stores the wave's 64 chunks contiguously at M0 + lane*16), two LDS stages.  The loop is skewed:
// the single barrier of an iteration sits BEFORE its last k-step, so the first fragments of the next tile
// are read while the matrix cores work on that last step, and the refill of the stage that was just
// drained (tile kt+2) is issued right after the barrier and has a full iteration to land.
//
// Matrix cores.  v_mfma_f32_16x16x32_bf16 (k = 32 per instruction: each accumulator register is touched
// half as often as with the 32x32x16 form).  W rows are the MFMA "A" operand and activation rows the "B"
// operand, so a lane owns output row m = lane%16 of a 16x16 block.  The W rows that feed fragment j of a
// wave are PERMUTED: fragment row 4q+r holds W row q*(4*NT) + 4j + r of the wave's WTN = 16*NT rows, which
// makes the 4*NT accumulator values a lane holds for one output row CONSECUTIVE in n.  The epilogue can
// therefore read bias/residual and write C in 8/16-byte pieces that tile whole 128-byte lines, with no
// trip through LDS.
//
// LDS layout.  A tile row is 128 bytes = 8 chunks of 16 bytes; logical chunk c of row r lives in slot
// c ^ key(r).  The LDS has 64 four-byte banks, so a 16-byte-per-lane read is served 16 lanes at a time and
// is conflict-free when those lanes hit 16 distinct 16-byte groups of a 256-byte span; with 128-byte rows
// the row parity picks the half and the key must differ across the 8 rows of equal parity.  Activation
// fragments read 16 consecutive rows (key = (r>>1)&7); W fragments read rows q*(4*NT)+4j+r
// (key = q*2 + ((r>>1)&1)).  Since a direct-to-LDS load fixes the LDS side (lane -> consecutive chunk),
// the swizzle is applied on the GLOBAL side: the lane that lands in slot s of row r fetches chunk s ^ key(r).
#include <type_traits>

#include "gemm_common.h"

namespace {

using namespace csgemm;

constexpr int NTHREADS = 512;  // 8 waves, 2 per SIMD

// s_waitcnt with only vmcnt set (lgkmcnt/expcnt left at "don't wait"), gfx9 encoding.
#define CS_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt((((n) & 0xF) | (((n) >> 4) << 14)) | 0x0F70)

typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void global_void_t;

CS_DEVICE void load_chunk_to_lds(const char* gptr, char* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((global_void_t*)gptr, (lds_void_t*)lds_wave_base, 16, 0, 0);
}
// Workgroup barrier without the full memory fence of __syncthreads(): the callers order LDS traffic with
// explicit waits, and the asm statements keep the compiler from moving memory operations across it.
CS_DEVICE void wg_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI>
__global__ __launch_bounds__(NTHREADS) void gemm_fast_kernel(const CsGemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  static_assert(WAVES_M * WAVES_N == 8, "8 waves");
  constexpr int A_BYTES = BM * BK * 2;
  constexpr int W_BYTES = BN * BK * 2;
  constexpr int STAGE = A_BYTES + W_BYTES;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0 && BM % 8 == 0 && BN % 8 == 0, "tile shape");
  constexpr int MT = WTM / 16, NT = WTN / 16;
  constexpr int A_BLK = BM / 8, W_BLK = BN / 8;            // 8-row blocks = direct loads per stage
  constexpr int A_LD = (A_BLK + 7) / 8, W_LD = (W_BLK + 7) / 8;  // per wave

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
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;

  // ---- global sources of the direct loads.  Row block rb = j*8 + wave covers tile rows 8rb..8rb+7; the
  //      lane lands in slot lane%8 of row 8rb + lane/8 and fetches chunk (lane%8) ^ key(row).
  const int l_row = lane >> 3, l_slot = lane & 7;
  const char* a_src[A_LD];
  const char* w_src[W_LD];
#pragma unroll
  for (int j = 0; j < A_LD; ++j) {
    const int row = (j * 8 + wave) * 8 + l_row;  // tile-local
    const int key = (row >> 1) & 7;
    int r = min(m0 + row, p.M - 1);
    if (p.a_rows) r = p.a_rows[r];
    a_src[j] = (const char*)p.A + ((int64_t)r * p.lda + ((l_slot ^ key) << 3)) * 2;
  }
#pragma unroll
  for (int j = 0; j < W_LD; ++j) {
    const int row = (j * 8 + wave) * 8 + l_row;
    const int key = ((((row % WTN) / (4 * NT)) & 3) << 1) | ((row >> 1) & 1);
    const int r = min(n0 + row, p.N - 1);
    w_src[j] = (const char*)p.W + ((int64_t)r * p.ldw + ((l_slot ^ key) << 3)) * 2;
  }
  auto issue_loads = [&](int kt, int stage) {
    char* As = smem + stage * STAGE;
    char* Ws = As + A_BYTES;
    const int koff = kt * BK * 2;
#pragma unroll
    for (int j = 0; j < A_LD; ++j)
      if ((A_BLK % 8 == 0) || j * 8 + wave < A_BLK) load_chunk_to_lds(a_src[j] + koff, As + (j * 8 + wave) * 1024);
#pragma unroll
    for (int j = 0; j < W_LD; ++j)
      if ((W_BLK % 8 == 0) || j * 8 + wave < W_BLK) load_chunk_to_lds(w_src[j] + koff, Ws + (j * 8 + wave) * 1024);
  };

  // ---- fragment addressing.  Lane (a = lane%16, kq = lane/16) reads chunk ks*4 + kq of its fragment row.
  //      Both keys depend only on the lane, so the per-lane part of the address is loop-invariant.
  const int fa = lane & 15, kq = lane >> 4;
  const int fq = fa >> 2, fr = fa & 3;
  const int x_key = (fa >> 1) & 7;
  const int w_key = (fq << 1) | ((fr >> 1) & 1);
  // byte offset inside a stage of fragment (i or j), k-step ks: row*128 + (((ks*4 + kq) ^ key) << 4)
  int x_off[2], w_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    x_off[ks] = (wm * WTM + fa) * 128 + (((ks * 4 + kq) ^ x_key) << 4);
    w_off[ks] = A_BYTES + (wn * WTN + fq * (4 * NT) + fr) * 128 + (((ks * 4 + kq) ^ w_key) << 4);
  }

  f32x4_t acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  bf16x8_t wf[2][NT], xf[2][MT];
  auto read_frags = [&](int stage, int ks, int b) {
    const char* base = smem + stage * STAGE;
#pragma unroll
    for (int j = 0; j < NT; ++j) wf[b][j] = *(const bf16x8_t*)(base + w_off[ks] + j * 4 * 128);
#pragma unroll
    for (int i = 0; i < MT; ++i) xf[b][i] = *(const bf16x8_t*)(base + x_off[ks] + i * 16 * 128);
  };
  auto mfmas = [&](int b) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[b][j], xf[b][i], acc[i][j], 0, 0, 0);
  };

  const int nk = p.K / BK;
  issue_loads(0, 0);
  if (nk > 1) issue_loads(1, 1);
  if (nk > 1 && A_BLK % 8 == 0 && W_BLK % 8 == 0) {
    CS_WAIT_VMCNT(A_LD + W_LD);  // tile 0 landed; tile 1 may still be in flight
  } else {
    CS_WAIT_VMCNT(0);
  }
  wg_barrier();
  read_frags(0, 0, 0);

  // One K iteration.  LOADS: tile kt+2 exists and is fetched; NEXT: tile kt+1 exists.
  auto body = [&](int kt, auto loads_c, auto next_c) {
    constexpr bool LOADS = decltype(loads_c)::value, NEXT = decltype(next_c)::value;
    const int cur = kt & 1;
    __builtin_amdgcn_sched_barrier(0);
    read_frags(cur, 1, 1);
    mfmas(0);
    __builtin_amdgcn_sched_barrier(0);
    // Tile kt+1 (issued one iteration ago) must have landed in every wave's part of the other stage, and
    // every wave must have requested its last fragments of this stage before it is refilled.
    CS_WAIT_VMCNT(0);
    wg_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (LOADS) issue_loads(kt + 2, cur);
    if (NEXT) read_frags(cur ^ 1, 0, 0);
    mfmas(1);
    __builtin_amdgcn_sched_barrier(0);
  };
  int kt = 0;
  for (; kt + 2 < nk; ++kt) body(kt, std::true_type{}, std::true_type{});
  if (kt + 1 < nk) {
    body(kt, std::false_type{}, std::true_type{});
    ++kt;
  }
  body(kt, std::false_type{}, std::false_type{});

  // ---- epilogue.  acc[i][j][r] = C[m][n], m = m0 + wm*WTM + 16i + lane%16,
  //      n = n0 + wn*WTN + (lane/16)*(4*NT) + 4j + r : 4*NT consecutive columns per lane and row.
  const bf16_t* const pBias = (const bf16_t*)p.bias;
  const bf16_t* const pRes = (const bf16_t*)p.residual;
  const bf16_t* const pPos = (const bf16_t*)p.pos;
  bf16_t* const pC = (bf16_t*)p.C;
  const int n_lane = n0 + wn * WTN + kq * (4 * NT);
  float bias_v[NT][4];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = n_lane + 4 * j;
    bf16x4_t b = {0, 0, 0, 0};
    if (pBias && n < p.N) b = *(const bf16x4_t*)(pBias + n);
#pragma unroll
    for (int r = 0; r < 4; ++r) bias_v[j][r] = bf2f(b[r]);
  }
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = m0 + wm * WTM + i * 16 + fa;
    if (m >= p.M) continue;
    const int64_t crow = p.c_rows ? (int64_t)p.c_rows[m] : (int64_t)m;
    bf16x4_t out[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = n_lane + 4 * j;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = acc[i][j][r] + bias_v[j][r];
      if (EPI == CS_EPI_SWIGLU) {
        const float g0 = rbf(silu(rbf(v[0]))), u0 = rbf(v[1]);
        const float g1 = rbf(silu(rbf(v[2]))), u1 = rbf(v[3]);
        out[j][0] = f2bf(g0 * u0);
        out[j][1] = f2bf(g1 * u1);
      } else {
        if (EPI == CS_EPI_GELU_ERF) {
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = gelu_erf(rbf(v[r]));
        } else if (EPI == CS_EPI_GELU_TANH) {
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = gelu_tanh(rbf(v[r]));
        } else if (EPI == CS_EPI_RESIDUAL) {
          if (n < p.N) {
            const bf16x4_t rr = *(const bf16x4_t*)(pRes + (int64_t)m * p.ldr + n);
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = rbf(v[r]) + bf2f(rr[r]);
          }
        }
        if (pPos && n < p.N) {
          const bf16x4_t rr = *(const bf16x4_t*)(pPos + (int64_t)(m % p.pos_period) * p.ldpos + n);
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = rbf(v[r]) + bf2f(rr[r]);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) out[j][r] = f2bf(v[r]);
      }
    }
    if (EPI == CS_EPI_SWIGLU) {
      bf16_t* dst = pC + crow * p.ldc + (n_lane >> 1);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        if (n_lane + 4 * j < p.N) {
          bf16x2_t o;
          o[0] = out[j][0];
          o[1] = out[j][1];
          *(bf16x2_t*)(dst + 2 * j) = o;
        }
      }
    } else {
      bf16_t* dst = pC + crow * p.ldc + n_lane;
#pragma unroll
      for (int j = 0; j < NT; ++j)
        if (n_lane + 4 * j < p.N) *(bf16x4_t*)(dst + 4 * j) = out[j];
    }
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI>
int launch(const CsGemmArgs& a, hipStream_t stream) {
  CsGemmArgs p = a;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  constexpr int lds = 2 * (BM + BN) * BK * 2;
  static bool attr_set = false;
  auto kern = gemm_fast_kernel<BM, BN, WAVES_M, WAVES_N, EPI>;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return CS_ERR_LAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(NTHREADS), lds, stream, p);
  return cs_launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int dispatch_epi(const CsGemmArgs& a, hipStream_t s) {
  switch (a.epilogue) {
    case CS_EPI_BIAS: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS>(a, s);
    case CS_EPI_RESIDUAL: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_RESIDUAL>(a, s);
    case CS_EPI_SWIGLU: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_SWIGLU>(a, s);
    case CS_EPI_GELU_ERF: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_GELU_ERF>(a, s);
    case CS_EPI_GELU_TANH: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_GELU_TANH>(a, s);
    default: return CS_ERR_INVALID_ARG;
  }
}

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
  if (a.w_fp8 || a.K % BK || a.M < 1 || a.w_scale) return CS_OK;
  *handled = true;
  // Tile shape: the one that needs the least chip time (tile quantisation over the 256 CUs).  The narrow
  // 256x160 tile exists for N = 1280 (8 column tiles: 8192 rows give exactly 256 workgroups).
  const double c256 = rounds_cost(a.M, a.N, 256, 256);
  const double c160 = rounds_cost(a.M, a.N, 256, 160) * 1.03;  // smaller tiles reuse less per byte loaded
  if (c160 < c256) return dispatch_epi<256, 160, 4, 2>(a, stream);
  return dispatch_epi<256, 256, 2, 4>(a, stream);
}
