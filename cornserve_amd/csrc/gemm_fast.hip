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
#include <stdlib.h>

#include <type_traits>

#include "gemm_common.h"

namespace {

using namespace csgemm;

constexpr int NTHREADS = 512;  // 8 waves, 2 per SIMD
constexpr int CS_EPI_BIAS_POS = 100;  // internal: CS_EPI_BIAS plus the (row % pos_period) position addend

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

#ifdef CS_GEMM_TS
__device__ long long* cs_ts_buf;  // [tiles][8]: 4 wall-clock stamps + 4 shader-clock stamps by wave 0 (profiling builds only)
#define CS_TS(slot) do { if (tid == 0 && cs_ts_buf) { cs_ts_buf[vb * 8 + (slot)] = wall_clock64(); cs_ts_buf[vb * 8 + 4 + (slot)] = clock64(); } } while (0)
#else
#define CS_TS(slot) do { } while (0)
#endif

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI>
__global__ __launch_bounds__(NTHREADS) void gemm_fast_kernel(const CsGemmArgs p, const int stagger) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  static_assert(WAVES_M * WAVES_N == 8, "8 waves");
  constexpr int A_BYTES = BM * BK * 2;
  constexpr int W_BYTES = BN * BK * 2;
  constexpr int STAGE = A_BYTES + W_BYTES;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0 && BM % 8 == 0 && BN % 8 == 0, "tile shape");
  constexpr int MT = WTM / 16, NT = WTN / 16;
  // Pinning a fine MFMA/LDS interleave costs registers; only tiles whose accumulators and two fragment
  // sets leave room for it use it (the 256x256 tile would spill).
  constexpr bool ILV = (MT * NT * 4 + (MT + NT) * 8) <= 176;
  constexpr int A_BLK = BM / 8, W_BLK = BN / 8;            // 8-row blocks = direct loads per stage
  constexpr int A_LD = (A_BLK + 7) / 8, W_LD = (W_BLK + 7) / 8;  // per wave

  // ---- tile coordinates of virtual block vb in [0, tiles): XCD-aware remap (workgroup i runs on XCD i%8,
  //      and the persistent stride gridDim.x is a multiple of 8, so a workgroup's tiles stay on its XCD),
  //      then bands of 8 tile-rows walked column-major so the 32 workgroups resident on one XCD share
  //      8 A panels and 4 W panels through that XCD's L2.
  const int ntiles = p.tiles_m * p.tiles_n;
  auto tile_origin = [&](int vb, int& m0, int& n0) {
    const int per = ntiles >> 3;
    if (vb < per * 8) vb = (vb & 7) * per + (vb >> 3);
    constexpr int GM = 8;
    const int band_sz = GM * p.tiles_n;
    const int band = vb / band_sz;
    const int within = vb - band * band_sz;
    const int rows_in_band = min(GM, p.tiles_m - band * GM);
    m0 = (band * GM + within % rows_in_band) * BM;
    n0 = (within / rows_in_band) * BN;
  };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;

  // ---- global sources of the direct loads.  Row block rb = j*8 + wave covers tile rows 8rb..8rb+7; the
  //      lane lands in slot lane%8 of row 8rb + lane/8 and fetches chunk (lane%8) ^ key(row).
  const int l_row = lane >> 3, l_slot = lane & 7;
  // 32-bit byte offsets from the (scalar) matrix bases: half the registers of full pointers, and the K
  // advance is one scalar add per operand instead of a vector add per load.
  uint32_t a_src[A_LD];
  uint32_t w_src[W_LD];
  auto setup_sources = [&](int m0, int n0) {
#pragma unroll
    for (int j = 0; j < A_LD; ++j) {
      const int row = (j * 8 + wave) * 8 + l_row;  // tile-local
      const int key = (row >> 1) & 7;
      const int r = min(m0 + row, p.M - 1);
      a_src[j] = (uint32_t)(((int64_t)r * p.lda + ((l_slot ^ key) << 3)) * 2);
    }
#pragma unroll
    for (int j = 0; j < W_LD; ++j) {
      const int row = (j * 8 + wave) * 8 + l_row;
      const int key = ((((row % WTN) / (4 * NT)) & 3) << 1) | ((row >> 1) & 1);
      const int r = min(n0 + row, p.N - 1);
      w_src[j] = (uint32_t)(((int64_t)r * p.ldw + ((l_slot ^ key) << 3)) * 2);
    }
  };
  auto issue_loads = [&](int kt, int stage) {
    char* As = smem + stage * STAGE;
    char* Ws = As + A_BYTES;
    const char* Ak = (const char*)p.A + (int64_t)kt * (BK * 2);
    const char* Wk = (const char*)p.W + (int64_t)kt * (BK * 2);
#pragma unroll
    for (int j = 0; j < A_LD; ++j)
      if ((A_BLK % 8 == 0) || j * 8 + wave < A_BLK) load_chunk_to_lds(Ak + a_src[j], As + (j * 8 + wave) * 1024);
#pragma unroll
    for (int j = 0; j < W_LD; ++j)
      if ((W_BLK % 8 == 0) || j * 8 + wave < W_BLK) load_chunk_to_lds(Wk + w_src[j], Ws + (j * 8 + wave) * 1024);
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
  bf16x8_t wf[2][NT], xf[2][MT];
  auto read_frags = [&](int stage, int ks, int b) {
    const char* base = smem + stage * STAGE;
#pragma unroll
    for (int j = 0; j < NT; ++j) wf[b][j] = *(const bf16x8_t*)(base + w_off[ks] + j * 4 * 128);
#ifdef CS_EXP_SKIP_X  // experiment: issue only half of the activation-fragment reads (results are wrong)
#pragma unroll
    for (int i = 0; i < MT / 2; ++i) xf[b][i] = *(const bf16x8_t*)(base + x_off[ks] + i * 16 * 128);
#pragma unroll
    for (int i = MT / 2; i < MT; ++i) xf[b][i] = xf[b][i - MT / 2];
#else
#pragma unroll
    for (int i = 0; i < MT; ++i) xf[b][i] = *(const bf16x8_t*)(base + x_off[ks] + i * 16 * 128);
#endif
  };
  auto mfmas = [&](int b) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[b][j], xf[b][i], acc[i][j], 0, 0, 0);
  };

  const int nk = p.K / BK;
  int vb = blockIdx.x;
  if (stagger > 0) {
    // Persistent launches: spread the 32 workgroups of each XCD in time (10 ns ticks per slot) so that the
    // output bursts of the 256 CUs do not hit HBM in the same few microseconds of every round.
    const long long until = wall_clock64() + (long long)((blockIdx.x >> 3) & 31) * stagger;
    while (wall_clock64() < until) __builtin_amdgcn_s_sleep(4);
  }
  int m0, n0;
  tile_origin(vb, m0, n0);
  setup_sources(m0, n0);
  issue_loads(0, 0);
  if (nk > 1) issue_loads(1, 1);

  // Persistent loop over this workgroup's tiles (vb, vb + gridDim.x, ...).  The first two K tiles of the
  // NEXT output tile are requested inside the last K iteration of the current one, so they travel while
  // the epilogue runs.
  for (;;) {
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  const int vb_next = vb + gridDim.x;
  const bool has_next = vb_next < ntiles;
  int m0_next = 0, n0_next = 0;

  CS_TS(0);
  CS_WAIT_VMCNT(0);  // K tiles 0 and 1 of this output tile (and the previous tile's stores)
  wg_barrier();
  CS_TS(1);
  read_frags(0, 0, 0);

  // One K iteration.  LOADS: tile kt+2 exists and is fetched; NEXT: tile kt+1 exists; LAST: final iteration.
  auto body = [&](int kt, auto loads_c, auto next_c) {
    constexpr bool LOADS = decltype(loads_c)::value, NEXT = decltype(next_c)::value;
    const int cur = kt & 1;
    __builtin_amdgcn_sched_barrier(0);
    read_frags(cur, 1, 1);
    mfmas(0);
    // Issue order: one fragment read after each of the first MFMAs, so the matrix cores never wait for
    // the wave to get through a block of LDS instructions.
    if (ILV) {
#pragma unroll
      for (int r = 0; r < MT + NT; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
      }
      __builtin_amdgcn_sched_group_barrier(0x008, MT * NT - (MT + NT), 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    // Tile kt+1 (issued one iteration ago) must have landed in every wave's part of the other stage, and
    // every wave must have received its last fragments of this stage before it is refilled.
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    wg_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (LOADS) issue_loads(kt + 2, cur);
    if (NEXT) read_frags(cur ^ 1, 0, 0);
    if (!NEXT && has_next) {  // both stages are free now: start on the next output tile
      tile_origin(vb_next, m0_next, n0_next);
      setup_sources(m0_next, n0_next);
      issue_loads(0, 0);
      if (nk > 1) issue_loads(1, 1);
    }
    mfmas(1);
    if (ILV && LOADS && NEXT) {
      constexpr int NLD = A_LD + W_LD;
#pragma unroll
      for (int r = 0; r < NLD; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // direct-to-LDS load
      }
#pragma unroll
      for (int r = 0; r < MT + NT; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, MT * NT - NLD - (MT + NT), 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  int kt = 0;
  for (; kt + 2 < nk; ++kt) body(kt, std::true_type{}, std::true_type{});
  if (kt + 1 < nk) {
    body(kt, std::false_type{}, std::true_type{});
    ++kt;
  }
  body(kt, std::false_type{}, std::false_type{});
  CS_TS(2);

  // ---- epilogue.  acc[i][j][r] = C[m][n], m = m0 + wm*WTM + 16i + lane%16,
  //      n = n0 + wn*WTN + (lane/16)*(4*NT) + 4j + r : 4*NT consecutive columns per lane and row.
  //      Every load the epilogue needs (row map, bias, residual / position rows) is issued up front, from
  //      clamped addresses so that no branch guards a load: a load inside the store loop would make the
  //      compiler wait for ALL outstanding memory operations (vmcnt counts stores too), i.e. for every
  //      store issued so far and for the next tile's prefetch, once per row block.
  {
    const bf16_t* const pBias = (const bf16_t*)p.bias;
    bf16_t* const pC = (bf16_t*)p.C;
    const int n_lane = n0 + wn * WTN + kq * (4 * NT);
    int mrow[MT];
    int64_t crow[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      mrow[i] = m0 + wm * WTM + i * 16 + fa;
      const int mc = min(mrow[i], p.M - 1);
      crow[i] = p.c_rows ? (int64_t)p.c_rows[mc] : (int64_t)mc;
    }
    float bias_v[NT][4];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int nc = min(n_lane + 4 * j, p.N - 4);
      bf16x4_t bb = {0, 0, 0, 0};
      if (pBias) bb = *(const bf16x4_t*)(pBias + nc);
#pragma unroll
      for (int r = 0; r < 4; ++r) bias_v[j][r] = bf2f(bb[r]);
    }
    constexpr bool ADDEND = (EPI == CS_EPI_RESIDUAL) || (EPI == CS_EPI_BIAS_POS);
    bf16x4_t addend[ADDEND ? MT : 1][ADDEND ? NT : 1];
    if (ADDEND) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int mc = min(mrow[i], p.M - 1);
        const bf16_t* row = (EPI == CS_EPI_RESIDUAL)
                                ? (const bf16_t*)p.residual + (int64_t)mc * p.ldr
                                : (const bf16_t*)p.pos + (int64_t)(mc % p.pos_period) * p.ldpos;
#pragma unroll
        for (int j = 0; j < NT; ++j) addend[i][j] = *(const bf16x4_t*)(row + min(n_lane + 4 * j, p.N - 4));
      }
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const bool mok = mrow[i] < p.M;
      bf16x4_t out[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = acc[i][j][r] + bias_v[j][r];
        if (EPI == CS_EPI_SWIGLU) {
          // gate and up are rounded to bf16 like the reference's two F.linear outputs; SiLU and the
          // product stay in fp32 until the single output rounding
          const float g0 = silu(rbf(v[0])), u0 = rbf(v[1]);
          const float g1 = silu(rbf(v[2])), u1 = rbf(v[3]);
          out[j][0] = f2bf(g0 * u0);
          out[j][1] = f2bf(g1 * u1);
        } else {
          if (EPI == CS_EPI_GELU_ERF) {
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = gelu_erf(rbf(v[r]));
          } else if (EPI == CS_EPI_GELU_TANH) {
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = gelu_tanh(rbf(v[r]));
          } else if (ADDEND) {
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = rbf(v[r]) + bf2f(addend[ADDEND ? i : 0][ADDEND ? j : 0][r]);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) out[j][r] = f2bf(v[r]);
        }
      }
      if (EPI == CS_EPI_SWIGLU) {
        bf16_t* dst = pC + crow[i] * p.ldc + (n_lane >> 1);
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          if (mok && n_lane + 4 * j < p.N) {
            bf16x2_t o;
            o[0] = out[j][0];
            o[1] = out[j][1];
            *(bf16x2_t*)(dst + 2 * j) = o;
          }
        }
      } else {
        bf16_t* dst = pC + crow[i] * p.ldc + n_lane;
#pragma unroll
        for (int j = 0; j < NT; ++j)
          if (mok && n_lane + 4 * j < p.N) *(bf16x4_t*)(dst + 4 * j) = out[j];
      }
    }
  }
  CS_TS(3);
  if (!has_next) break;
  vb = vb_next;
  m0 = m0_next;
  n0 = n0_next;
  }  // persistent tile loop
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
  const int tiles = p.tiles_m * p.tiles_n;
  // One resident workgroup per CU (LDS-bound); with more tiles than CUs the kernel is persistent.
  const int grid = tiles <= 256 ? tiles : 256;
  static const char* st_env = getenv("CS_GEMM_STAGGER");  // experiment knob: ticks of 10 ns per slot
  const int stagger = tiles > 256 ? (st_env ? atoi(st_env) : 0) : 0;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NTHREADS), lds, stream, p, stagger);
  return cs_launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int dispatch_epi(const CsGemmArgs& a, hipStream_t s) {
  switch (a.epilogue) {
    case CS_EPI_BIAS:
      if (a.pos) return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS_POS>(a, s);
      return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS>(a, s);
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
  if (a.w_fp8 || a.K % BK || a.M < 1 || a.w_scale || a.N < 4) return CS_OK;
  if (a.pos && a.epilogue != CS_EPI_BIAS) return CS_OK;
  // per-lane source offsets are 32-bit byte offsets from the matrix bases
  if (a.a_rows) return CS_OK;  // gathered A rows can lie anywhere: the general kernel keeps 64-bit pointers
  if ((int64_t)a.M * a.lda * 2 >= (int64_t)UINT32_MAX || (int64_t)a.N * a.ldw * 2 >= (int64_t)UINT32_MAX) return CS_OK;  // position addend only pairs with the plain epilogue here
  *handled = true;
  // Tile shape: the one that needs the least chip time (tile quantisation over the 256 CUs).  The narrow
  // 256x160 tile exists for N = 1280 (8 column tiles: 8192 rows give exactly 256 workgroups).
  const double c256 = rounds_cost(a.M, a.N, 256, 256);
  const double c160 = rounds_cost(a.M, a.N, 256, 160) * 1.15;  // narrower tiles: more LDS and L2 traffic per FLOP
  static const char* force = getenv("CS_GEMM_TILE");        // benchmarking aid: "160" or "256"
  if (force ? force[0] == '1' : c160 < c256) return dispatch_epi<256, 160, 4, 2>(a, stream);
  // Column split.  When the last round of 256x256 tiles would leave most CUs idle, the leading columns
  // that fill whole rounds go to one launch and the remaining columns to a second launch with 256x128
  // tiles (twice as many workgroups, half as long).  The two launches write disjoint column ranges of C.
  if (!force) {
    const int tm = (a.M + 255) / 256, tn = (a.N + 255) / 256;
    double best = c256;
    int best_cols = 0;
    for (int c = tn - 1; c >= 1 && c >= tn - 12; --c) {
      const int rest = a.N - c * 256;
      const double cost = rounds_cost(a.M, c * 256, 256, 256) + rounds_cost(a.M, rest, 256, 128) * 1.10;
      if (cost < best - 0.05) {
        best = cost;
        best_cols = c;
      }
    }
    (void)tm;
    if (best_cols > 0) {
      const int n1 = best_cols * 256;
      CsGemmArgs lo = a, hi = a;
      lo.N = n1;
      hi.N = a.N - n1;
      hi.W = (const char*)a.W + (int64_t)n1 * a.ldw * 2;
      if (a.bias) hi.bias = (const char*)a.bias + (int64_t)n1 * 2;
      if (a.residual) hi.residual = (const char*)a.residual + (int64_t)n1 * 2;
      if (a.pos) hi.pos = (const char*)a.pos + (int64_t)n1 * 2;
      hi.C = (char*)a.C + (int64_t)(a.epilogue == CS_EPI_SWIGLU ? n1 / 2 : n1) * 2;
      const int st = dispatch_epi<256, 256, 2, 4>(lo, stream);
      if (st != CS_OK) return st;
      return dispatch_epi<256, 128, 4, 2>(hi, stream);
    }
  }
  return dispatch_epi<256, 256, 2, 4>(a, stream);
}
