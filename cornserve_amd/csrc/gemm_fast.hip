// Fast-path bf16 MFMA GEMM for gfx950:  C[M,N] = epilogue(A[M,K] . W[N,K]^T),  K % 64 == 0, bf16 weights.
//
// Pipeline.  One workgroup owns a BM x BN tile of C and walks K in steps of 64.  Tiles go global -> LDS
// directly (buffer_load_dwordx4 ... lds: each lane fetches 16 bytes and the hardware stores the wave's 64
// chunks contiguously at M0 + lane*16), two LDS stages.  The loop is skewed: the single barrier of an
// iteration sits BEFORE its last k-step, so the first fragments of the next tile are read while the matrix
// cores work on that last step, and the refill of the stage that was just drained (tile kt+2) is issued
// right after the barrier and has a full iteration to land.
//
// Two forms share the code.  The 256x256 tile runs with FOUR waves, one per SIMD, 128x128 outputs and all
// 512 registers per lane: 256 accumulation registers hold the accumulators and are driven by inline
// assembly in a fixed instruction order (LDS traffic per FLOP is a third lower than with eight waves, and
// the compiler cannot shuffle or spill the accumulators).  The narrower tiles (256x160, 256x128) run with
// EIGHT waves, two per SIMD, compiler-scheduled builtins.
//
// Matrix cores.  v_mfma_f32_16x16x32_bf16 (k = 32 per instruction: each accumulator register is touched
// half as often as with the 32x32x16 form).  W rows are the MFMA "A" operand and activation rows the "B"
// operand, so a lane owns output row m = lane%16 of a 16x16 block.  The W rows that feed the fragments of a
// wave are PERMUTED in groups of G fragments (G = 2 when the wave has an even number of them): fragment j,
// fragment row 4q+r holds W row (j/G)*16G + q*4G + (j%G)*4 + r of the wave's rows.  The 4G accumulator
// values a lane holds for one output row and group are then CONSECUTIVE in n, and the four lanes of that
// output row hold 16G consecutive columns: with G = 2 every store instruction writes 16 bytes per lane and
// 64 contiguous bytes per output row, with no trip through LDS.
//
// LDS layout.  A tile row is 128 bytes = 8 chunks of 16 bytes; logical chunk c of row r lives in slot
// c ^ key(r).  The LDS has 64 four-byte banks, so a 16-byte-per-lane read is served 16 lanes at a time and
// is conflict-free when those lanes hit 16 distinct 16-byte groups of a 256-byte span; with 128-byte rows
// the row parity picks the half and the key must differ across the 8 rows of equal parity.  Activation
// fragments read 16 consecutive rows (key = (r>>1)&7); W fragments read rows q*4G + r plus a multiple of 4
// (key = q*2 + ((r>>1)&1)).  Since a direct-to-LDS load fixes the LDS side (lane -> consecutive chunk),
// the swizzle is applied on the GLOBAL side: the lane that lands in slot s of row r fetches chunk s ^ key(r).
#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "gemm_common.h"

namespace {

using namespace csgemm;

constexpr int CS_EPI_BIAS_POS = 100;  // internal: CS_EPI_BIAS plus the (row % pos_period) position addend

// s_waitcnt with only vmcnt set (lgkmcnt/expcnt left at "don't wait"), gfx9 encoding.
#define CS_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt((((n) & 0xF) | (((n) >> 4) << 14)) | 0x0F70)

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void_t;

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

// every accumulation register, as an inline-asm clobber list
#define CS_ALL_ACC_REGS \
  "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", \
  "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31", \
  "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", \
  "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63", \
  "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", \
  "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", \
  "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111", \
  "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127", \
  "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141", "a142", "a143", \
  "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159", \
  "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", \
  "a176", "a177", "a178", "a179", "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191", \
  "a192", "a193", "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", "a206", "a207", \
  "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", "a219", "a220", "a221", "a222", "a223", \
  "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", "a232", "a233", "a234", "a235", "a236", "a237", "a238", "a239", \
  "a240", "a241", "a242", "a243", "a244", "a245", "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255"

template <int V>
using ic = std::integral_constant<int, V>;
template <class F, int... Is>
CS_DEVICE void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(ic<Is>{}), ...);
}
// f(ic<0>{}), f(ic<1>{}), ... f(ic<N-1>{}): a loop whose index is a constant expression in the body
template <int N, class F>
CS_DEVICE void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_fast_kernel(const CsGemmArgs p, const int stagger) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int NW = WAVES_M * WAVES_N;
  static_assert(NW == 8 || NW == 4, "8 waves (2 per SIMD, 256 registers each) or 4 waves (1 per SIMD, 512 registers)");
  static_assert(NW == 8 || (BM / WAVES_M) * (BN / WAVES_N) <= 128 * 128, "the 4-wave form has 256 accumulation registers");
  constexpr int A_BYTES = BM * BK * 2;
  constexpr int W_BYTES = BN * BK * 2;
  constexpr int STAGE = A_BYTES + W_BYTES;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0 && BM % 8 == 0 && BN % 8 == 0, "tile shape");
  constexpr int MT = WTM / 16, NT = WTN / 16;
  // W fragments come in groups of G: fragment j, fragment row 4q+r holds W row (j/G)*16G + q*4G + (j%G)*4 + r of
  // the wave's rows, so a lane owns 4G consecutive output columns per group and the four lanes q = 0..3 of
  // one output row own 16G consecutive columns.
  constexpr int G = (NT % 2 == 0) ? 2 : NT;
  auto piece_col = [](int j) { return (j / G) * 16 * G + (j % G) * 4; };  // first column of fragment j's piece
  // Pinning a fine MFMA/LDS interleave costs registers; only tiles whose accumulators and two fragment
  // sets leave room for it use it (the 256x256 tile would spill).
  constexpr bool ILV = NW == 4 || (MT * NT * 4 + (MT + NT) * 8) <= 176;
  constexpr int A_BLK = BM / 8, W_BLK = BN / 8;            // 8-row blocks = direct loads per stage
  constexpr int A_LD = (A_BLK + NW - 1) / NW, W_LD = (W_BLK + NW - 1) / NW;  // per wave
  // Tiles whose stage is small enough get a ring of THREE stages (one-wave-per-SIMD form only): the direct
  // loads of a K tile are then spread over two half-iterations and have a whole iteration more to land.
  constexpr bool RING = NW == 4 && 3 * STAGE <= 160 * 1024;
  constexpr int NLD = A_LD + W_LD, H1 = NLD / 2, H2 = NLD - H1;  // direct loads per wave and K tile; its two halves
  // The 256x256 tile (two 32 KB operand tiles per K tile) uses the whole 160 KB as a ring of FIVE 32 KB units
  // holding A(kt), W(kt), A(kt+1), W(kt+1) and one unit in flight: A(kt+2) is requested in the first half
  // of iteration kt, W(kt+2) in the second half into the unit the barrier has just freed.
  constexpr bool RING5 = NW == 4 && !RING && A_BYTES == W_BYTES && 5 * A_BYTES <= 160 * 1024;
  constexpr int UNIT = A_BYTES;

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

  if constexpr (NW == 4) asm volatile("" ::: CS_ALL_ACC_REGS);  // accounts a[0:255] to this kernel
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
      const int row = (j * NW + wave) * 8 + l_row;  // tile-local
      const int key = (row >> 1) & 7;
      const int r = min(m0 + row, p.M - 1);
      a_src[j] = (uint32_t)(((int64_t)r * p.lda + ((l_slot ^ key) << 3)) * 2);
    }
#pragma unroll
    for (int j = 0; j < W_LD; ++j) {
      const int row = (j * NW + wave) * 8 + l_row;
      const int key = ((((row % (16 * G)) / (4 * G)) & 3) << 1) | ((row >> 1) & 1);
      const int r = min(n0 + row, p.N - 1);
      w_src[j] = (uint32_t)(((int64_t)r * p.ldw + ((l_slot ^ key) << 3)) * 2);
    }
  };
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)p.A, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc((void*)p.W, 0, -1, 0x00020000);
  // Direct loads are buffer loads: a 32-bit per-lane byte offset plus a scalar K offset on a scalar descriptor,
  // so an address costs one register and no vector arithmetic.
  auto load_a = [&](int kt, char* lds_dst, uint32_t off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t*)lds_dst, 16, off, kt * (BK * 2), 0, 0);
  };
  auto load_w = [&](int kt, char* lds_dst, uint32_t off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_void_t*)lds_dst, 16, off, kt * (BK * 2), 0, 0);
  };
  // one direct load of K tile kt into `stage`: IDX < A_LD activation row blocks, then the W row blocks
  auto issue_one_load = [&](int kt, int stage, auto idx_c) {
    constexpr int IDX = decltype(idx_c)::value;
    char* As = smem + stage * STAGE;
    if constexpr (IDX < A_LD) {
      if ((A_BLK % NW == 0) || IDX * NW + wave < A_BLK) load_a(kt, As + (IDX * NW + wave) * 1024, a_src[IDX]);
    } else {
      constexpr int J = IDX - A_LD;
      if ((W_BLK % NW == 0) || J * NW + wave < W_BLK) load_w(kt, As + A_BYTES + (J * NW + wave) * 1024, w_src[J]);
    }
  };
  // five-unit ring: one direct load of operand tile (A or W) of K tile kt into ring unit `slot`
  auto issue_unit_load = [&](int kt, auto is_w_c, int slot, auto idx_c) {
    constexpr int IDX = decltype(idx_c)::value;
    char* dst = smem + slot * UNIT + (IDX * NW + wave) * 1024;
    if constexpr (decltype(is_w_c)::value) load_w(kt, dst, w_src[IDX]);
    else load_a(kt, dst, a_src[IDX]);
  };
  auto issue_loads = [&](int kt, int stage) { static_for<A_LD + W_LD>([&](auto n) { issue_one_load(kt, stage, n); }); };

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
    w_off[ks] = A_BYTES + (wn * WTN + fq * (4 * G) + fr) * 128 + (((ks * 4 + kq) ^ w_key) << 4);
  }

  f32x4_t acc[MT][NT];
  bf16x8_t wf[2][NT], xf[2][MT];
  auto read_frags = [&](int stage, int ks, int b) {
    const char* base = smem + stage * STAGE;
#pragma unroll
    for (int j = 0; j < NT; ++j) wf[b][j] = *(const bf16x8_t*)(base + w_off[ks] + piece_col(j) * 128);
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

  // ---- one-wave-per-SIMD form (NW == 4, 8x8 fragments per wave, 512 registers per lane).  The 64
  //      accumulators live in the accumulation registers a[0:255], accumulator (i, j) in a[4(8i+j) .. +3],
  //      and are touched ONLY by the inline-asm statements below (MFMAs here, v_accvgpr_read in the
  //      epilogue): the compiler sees no accumulator values at all, so it cannot copy, rotate or spill them.
  //      It is told once that the 256 registers are in use (the clobber list at the top of the kernel) so
  //      that the kernel's register allocation covers them, and it has no reason to use them itself as long
  //      as the rest of the kernel fits the 256 architectural registers (the build checks the generated
  //      code for that).  asm volatile statements keep their program order, so the hook called after each
  //      MFMA places LDS reads and direct loads at fixed points of the instruction stream.  The first k-step
  //      of an output tile takes a zero addend, which saves clearing the accumulators.
  auto read_one = [&](int stage, int ks, int b, auto idx_c) {
    constexpr int IDX = decltype(idx_c)::value;
    const char* base = smem + stage * STAGE;
    if constexpr (IDX < NT) wf[b][IDX] = *(const bf16x8_t*)(base + w_off[ks] + piece_col(IDX) * 128);
    else xf[b][IDX - NT] = *(const bf16x8_t*)(base + x_off[ks] + (IDX - NT) * 16 * 128);
  };
  // five-unit ring: fragment IDX of k-step ks from the units holding the A and W tiles
  auto read_one5 = [&](int slot_a, int slot_w, int ks, int b, auto idx_c) {
    constexpr int IDX = decltype(idx_c)::value;
    if constexpr (IDX < NT)
      wf[b][IDX] = *(const bf16x8_t*)(smem + slot_w * UNIT + (w_off[ks] - A_BYTES) + piece_col(IDX) * 128);
    else
      xf[b][IDX - NT] = *(const bf16x8_t*)(smem + slot_a * UNIT + x_off[ks] + (IDX - NT) * 16 * 128);
  };
  auto mfmas_pinned = [&](auto b_c, auto zero_c, auto&& hook) {
    constexpr int B = decltype(b_c)::value;
    constexpr bool ZERO = decltype(zero_c)::value;
    static_for<MT * NT>([&](auto n) {
      constexpr int N = decltype(n)::value, I = N / NT, J = N % NT, R = N * 4;
      if constexpr (ZERO)
        asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" ::"v"(wf[B][J]), "v"(xf[B][I]), "n"(R), "n"(R + 3));
      else
        asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(wf[B][J]), "v"(xf[B][I]), "n"(R), "n"(R + 3));
      hook(n);
    });
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
  if constexpr (RING5) {  // units 0..3 = A(0), W(0), A(1), W(1); nk >= 3 (checked on the host)
    static_for<A_LD>([&](auto n) { issue_unit_load(0, std::false_type{}, 0, n); });
    static_for<W_LD>([&](auto n) { issue_unit_load(0, std::true_type{}, 1, n); });
    static_for<A_LD>([&](auto n) { issue_unit_load(1, std::false_type{}, 2, n); });
    static_for<W_LD>([&](auto n) { issue_unit_load(1, std::true_type{}, 3, n); });
  } else {
    issue_loads(0, 0);
    if (nk > 1) issue_loads(1, 1);
  }
  int ua = 0;  // five-unit ring: unit of A(kt); W(kt), A(kt+1), W(kt+1), A(kt+2) follow cyclically
  if constexpr (RING) static_for<H1>([&](auto n) { issue_one_load(2, 2, n); });  // nk >= 3 (checked on the host)
  int st = 0;  // ring form: LDS stage of the current K tile; keeps rotating across output tiles

  // Persistent loop over this workgroup's tiles (vb, vb + gridDim.x, ...).  The first two K tiles of the
  // NEXT output tile are requested inside the last K iteration of the current one, so they travel while
  // the epilogue runs.
  for (;;) {
  if constexpr (NW == 8) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  }
  const int vb_next = vb + gridDim.x;
  const bool has_next = vb_next < ntiles;
  int m0_next = 0, n0_next = 0;

  CS_TS(0);
  if constexpr (RING5) {
    CS_WAIT_VMCNT(NLD);  // K tile 0 has landed once at most K tile 1's loads are outstanding
    wg_barrier();
    CS_TS(1);
    static_for<MT + NT>([&](auto n) { read_one5(ua, (ua + 1) % 5, 0, 0, n); });
  } else if constexpr (RING) {
    // K tile 0 has landed once at most the loads issued after it are outstanding: K tile 1 and the first
    // half of K tile 2.  (Loads complete in order; stores of the previous epilogue that are still in
    // flight only make this wait longer, never shorter.)
    CS_WAIT_VMCNT(NLD + H1);
    wg_barrier();
    CS_TS(1);
    read_frags(st, 0, 0);
  } else {
    CS_WAIT_VMCNT(0);  // K tiles 0 and 1 of this output tile (and the previous tile's stores)
    wg_barrier();
    CS_TS(1);
    read_frags(0, 0, 0);
  }

  // Ring form of one K iteration.  MODE 0: steady state; 3, 2, 1: that many iterations before the end of
  // the output tile, where the loads switch over to the next output tile's first K tiles.  In iteration kt
  // the first half requests the SECOND half of K tile kt+2 (stage freed one barrier ago) and the second
  // half requests the FIRST half of K tile kt+3 (the stage this iteration's barrier has just freed).
  auto body_ring = [&](int kt, auto first_c, auto mode_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr int MODE = decltype(mode_c)::value;
    constexpr int NFR = MT + NT;
    constexpr int EA = (MT * NT) / H2, EB = (MT * NT) / H1;  // MFMAs per direct load in each half
    static_assert(2 * NFR <= MT * NT && EA >= 1 && EB >= 1, "one slot after an MFMA per LDS read / direct load");
    const int s_cur = st, s_nxt = st == 2 ? 0 : st + 1, s_prv = st == 0 ? 2 : st - 1;
    const int k_a = (MODE == 0 || MODE == 3) ? kt + 2 : 2 - MODE;  // MODE 2 -> next tile's 0, MODE 1 -> 1
    const int k_b = MODE == 0 ? kt + 3 : 3 - MODE;                 // MODE 3 -> next tile's 0, 2 -> 1, 1 -> 2
    __builtin_amdgcn_sched_barrier(0);
    mfmas_pinned(ic<0>{}, std::bool_constant<FIRST>{}, [&](auto n) {
      constexpr int N = decltype(n)::value;
      if constexpr (N < NFR) read_one(s_cur, 1, 1, n);
      if constexpr (N < EA * H2 && N % EA == EA - 1) {
        if constexpr (MODE == 0 || MODE == 3) issue_one_load(k_a, s_prv, ic<H1 + N / EA>{});
        else if (has_next) issue_one_load(k_a, s_prv, ic<H1 + N / EA>{});
      }
    });
    // K tile kt+1 has landed once at most the NLD loads issued after it (K tile kt+2) are outstanding
    if constexpr (MODE == 1) {
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): nothing more is read from LDS for this output tile
    } else if (MODE == 2 && !has_next) {
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    } else {
      __builtin_amdgcn_s_waitcnt(((NLD & 0xF) | ((NLD >> 4) << 14)) | 0x0070);  // vmcnt(NLD) lgkmcnt(0)
    }
    wg_barrier();
    if constexpr (MODE == 3) {
      if (has_next) {
        tile_origin(vb_next, m0_next, n0_next);
        setup_sources(m0_next, n0_next);
      }
    }
    mfmas_pinned(ic<1>{}, std::false_type{}, [&](auto n) {
      constexpr int N = decltype(n)::value;
      if constexpr (MODE != 1 && N < 2 * NFR && N % 2 == 0) read_one(s_nxt, 0, 0, ic<N / 2>{});
      if constexpr (N < EB * H1 && N % EB == EB - 1) {
        if constexpr (MODE == 0) issue_one_load(k_b, s_cur, ic<N / EB>{});
        else if (has_next) issue_one_load(k_b, s_cur, ic<N / EB>{});
      }
    });
    st = s_nxt;
  };

  // Five-unit-ring form of one K iteration.  MODE 0: steady state; 2, 1: that many iterations before the
  // end of the output tile, where the loads belong to the next output tile.
  auto body_ring5 = [&](int kt, auto first_c, auto mode_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr int MODE = decltype(mode_c)::value;
    constexpr int NFR = MT + NT;
    constexpr int EA = (MT * NT) / A_LD, EB = (MT * NT) / W_LD;
    static_assert(2 * NFR <= MT * NT, "one slot after an MFMA per LDS read");
    const int u_a0 = ua, u_w0 = (ua + 1) % 5, u_a1 = (ua + 2) % 5, u_w1 = (ua + 3) % 5, u_a2 = (ua + 4) % 5;
    const int k_ld = MODE == 0 ? kt + 2 : 2 - MODE;  // MODE 2 -> next tile's K tile 0, MODE 1 -> 1
    if constexpr (MODE == 2) {
      if (has_next) {  // every load of this output tile has been issued
        tile_origin(vb_next, m0_next, n0_next);
        setup_sources(m0_next, n0_next);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    mfmas_pinned(ic<0>{}, std::bool_constant<FIRST>{}, [&](auto n) {
      constexpr int N = decltype(n)::value;
      if constexpr (N < NFR) read_one5(u_a0, u_w0, 1, 1, n);
      if constexpr (N < EA * A_LD && N % EA == EA - 1) {
        if constexpr (MODE == 0) issue_unit_load(k_ld, std::false_type{}, u_a2, ic<N / EA>{});
        else if (has_next) issue_unit_load(k_ld, std::false_type{}, u_a2, ic<N / EA>{});
      }
    });
    // K tile kt+1 has landed once at most the A_LD loads issued after it (A of K tile kt+2) are outstanding
    if constexpr (MODE == 1) {
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): nothing more is read from LDS for this output tile
    } else if (MODE == 2 && !has_next) {
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    } else {
      __builtin_amdgcn_s_waitcnt(((A_LD & 0xF) | ((A_LD >> 4) << 14)) | 0x0070);  // vmcnt(A_LD) lgkmcnt(0)
    }
    wg_barrier();
    mfmas_pinned(ic<1>{}, std::false_type{}, [&](auto n) {
      constexpr int N = decltype(n)::value;
      if constexpr (MODE != 1 && N < 2 * NFR && N % 2 == 0) read_one5(u_a1, u_w1, 0, 0, ic<N / 2>{});
      if constexpr (N < EB * W_LD && N % EB == EB - 1) {
        if constexpr (MODE == 0) issue_unit_load(k_ld, std::true_type{}, u_a0, ic<N / EB>{});
        else if (has_next) issue_unit_load(k_ld, std::true_type{}, u_a0, ic<N / EB>{});
      }
    });
    ua = u_a1;
  };

  // One K iteration.  LOADS: tile kt+2 exists and is fetched; NEXT: tile kt+1 exists; LAST: final iteration.
  auto body = [&](int kt, auto first_c, auto loads_c, auto next_c) {
    constexpr bool FIRST = decltype(first_c)::value, LOADS = decltype(loads_c)::value, NEXT = decltype(next_c)::value;
    const int cur = kt & 1;
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (NW == 4) {
      constexpr int NLD = A_LD + W_LD, NFR = MT + NT;
      static_assert(2 * NLD <= MT * NT && 2 * NFR <= MT * NT, "one slot after an MFMA per LDS read / direct load");
      // first k-step; meanwhile the fragments of the second k-step
      mfmas_pinned(ic<0>{}, std::bool_constant<FIRST>{}, [&](auto n) {
        constexpr int N = decltype(n)::value;
        if constexpr (N < NFR) read_one(cur, 1, 1, n);
      });
      // K tile kt+1 (requested one iteration ago) has landed in this wave's part of the other stage, and
      // this wave has received its last fragments of the current stage
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
      wg_barrier();
      if (!NEXT && has_next) {
        tile_origin(vb_next, m0_next, n0_next);
        setup_sources(m0_next, n0_next);
      }
      // second k-step; meanwhile the first fragments of K tile kt+1 and the request for K tile kt+2 into
      // the stage that was just drained (or, at the end, for the next output tile's first two K tiles)
      mfmas_pinned(ic<1>{}, std::false_type{}, [&](auto n) {
        constexpr int N = decltype(n)::value;
        if constexpr (NEXT && N < 2 * NFR && N % 2 == 0) read_one(cur ^ 1, 0, 0, ic<N / 2>{});
        // four waves share the CU's one memory pipeline: space the direct loads as widely as the half allows
        constexpr int LD_EVERY = (MT * NT) / NLD >= 4 ? 4 : ((MT * NT) / NLD >= 3 ? 3 : 2);
        if constexpr (LOADS && N < LD_EVERY * NLD && N % LD_EVERY == LD_EVERY - 1)
          issue_one_load(kt + 2, cur, ic<N / LD_EVERY>{});
        constexpr int PF_EVERY = (MT * NT) / (2 * NLD);
        if constexpr (!NEXT && N < PF_EVERY * 2 * NLD && N % PF_EVERY == PF_EVERY - 1) {
          constexpr int L = N / PF_EVERY;
          if (has_next && (nk > 1 || L < NLD)) issue_one_load(L / NLD, L / NLD, ic<L % NLD>{});
        }
      });
      return;
    }
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
  if constexpr (RING5) {
    constexpr std::true_type T{};
    constexpr std::false_type F{};
    body_ring5(0, T, ic<0>{});
    for (int kt = 1; kt < nk - 2; ++kt) body_ring5(kt, F, ic<0>{});
    body_ring5(nk - 2, F, ic<2>{});
    body_ring5(nk - 1, F, ic<1>{});
  } else if constexpr (RING) {
    constexpr std::true_type T{};
    constexpr std::false_type F{};
    if (nk == 3) {
      body_ring(0, T, ic<3>{});
    } else {
      body_ring(0, T, ic<0>{});
      int kt = 1;
      for (; kt < nk - 3; ++kt) body_ring(kt, F, ic<0>{});
      body_ring(nk - 3, F, ic<3>{});
    }
    body_ring(nk - 2, F, ic<2>{});
    body_ring(nk - 1, F, ic<1>{});
  } else {
    constexpr std::true_type T{};
    constexpr std::false_type F{};
    if (nk >= 3) {
      body(0, T, T, T);
      int kt = 1;
      for (; kt + 2 < nk; ++kt) body(kt, F, T, T);
      body(kt, F, F, T);
      body(kt + 1, F, F, F);
    } else if (nk == 2) {
      body(0, T, F, T);
      body(1, F, F, F);
    } else {
      body(0, T, F, F);
    }
  }
  // inline-asm MFMAs are opaque to the compiler's hazard tracking: let the last results land before the
  // epilogue reads the accumulation registers
  if constexpr (NW == 4) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  CS_TS(2);

  // ---- epilogue.  acc[i][j][r] = C[m][n], m = m0 + wm*WTM + 16i + lane%16,
  //      n = n0 + wn*WTN + (j/G)*16G + (lane/16)*4G + (j%G)*4 + r : 4G consecutive columns per lane, row and group.
  //      Every load the epilogue needs (row map, bias, residual / position rows) is issued up front, from
  //      clamped addresses so that no branch guards a load: a load inside the store loop would make the
  //      compiler wait for ALL outstanding memory operations (vmcnt counts stores too), i.e. for every
  //      store issued so far and for the next tile's prefetch, once per row block.
  {
    const bf16_t* const pBias = (const bf16_t*)p.bias;
    bf16_t* const pC = (bf16_t*)p.C;
    const int n_lane = n0 + wn * WTN + kq * (4 * G);
    int mrow[MT];
    int crow[MT];  // 32-bit row numbers; the 64-bit address is formed at the store
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      mrow[i] = m0 + wm * WTM + i * 16 + fa;
      const int mc = min(mrow[i], p.M - 1);
      crow[i] = p.c_rows ? p.c_rows[mc] : mc;
    }
    bf16x4_t bias_v[NT];  // kept packed: half the registers of fp32 copies
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int nc = min(n_lane + piece_col(j), p.N - 4);
      bias_v[j] = bf16x4_t{0, 0, 0, 0};
      if (pBias) bias_v[j] = *(const bf16x4_t*)(pBias + nc);
    }
    constexpr bool ADDEND = (EPI == CS_EPI_RESIDUAL) || (EPI == CS_EPI_BIAS_POS);
    bf16x4_t addend[ADDEND ? MT : 1][ADDEND ? NT : 1];
    auto load_addend = [&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      const int mc = min(mrow[i], p.M - 1);
      const bf16_t* row = (EPI == CS_EPI_RESIDUAL)
                              ? (const bf16_t*)p.residual + (int64_t)mc * p.ldr
                              : (const bf16_t*)p.pos + (int64_t)(mc % p.pos_period) * p.ldpos;
#pragma unroll
      for (int j = 0; j < NT; ++j)
        addend[ADDEND ? i : 0][ADDEND ? j : 0] = *(const bf16x4_t*)(row + min(n_lane + piece_col(j), p.N - 4));
    };
    // The one-wave-per-SIMD form must stay inside the architectural registers (its accumulation registers
    // are not the compiler's to use), so it fetches the addend rows in two batches.
    constexpr int ADD_BATCH = (NW == 4) ? MT / 2 : MT;
    if constexpr (ADDEND) static_for<ADD_BATCH>(load_addend);
    static_for<MT>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      if constexpr (ADDEND && i == ADD_BATCH && ADD_BATCH < MT)
        static_for<MT - ADD_BATCH>([&](auto k_c) { load_addend(ic<ADD_BATCH + decltype(k_c)::value>{}); });
      const bool mok = mrow[i] < p.M;
      f32x4_t racc[NT];
      if constexpr (NW == 4) {
        static_for<NT * 4>([&](auto e_c) {
          constexpr int E = decltype(e_c)::value;
          float t;
          asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"(i * NT * 4 + E));
          racc[E / 4][E % 4] = t;
        });
      } else {
#pragma unroll
        for (int j = 0; j < NT; ++j) racc[j] = acc[i][j];
      }
      bf16x4_t out[NT];
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = racc[j][r] + bf2f(bias_v[j][r]);
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
      // With G == 2 the pieces of fragments 2g and 2g+1 are adjacent: one 16-byte store per lane, and the
      // four lanes of an output row write 64 consecutive bytes (32 with the halved SwiGLU output).
      if (EPI == CS_EPI_SWIGLU) {
        bf16_t* dst = pC + (int64_t)crow[i] * p.ldc + (n_lane >> 1);
        if constexpr (G == 2) {
#pragma unroll
          for (int j = 0; j < NT; j += 2) {
            if (mok && n_lane + piece_col(j) < p.N) {
              bf16x4_t o = {out[j][0], out[j][1], out[j + 1][0], out[j + 1][1]};
              *(bf16x4_t*)(dst + (piece_col(j) >> 1)) = o;
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            if (mok && n_lane + piece_col(j) < p.N) {
              bf16x2_t o;
              o[0] = out[j][0];
              o[1] = out[j][1];
              *(bf16x2_t*)(dst + (piece_col(j) >> 1)) = o;
            }
          }
        }
      } else {
        bf16_t* dst = pC + (int64_t)crow[i] * p.ldc + n_lane;
        if constexpr (G == 2) {
#pragma unroll
          for (int j = 0; j < NT; j += 2) {
            if (mok && n_lane + piece_col(j) < p.N) {
              bf16x8_t o = {out[j][0], out[j][1], out[j][2], out[j][3], out[j + 1][0], out[j + 1][1], out[j + 1][2], out[j + 1][3]};
              *(bf16x8_t*)(dst + piece_col(j)) = o;
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < NT; ++j)
            if (mok && n_lane + piece_col(j) < p.N) *(bf16x4_t*)(dst + piece_col(j)) = out[j];
        }
      }
    });
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
  constexpr int stage_bytes = (BM + BN) * BK * 2;
  constexpr bool ring3 = WAVES_M * WAVES_N == 4 && 3 * stage_bytes <= 160 * 1024;
  constexpr bool ring5 = WAVES_M * WAVES_N == 4 && !ring3 && BM == BN && 5 * BM * BK * 2 <= 160 * 1024;
  constexpr int lds = ring5 ? 5 * BM * BK * 2 : (ring3 ? 3 : 2) * stage_bytes;
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
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WAVES_M * WAVES_N), lds, stream, p, stagger);
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
  if (a.w_fp8 || a.K % BK || a.K < 3 * BK || a.M < 1 || a.w_scale || a.N < 8) return CS_OK;
  // 16-byte output stores
  if (a.N % 8 || a.ldc % 8 || ((uintptr_t)a.C & 15)) return CS_OK;
  if (a.pos && a.epilogue != CS_EPI_BIAS) return CS_OK;
  // per-lane source offsets are 32-bit byte offsets from the matrix bases
  if (a.a_rows) return CS_OK;  // gathered A rows can lie anywhere: the general kernel keeps 64-bit pointers
  if ((int64_t)a.M * a.lda * 2 >= (int64_t)UINT32_MAX || (int64_t)a.N * a.ldw * 2 >= (int64_t)UINT32_MAX) return CS_OK;  // position addend only pairs with the plain epilogue here
  *handled = true;
  // Tile shape: the one that needs the least chip time (tile quantisation over the 256 CUs).  The narrow
  // 256x160 tile exists for N = 1280 (8 column tiles: 8192 rows give exactly 256 workgroups).
  const double c256 = rounds_cost(a.M, a.N, 256, 256);
  const double c160 = rounds_cost(a.M, a.N, 256, 160) * 1.15;  // narrower tiles: more LDS and L2 traffic per FLOP
  static const char* force = getenv("CS_GEMM_TILE");        // benchmarking aid: "160", "256" or "8" (8-wave 256x256)
  if (force && force[0] == '8') return dispatch_epi<256, 256, 2, 4>(a, stream);
  if (force ? force[0] == '1' : c160 < c256) return dispatch_epi<256, 160, 4, 1>(a, stream);
  // Column split.  When the last round of 256x256 tiles would leave most CUs idle, the leading columns
  // that fill whole rounds go to one launch and the remaining columns to a second launch with smaller
  // tiles (256x128 or 128x192: more workgroups, each shorter).  The two launches write disjoint column
  // ranges of C.
  if (!force) {
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
      hi.N = a.N - n1;
      hi.W = (const char*)a.W + (int64_t)n1 * a.ldw * 2;
      if (a.bias) hi.bias = (const char*)a.bias + (int64_t)n1 * 2;
      if (a.residual) hi.residual = (const char*)a.residual + (int64_t)n1 * 2;
      if (a.pos) hi.pos = (const char*)a.pos + (int64_t)n1 * 2;
      hi.C = (char*)a.C + (int64_t)(a.epilogue == CS_EPI_SWIGLU ? n1 / 2 : n1) * 2;
      const int st = dispatch_epi<256, 256, 2, 2>(lo, stream);
      if (st != CS_OK) return st;
      if (best_192) return dispatch_epi<128, 192, 2, 2>(hi, stream);
      return dispatch_epi<256, 128, 2, 2>(hi, stream);
    }
  }
  return dispatch_epi<256, 256, 2, 2>(a, stream);
}
