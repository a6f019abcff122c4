// Fast-path bf16 MFMA GEMM for gfx950:  C[M,N] = epilogue(A[M,K] . W[N,K]^T),  K % 64 == 0, bf16 weights.
//
// Shape of a workgroup.  FOUR waves, one per SIMD, each with all 512 registers of a lane: the 256
// accumulation registers hold the wave's accumulators (up to 128x128 outputs), the architectural registers
// hold two sets of operand fragments and the addresses.  The accumulators are driven by inline assembly in a
// fixed instruction order: the compiler never sees them, so it cannot copy, rotate or spill them, and the LDS
// reads and direct loads sit at chosen places between the MFMAs.  One workgroup per CU (LDS-bound), the
// kernel is persistent over output tiles.
//
// Pipeline.  K is walked in steps of 64.  Tiles go global -> LDS directly (buffer_load_dwordx4 ... lds: each
// lane fetches 16 bytes and the hardware stores the wave's 64 chunks contiguously at M0 + lane*16).  The loop
// is skewed: the single barrier of an iteration sits BEFORE its last k-step, so the first fragments of the
// next K tile are read while the matrix cores work on that last step.  The four waves share the CU's one
// memory pipeline, and a K tile costs it about half an iteration, so the direct loads must not come in
// bursts: LDS is organised as a RING with more than two K tiles of room, which lets the loads of a K tile be
// issued in two different half-iterations, evenly spaced between the MFMAs, and gives them a whole
// iteration more to land (the weights of an encoder block come from HBM, not from a cache):
//   * 256x256 tile: five 32 KB units = A(kt), W(kt), A(kt+1), W(kt+1) and one in flight.  A(kt+2) is
//     requested in the first half of iteration kt, W(kt+2) in the second half, into the unit that the
//     barrier has just freed.
//   * narrower tiles (256x160, 128x160, 256x128, 128x192): three whole stages.  The second half of K tile kt+2 is
//     requested in the first half of iteration kt, the first half of K tile kt+3 in the second half.
// The sequence of K tiles runs on across output tiles: the next output tile's first K tiles are requested
// in the last iterations of the current one and travel while the epilogue runs.  Waits use the in-order
// completion of loads: "K tile j has landed" == "at most the loads issued after it are outstanding".
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
//
// This header holds the kernel and its launch / epilogue dispatch as templates.  Every tile form is instantiated
// in a translation unit of its own (gemm_fast_t*.hip), so that the forms compile side by side; gemm_fast.hip
// chooses among them.  CS_ALL_ACC_REGS: the accumulation registers belong to inline assembly in every file that
// includes this header (the build checks the compiler's output of each of them).
#pragma once

#include <stdlib.h>

#include <type_traits>
#include <utility>

#include "gemm_common.h"

namespace {

using namespace csgemm;

constexpr int CS_EPI_BIAS_POS = 100;  // internal: CS_EPI_BIAS plus the (row % pos_period) position addend
// internal: the QKV projection of one head per column tile with rotary and window attention as its epilogue (see
// cs_qkv_window_attn): the tile's 256 columns are the head's q (5 fragments), k (5), v (5) and one all-zero fragment
constexpr int CS_EPI_QKV_WATTN = 101;
// internal: the same with windows of 4 .. 64 rows, each in a 64-row slot of its own: the tile's rows are VIRTUAL rows,
// slot v/64, place v%64; place >= the window's row count repeats the window's last row (operand loads), is masked
// (keys) or not stored (queries)
constexpr int CS_EPI_QKV_WATTN_RAGGED = 102;
constexpr int NW = 4;                 // waves per workgroup, one per SIMD
constexpr int LDS_BYTES = 160 * 1024;

// s_waitcnt encodings (gfx9): vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8.
constexpr int waitcnt_vm(int n) { return ((n & 0xF) | ((n >> 4) << 14)) | 0x0F70; }       // vmcnt(n) only
constexpr int waitcnt_vm_lgkm0(int n) { return ((n & 0xF) | ((n >> 4) << 14)) | 0x0070; }  // vmcnt(n) lgkmcnt(0)
constexpr int WAITCNT_LGKM0 = 0xC07F;                                                      // lgkmcnt(0) only

typedef __attribute__((address_space(3))) void lds_void_t;

// Buffer accesses: a scalar descriptor, one 32-bit byte offset per lane and an immediate, so that an address costs no
// 64-bit vector arithmetic.  (Plain functions on purpose: the device-only builtins must not sit in generic lambdas.)
CS_DEVICE u32x4_t buf_ld_u32x4(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0); }
CS_DEVICE u32x2_t buf_ld_u32x2(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0); }
CS_DEVICE uint32_t buf_ld_u32(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0); }
CS_DEVICE f32x4_t buf_ld_f32x4(__amdgpu_buffer_rsrc_t r, uint32_t off) { return __builtin_bit_cast(f32x4_t, buf_ld_u32x4(r, off)); }
CS_DEVICE void buf_st_u32x4(__amdgpu_buffer_rsrc_t r, uint32_t off, u32x4_t v) { __builtin_amdgcn_raw_buffer_store_b128(v, r, off, 0, 0); }
CS_DEVICE void buf_st_u32x2(__amdgpu_buffer_rsrc_t r, uint32_t off, u32x2_t v) { __builtin_amdgcn_raw_buffer_store_b64(v, r, off, 0, 0); }
CS_DEVICE void buf_st_u32(__amdgpu_buffer_rsrc_t r, uint32_t off, uint32_t v) { __builtin_amdgcn_raw_buffer_store_b32(v, r, off, 0, 0); }

// acc + a.lo * b.lo + a.hi * b.hi on words of two bf16 each (v_dot2c_f32_bf16): the row sums of the folded norms are
// taken over the packed output words with it, by every form of the epilogue in the same order.
CS_DEVICE float dot2_bf16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc, false);
}
constexpr uint32_t BF16_ONE_PAIR = 0x3F803F80u;   // {1.0, 1.0}

// Workgroup barrier without the full memory fence of __syncthreads(): the callers order LDS traffic with
// explicit waits, and the asm statements keep the compiler from moving memory operations across it.
CS_DEVICE void wg_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

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

// LDS organisation of a tile shape (shared by the kernel and its launcher).
template <int BM, int BN, bool W_FP8>
struct RingShape {
  static constexpr int A_BYTES = BM * BK * 2, W_BYTES = BN * BK * (W_FP8 ? 1 : 2);
  static constexpr bool FIVE_UNITS = A_BYTES == W_BYTES && 5 * A_BYTES <= LDS_BYTES && 3 * (A_BYTES + W_BYTES) > LDS_BYTES;
  static constexpr int BYTES = FIVE_UNITS ? 5 * A_BYTES : 3 * (A_BYTES + W_BYTES);
  static_assert(BYTES <= LDS_BYTES, "tile does not fit a ring");
};

// W_FP8: the weights are e4m3 bytes with a per-output-channel fp32 scale.  W tiles travel and sit in LDS as bytes
// (half the traffic); a fragment is converted to bf16 in registers right before its MFMAs (exact: every e4m3
// value is a bf16 value) and the scale is applied to the fp32 accumulators in the epilogue.
//
// FUSE: 0 = plain; FUSE_NORM_A = the rows of A stand for their RMS-normalised form: the accumulators are multiplied
// by rsqrt(sum of squares of the A row / K + eps) before the bias (the norm's weight is folded into W by the
// caller); FUSE_SUMSQ_C = besides C, the sum of squares of every output row over this tile's columns goes to
// c_row_sumsq (what the next FUSE_NORM_A launch reads).
// FUSE_LN_A / FUSE_STATS_C: the same for LayerNorm -- the producer also emits the row sums, the consumer computes
// rstd * (acc - mean * w_col_sum[n]) + bias[n] with mean and rstd from the two sets of parts (the norm's weight is
// folded into W, its bias into the GEMM bias, and w_col_sum[n] = sum_k W'[n,k] carries the mean term).
constexpr int FUSE_NORM_A = 1, FUSE_SUMSQ_C = 2, FUSE_LN_A = 3, FUSE_STATS_C = 4;
// The forms whose epilogue takes its residual piece through the LDS ring (see the kernel): residual epilogue on the split
// stream, one wave spanning the tile's columns, bf16 weights.  They use 4 KB of LDS behind the ring.
template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI, bool W_FP8, int FUSE, bool SPLIT_RES>
constexpr bool residual_piece_through_ring() {
  constexpr int MT = BM / WAVES_M / 16, NT = BN / WAVES_N / 16;
  return SPLIT_RES && EPI == CS_EPI_RESIDUAL && NT % 2 == 0 && !W_FP8 && !RingShape<BM, BN, W_FP8>::FIVE_UNITS && WAVES_N == 1 &&
         (MT == 2 || MT == 4) && FUSE != FUSE_NORM_A && FUSE != FUSE_LN_A;
}
template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI, bool W_FP8, int FUSE, bool SPLIT_RES>
__global__ __launch_bounds__(64 * NW) void gemm_fast_kernel(const CsGemmArgs p) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  static_assert(WAVES_M * WAVES_N == NW, "four waves, one per SIMD");
  using Ring = RingShape<BM, BN, W_FP8>;
  constexpr bool WATTN = EPI == CS_EPI_QKV_WATTN || EPI == CS_EPI_QKV_WATTN_RAGGED, RAGGED = EPI == CS_EPI_QKV_WATTN_RAGGED;
  constexpr int A_BYTES = Ring::A_BYTES, W_BYTES = Ring::W_BYTES;
  constexpr bool RING5 = Ring::FIVE_UNITS;
  // Byte offsets of operand tile slots.  Three-stage ring: slot s holds A at s*STAGE and W behind it.
  // Five-unit ring: every unit is one operand tile.
  constexpr int STAGE = A_BYTES + W_BYTES;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0 && BM % 8 == 0 && BN % 8 == 0, "tile shape");
  constexpr int MT = WTM / 16, NT = WTN / 16;
  static_assert(MT * NT * 4 <= 256, "the accumulators of a wave live in its 256 accumulation registers");
  // W fragments come in groups of G: fragment j, fragment row 4q+r holds W row (j/G)*16G + q*4G + (j%G)*4 + r of
  // the wave's rows, so a lane owns 4G consecutive output columns per group and the four lanes q = 0..3 of
  // one output row own 16G consecutive columns.
  constexpr int G = (NT % 2 == 0) ? 2 : NT;
  auto piece_col = [](int j) { return (j / G) * 16 * G + (j % G) * 4; };  // first column of fragment j's piece
  constexpr int W_ROW = W_FP8 ? BK : BK * 2;     // bytes per W tile row
  constexpr int W_ROWS_LD = 1024 / W_ROW;         // W rows per direct load (one load moves 64 x 16 bytes)
  static_assert(BN % W_ROWS_LD == 0, "tile shape");
  constexpr int A_BLK = BM / 8, W_BLK = BN / W_ROWS_LD;  // row blocks = direct loads per operand tile
  static_assert(A_BLK % NW == 0, "every wave issues the same number of direct loads");
  // When W_BLK is not a multiple of the wave count, the waves that have no block left repeat the last one
  // (the same bytes to the same place): every wave must issue the same number of loads, because the waits
  // count loads.
  constexpr int A_LD = A_BLK / NW, W_LD = (W_BLK + NW - 1) / NW;  // per wave
  constexpr int NLD = A_LD + W_LD;                      // direct loads per wave and K tile
  constexpr int NFR = MT + NT;                          // fragment reads per wave and k-step
  constexpr int NMFMA = MT * NT;                        // MFMAs per wave and k-step
  // Fragment reads of the second k-step go after every other MFMA where there are enough of them, else after each.
  constexpr int READ_STRIDE = (2 * NFR <= NMFMA) ? 2 : 1;
  static_assert(READ_STRIDE * NFR <= NMFMA, "one slot after an MFMA per LDS read");

  // ---- tile coordinates of virtual block vb in [0, tiles): XCD-aware remap (workgroup i runs on XCD i%8,
  //      and the persistent stride gridDim.x is a multiple of 8, so a workgroup's tiles stay on its XCD),
  //      then bands of 8 tile-rows walked column-major so the 32 workgroups resident on one XCD share
  //      8 A panels and 4 W panels through that XCD's L2.
  const int ntiles = p.tiles_m * p.tiles_n;
  // ---- workgroups past the computing ones (a launch with few tiles and a prefetch hint): read the hinted bytes once,
  //      16 per lane and four loads in flight, and leave.  They take no part in barriers or in the tile loop.
  if ((int)blockIdx.x >= ntiles) {
    const int pw = (int)blockIdx.x - ntiles, npw = (int)gridDim.x - ntiles;
    const char* const base = (const char*)p.prefetch;
    const int64_t n16 = p.prefetch_bytes >> 4, stride = (int64_t)npw * (64 * NW);
    u32x4_t sink = {0u, 0u, 0u, 0u};
    for (int64_t i = (int64_t)pw * (64 * NW) + threadIdx.x; i < n16; i += 4 * stride) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t j = i + u * stride;
        if (j < n16) {
          const u32x4_t v = *(const u32x4_t*)(base + 16 * j);
          sink[0] |= v[0] & v[1] & v[2] & v[3];
        }
      }
    }
    // (a store that never happens -- M is positive -- keeps the loads alive)
    if (sink[0] == 0xFFFFFFFFu && p.M < 0) *(volatile uint32_t*)p.C = sink[0];
    return;
  }
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

  // The accumulation registers a[0:255] belong to the inline assembly below (MFMAs in the main loop,
  // v_accvgpr_read in the epilogue), accumulator (i, j) in a[4(i*NT+j) .. +3].  The compiler is told once
  // that they are in use, so that the kernel's register allocation covers them; it has no reason to touch
  // them itself as long as the rest of the kernel fits the 256 architectural registers, and the build
  // checks the generated code for exactly that.
  asm volatile("" ::: CS_ALL_ACC_REGS);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WAVES_M, wn = wave / WAVES_M;

  // ---- global sources of the direct loads.  Row block rb = j*NW + wave covers tile rows 8rb..8rb+7; the
  //      lane lands in slot lane%8 of row 8rb + lane/8 and fetches chunk (lane%8) ^ key(row).  Buffer
  //      loads: a 32-bit per-lane byte offset plus a scalar K offset on a scalar descriptor, so an address
  //      costs one register and no vector arithmetic.
  uint32_t a_src[A_LD];
  uint32_t w_src[W_LD];
  auto setup_sources = [&](int m0, int n0) {
    // (the lane number afresh from the hardware, behind an opaque copy: the swizzled chunk offsets are recomputed at
    // every call instead of being kept in registers across the main loop)
    int lane_s = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(lane_s));
    const int l_row = lane_s >> 3, l_slot = lane_s & 7;
#pragma unroll
    for (int j = 0; j < A_LD; ++j) {
      const int row = (j * NW + wave) * 8 + l_row;  // tile-local
      const int key = (row >> 1) & 7;
      int r;
      if constexpr (RAGGED) {
        // the 8 rows of this load lie in one slot (8 divides 64): slot, start and count are wave-uniform
        const int v0 = m0 + (j * NW + wave) * 8;
        const int slot = min(v0 >> 6, p.attn_n_win - 1);
        const int start = p.attn_win_start[slot];
        const int cnt = min(max(p.attn_win_start[slot + 1] - start, 1), 64);
        r = start + min((v0 & 63) + l_row, cnt - 1);
      } else {
        r = min(m0 + row, p.M - 1);
      }
      a_src[j] = (uint32_t)(((int64_t)r * p.lda + ((l_slot ^ key) << 3)) * 2);
    }
#pragma unroll
    for (int j = 0; j < W_LD; ++j) {
      const int blk = min(j * NW + wave, W_BLK - 1);
      if constexpr (W_FP8) {  // 64-byte rows: the lane lands in slot lane%4 of row 16 blk + lane/4
        const int row = blk * 16 + (lane_s >> 2);
        const int key = ((row % (16 * G)) / (4 * G)) & 3;
        const int r = min(n0 + row, p.N - 1);
        w_src[j] = (uint32_t)((int64_t)r * p.ldw + (((lane_s & 3) ^ key) << 4));
      } else {
        const int row = blk * 8 + l_row;
        const int key = ((((row % (16 * G)) / (4 * G)) & 3) << 1) | ((row >> 1) & 1);
        const int r = min(n0 + row, p.N - 1);
        w_src[j] = (uint32_t)(((int64_t)r * p.ldw + ((l_slot ^ key) << 3)) * 2);
      }
    }
  };
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)p.A, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc((void*)p.W, 0, -1, 0x00020000);
  // descriptors of what the epilogue's fast form reads and writes
  const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc((void*)p.C, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_clo = __builtin_amdgcn_make_buffer_rsrc((void*)p.c_lo, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_res = __builtin_amdgcn_make_buffer_rsrc((void*)p.residual, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_reslo = __builtin_amdgcn_make_buffer_rsrc((void*)p.residual_lo, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_bias = __builtin_amdgcn_make_buffer_rsrc((void*)p.bias, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_asumsq = __builtin_amdgcn_make_buffer_rsrc((void*)p.a_row_sumsq, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_asum = __builtin_amdgcn_make_buffer_rsrc((void*)p.a_row_sum, 0, -1, 0x00020000);
  // (The builtin is called from non-generic lambdas on purpose: inside a generic lambda the host pass of the
  // compiler rejects the device-only builtin, silently drops the kernel and leaves its launch stub undefined.)
  auto load_a = [&](int kt, char* lds_dst, uint32_t off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_void_t*)lds_dst, 16, off, kt * (BK * 2), 0, 0);
  };
  auto load_w = [&](int kt, char* lds_dst, uint32_t off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_void_t*)lds_dst, 16, off, kt * W_ROW, 0, 0);
  };
  // Direct load number IDX (A row blocks first, then W row blocks) of K tile kt; a_base / w_base are the
  // LDS byte offsets of the operand tiles it goes to.
  auto direct_load = [&](int kt, int a_base, int w_base, auto idx_c) {
    constexpr int IDX = decltype(idx_c)::value;
    if constexpr (IDX < A_LD) {
      load_a(kt, smem + a_base + (IDX * NW + wave) * 1024, a_src[IDX]);
    } else {
      constexpr int J = IDX - A_LD;
      load_w(kt, smem + w_base + min(J * NW + wave, W_BLK - 1) * 1024, w_src[J]);
    }
  };

  // ---- fragment addressing.  Lane (a = lane%16, kq = lane/16) reads chunk ks*4 + kq of its fragment row.
  //      Both keys depend only on the lane, so the per-lane part of the address is loop-invariant.
  const int fa = lane & 15, kq = lane >> 4;
  // byte offset inside an operand tile of fragment (i or j), k-step ks: row*128 + (((ks*4 + kq) ^ key) << 4)
  int x_off[2], w_off[2];
  auto setup_frag_offsets = [&](int ln) {
    const int fa = ln & 15, kq = ln >> 4;
    const int fq = fa >> 2, fr = fa & 3;
    const int x_key = (fa >> 1) & 7;
    const int w_key = (fq << 1) | ((fr >> 1) & 1);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      x_off[ks] = (wm * WTM + fa) * 128 + (((ks * 4 + kq) ^ x_key) << 4);
      if constexpr (W_FP8)  // 8 bytes: half (kq%2) of chunk 2ks + kq/2, which sits in slot chunk ^ q
        w_off[ks] = (wn * WTN + fq * (4 * G) + fr) * W_ROW + (((ks * 2 + (kq >> 1)) ^ fq) << 4) + (kq & 1) * 8;
      else
        w_off[ks] = (wn * WTN + fq * (4 * G) + fr) * W_ROW + (((ks * 4 + kq) ^ w_key) << 4);
    }
  };
  setup_frag_offsets(lane);
  // Operand fragments: two sets.  fp8 weights are read as 8 raw bytes per fragment and converted into one of
  // two bf16 registers sets right before use.
  bf16x8_t wf[2][W_FP8 ? 1 : NT], xf[2][MT];
  i32x2_t wraw[2][W_FP8 ? NT : 1];
  bf16x8_t wcv[2];
  // Fragment read number IDX of k-step ks into set b.  bf16 weights: W fragments first (MFMAs run i-major and
  // need every W fragment at once); fp8 weights: activation fragments first (MFMAs run j-major).
  auto read_frag = [&](int a_base, int w_base, int ks, int b, auto idx_c) {
    constexpr int IDX = decltype(idx_c)::value;
    if constexpr (W_FP8) {
      if constexpr (IDX < MT) xf[b][IDX] = *(const bf16x8_t*)(smem + a_base + x_off[ks] + IDX * 16 * 128);
      else wraw[b][IDX - MT] = *(const i32x2_t*)(smem + w_base + w_off[ks] + piece_col(IDX - MT) * W_ROW);
    } else {
      if constexpr (IDX < NT) wf[b][IDX] = *(const bf16x8_t*)(smem + w_base + w_off[ks] + piece_col(IDX) * W_ROW);
      else xf[b][IDX - NT] = *(const bf16x8_t*)(smem + a_base + x_off[ks] + (IDX - NT) * 16 * 128);
    }
  };
  auto convert_w = [&](int b, auto j_c) {  // 8 e4m3 bytes -> 8 bf16 (exact)
    constexpr int J = decltype(j_c)::value;
    bf16x8_t o;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const auto p0 = __builtin_amdgcn_cvt_pk_f32_fp8(wraw[b][W_FP8 ? J : 0][h], false);
      const auto p1 = __builtin_amdgcn_cvt_pk_f32_fp8(wraw[b][W_FP8 ? J : 0][h], true);
      o[4 * h + 0] = (bf16_t)p0[0];
      o[4 * h + 1] = (bf16_t)p0[1];
      o[4 * h + 2] = (bf16_t)p1[0];
      o[4 * h + 3] = (bf16_t)p1[1];
    }
    wcv[J & 1] = o;
  };
  // The MFMAs of one k-step on fragment set B, in program order (asm volatile statements keep it), with a
  // hook call after each: that is where LDS reads and direct loads are placed.  ZERO: the first k-step of an
  // output tile takes a zero addend, which saves clearing the accumulators.
  auto mfmas = [&](auto b_c, auto zero_c, auto&& hook) {
    constexpr int B = decltype(b_c)::value;
    constexpr bool ZERO = decltype(zero_c)::value;
    if constexpr (W_FP8) convert_w(B, ic<0>{});
    static_for<NMFMA>([&](auto n) {
      constexpr int N = decltype(n)::value;
      // bf16 weights: i-major; fp8 weights: j-major, the next W fragment is converted while this one is used
      constexpr int I = W_FP8 ? N % MT : N / NT, J = W_FP8 ? N / MT : N % NT, R = (I * NT + J) * 4;
      const bf16x8_t& w = W_FP8 ? wcv[J & 1] : wf[B][W_FP8 ? 0 : J];
      // A register written by a vector instruction must not be read by an MFMA in the next few cycles; the
      // compiler pads that for its own MFMAs but cannot see into these.  Only the first MFMA after a
      // conversion can be that close.
      if constexpr (W_FP8 && I == 0) asm volatile("s_nop 3");
      if constexpr (WATTN && J >= 10) {
        // The V fragments are computed TRANSPOSED (activation rows as the first operand): a lane then owns one
        // head dim and four consecutive keys, the operand layout of the P.V product.  Fragment 15 is padding.
        if constexpr (J < 15) {
          if constexpr (ZERO)
            asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %1, %0, 0" ::"v"(w), "v"(xf[B][I]), "n"(R), "n"(R + 3));
          else
            asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %1, %0, a[%2:%3]" ::"v"(w), "v"(xf[B][I]), "n"(R), "n"(R + 3));
        }
      } else if constexpr (ZERO)
        asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" ::"v"(w), "v"(xf[B][I]), "n"(R), "n"(R + 3));
      else
        asm volatile("v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(w), "v"(xf[B][I]), "n"(R), "n"(R + 3));
      if constexpr (W_FP8 && I == 0 && J + 1 < NT) convert_w(B, ic<J + 1>{});
      hook(n);
    });
  };

  // ---- ring state.  `ring` is the slot of the current K tile: a stage number (three-stage ring) or the
  //      unit of A(kt) with W(kt), A(kt+1), W(kt+1), A(kt+2) following cyclically (five-unit ring).  It
  //      keeps rotating across output tiles.
  constexpr int RING_N = RING5 ? 5 : 3;
  auto slot_add = [](int s, int d) { return (s + d) % RING_N; };
  auto a_base_of = [&](int tile_ahead, int ring) {  // LDS offset of the A tile of K tile kt + tile_ahead
    return RING5 ? slot_add(ring, 2 * tile_ahead) * A_BYTES : slot_add(ring, tile_ahead) * STAGE;
  };
  auto w_base_of = [&](int tile_ahead, int ring) {
    return RING5 ? slot_add(ring, 2 * tile_ahead + 1) * A_BYTES : slot_add(ring, tile_ahead) * STAGE + A_BYTES;
  };
  // Loads of a K tile are issued in two portions; PA of them in the first half of an iteration.
  // Five-unit ring: A(kt+2) in the first half, W(kt+2) in the second (same K tile, AHEAD_B == AHEAD_A).
  // Three-stage ring: the second portion of K tile kt+2 in the first half, the first portion of K tile kt+3
  // in the second half.
  constexpr int PA = RING5 ? A_LD : NLD - NLD / 2;  // loads issued in a first half
  constexpr int PB = NLD - PA;                       // loads issued in a second half
  constexpr int PA_FIRST = RING5 ? 0 : PB;           // index of the first load of the first-half portion
  constexpr int PB_FIRST = RING5 ? A_LD : 0;
  constexpr int AHEAD_A = 2, AHEAD_B = RING5 ? 2 : 3;
  constexpr int EA = NMFMA / PA, EB = NMFMA / PB;    // MFMAs per direct load in each half
  static_assert(EA >= 1 && EB >= 1, "one slot after an MFMA per direct load");
  // Loads outstanding by design at the two wait points: everything issued after the K tile that is needed.
  constexpr int PENDING_AT_BARRIER = RING5 ? PA : NLD;           // after K tile kt+1
  constexpr int PENDING_AT_TILE_START = RING5 ? NLD : NLD + PB;  // after K tile 0 of an output tile

  const int nk = p.K / BK;  // >= 3 (checked on the host)
  int vb = blockIdx.x;
  int m0, n0;
  tile_origin(vb, m0, n0);
  setup_sources(m0, n0);
  int ring = 0;
  // in flight before the first iteration: K tiles 0 and 1, and what a second half would have requested
  static_for<NLD>([&](auto n) { direct_load(0, a_base_of(0, ring), w_base_of(0, ring), n); });
  static_for<NLD>([&](auto n) { direct_load(1, a_base_of(1, ring), w_base_of(1, ring), n); });
  if constexpr (!RING5)
    static_for<PB>([&](auto n) { direct_load(2, a_base_of(2, ring), w_base_of(2, ring), ic<PB_FIRST + decltype(n)::value>{}); });

  for (;;) {  // persistent loop over this workgroup's output tiles (vb, vb + gridDim.x, ...)
    const int vb_next = vb + gridDim.x;
    const bool has_next = vb_next < ntiles;
    int m0_next = 0, n0_next = 0;
    // ---- Residual GEMMs on the split 16-bit stream (the 160-column forms: one wave spans the tile's columns).  Their
    //      epilogue reads a [rows x 160] piece of the residual stream, three bytes per value, that nothing has touched
    //      since the previous encoder block, and with one wave per SIMD nothing hides that latency.  The last output
    //      tile of a workgroup requests no further K tiles, so the slots of the ring fall free one by one in its last
    //      iterations, and the piece is requested straight into them with the same direct-to-LDS loads as the operands
    //      (no registers), per row block of 16 rows: NP loads of the bf16 plane (every lane fetches the 16 bytes of each
    //      pair of pieces it will need, so it reads back its own bytes) and LO_LD loads of the byte plane (the row
    //      block's [16][BN] bytes as one run of 16-byte chunks; 4-byte loads would cost the memory pipeline as much per
    //      load as 16-byte ones).  A wave reads back only what it requested itself, so no barrier is involved.  The
    //      memory pipeline takes about two clocks per cache line a load touches, whoever waits for it, so the loads
    //      are spread: row block 0 (and the bias, into the 4 KB behind the ring) over the second half of the
    //      third-last K iteration and the first half of the second-last, row block 1 over the two half-iterations
    //      after that; row blocks 2 and 3 are requested during the epilogue itself, while row blocks 0 and 1 are
    //      worked on.
    constexpr bool PRE = residual_piece_through_ring<BM, BN, WAVES_M, WAVES_N, EPI, W_FP8, FUSE, SPLIT_RES>();
    constexpr int NP = NT / 2;                          // pairs of pieces: 16 bytes of the bf16 plane per lane
    constexpr int LO_CHUNKS = 16 * BN / 16;             // 16-byte chunks of a row block's byte plane
    constexpr int LO_LD = (LO_CHUNKS + 63) / 64;        // ... and the loads that move them
    constexpr int ROW_LD = NP + LO_LD;                  // direct loads per wave and row block
    constexpr int ROW_HI_BYTES = NW * NP * 1024, ROW_LO_BYTES = NW * LO_LD * 1024, ROW_BYTES = ROW_HI_BYTES + ROW_LO_BYTES;
    static_assert(!PRE || ((MT <= 2 ? ROW_BYTES : ROW_BYTES + ROW_HI_BYTES) <= STAGE && Ring::BYTES + NW * 1024 <= LDS_BYTES && BN * 2 <= 1024 &&
                           2 * (ROW_LD + 1) <= NMFMA && MT <= 4),
                  "two row blocks' bf16 planes and one byte plane fit a ring slot, the bias the room behind the ring");
    const bool fast_tile = p.fast_epilogue && m0 + BM <= p.M && n0 + BN <= p.N;
    const bool pre_on = PRE && fast_tile && !has_next;
    // lane-only byte offsets of the direct loads (the tile and the row block go into the scalar offset)
    uint32_t pre_hi_v = 0, pre_lo_v[PRE ? LO_LD : 1] = {}, pre_bias_v = 0;
    int pre_sbase = 0;   // element offset of the wave's first row and the tile's first column in the residual matrix
    if constexpr (PRE) {
      if (pre_on) {
        int lane_p = lane;
        asm volatile("" : "+v"(lane_p));
        pre_hi_v = ((uint32_t)(lane_p & 15) * (uint32_t)p.ldr + (uint32_t)(lane_p >> 4) * (4 * G)) * 2;
#pragma unroll
        for (int k = 0; k < LO_LD; ++k) {
          const uint32_t g = (uint32_t)min(k * 64 + lane_p, LO_CHUNKS - 1), r = g / (BN / 16), c = g - r * (BN / 16);
          pre_lo_v[k] = r * (uint32_t)p.ldr + c * 16;
        }
        pre_bias_v = (uint32_t)min(lane_p, BN * 2 / 16 - 1) * 16;
        pre_sbase = (m0 + wm * WTM) * (int)p.ldr + n0;
      }
    }
    // Direct load IDX (bf16 plane of pair IDX, then the byte plane's chunks, then -- IDX == ROW_LD -- the bias) of row
    // block I; hi_base / lo_base are the LDS byte offsets of the row block's two regions.  A missing byte plane or
    // bias is replaced by loads of the same size from the bf16 plane (never read back): the waits count loads, so every
    // wave always issues the same number.  (Row block and piece go into the scalar offset: an immediate offset of a
    // direct load would move the LDS side as well.)
    // (a plain lambda around the device-only builtin: see load_a)
    auto dma16 = [&](const __amdgpu_buffer_rsrc_t rs, char* lds_dst, uint32_t voff, int soff) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (lds_void_t*)lds_dst, 16, voff, soff, 0, 0);
    };
    auto residual_to_lds = [&](auto i_c, auto idx_c, int hi_base, int lo_base) {
      constexpr int I = decltype(i_c)::value, IDX = decltype(idx_c)::value;
      if constexpr (IDX < NP) {
        constexpr int COL = (2 * IDX / G) * 16 * G + (2 * IDX % G) * 4;
        dma16(rsrc_res, smem + hi_base + (wave * NP + IDX) * 1024, pre_hi_v, (pre_sbase + I * 16 * (int)p.ldr + COL) * 2);
      } else if constexpr (IDX < ROW_LD) {
        constexpr int Kk = IDX - NP;
        dma16(p.residual_lo ? rsrc_reslo : rsrc_res, smem + lo_base + (wave * LO_LD + Kk) * 1024, pre_lo_v[PRE ? Kk : 0],
              pre_sbase + I * 16 * (int)p.ldr);
      } else {
        dma16(p.bias ? rsrc_bias : rsrc_res, smem + Ring::BYTES + wave * 1024, pre_bias_v, p.bias ? n0 * 2 : 0);
      }
    };
    // loads of row block 0 (+ bias) issued in the second half of the third-last iteration; the rest follows in the
    // first half of the second-last.  Row block 1 likewise, one half-iteration later.
    constexpr int PRE_N0 = ROW_LD + 1, PRE_N0A = (PRE_N0 + 1) / 2, PRE_N1 = ROW_LD, PRE_N1A = (PRE_N1 + 1) / 2;
    // K tile 0 has landed once at most the loads issued after it are outstanding.  (Loads complete in
    // order; stores of the previous epilogue that are still in flight only make this wait longer.)
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(PENDING_AT_TILE_START));
    wg_barrier();
    static_for<NFR>([&](auto n) { read_frag(a_base_of(0, ring), w_base_of(0, ring), 0, 0, n); });

    // One K iteration.  TAIL 0: steady state.  TAIL t > 0: t iterations before the end of the output tile,
    // where the K tiles being requested belong to the next output tile (if there is one).
    auto iteration = [&](int kt, auto first_c, auto tail_c) {
      constexpr bool FIRST = decltype(first_c)::value;
      constexpr int TAIL = decltype(tail_c)::value;
      // Does the portion requested in each half belong to this output tile?  K tile kt + AHEAD exists iff
      // AHEAD < TAIL (or TAIL == 0).
      constexpr bool CUR_A = TAIL == 0 || AHEAD_A < TAIL, CUR_B = TAIL == 0 || AHEAD_B < TAIL;
      const int k_a = CUR_A ? kt + AHEAD_A : AHEAD_A - TAIL;  // K tile number inside its output tile
      const int k_b = CUR_B ? kt + AHEAD_B : AHEAD_B - TAIL;
      // The sources switch to the next output tile once, right before its first load is issued: that is the
      // second-half portion when it runs further ahead than the first-half portion, else the first-half one.
      constexpr bool SWITCH_BEFORE_B = AHEAD_B > AHEAD_A && TAIL == AHEAD_B;
      constexpr bool SWITCH_BEFORE_A = AHEAD_B == AHEAD_A && TAIL == AHEAD_A;
      auto switch_sources = [&]() {
        if (has_next) {
          tile_origin(vb_next, m0_next, n0_next);
          setup_sources(m0_next, n0_next);
        }
      };
      if constexpr (SWITCH_BEFORE_A) switch_sources();
      __builtin_amdgcn_sched_barrier(0);
      // first k-step; meanwhile the fragments of the second k-step and the first-half portion of loads
      mfmas(ic<0>{}, std::bool_constant<FIRST>{}, [&](auto n) {
        constexpr int N = decltype(n)::value;
        if constexpr (N < NFR) read_frag(a_base_of(0, ring), w_base_of(0, ring), 1, 1, n);
        if constexpr (N < EA * PA && N % EA == EA - 1) {
          auto ld = [&]() { direct_load(k_a, a_base_of(AHEAD_A, ring), w_base_of(AHEAD_A, ring), ic<PA_FIRST + N / EA>{}); };
          if constexpr (CUR_A) ld();
          else if (has_next) ld();
        }
        // the rest of row block 0 (second-last iteration) / row block 1 (last): their slot was the current one an
        // iteration ago
        if constexpr (PRE && (TAIL == 2 || TAIL == 1)) {
          constexpr int FIRST_LD = TAIL == 2 ? PRE_N0A : PRE_N1A, COUNT = (TAIL == 2 ? PRE_N0 : PRE_N1) - FIRST_LD, EVERY = NMFMA / COUNT;
          if constexpr (N % EVERY == 0 && N / EVERY < COUNT) {
            if (pre_on) residual_to_lds(ic<2 - TAIL>{}, ic<FIRST_LD + N / EVERY>{}, a_base_of(2, ring), a_base_of(2, ring) + ROW_HI_BYTES);
          }
        }
      });
      // K tile kt+1 has landed in this wave's part of LDS once at most the loads issued after it are
      // outstanding, and this wave has received its last fragments of K tile kt.
      if constexpr (TAIL == 1) {
        __builtin_amdgcn_s_waitcnt(WAITCNT_LGKM0);  // nothing more is read from LDS for this output tile
      } else if (!CUR_A && !has_next) {
        // nothing was requested after K tile kt+1 -- except row block 0 of the residual piece, which may stay in flight
        if (PRE && pre_on) __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(PRE ? PRE_N0 : 0));
        else __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
      } else {
        __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(PENDING_AT_BARRIER));
      }
      wg_barrier();
      if constexpr (SWITCH_BEFORE_B) switch_sources();
      // second k-step; meanwhile the first fragments of K tile kt+1 and the second-half portion of loads,
      // which goes to LDS space that the barrier has just freed
      mfmas(ic<1>{}, std::false_type{}, [&](auto n) {
        constexpr int N = decltype(n)::value;
        if constexpr (TAIL != 1 && N < READ_STRIDE * NFR && N % READ_STRIDE == 0)
          read_frag(a_base_of(1, ring), w_base_of(1, ring), 0, 0, ic<N / READ_STRIDE>{});
        if constexpr (N < EB * PB && N % EB == EB - 1) {
          auto ld = [&]() { direct_load(k_b, a_base_of(AHEAD_B, ring), w_base_of(AHEAD_B, ring), ic<PB_FIRST + N / EB>{}); };
          if constexpr (CUR_B) ld();
          else if (has_next) ld();
        }
        // the residual piece of the workgroup's last tile: first loads of row block 0 (third-last iteration) / row
        // block 1 (second-last) into the slot that the barrier has just freed (the tile requests no K tile any more)
        if constexpr (PRE && (TAIL == 3 || TAIL == 2)) {
          constexpr int COUNT = TAIL == 3 ? PRE_N0A : PRE_N1A, EVERY = NMFMA / COUNT;
          if constexpr (N % EVERY == 0 && N / EVERY < COUNT) {
            if (pre_on) residual_to_lds(ic<3 - TAIL>{}, ic<N / EVERY>{}, a_base_of(0, ring), a_base_of(0, ring) + ROW_HI_BYTES);
          }
        }
      });
      ring = slot_add(ring, RING5 ? 2 : 1);
    };
    {
      constexpr std::true_type T{};
      constexpr std::false_type F{};
      // the last AHEAD_B iterations are tails; everything before is steady state
      if (nk == 3 && AHEAD_B == 3) {
        iteration(0, T, ic<3>{});
      } else {
        iteration(0, T, ic<0>{});
        for (int kt = 1; kt < nk - AHEAD_B; ++kt) iteration(kt, F, ic<0>{});
        if constexpr (AHEAD_B == 3) iteration(nk - 3, F, ic<3>{});
      }
      iteration(nk - 2, F, ic<2>{});
      iteration(nk - 1, F, ic<1>{});
    }
    // inline-asm MFMAs are opaque to the compiler's hazard tracking: let the last results land before the
    // epilogue reads the accumulation registers
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- QKV projection + rotary + window attention for one head and four windows (one window of 64 rows per
    //      wave), entirely in registers.  Accumulator fragment (I, J) of a wave: rows 16I .. 16I+15 of its window;
    //      J = 0..4 q, 5..9 k, 10..14 v (transposed), 15 padding.  For q and k a lane (row lr = lane%16, kq = lane/16)
    //      holds four values per fragment, 20 per tensor: "slot" s = 4(J mod 5) + r stands for head dim 10kq + s
    //      (s < 10) or 40 + 10kq + (s - 10): the caller packs the weight rows in that order, so that both halves of
    //      every rotary pair sit in one lane, and so that eight slots of a lane are exactly one MFMA operand: S^T =
    //      K.Q^T is two 16x16x32 steps and one 16x16x16 step per 16x16 block, straight from the rotated registers.
    //      S^T's accumulators hold four consecutive keys per lane, the layout of the second product's operand, and
    //      the transposed V fragments hold four consecutive keys per head dim: O^T = V^T.P^T needs no transposition.
    auto wattn_epilogue = [&](auto) {   // (generic: only instantiated for the kernel that calls it)
      static_assert(!WATTN || (BM == 256 && BN == 256 && WAVES_M == 4 && WAVES_N == 1),
                    "one 64-row window per wave, one head per column tile");
      constexpr int HD = 80, HALF = 40;
      // A register written by a vector instruction must not be read by an MFMA in the next few cycles.  The compiler
      // pads that for its own MFMAs but cannot see into these, and it is free to place the instruction that produces
      // an operand right in front of the statement that uses it: every MFMA of this epilogue carries its own wait
      // (the previous MFMA still occupies the pipeline meanwhile, so the wait costs nothing).
#define CS_OPERAND_SETTLE "s_nop 3\n\t"
      constexpr bool NORM_A = FUSE == FUSE_NORM_A;
      auto s_reg = [](int b) constexpr { return b < 10 ? 4 * b : 64 + 4 * (b - 10); };   // first register of S^T block b
      int lane_e = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));   // the lane number, afresh
      asm volatile("" : "+v"(lane_e));
      const int lr = lane_e & 15, kq = lane_e >> 4;
      // lane exchanges through bpermute with addresses derived from the opaque lane number: the library shuffles
      // derive them from a lane id that the compiler computes once per kernel and would keep in a register -- an
      // accumulation register -- across the main loop
      const int x16 = (lane_e ^ 16) << 2, x32 = (lane_e ^ 32) << 2;
      auto lane_xchg = [](float v, int byte_addr) {
        return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(byte_addr, __builtin_bit_cast(int, v)));
      };
      // first row and row count of this wave's window (RAGGED: the window of slot (m0 + 64 wm) / 64)
      int row0 = m0 + wm * 64, cnt = 64;
      if (row0 >= p.M) return;                       // (no barrier below: waves may leave independently)
      if constexpr (RAGGED) {
        const int slot = row0 >> 6;
        row0 = p.attn_win_start[slot];
        cnt = min(max(p.attn_win_start[slot + 1] - row0, 1), 64);
      }
      // row of the window at place `local` (rows past the window's last repeat it: finite values that are never used)
      auto row_at = [&](int local) { return RAGGED ? row0 + min(local, cnt - 1) : row0 + local; };
      const int head = n0 / BN;
      const bf16_t* const pBias = (const bf16_t*)p.bias + n0;
      const float* const pScale = p.w_scale + n0;   // fp8 weights: the per-output-channel scales, packed like the bias
      const float sl2 = p.attn_scale_log2e;
      // per-row scale of the folded RMSNorm: rows row0 + 16I + lr
      float rstd[4];
#pragma unroll
      for (int I = 0; I < 4; ++I) {
        rstd[I] = 1.0f;
        if constexpr (NORM_A) {
          const float* parts = p.a_row_sumsq + (int64_t)row_at(16 * I + lr) * CS_SUMSQ_PARTS;
          const f32x4_t s0 = *(const f32x4_t*)parts, s1 = *(const f32x4_t*)(parts + 4);
          const float ss = ((s0[0] + s0[1]) + (s0[2] + s0[3])) + ((s1[0] + s1[1]) + (s1[2] + s1[3]));
          rstd[I] = rsqrtf(ss / (float)p.K + p.norm_eps);
        }
      }
      // bias of the lane's q / k slots (packed like the weight rows: fragment J, lane kq -> 4 consecutive entries)
      // (fp8 weights: fetched per row block next to the scales instead, five at a time)
      bf16x4_t bias_qk[10];
      if constexpr (!W_FP8) {
#pragma unroll
        for (int J = 0; J < 10; ++J) bias_qk[J] = *(const bf16x4_t*)(pBias + (J / 2) * 32 + kq * 8 + (J % 2) * 4);
      }
      bf16x8_t qf8[4][2], kf8[4][2];
      bf16x4_t qf4[4], kf4[4];
      // q and k: scale, bias, rotary (fp32, one rounding), packed as operands
      static_for<4>([&](auto i_c) {
        constexpr int I = decltype(i_c)::value;
        const float* cs = p.attn_cos_sin + (int64_t)row_at(16 * I + lr) * HD + 10 * kq;
        float co[10], si[10];
#pragma unroll
        for (int t = 0; t < 10; t += 2) {   // 8-byte aligned: 40 kq bytes into a 320-byte row
          const f32x2_t c2 = *(const f32x2_t*)(cs + t), s2 = *(const f32x2_t*)(cs + HALF + t);
          co[t] = c2[0];
          co[t + 1] = c2[1];
          si[t] = s2[0];
          si[t + 1] = s2[1];
        }
        static_for<2>([&](auto which_c) {
          constexpr int WHICH = decltype(which_c)::value;   // 0: q (fragments 0..4), 1: k (fragments 5..9)
          // fp8 weights: the scales of these 20 output channels, fetched for every row block anew (behind an opaque
          // offset, so that the compiler does not keep all 40 registers of them across the row blocks)
          f32x4_t wsc[W_FP8 ? 5 : 1];
          if constexpr (W_FP8) {
            int kq_s = kq * 8;
            asm volatile("" : "+v"(kq_s));
#pragma unroll
            for (int J5 = 0; J5 < 5; ++J5) {
              const int ch = ((WHICH * 5 + J5) / 2) * 32 + kq_s + ((WHICH * 5 + J5) % 2) * 4;
              wsc[W_FP8 ? J5 : 0] = *(const f32x4_t*)(pScale + ch);
              bias_qk[WHICH * 5 + J5] = *(const bf16x4_t*)(pBias + ch);
            }
          }
          float x[20];
          static_for<20>([&](auto s_c) {
            constexpr int S = decltype(s_c)::value, J = WHICH * 5 + S / 4, R = (I * NT + J) * 4 + S % 4;
            float t;
            asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"(R));
            if constexpr (W_FP8) t *= wsc[W_FP8 ? S / 4 : 0][S % 4];
            x[S] = t * rstd[I] + bf2f(bias_qk[J][S % 4]);
          });
          float o[20];
#pragma unroll
          for (int t = 0; t < 10; ++t) {
            // (fused multiply-adds: one rounding less than the stand-alone rotary kernel, one instruction less too)
            o[t] = __builtin_fmaf(x[t], co[t], -(x[t + 10] * si[t]));
            o[t + 10] = __builtin_fmaf(x[t + 10], co[t], x[t] * si[t]);
          }
          bf16x8_t f0, f1;
          bf16x4_t f2;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            f0[e] = f2bf(o[e]);
            f1[e] = f2bf(o[8 + e]);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) f2[e] = f2bf(o[16 + e]);
          bf16x8_t(&dst8)[4][2] = WHICH == 0 ? qf8 : kf8;
          bf16x4_t(&dst4)[4] = WHICH == 0 ? qf4 : kf4;
          dst8[I][0] = f0;
          dst8[I][1] = f1;
          dst4[I] = f2;
        });
      });
      // ---- S^T[key][query] = K.Q^T, block b = 4kb + qb in registers that the q and k accumulators have left free
      //      (the transposed V accumulators are still where the main loop put them: fragments 10..14 of every row
      //      block): a[4b ..] for b < 10, a[64 + 4(b - 10) ..] above.  Steps outermost, so that consecutive MFMAs
      //      never depend on each other.
      static_for<16>([&](auto b_c) {
        constexpr int KB = decltype(b_c)::value / 4, QB = decltype(b_c)::value % 4, R = s_reg(KB * 4 + QB);
        const bf16x8_t ka = kf8[KB][0], qb = qf8[QB][0];   // (named copies: asm operands alone do not capture)
        asm volatile(CS_OPERAND_SETTLE "v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" ::"v"(ka), "v"(qb), "n"(R), "n"(R + 3));
      });
      static_for<16>([&](auto b_c) {
        constexpr int KB = decltype(b_c)::value / 4, QB = decltype(b_c)::value % 4, R = s_reg(KB * 4 + QB);
        const bf16x8_t ka = kf8[KB][1], qb = qf8[QB][1];
        asm volatile(CS_OPERAND_SETTLE "v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(ka), "v"(qb), "n"(R), "n"(R + 3));
      });
      static_for<16>([&](auto b_c) {
        constexpr int KB = decltype(b_c)::value / 4, QB = decltype(b_c)::value % 4, R = s_reg(KB * 4 + QB);
        const bf16x4_t ka = kf4[KB], qb = qf4[QB];
        asm volatile(CS_OPERAND_SETTLE "v_mfma_f32_16x16x16_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(ka), "v"(qb), "n"(R), "n"(R + 3));
      });
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
      // ---- softmax over the 64 keys of a query row (16 per lane, 4 lanes per row); P packed as the operand of the
      //      second product: key step t = blocks 2t, 2t+1
      bf16x8_t pf8[4][2];
      static_for<4>([&](auto q_c) {
        constexpr int QB = decltype(q_c)::value;
        float sv[16];
        static_for<16>([&](auto e_c) {
          constexpr int E = decltype(e_c)::value, KB = E / 4, R = s_reg(KB * 4 + QB) + E % 4;
          float t;
          asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"(R));
          // (a lane's four keys of a block are keys 16 KB + 4 kq .. + 3, and a window's row count is a multiple of 4)
          if constexpr (RAGGED) sv[E] = 16 * KB + 4 * kq < cnt ? t : -__builtin_inff();
          else sv[E] = t;
        });
        float mx = sv[0];
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, sv[e]);
        mx = fmaxf(mx, lane_xchg(mx, x16));
        mx = fmaxf(mx, lane_xchg(mx, x32));
        const float mb = mx * sl2;
        bf16x8_t f[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) f[e >> 3][e & 7] = f2bf(__builtin_amdgcn_exp2f(sv[e] * sl2 - mb));
        pf8[QB][0] = f[0];
        pf8[QB][1] = f[1];
      });
      // v (transposed fragments): lane (head dim 16d + lr, kq) holds keys 16I + 4kq + r; operand of key step t = keys
      // of row blocks 2t and 2t+1
      bf16x8_t vf8[5][2];
      {
        // (addresses re-derived behind an opaque copy of the lane number, so that these loads are not hoisted to the
        // top of the epilogue, where the registers are needed for the q and k operands)
        int lane_v = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        asm volatile("" : "+v"(lane_v));
        const int lrv = lane_v & 15;
        float bias_v[5], scale_v[W_FP8 ? 5 : 1];   // fragment row lr of the transposed V fragments
#pragma unroll
        for (int d = 0; d < 5; ++d) {
          const int ch = ((10 + d) / 2) * 32 + (lrv >> 2) * 8 + ((10 + d) % 2) * 4 + (lrv & 3);
          bias_v[d] = bf2f(pBias[ch]);
          if constexpr (W_FP8) scale_v[W_FP8 ? d : 0] = pScale[ch];
        }
        // the folded norm's scale of rows 16I + 4kq + r: recomputed for rows 16I + lr (not kept in registers since the
        // q / k phase) and fetched from the lanes that hold them
        float rv[4][4];
#pragma unroll
        for (int I = 0; I < 4; ++I) {
          float rs = 1.0f;
          if constexpr (NORM_A) {
            const float* parts = p.a_row_sumsq + (int64_t)row_at(16 * I + lrv) * CS_SUMSQ_PARTS;
            const f32x4_t s0 = *(const f32x4_t*)parts, s1 = *(const f32x4_t*)(parts + 4);
            const float ss = ((s0[0] + s0[1]) + (s0[2] + s0[3])) + ((s1[0] + s1[1]) + (s1[2] + s1[3]));
            rs = rsqrtf(ss / (float)p.K + p.norm_eps);
          }
#pragma unroll
          for (int r = 0; r < 4; ++r) rv[I][r] = NORM_A ? lane_xchg(rs, ((lane_v >> 4) * 4 + r) << 2) : 1.0f;
        }
        static_for<5>([&](auto d_c) {
          constexpr int Dd = decltype(d_c)::value, J = 10 + Dd;
          static_for<2>([&](auto t_c) {
            constexpr int T = decltype(t_c)::value;
            bf16x8_t f;
            static_for<8>([&](auto e_c) {
              constexpr int E = decltype(e_c)::value, I = 2 * T + E / 4, R = (I * NT + J) * 4 + E % 4;
              float t;
              asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"(R));
              if constexpr (W_FP8) t *= scale_v[W_FP8 ? Dd : 0];
              f[E] = f2bf(t * rv[I][E % 4] + bias_v[Dd]);
            });
            vf8[Dd][T] = f;
          });
        });
      }
      // ---- O^T[dim][query] = V^T.P^T: block (d, qb) in a[4(4d + qb) ..] (every accumulator has been read by now)
      static_for<20>([&](auto b_c) {
        constexpr int Dd = decltype(b_c)::value / 4, QB = decltype(b_c)::value % 4, R = (Dd * 4 + QB) * 4;
        const bf16x8_t va = vf8[Dd][0], pb = pf8[QB][0];
        asm volatile(CS_OPERAND_SETTLE "v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" ::"v"(va), "v"(pb), "n"(R), "n"(R + 3));
      });
      static_for<20>([&](auto b_c) {
        constexpr int Dd = decltype(b_c)::value / 4, QB = decltype(b_c)::value % 4, R = (Dd * 4 + QB) * 4;
        const bf16x8_t va = vf8[Dd][1], pb = pf8[QB][1];
        asm volatile(CS_OPERAND_SETTLE "v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(va), "v"(pb), "n"(R), "n"(R + 3));
      });
      // the softmax denominators come from the matrix cores as well: a row block of ones in place of V^T sums exactly
      // the rounded weights that the product above used, and leaves the sum of query lr in every register of the lane
      {
        bf16x8_t ones;
#pragma unroll
        for (int e = 0; e < 8; ++e) ones[e] = f2bf(1.0f);
        static_for<4>([&](auto q_c) {
          constexpr int QB = decltype(q_c)::value, R = 80 + 4 * QB;
          const bf16x8_t pb = pf8[QB][0], one = ones;
          asm volatile(CS_OPERAND_SETTLE "v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, 0" ::"v"(one), "v"(pb), "n"(R), "n"(R + 3));
        });
        static_for<4>([&](auto q_c) {
          constexpr int QB = decltype(q_c)::value, R = 80 + 4 * QB;
          const bf16x8_t pb = pf8[QB][1], one = ones;
          asm volatile(CS_OPERAND_SETTLE "v_mfma_f32_16x16x32_bf16 a[%2:%3], %0, %1, a[%2:%3]" ::"v"(one), "v"(pb), "n"(R), "n"(R + 3));
        });
      }
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
      // ---- out[row0 + 16qb + lr][head*80 + 16d + 4kq ..+3] = O^T / l
      bf16_t* const out0 = (bf16_t*)p.C + (int64_t)(row0 + lr) * p.ldc + head * HD + 4 * kq;
      static_for<4>([&](auto q_c) {
        constexpr int QB = decltype(q_c)::value;
        float l_sum;
        asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(l_sum) : "n"(80 + 4 * QB));
        const float inv = 1.0f / l_sum;
        static_for<5>([&](auto d_c) {
          constexpr int Dd = decltype(d_c)::value, R = (Dd * 4 + QB) * 4;
          bf16x4_t o;
          static_for<4>([&](auto r_c) {
            constexpr int Rr = decltype(r_c)::value;
            float t;
            asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"(R + Rr));
            o[Rr] = f2bf(t * inv);
          });
          if (!RAGGED || 16 * QB + lr < cnt) *(bf16x4_t*)(out0 + (int64_t)(16 * QB) * p.ldc + 16 * Dd) = o;
        });
      });
    };
#undef CS_OPERAND_SETTLE
    // ---- epilogue.  Accumulator (i, j), element r = C[m][n], m = m0 + wm*WTM + 16i + lane%16,
    //      n = n0 + wn*WTN + (j/G)*16G + (lane/16)*4G + (j%G)*4 + r : 4G consecutive columns per lane, row and group.
    //      With one wave per SIMD nothing overlaps the epilogue and it is bound by instruction issue (a vector
    //      instruction every four to five clocks), so it comes in two forms.  FAST: the tile lies inside the matrix
    //      and rows are not scattered -- no guards, no clamps, and every access is a buffer instruction (scalar
    //      descriptor + one 32-bit lane offset + an immediate), so an address costs no vector arithmetic.  General:
    //      edge tiles and scattered rows, with guards and 64-bit addresses.  In both, the loads the epilogue needs
    //      (row map, bias, residual / position rows) are issued ahead of the stores that follow them: a load inside the
    //      store loop would make the compiler wait for ALL outstanding memory operations (vmcnt counts stores too),
    //      i.e. for every store issued so far and for the next tile's prefetch, once per row block.
    // ---- epilogue of a residual tile whose residual piece travels through the ring (pre_on).  Per value: accumulator
    //      read, + bias (converted to fp32 once per tile), join / add / split by byte selects (add_split24), the row sums
    //      over the packed output words.  `ring` has moved on three slots since row block 0 was requested, so row block 0
    //      sits in slot ring, row block 1 in slot ring + 1; row block 2 goes to slot ring + 2 and row block 3 behind it
    //      (bf16 plane) and behind row block 0 (byte plane), requested while row blocks 0 and 1 are worked on.
    auto epilogue_from_lds = [&](auto) {
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      const int kq = lane_e >> 4, fa = lane_e & 15;
      const uint32_t row0 = (uint32_t)(m0 + wm * WTM + fa);
      const uint32_t n_lane = (uint32_t)(n0 + wn * WTN + kq * (4 * G));
      const int slot0 = a_base_of(0, ring), slot1 = a_base_of(1, ring), slot2 = a_base_of(2, ring);
      auto hi_base_of = [&](int i) { return i == 0 ? slot0 : i == 1 ? slot1 : i == 2 ? slot2 : slot2 + ROW_BYTES; };
      auto lo_base_of = [&](int i) { return i == 0 ? slot0 + ROW_HI_BYTES : i == 1 ? slot1 + ROW_HI_BYTES : i == 2 ? slot2 + ROW_HI_BYTES : slot0 + ROW_BYTES; };
      // Row block 0 and the bias have landed once at most row block 1, requested after them, is outstanding: loads and
      // stores complete in the order issued.  Row block i > 0 was requested before row block i - 1 was worked on, so it
      // has landed once at most what that work issued is outstanding: 2 NP stores and the loads of row block i + 1.
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(ROW_LD) : "memory");
      const uint32_t lo_mask = p.residual_lo ? 0xFFFFFFFFu : 0u, bias_mask = p.bias ? 0xFFFFFFFFu : 0u;
      float bias_f[NT][4];
      {
        const char* const bsrc = smem + Ring::BYTES + wave * 1024 + kq * (4 * G) * 2;
#pragma unroll
        for (int jp = 0; jp < NP; ++jp) {
          const u32x4_t bw = *(const u32x4_t*)(bsrc + piece_col(2 * jp) * 2);
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            bias_f[2 * jp + w / 2][2 * (w % 2)] = __builtin_bit_cast(float, (bw[w] & bias_mask) << 16);
            bias_f[2 * jp + w / 2][2 * (w % 2) + 1] = __builtin_bit_cast(float, bw[w] & bias_mask & 0xFFFF0000u);
          }
        }
      }
      static_for<MT>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        if constexpr (i > 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NP + (i + 1 < MT ? ROW_LD : 0)) : "memory");
        // (a wave's chunk of a direct load is 64 lanes x 16 bytes; the bf16 plane: every lane reads back what it
        // requested; the byte plane: rows of BN bytes, one after the other)
        const char* const hi_src = smem + hi_base_of(i) + (wave * NP) * 1024 + lane_e * 16;
        const char* const lo_src = smem + lo_base_of(i) + (wave * LO_LD) * 1024 + fa * BN + kq * (4 * G);
        const uint32_t off = (row0 + 16 * i) * (uint32_t)p.ldc + n_lane;   // in elements
        float ss = 0.f, sm = 0.f;
        static_for<NP>([&](auto jp_c) {
          constexpr int JP = decltype(jp_c)::value;
          // row block i + 2 is requested while this one is worked on: its loads are spread over the pairs
          if constexpr (i + 2 < MT) {
            constexpr int PER = (ROW_LD + NP - 1) / NP;
            static_for<PER>([&](auto q_c) {
              constexpr int Q = JP * PER + decltype(q_c)::value;
              if constexpr (Q < ROW_LD) residual_to_lds(ic<i + 2>{}, ic<Q>{}, hi_base_of(i + 2), lo_base_of(i + 2));
            });
          }
          const u32x4_t hi_in = *(const u32x4_t*)(hi_src + JP * 1024);
          // (without a byte plane the ring holds stand-in bytes: masked to zero, no branch)
          const u32x2_t lo_raw = *(const u32x2_t*)(lo_src + piece_col(2 * JP));
          const u32x2_t lo_in = {lo_raw[0] & lo_mask, lo_raw[1] & lo_mask};
          u32x2_t hi_o[2];
          uint32_t lo_o[2];
          static_for<2>([&](auto h_c) {
            constexpr int Hh = decltype(h_c)::value, J = 2 * JP + Hh;
            float v[4];
            static_for<4>([&](auto r_c) {
              constexpr int Rr = decltype(r_c)::value;
              float t;
              asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"((i * NT + J) * 4 + Rr));
              v[Rr] = t + bias_f[J][Rr];
            });
            add_split24(v, u32x2_t{hi_in[2 * Hh], hi_in[2 * Hh + 1]}, lo_in[Hh], hi_o[Hh], lo_o[Hh]);
            if constexpr (FUSE == FUSE_SUMSQ_C || FUSE == FUSE_STATS_C) {
              ss = dot2_bf16(hi_o[Hh][0], hi_o[Hh][0], ss);
              ss = dot2_bf16(hi_o[Hh][1], hi_o[Hh][1], ss);
            }
            if constexpr (FUSE == FUSE_STATS_C) {
              sm = dot2_bf16(hi_o[Hh][0], BF16_ONE_PAIR, sm);
              sm = dot2_bf16(hi_o[Hh][1], BF16_ONE_PAIR, sm);
            }
          });
          buf_st_u32x4(rsrc_c, (off + piece_col(2 * JP)) * 2, u32x4_t{hi_o[0][0], hi_o[0][1], hi_o[1][0], hi_o[1][1]});
          buf_st_u32x2(rsrc_clo, off + piece_col(2 * JP), u32x2_t{lo_o[0], lo_o[1]});
        });
        if constexpr (FUSE == FUSE_SUMSQ_C || FUSE == FUSE_STATS_C) {
          ss += __shfl_xor(ss, 16);
          ss += __shfl_xor(ss, 32);
          if (kq == 0) p.c_row_sumsq[(int64_t)(row0 + 16 * i) * CS_SUMSQ_PARTS + n0 / BN] = ss;
        }
        if constexpr (FUSE == FUSE_STATS_C) {
          sm += __shfl_xor(sm, 16);
          sm += __shfl_xor(sm, 32);
          if (kq == 0) p.c_row_sum[(int64_t)(row0 + 16 * i) * CS_SUMSQ_PARTS + n0 / BN] = sm;
        }
      });
    };
    auto epilogue = [&](auto fast_c) {
      constexpr bool FAST = decltype(fast_c)::value;
      const bf16_t* const pBias = (const bf16_t*)p.bias;
      bf16_t* const pC = (bf16_t*)p.C;
      // The lane's column and row are re-derived behind an opaque copy of the lane number: otherwise the compiler
      // hoists the lane-dependent halves of the epilogue's addresses out of the tile loop and keeps them in registers
      // across the main loop, which has none to spare.
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      const int fa = lane_e & 15, kq = lane_e >> 4;
      const int n_lane = n0 + wn * WTN + kq * (4 * G);
      const int m_lane = m0 + wm * WTM + fa;   // the lane's row of row block 0; block i is 16 i rows further
      int mrow[MT];
      int crow[MT];  // 32-bit row numbers; the 64-bit address is formed at the store
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        mrow[i] = m_lane + i * 16;
        if constexpr (FAST) {
          crow[i] = mrow[i];
        } else {
          const int mc = min(mrow[i], p.M - 1);
          crow[i] = p.c_rows ? p.c_rows[mc] : mc;
        }
      }
      auto clamp_m = [&](int m) { return FAST ? m : min(m, p.M - 1); };
      auto clamp_n = [&](int n) { return FAST ? n : min(n, p.N - 4); };
      constexpr bool NORM_A = FUSE == FUSE_NORM_A || FUSE == FUSE_LN_A;
      float rstd[NORM_A ? MT : 1];
      float nmean_rstd[FUSE == FUSE_LN_A ? MT : 1];   // -mean * rstd
      auto total8 = [&](const float* base, const __amdgpu_buffer_rsrc_t rs, int row) {
        f32x4_t s0, s1;
        if constexpr (FAST) {
          s0 = buf_ld_f32x4(rs, (uint32_t)row * (CS_SUMSQ_PARTS * 4));
          s1 = buf_ld_f32x4(rs, (uint32_t)row * (CS_SUMSQ_PARTS * 4) + 16);
        } else {
          const float* parts = base + (int64_t)row * CS_SUMSQ_PARTS;
          s0 = *(const f32x4_t*)parts;
          s1 = *(const f32x4_t*)(parts + 4);
        }
        return ((s0[0] + s0[1]) + (s0[2] + s0[3])) + ((s1[0] + s1[1]) + (s1[2] + s1[3]));
      };
      if constexpr (FUSE == FUSE_LN_A) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const float mean = total8(p.a_row_sum, rsrc_asum, clamp_m(mrow[i])) / (float)p.K;
          const float var = fmaxf(total8(p.a_row_sumsq, rsrc_asumsq, clamp_m(mrow[i])) / (float)p.K - mean * mean, 0.f);
          rstd[i] = rsqrtf(var + p.norm_eps);
          nmean_rstd[i] = -mean * rstd[i];
        }
      }
      if constexpr (FUSE == FUSE_NORM_A) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const float ss = total8(p.a_row_sumsq, rsrc_asumsq, clamp_m(mrow[i]));
          rstd[i] = rsqrtf(ss / (float)p.K + p.norm_eps);
        }
      }
      f32x4_t csum_v[FUSE == FUSE_LN_A ? NT : 1];
      if constexpr (FUSE == FUSE_LN_A) {
#pragma unroll
        for (int j = 0; j < NT; ++j) csum_v[j] = *(const f32x4_t*)(p.w_col_sum + clamp_n(n_lane + piece_col(j)));
      }
      bf16x4_t bias_v[NT];  // kept packed: half the registers of fp32 copies
      if (pBias) {   // (one branch around all the loads, not one per load)
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          if constexpr (FAST) bias_v[j] = __builtin_bit_cast(bf16x4_t, buf_ld_u32x2(rsrc_bias, (uint32_t)(n_lane + piece_col(j)) * 2));
          else bias_v[j] = *(const bf16x4_t*)(pBias + clamp_n(n_lane + piece_col(j)));
        }
      } else {
#pragma unroll
        for (int j = 0; j < NT; ++j) bias_v[j] = bf16x4_t{0, 0, 0, 0};
      }
      f32x4_t scale_v[W_FP8 ? NT : 1];
      if constexpr (W_FP8) {
#pragma unroll
        for (int j = 0; j < NT; ++j) scale_v[j] = *(const f32x4_t*)(p.w_scale + clamp_n(n_lane + piece_col(j)));
      }
      constexpr bool ADDEND = (EPI == CS_EPI_RESIDUAL) || (EPI == CS_EPI_BIAS_POS);
      // SPLIT: the residual stream is carried with 16 significant bits (bf16 plane + byte plane, see split24)
      constexpr bool SPLIT = SPLIT_RES && EPI == CS_EPI_RESIDUAL;
      bf16x4_t addend[ADDEND ? MT : 1][ADDEND ? NT : 1];
      uint32_t addend_lo[SPLIT ? MT : 1][SPLIT ? NT : 1];   // the four bytes of a piece
      auto load_addend = [&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        if constexpr (FAST && EPI == CS_EPI_RESIDUAL) {
          // lane offset of the row inside the residual matrix; the piece's column is an immediate of the instruction
          const uint32_t off = (uint32_t)mrow[i] * (uint32_t)p.ldr + (uint32_t)n_lane;
          if constexpr (G == 2) {
#pragma unroll
            for (int j = 0; j < NT; j += 2) {
              const u32x4_t w = buf_ld_u32x4(rsrc_res, (off + piece_col(j)) * 2);
              addend[ADDEND ? i : 0][ADDEND ? j : 0] = __builtin_bit_cast(bf16x4_t, u32x2_t{w[0], w[1]});
              addend[ADDEND ? i : 0][ADDEND ? j + 1 : 0] = __builtin_bit_cast(bf16x4_t, u32x2_t{w[2], w[3]});
            }
          } else {
#pragma unroll
            for (int j = 0; j < NT; ++j)
              addend[ADDEND ? i : 0][ADDEND ? j : 0] = __builtin_bit_cast(bf16x4_t, buf_ld_u32x2(rsrc_res, (off + piece_col(j)) * 2));
          }
          if constexpr (SPLIT) {
            if constexpr (G == 2) {
#pragma unroll
              for (int j = 0; j < NT; j += 2) {
                u32x2_t w = {0u, 0u};
                if (p.residual_lo) w = buf_ld_u32x2(rsrc_reslo, off + piece_col(j));
                addend_lo[SPLIT ? i : 0][SPLIT ? j : 0] = w[0];
                addend_lo[SPLIT ? i : 0][SPLIT ? j + 1 : 0] = w[1];
              }
            } else {
#pragma unroll
              for (int j = 0; j < NT; ++j)
                addend_lo[SPLIT ? i : 0][SPLIT ? j : 0] = p.residual_lo ? buf_ld_u32(rsrc_reslo, off + piece_col(j)) : 0u;
            }
          }
        } else {
          const int mc = clamp_m(mrow[i]);
          const bf16_t* row = (EPI == CS_EPI_RESIDUAL)
                                  ? (const bf16_t*)p.residual + (int64_t)mc * p.ldr
                                  : (const bf16_t*)p.pos + (int64_t)(mc % p.pos_period) * p.ldpos;
#pragma unroll
          for (int j = 0; j < NT; ++j)
            addend[ADDEND ? i : 0][ADDEND ? j : 0] = *(const bf16x4_t*)(row + clamp_n(n_lane + piece_col(j)));
          if constexpr (SPLIT) {
            const uint8_t* row_lo = p.residual_lo + (int64_t)mc * p.ldr;
#pragma unroll
            for (int j = 0; j < NT; ++j)
              addend_lo[SPLIT ? i : 0][SPLIT ? j : 0] = p.residual_lo ? *(const uint32_t*)(row_lo + clamp_n(n_lane + piece_col(j))) : 0u;
          }
        }
      };
      // The kernel must stay inside the architectural registers (the accumulation registers are not the
      // compiler's to use), so the addend rows are fetched in batches, the first ahead of the accumulator reads, every
      // later one right before its rows: two batches normally, row by row where the split stream's three registers
      // per piece meet the fp8 scales.
      constexpr int ADD_BATCH = (SPLIT && W_FP8 && MT >= 8) ? 1 : MT / 2;
      auto load_addend_batch = [&](auto b_c) {
        static_for<ADD_BATCH>([&](auto k_c) { load_addend(ic<decltype(b_c)::value * ADD_BATCH + decltype(k_c)::value>{}); });
      };
      if constexpr (ADDEND) load_addend_batch(ic<0>{});
      static_for<MT>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        if constexpr (ADDEND && i % ADD_BATCH == 0 && i > 0) load_addend_batch(ic<i / ADD_BATCH>{});
        const bool mok = FAST || mrow[i] < p.M;
        f32x4_t racc[NT];
        static_for<NT * 4>([&](auto e_c) {
          constexpr int E = decltype(e_c)::value;
          float t;
          asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(t) : "n"(i * NT * 4 + E));
          racc[E / 4][E % 4] = t;
        });
        bf16x4_t out[NT];
        uint32_t out_lo[SPLIT ? NT : 1];
#pragma unroll
        for (int j = 0; j < NT; ++j) {
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float t = racc[j][r];
            if constexpr (W_FP8) t *= scale_v[W_FP8 ? j : 0][r];
            if constexpr (NORM_A) t *= rstd[NORM_A ? i : 0];
            if constexpr (FUSE == FUSE_LN_A) t += nmean_rstd[FUSE == FUSE_LN_A ? i : 0] * csum_v[FUSE == FUSE_LN_A ? j : 0][r];
            v[r] = t + bf2f(bias_v[j][r]);
          }
          if (EPI == CS_EPI_SWIGLU) {
            // SiLU(gate) * up on the fp32 sums, one rounding of the product (the reference rounds gate, SiLU(gate)
            // and up to bf16 on the way, qwen2_5_vl.py:143-148: three roundings this epilogue does not spend
            // instructions on)
            out[j][0] = f2bf(silu(v[0]) * v[1]);
            out[j][1] = f2bf(silu(v[2]) * v[3]);
          } else {
            if (EPI == CS_EPI_GELU_ERF) {
#pragma unroll
              for (int r = 0; r < 4; ++r) v[r] = gelu_erf(v[r]);
            } else if (EPI == CS_EPI_GELU_TANH) {
#pragma unroll
              for (int r = 0; r < 4; ++r) v[r] = gelu_tanh(v[r]);
            } else if (EPI == CS_EPI_QUICK_GELU) {
#pragma unroll
              for (int r = 0; r < 4; ++r) v[r] = quick_gelu(v[r]);
            } else if (ADDEND && !SPLIT) {
#pragma unroll
              for (int r = 0; r < 4; ++r) v[r] = rbf(v[r]) + bf2f(addend[ADDEND ? i : 0][ADDEND ? j : 0][r]);
            }
            if constexpr (SPLIT) {
              u32x2_t hi_words;
              add_split24(v, __builtin_bit_cast(u32x2_t, addend[ADDEND ? i : 0][ADDEND ? j : 0]),
                          addend_lo[SPLIT ? i : 0][SPLIT ? j : 0], hi_words, out_lo[SPLIT ? j : 0]);
              out[j] = __builtin_bit_cast(bf16x4_t, hi_words);
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r) out[j][r] = f2bf(v[r]);
            }
          }
        }
        if constexpr (FUSE == FUSE_SUMSQ_C || FUSE == FUSE_STATS_C) {
          // Sum of squares of the row's ROUNDED outputs over this wave's columns: lane-local over the lane's
          // pieces, then over the four lanes of the row (fixed order: the result does not depend on timing, and
          // neither form of the epilogue changes it: a piece outside the matrix adds exact zeros).
          static_assert(WAVES_N == 1 && EPI != CS_EPI_SWIGLU, "one wave spans the tile's columns: one part per tile");
          float ss = 0.f, sm = 0.f;
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            const bool nok = FAST || n_lane + piece_col(j) < p.N;
            const u32x2_t ow = nok ? __builtin_bit_cast(u32x2_t, out[j]) : u32x2_t{0u, 0u};
            ss = dot2_bf16(ow[0], ow[0], ss);
            ss = dot2_bf16(ow[1], ow[1], ss);
            if constexpr (FUSE == FUSE_STATS_C) {
              sm = dot2_bf16(ow[0], BF16_ONE_PAIR, sm);
              sm = dot2_bf16(ow[1], BF16_ONE_PAIR, sm);
            }
          }
          ss += __shfl_xor(ss, 16);
          ss += __shfl_xor(ss, 32);
          if (mok && kq == 0) p.c_row_sumsq[(int64_t)crow[i] * CS_SUMSQ_PARTS + n0 / BN] = ss;
          if constexpr (FUSE == FUSE_STATS_C) {
            sm += __shfl_xor(sm, 16);
            sm += __shfl_xor(sm, 32);
            if (mok && kq == 0) p.c_row_sum[(int64_t)crow[i] * CS_SUMSQ_PARTS + n0 / BN] = sm;
          }
        }
        // With G == 2 the pieces of fragments 2g and 2g+1 are adjacent: one 16-byte store per lane, and the
        // four lanes of an output row write 64 consecutive bytes (32 with the halved SwiGLU output).
        if constexpr (FAST) {
          if (EPI == CS_EPI_SWIGLU) {
            const uint32_t off = ((uint32_t)mrow[i] * (uint32_t)p.ldc + (uint32_t)(n_lane >> 1)) * 2;
            if constexpr (G == 2) {
#pragma unroll
              for (int j = 0; j < NT; j += 2) {
                const bf16x4_t o = {out[j][0], out[j][1], out[j + 1][0], out[j + 1][1]};
                buf_st_u32x2(rsrc_c, off + (piece_col(j) >> 1) * 2, __builtin_bit_cast(u32x2_t, o));
              }
            } else {
#pragma unroll
              for (int j = 0; j < NT; ++j) {
                const bf16x2_t o = {out[j][0], out[j][1]};
                buf_st_u32(rsrc_c, off + (piece_col(j) >> 1) * 2, __builtin_bit_cast(uint32_t, o));
              }
            }
          } else {
            const uint32_t off = (uint32_t)mrow[i] * (uint32_t)p.ldc + (uint32_t)n_lane;   // in elements
            if constexpr (G == 2) {
#pragma unroll
              for (int j = 0; j < NT; j += 2) {
                const u32x2_t a0 = __builtin_bit_cast(u32x2_t, out[j]), a1 = __builtin_bit_cast(u32x2_t, out[j + 1]);
                buf_st_u32x4(rsrc_c, (off + piece_col(j)) * 2, u32x4_t{a0[0], a0[1], a1[0], a1[1]});
              }
            } else {
#pragma unroll
              for (int j = 0; j < NT; ++j) buf_st_u32x2(rsrc_c, (off + piece_col(j)) * 2, __builtin_bit_cast(u32x2_t, out[j]));
            }
            if constexpr (SPLIT) {
              if constexpr (G == 2) {
#pragma unroll
                for (int j = 0; j < NT; j += 2)
                  buf_st_u32x2(rsrc_clo, off + piece_col(j), u32x2_t{out_lo[SPLIT ? j : 0], out_lo[SPLIT ? j + 1 : 0]});
              } else {
#pragma unroll
                for (int j = 0; j < NT; ++j) buf_st_u32(rsrc_clo, off + piece_col(j), out_lo[SPLIT ? j : 0]);
              }
            }
          }
        } else if (EPI == CS_EPI_SWIGLU) {
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
          if constexpr (SPLIT) {
            uint8_t* dst_lo = p.c_lo + (int64_t)crow[i] * p.ldc + n_lane;
            if constexpr (G == 2) {
#pragma unroll
              for (int j = 0; j < NT; j += 2) {
                if (mok && n_lane + piece_col(j) < p.N) {
                  u32x2_t o = {out_lo[SPLIT ? j : 0], out_lo[SPLIT ? j + 1 : 0]};
                  *(u32x2_t*)(dst_lo + piece_col(j)) = o;
                }
              }
            } else {
#pragma unroll
              for (int j = 0; j < NT; ++j)
                if (mok && n_lane + piece_col(j) < p.N) *(uint32_t*)(dst_lo + piece_col(j)) = out_lo[SPLIT ? j : 0];
            }
          }
        }
      });
    };
    // (p.fast_epilogue: the host has checked that every matrix the epilogue touches lies within 32-bit byte offsets)
    if constexpr (WATTN) {
      wattn_epilogue(0);
      // the next tile's source offsets and the fragment offsets are recomputed rather than kept in registers across
      // this epilogue (the lane number comes from the hardware again, not from a register held since the start)
      if (!has_next) break;
      setup_sources(m0_next, n0_next);
      int lane_again = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
      asm volatile("" : "+v"(lane_again));   // else the compiler proves the offsets loop-invariant and keeps them
      setup_frag_offsets(lane_again);
    }
    else if (PRE && pre_on) {
      if constexpr (PRE) epilogue_from_lds(0);
    } else if (fast_tile) epilogue(std::true_type{});
    else epilogue(std::false_type{});
    if (!has_next) break;
    vb = vb_next;
    m0 = m0_next;
    n0 = n0_next;
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI, bool W_FP8, int FUSE = 0, bool SPLIT_RES = false>
int launch(const CsGemmArgs& a, hipStream_t stream) {
  CsGemmArgs p = a;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  // The epilogue's fast form addresses C, the residual and their byte planes with 32-bit byte offsets from the
  // matrix bases, and takes output row m for accumulator row m.
  const int64_t lim = (int64_t)UINT32_MAX - 64;
  p.fast_epilogue = !p.c_rows && (int64_t)p.M * p.ldc * 2 < lim && (!p.residual || (int64_t)p.M * p.ldr * 2 < lim);
  constexpr int lds = RingShape<BM, BN, W_FP8>::BYTES +
                      (residual_piece_through_ring<BM, BN, WAVES_M, WAVES_N, EPI, W_FP8, FUSE, SPLIT_RES>() ? NW * 1024 : 0);
  static bool attr_set = false;
  auto kern = gemm_fast_kernel<BM, BN, WAVES_M, WAVES_N, EPI, W_FP8, FUSE, SPLIT_RES>;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return CS_ERR_LAUNCH;
    attr_set = true;
  }
  const int tiles = p.tiles_m * p.tiles_n;
  // One resident workgroup per CU (LDS-bound); with more tiles than CUs the kernel is persistent.
  int grid = tiles <= 256 ? tiles : 256;
  // few tiles and a prefetch hint: the idle compute units read the hinted bytes (see the kernel)
  if (p.prefetch && p.prefetch_bytes >= 16 && tiles <= 192) grid = tiles + (256 - tiles < 128 ? 256 - tiles : 128);
  else p.prefetch = nullptr;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), lds, stream, p);
  return cs_launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool W_FP8>
int dispatch_epi_w(const CsGemmArgs& a, hipStream_t s) {
  if constexpr (!W_FP8) {
    // the fused-norm forms exist for the epilogues an encoder block pairs them with
    if (a.a_row_sum) {   // LayerNorm in front of this GEMM
      if (!a.a_row_sumsq || !a.w_col_sum || a.pos || a.c_row_sumsq || a.c_row_sum) return CS_ERR_UNSUPPORTED;
      // (the per-column sums take 4 registers per piece on top of the bias: with the 64 pieces of a 256x256 tile's
      // wave the epilogue no longer fits the architectural registers, so that tile is not built; cs_gemm_fast
      // sends these launches to the 256x160 tile)
      if constexpr (BM == 256 && BN == 256) return CS_ERR_UNSUPPORTED;
      else switch (a.epilogue) {
        case CS_EPI_BIAS: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS, false, FUSE_LN_A>(a, s);
        case CS_EPI_GELU_TANH: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_GELU_TANH, false, FUSE_LN_A>(a, s);
        case CS_EPI_QUICK_GELU: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_QUICK_GELU, false, FUSE_LN_A>(a, s);
        default: return CS_ERR_UNSUPPORTED;
      }
    }
    if (a.c_row_sum) {   // ... and behind it: sums and sums of squares of the output rows
      if (!a.c_row_sumsq || a.pos) return CS_ERR_UNSUPPORTED;
      if constexpr (BN == 160 && WAVES_N == 1) {
        if (a.epilogue == CS_EPI_RESIDUAL)
          return a.c_lo ? launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_RESIDUAL, false, FUSE_STATS_C, true>(a, s)
                        : launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_RESIDUAL, false, FUSE_STATS_C>(a, s);
      }
      return CS_ERR_UNSUPPORTED;
    }
    if (a.a_row_sumsq) {
      if (a.pos || a.c_row_sumsq) return CS_ERR_UNSUPPORTED;
      if (a.epilogue == CS_EPI_BIAS) return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS, false, FUSE_NORM_A>(a, s);
      if (a.epilogue == CS_EPI_SWIGLU) return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_SWIGLU, false, FUSE_NORM_A>(a, s);
      return CS_ERR_UNSUPPORTED;
    }
    if (a.c_row_sumsq) {
      if constexpr (BN == 160 && WAVES_N == 1) {
        if (a.epilogue == CS_EPI_RESIDUAL)
          return a.c_lo ? launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_RESIDUAL, false, FUSE_SUMSQ_C, true>(a, s)
                        : launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_RESIDUAL, false, FUSE_SUMSQ_C>(a, s);
        if (a.epilogue == CS_EPI_BIAS && !a.pos) return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS, false, FUSE_SUMSQ_C>(a, s);
      }
      return CS_ERR_UNSUPPORTED;
    }
  } else {
    if (a.a_row_sumsq || a.c_row_sumsq || a.a_row_sum || a.c_row_sum) return CS_ERR_UNSUPPORTED;
  }
  switch (a.epilogue) {
    case CS_EPI_BIAS:
      if constexpr (!W_FP8) {
        if (a.pos) return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS_POS, false>(a, s);
      }
      return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_BIAS, W_FP8>(a, s);
    case CS_EPI_RESIDUAL:
      return a.c_lo ? launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_RESIDUAL, W_FP8, 0, true>(a, s)
                    : launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_RESIDUAL, W_FP8>(a, s);
    case CS_EPI_SWIGLU: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_SWIGLU, W_FP8>(a, s);
    case CS_EPI_GELU_ERF: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_GELU_ERF, W_FP8>(a, s);
    case CS_EPI_GELU_TANH: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_GELU_TANH, W_FP8>(a, s);
    case CS_EPI_QUICK_GELU: return launch<BM, BN, WAVES_M, WAVES_N, CS_EPI_QUICK_GELU, W_FP8>(a, s);
    default: return CS_ERR_INVALID_ARG;
  }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int dispatch_epi(const CsGemmArgs& a, hipStream_t s) {
  if (a.w_fp8) {
    // (the few-rows form is only dispatched for bf16 weights: its fp8 kernels are not built)
    if constexpr (BM == 128 && BN == 160) return CS_ERR_UNSUPPORTED;
    else return dispatch_epi_w<BM, BN, WAVES_M, WAVES_N, true>(a, s);
  }
  return dispatch_epi_w<BM, BN, WAVES_M, WAVES_N, false>(a, s);
}

}  // namespace
