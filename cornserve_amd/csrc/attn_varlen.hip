// Variable-length, non-causal flash attention on MFMA for gfx950.
//
// Replaces flash_attn_varlen_func (eric/models/qwen2_5_vl.py:110-120: block-diagonal attention over
// cu_seqlens segments, softmax scale head_dim^-0.5, no dropout, no mask inside a segment) and
// xformers memory_efficient_attention_forward (eric/models/layers/attention.py:51, one segment per
// image).  Optionally applies the Qwen2.5-VL rotary embedding (qwen2_5_vl.py:26-33) to q and k while
// they are staged into LDS, so the rotated tensors never exist in HBM.
//
// Decomposition.  A workgroup owns one query block (<= 32*NWAVES rows of one segment) of one head and
// streams that segment's keys/values through LDS in tiles of 64.  Each wave owns 32 query rows.
// Both products are computed TRANSPOSED so that a lane owns one query column of every accumulator:
//     S^T[key][q] = K[key][:] . Q[q][:]      (MFMA A operand = K rows, B operand = Q rows, k = head dim)
//     O^T[d][q]  += V^T[d][key] . P^T[key][q] (A operand = V^T rows, B operand = P, k = keys)
// With the 32x32 accumulator layout (lane -> column q = lane%32, 16 rows per lane) the online-softmax
// max / sum over keys is 32 in-register operations plus one exchange with lane^32, the rescale of O is
// a per-lane scalar, and P goes from the S accumulators straight into the B operand of the second
// product without touching LDS: accumulator rows 8kk..8kk+7 of a lane are keys
// {16kk+4h+0..3, 16kk+8+4h+0..3} (h = lane/32); the V^T fragment is read from LDS with the same key
// order, which is legal because a dot product does not care about the order of its terms.
// V goes to LDS row-major like K; the transposition happens in the LDS read: ds_read_b64_tr_b16 hands each
// lane of a 16-lane group four 16-bit values gathered from four other lanes' addresses, which turns a
// [4 keys x 16 dims] block into "lane l holds 4 consecutive keys of dim l".
// Head dims that are not multiples of 16 (SigLIP's 72) are zero-padded in LDS only.
#include <type_traits>

#include "common.h"

namespace {

constexpr int BKV = 64;        // keys per LDS tile
constexpr int V_RS = 192;      // bytes per key row of a V tile in LDS (96 head-dim slots).  192 = 64 mod 256: the four
                               // key rows x 64 bytes that 32 lanes of a transposing read touch fall into distinct banks.

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4_t lds_s16x4_t;

// A-operand fragment of V^T for the 32x32x16 MFMA: lane (fr = lane%32, hf = lane/32) gets dim 32t + fr and the
// keys {16g + 4hf + 0..3, 16g + 8 + 4hf + 0..3} of key group g -- the key order in which the S^T accumulators
// hold P.  ds_read_b64_tr_b16 works on groups of 16 lanes: destination lane l receives element l%4 of the
// 8 bytes addressed by source lanes l/4 + 4e, e = 0..3.  So source lane s = 4e + j of a group addresses key
// k0 + e, dims d0 + 4j .. 4j+3, and destination lane l ends up with dim d0 + l, keys k0 .. k0+3.
CS_DEVICE bf16x8_t read_vt_frag(const char* v_tile, int t, int g, int lane) {
  const int hf = lane >> 5, s = lane & 15;
  const int key = 16 * g + 4 * hf + (s >> 2);
  const int dim = 32 * t + 16 * ((lane >> 4) & 1) + 4 * (s & 3);
  const char* p = v_tile + key * V_RS + dim * 2;
  const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)p);
  const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(p + 8 * V_RS));
  return __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

struct AttnArgs {
  const bf16_t* q;
  const bf16_t* k;
  const bf16_t* v;
  int64_t ld;
  bf16_t* out;
  int64_t ldo;
  const int32_t* work;
  const float* cos_sin;
  float scale_log2e;
  // full-attention kernel only: 1-D launch, see its workgroup mapping
  int n_work, heads, chunk, n_chunks_x;
};

// ---- pieces shared by the attention kernels.  A wave owns 32 query rows (lane % 32 = query, lane / 32 = which
//      half of the 8-row groups of a 32x32 MFMA result it holds) and works on tiles of BKV = 64 keys.

// S^T = K.Q^T for one key tile in LDS (row stride RS bytes), keys past `nvalid` masked to -inf.
template <int KS, int RS>
CS_DEVICE void score_tile(f32x16_t (&sacc)[2], const char* k_tile, const bf16x8_t (&qf)[KS], int nvalid, int fr, int hf) {
#pragma unroll
  for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[kt][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8_t kf = *(const bf16x8_t*)(k_tile + (kt * 32 + fr) * RS + (2 * ks + hf) * 16);
      sacc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], sacc[kt], 0, 0, 0);
    }
  }
  if (nvalid < BKV) {  // uniform: only the last tile of a segment can be partial
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = kt * 32 + 8 * (r >> 2) + 4 * hf + (r & 3);
        if (key >= nvalid) sacc[kt][r] = -INFINITY;
      }
  }
}

// Online softmax of one tile's scores -> P (bf16 fragments for the P.V product).
// Lazy reference maximum: P = exp2((s - m_run) * scale) with an m_run that is only raised when some query of the
// wave sees a score more than LAZY_LOG2 (in log2 units) above it.  P then ranges up to 2^LAZY_LOG2 instead of 1,
// which fp32 accumulation and bf16's exponent range do not care about, the final division by the denominator
// (built from the same P) cancels the reference, and the rescale of O -- DT*16 multiplies and an exponential per
// tile -- runs only in the first tiles of a segment.  m_run starts at -inf, so the first tile always sets it to
// its own maximum.  With L_FROM_MFMA the denominator is not summed here (see attn_full_kernel).
// FIRST_TILE: the caller knows that nothing has been accumulated yet (O = 0, m_run = -inf): no rescale to consider.
template <int DT, bool L_FROM_MFMA, bool FIRST_TILE = false>
CS_DEVICE void softmax_tile(const f32x16_t (&sacc)[2], bf16x8_t (&pf)[2][2], f32x16_t (&oacc)[DT], float& m_run,
                            float& l_run, float sl2) {
  float mx = -INFINITY;
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kt][r]);
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  constexpr float LAZY_LOG2 = 6.0f;
  float alpha = 1.0f;
  if constexpr (FIRST_TILE) {
    m_run = mx;
  } else if (__any((mx - m_run) * sl2 > LAZY_LOG2)) {
    const float m_new = fmaxf(m_run, mx);
    alpha = __builtin_amdgcn_exp2f((m_run - m_new) * sl2);
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[t][r] *= alpha;
    m_run = m_new;
  }
  const float mb = m_run * sl2;
  float psum = 0.f;
#pragma unroll
  for (int kt = 0; kt < 2; ++kt)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float pv = __builtin_amdgcn_exp2f(sacc[kt][r] * sl2 - mb);
      if constexpr (!L_FROM_MFMA) psum += pv;
      pf[kt][r >> 3][r & 7] = f2bf(pv);
    }
  if constexpr (!L_FROM_MFMA) {
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
  }
}

// O^T[d][q] / l -> out[q][d0 ...]: a lane owns query `qi` and 4 consecutive d per 8-row group.  With L_FROM_MFMA the
// denominator is row D of O^T (block D/32, row D%32 = 8g + 4*half + e), held by the lanes of one half.
template <int D, int DT, bool L_FROM_MFMA>
CS_DEVICE void write_output(const f32x16_t (&oacc)[DT], float l_run, bf16_t* orow, bool valid, int hf) {
  if constexpr (L_FROM_MFMA) {
    constexpr int RR = D % 32, G_L = RR / 8, HF_L = (RR % 8) / 4, E_L = RR % 4;
    const float mine = oacc[D / 32][4 * G_L + E_L];
    const float other = __shfl_xor(mine, 32, 64);
    l_run = hf == HF_L ? mine : other;
  }
  if (!valid) return;
  const float inv = 1.0f / l_run;
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d0 = t * 32 + 8 * g + 4 * hf;
      if (d0 < D) {
        bf16x4_t o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = f2bf(oacc[t][4 * g + e] * inv);
        *(bf16x4_t*)(orow + d0) = o;
      }
    }
}

template <int D, int NWAVES, bool ROPE, int HPW>
__global__ __launch_bounds__(NWAVES * 64, 2) void attn_kernel(const AttnArgs a) {
  constexpr int NT = NWAVES * 64;
  constexpr int BQ = NWAVES * 32;
  constexpr int KS = (D + 15) / 16;    // MFMA k-steps over the head dim
  constexpr int DT = (D + 31) / 32;    // 32-row tiles of O^T
  constexpr int DC = D / 8;            // real 16-byte chunks per row
  constexpr int DKC = KS * 2;          // chunks per row after zero padding
  constexpr int RS = (DKC | 1) * 16;   // LDS row stride in bytes, odd chunk count: conflict-free b128 reads
  static_assert(D % 8 == 0 && D <= 96, "head dim");
  static_assert(!ROPE || D % 16 == 0, "rotary needs an even number of chunks per half");
  // The softmax denominator comes out of the P.V product through a column of ones in the V tile when the head
  // dim leaves spare rows in the last 32-row block of O^T (see attn_full_kernel; the same arithmetic in every
  // attention kernel keeps an item's result independent of which of them a batch's longest segment selects).
  constexpr bool L_FROM_MFMA = (D % 32) != 0;

  __shared__ __attribute__((aligned(16))) char q_lds[BQ * RS];
  __shared__ __attribute__((aligned(16))) char k_lds[BKV * RS];
  __shared__ __attribute__((aligned(16))) char v_lds[BKV * V_RS];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int fr = lane & 31, hf = lane >> 5;
  const int head0 = blockIdx.y * HPW;  // this workgroup's HPW consecutive heads
  const int seg_start = a.work[blockIdx.x * 4 + 0];
  const int seg_end = a.work[blockIdx.x * 4 + 1];
  const int q0 = a.work[blockIdx.x * 4 + 2];
  const int nq = a.work[blockIdx.x * 4 + 3];
  int64_t hoff = (int64_t)head0 * D;  // column offset of the head being processed
  if constexpr (L_FROM_MFMA) {  // chunk DC of every V row := (1, 0, ..., 0); the staging below never writes there
    bf16x8_t one = {0, 0, 0, 0, 0, 0, 0, 0};
    one[0] = f2bf(1.0f);
    for (int r = tid; r < BKV; r += NT) *(bf16x8_t*)(v_lds + r * V_RS + DC * 16) = one;
  }

  // Stage `nrows` rows starting at global row g0 (valid rows: < g0 + nvalid) of a [*, ld] tensor into an
  // LDS tile with row stride RS, zero-filling invalid rows and pad chunks, optionally rotating.
  auto stage_rows = [&](const bf16_t* src, char* dst, int g0, int nrows, int nvalid) {
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    if (ROPE) {
      constexpr int HC = DC / 2;  // chunks per half
      for (int i = tid; i < nrows * HC; i += NT) {
        const int r = i / HC, jc = i - r * HC;
        bf16x8_t o1 = zero, o2 = zero;
        if (r < nvalid) {
          const int64_t g = g0 + r;
          const bf16_t* p = src + g * a.ld + hoff + jc * 8;
          const bf16x8_t x1 = *(const bf16x8_t*)p;
          const bf16x8_t x2 = *(const bf16x8_t*)(p + D / 2);
          const float* cs = a.cos_sin + g * D + jc * 8;
          const f32x4_t c0 = *(const f32x4_t*)cs, c1 = *(const f32x4_t*)(cs + 4);
          const f32x4_t s0 = *(const f32x4_t*)(cs + D / 2), s1 = *(const f32x4_t*)(cs + D / 2 + 4);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float co = e < 4 ? c0[e] : c1[e - 4];
            const float si = e < 4 ? s0[e] : s1[e - 4];
            const float xa = bf2f(x1[e]), xb = bf2f(x2[e]);
            o1[e] = f2bf(rot_first(xa, xb, co, si));
            o2[e] = f2bf(rot_second(xa, xb, co, si));
          }
        }
        *(bf16x8_t*)(dst + r * RS + jc * 16) = o1;
        *(bf16x8_t*)(dst + r * RS + (jc + HC) * 16) = o2;
      }
    } else {
      for (int i = tid; i < nrows * DKC; i += NT) {
        const int r = i / DKC, c = i - r * DKC;
        bf16x8_t x = zero;
        if (r < nvalid && c < DC) x = *(const bf16x8_t*)(src + (int64_t)(g0 + r) * a.ld + hoff + c * 8);
        *(bf16x8_t*)(dst + r * RS + c * 16) = x;
      }
    }
    if (ROPE && DKC > DC) {
      for (int i = tid; i < nrows * (DKC - DC); i += NT) {
        const int r = i / (DKC - DC), c = DC + i % (DKC - DC);
        *(bf16x8_t*)(dst + r * RS + c * 16) = zero;
      }
    }
  };

  // V tile -> LDS, row-major; rows past the segment end are zero (they meet P = 0, which must not be 0 * NaN).
  auto stage_v = [&](int g0, int nvalid) {
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = tid; i < BKV * DC; i += NT) {
      const int r = i / DC, c = i - r * DC;
      bf16x8_t x = zero;
      if (r < nvalid) x = *(const bf16x8_t*)(a.v + (int64_t)(g0 + r) * a.ld + hoff + c * 8);
      *(bf16x8_t*)(v_lds + r * V_RS + c * 16) = x;
    }
  };

  f32x16_t oacc[DT];
  float m_run, l_run;
  auto reset_state = [&]() {
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[t][r] = 0.f;
    m_run = -INFINITY;
    l_run = 0.f;
  };
  const bool wave_active = wave * 32 < nq;
  auto write_out = [&]() {
    const int qi = wave * 32 + fr;
    write_output<D, DT, L_FROM_MFMA>(oacc, l_run, a.out + (int64_t)(q0 + min(qi, nq - 1)) * a.ldo + hoff, qi < nq, hf);
  };
  bf16x8_t qf[KS];
  auto load_q_frags = [&]() {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const bf16x8_t*)(q_lds + (wave * 32 + fr) * RS + (2 * ks + hf) * 16);
  };

  // One K/V tile in LDS (nvalid keys): S^T = K Q^T, online softmax, O^T += V^T P^T.
  auto compute_tile = [&](int nvalid, auto first_c) {
    f32x16_t sacc[2];
    bf16x8_t pf[2][2];
    score_tile<KS, RS>(sacc, k_lds, qf, nvalid, fr, hf);
    softmax_tile<DT, L_FROM_MFMA, decltype(first_c)::value>(sacc, pf, oacc, m_run, l_run, a.scale_log2e);
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const bf16x8_t vf = read_vt_frag(v_lds, t, kt * 2 + kk, lane);
          oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kt][kk], oacc[t], 0, 0, 0);
        }
    }
  };

  const int seg_len = seg_end - seg_start;
  if (ROPE && BQ == BKV && seg_len <= BKV && q0 == seg_start) {
    // A whole segment in one tile (window attention): the query rows ARE the key rows.  Every global load
    // of a head -- q, k, v -- is issued in one batch into registers, the rotary table is fetched once
    // for all HPW heads, and the batch of head h+1 is requested before the matrix-core work on head h,
    // so after the first head the memory latency hides behind compute.
    constexpr int HC = DC / 2;
    constexpr int NI = (BKV * HC + NT - 1) / NT, NV = (BKV * DC + NT - 1) / NT;
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8_t q1[NI], q2[NI], k1[NI], k2[NI], vx[NV];
    f32x4_t c0[NI], c1[NI], s0[NI], s1[NI];
    // Unconditional loads from clamped rows (no branch between them, so they are all in flight together).
    // Rows past the segment end therefore hold copies of the last row: as keys they are masked (P = 0, and
    // 0 times a finite V row is 0), as queries their outputs are never written.
#pragma unroll
    for (int it = 0; it < NI; ++it) {
      const int i = min(tid + it * NT, BKV * HC - 1), r = i / HC, jc = i - r * HC;
      const float* cs = a.cos_sin + (int64_t)(seg_start + min(r, seg_len - 1)) * D + jc * 8;
      c0[it] = *(const f32x4_t*)cs;
      c1[it] = *(const f32x4_t*)(cs + 4);
      s0[it] = *(const f32x4_t*)(cs + D / 2);
      s1[it] = *(const f32x4_t*)(cs + D / 2 + 4);
    }
    auto issue_qkv = [&](int64_t ho) {
#pragma unroll
      for (int it = 0; it < NI; ++it) {
        const int i = min(tid + it * NT, BKV * HC - 1), r = i / HC, jc = i - r * HC;
        const int64_t off = (int64_t)(seg_start + min(r, seg_len - 1)) * a.ld + ho + jc * 8;
        q1[it] = *(const bf16x8_t*)(a.q + off);
        q2[it] = *(const bf16x8_t*)(a.q + off + D / 2);
        k1[it] = *(const bf16x8_t*)(a.k + off);
        k2[it] = *(const bf16x8_t*)(a.k + off + D / 2);
      }
#pragma unroll
      for (int it = 0; it < NV; ++it) {
        const int i = min(tid + it * NT, BKV * DC - 1), r = i / DC, c = i - r * DC;
        vx[it] = *(const bf16x8_t*)(a.v + (int64_t)(seg_start + min(r, seg_len - 1)) * a.ld + ho + c * 8);
      }
    };
    issue_qkv(hoff);
    if (DKC > DC) {  // pad chunks of the q and k tiles: written once, never overwritten
      for (int i = tid; i < BKV * (DKC - DC); i += NT) {
        const int r = i / (DKC - DC), c = DC + i % (DKC - DC);
        *(bf16x8_t*)(q_lds + r * RS + c * 16) = zero;
        *(bf16x8_t*)(k_lds + r * RS + c * 16) = zero;
      }
    }
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      if (hh > 0) __syncthreads();  // every wave is done reading the previous head's tiles
#pragma unroll
      for (int it = 0; it < NI; ++it) {
        const int i = tid + it * NT, r = i / HC, jc = i - r * HC;
        if (i < BKV * HC) {
          bf16x8_t qa, qb, ka, kb;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float co = e < 4 ? c0[it][e] : c1[it][e - 4];
            const float si = e < 4 ? s0[it][e] : s1[it][e - 4];
            const float xa = bf2f(q1[it][e]), xb = bf2f(q2[it][e]);
            qa[e] = f2bf(rot_first(xa, xb, co, si));
            qb[e] = f2bf(rot_second(xa, xb, co, si));
            const float ya = bf2f(k1[it][e]), yb = bf2f(k2[it][e]);
            ka[e] = f2bf(rot_first(ya, yb, co, si));
            kb[e] = f2bf(rot_second(ya, yb, co, si));
          }
          *(bf16x8_t*)(q_lds + r * RS + jc * 16) = qa;
          *(bf16x8_t*)(q_lds + r * RS + (jc + HC) * 16) = qb;
          *(bf16x8_t*)(k_lds + r * RS + jc * 16) = ka;
          *(bf16x8_t*)(k_lds + r * RS + (jc + HC) * 16) = kb;
        }
      }
#pragma unroll
      for (int it = 0; it < NV; ++it) {
        const int i = tid + it * NT, r = i / DC, c = i - r * DC;
        if (i < BKV * DC) *(bf16x8_t*)(v_lds + r * V_RS + c * 16) = vx[it];
      }
      __syncthreads();
      if (hh + 1 < HPW) issue_qkv(hoff + D);  // the staging registers are free again
      reset_state();
      if (wave_active) {
        load_q_frags();
        compute_tile(seg_len, std::true_type{});
      }
      write_out();
      hoff += D;
    }
  } else {
    for (int hh = 0; hh < HPW; ++hh) {
      if (hh > 0) __syncthreads();
      reset_state();
      stage_rows(a.q, q_lds, q0, BQ, nq);
      __syncthreads();
      load_q_frags();
      for (int kv0 = 0; kv0 < seg_len; kv0 += BKV) {
        const int nvalid = min(BKV, seg_len - kv0);
        __syncthreads();  // previous tile fully consumed
        stage_rows(a.k, k_lds, seg_start + kv0, BKV, nvalid);
        stage_v(seg_start + kv0, nvalid);
        __syncthreads();
        if (!wave_active) continue;
        compute_tile(nvalid, std::false_type{});
      }
      write_out();
      hoff += D;
    }
  }
}

// Full-attention variant (segments longer than 64 rows): 4 waves x 32 query rows, K/V tiles double-buffered.
// The global loads of tile t+1 are issued before the matrix-core work on tile t and land in registers;
// rotary (K) and the transpose (V) are applied when those registers are written to the other LDS buffer
// after the compute, so one barrier per tile is enough and memory latency hides behind the MFMAs.  The Q
// tile shares its LDS region with the second K/V buffer: Q is only needed until its fragments are in
// registers.
template <int D, bool ROPE>
__global__ __launch_bounds__(256, 2) void attn_full_kernel(const AttnArgs a) {
  constexpr int NT = 256, BQ = 128;
  constexpr int KS = (D + 15) / 16, DT = (D + 31) / 32, DC = D / 8, DKC = KS * 2;
  constexpr int RS = (DKC | 1) * 16;
  constexpr int HC = DC / 2;
  static_assert(D % 8 == 0 && D <= 96, "head dim");
  static_assert(!ROPE || D % 16 == 0, "rotary needs an even number of chunks per half");
  // When the head dim does not fill its last 32-row block of O^T, one of the spare V columns is set to 1:
  // row D of O^T is then sum_k P[k], the softmax denominator, accumulated (and rescaled) by the matrix cores
  // together with O instead of 32 vector additions and a shuffle per tile.
  constexpr bool L_FROM_MFMA = (D % 32) != 0;
  constexpr int K_BYTES = BKV * RS, V_BYTES = BKV * V_RS, Q_BYTES = BQ * RS;
  constexpr int REGION_B = (K_BYTES + V_BYTES) > Q_BYTES ? (K_BYTES + V_BYTES) : Q_BYTES;
  __shared__ __attribute__((aligned(16))) char lds[K_BYTES + V_BYTES + REGION_B];
  auto k_buf = [&](int b) -> char* { return lds + b * (K_BYTES + V_BYTES); };
  auto v_buf = [&](int b) -> char* { return lds + b * (K_BYTES + V_BYTES) + K_BYTES; };
  char* const q_lds = lds + K_BYTES + V_BYTES;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int fr = lane & 31, hf = lane >> 5;
  // Workgroup mapping.  Workgroup i runs on XCD i % 8, each with its own L2.  Query blocks of one segment
  // and head read the same K/V, so they should meet in one L2: the (work item, head) space is cut into
  // chunks of `chunk` consecutive work items of one head (a segment's query blocks are consecutive work
  // items), chunk c goes to XCD c % 8, and an XCD walks its chunks in order.
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int cid = (j / a.chunk) * 8 + xcd;           // chunk id in [0, n_chunks_x * heads)
  const int item = (cid % a.n_chunks_x) * a.chunk + j % a.chunk;
  const int head = cid / a.n_chunks_x;
  if (item >= a.n_work || head >= a.heads) return;   // padding of the last chunks (uniform per workgroup)
  const int seg_start = a.work[item * 4 + 0];
  const int seg_end = a.work[item * 4 + 1];
  const int q0 = a.work[item * 4 + 2];
  const int nq = a.work[item * 4 + 3];
  const int64_t hoff = (int64_t)head * D;
  const int seg_len = seg_end - seg_start;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const f32x4_t zero4 = {0, 0, 0, 0};

  // ---- register staging of one K/V tile
  constexpr int K_ITEMS = ROPE ? BKV * HC : BKV * DC;
  constexpr int K_PER = (K_ITEMS + NT - 1) / NT;
  constexpr int V_ITEMS = BKV * DC;
  constexpr int V_PER = (V_ITEMS + NT - 1) / NT;
  bf16x8_t kx1[K_PER], kx2[ROPE ? K_PER : 1];
  f32x4_t kc0[ROPE ? K_PER : 1], kc1[ROPE ? K_PER : 1], ks0[ROPE ? K_PER : 1], ks1[ROPE ? K_PER : 1];
  bf16x8_t vx[V_PER];

  // Unconditional loads from clamped rows and items (no branch between them, so they are all in flight
  // together).  Rows past the segment end then hold copies of the last valid row: as keys they are masked
  // (P = 0, and 0 times a finite V row is 0).
  auto gload_tile = [&](int kv0, int nvalid) {
#pragma unroll
    for (int u = 0; u < K_PER; ++u) {
      const int i = min(tid + u * NT, K_ITEMS - 1);
      constexpr int PER_ROW = ROPE ? HC : DC;
      const int r = i / PER_ROW, jc = i - r * PER_ROW;
      const int64_t g = seg_start + kv0 + min(r, nvalid - 1);
      const bf16_t* p = a.k + g * a.ld + hoff + jc * 8;
      kx1[u] = *(const bf16x8_t*)p;
      if (ROPE) {
        kx2[u] = *(const bf16x8_t*)(p + D / 2);
        const float* cs = a.cos_sin + g * D + jc * 8;
        kc0[u] = *(const f32x4_t*)cs;
        kc1[u] = *(const f32x4_t*)(cs + 4);
        ks0[u] = *(const f32x4_t*)(cs + D / 2);
        ks1[u] = *(const f32x4_t*)(cs + D / 2 + 4);
      }
    }
#pragma unroll
    for (int u = 0; u < V_PER; ++u) {
      const int i = min(tid + u * NT, V_ITEMS - 1);
      const int r = i / DC, c = i - r * DC;   // consecutive lanes: consecutive chunks of one key row
      vx[u] = *(const bf16x8_t*)(a.v + (int64_t)(seg_start + kv0 + min(r, nvalid - 1)) * a.ld + hoff + c * 8);
    }
  };
  auto lstore_tile = [&](int b) {
    char* kd = k_buf(b);
    char* vd = v_buf(b);
#pragma unroll
    for (int u = 0; u < K_PER; ++u) {
      const int i = tid + u * NT;
      if (i < K_ITEMS) {
        constexpr int PER_ROW = ROPE ? HC : DC;
        const int r = i / PER_ROW, jc = i - r * PER_ROW;
        if (ROPE) {
          bf16x8_t o1, o2;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float co = e < 4 ? kc0[u][e] : kc1[u][e - 4];
            const float si = e < 4 ? ks0[u][e] : ks1[u][e - 4];
            const float xa = bf2f(kx1[u][e]), xb = bf2f(kx2[u][e]);
            o1[e] = f2bf(rot_first(xa, xb, co, si));
            o2[e] = f2bf(rot_second(xa, xb, co, si));
          }
          *(bf16x8_t*)(kd + r * RS + jc * 16) = o1;
          *(bf16x8_t*)(kd + r * RS + (jc + HC) * 16) = o2;
        } else {
          *(bf16x8_t*)(kd + r * RS + jc * 16) = kx1[u];
        }
      }
    }
    if (!ROPE && DKC > DC) {  // zero the pad chunks of the K rows (head dims that are not multiples of 16)
      for (int i = tid; i < BKV * (DKC - DC); i += NT) {
        const int r = i / (DKC - DC), c = DC + i % (DKC - DC);
        *(bf16x8_t*)(kd + r * RS + c * 16) = zero8;
      }
    }
#pragma unroll
    for (int u = 0; u < V_PER; ++u) {
      const int i = tid + u * NT;
      if (i < V_ITEMS) {
        const int r = i / DC, c = i - r * DC;
        *(bf16x8_t*)(vd + r * V_RS + c * 16) = vx[u];
      }
    }
  };

  // chunk DC (dims D .. D+7) of every key row of V buffer b := (1, 0, ..., 0); lstore_tile never writes there
  auto store_ones_column = [&](int b) {
    if constexpr (L_FROM_MFMA) {
      bf16x8_t one = zero8;
      one[0] = f2bf(1.0f);
      for (int r = tid; r < BKV; r += NT) *(bf16x8_t*)(v_buf(b) + r * V_RS + DC * 16) = one;
    }
  };

  // ---- prologue: Q -> LDS (rotated), tile 0 -> LDS buffer 0
  gload_tile(0, min(BKV, seg_len));
  {
    if (ROPE) {
      for (int i = tid; i < BQ * HC; i += NT) {
        const int r = i / HC, jc = i - r * HC;
        bf16x8_t o1 = zero8, o2 = zero8;
        if (r < nq) {
          const int64_t g = q0 + r;
          const bf16_t* p = a.q + g * a.ld + hoff + jc * 8;
          const bf16x8_t x1 = *(const bf16x8_t*)p;
          const bf16x8_t x2 = *(const bf16x8_t*)(p + D / 2);
          const float* cs = a.cos_sin + g * D + jc * 8;
          const f32x4_t c0 = *(const f32x4_t*)cs, c1 = *(const f32x4_t*)(cs + 4);
          const f32x4_t s0 = *(const f32x4_t*)(cs + D / 2), s1 = *(const f32x4_t*)(cs + D / 2 + 4);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float co = e < 4 ? c0[e] : c1[e - 4];
            const float si = e < 4 ? s0[e] : s1[e - 4];
            const float xa = bf2f(x1[e]), xb = bf2f(x2[e]);
            o1[e] = f2bf(rot_first(xa, xb, co, si));
            o2[e] = f2bf(rot_second(xa, xb, co, si));
          }
        }
        *(bf16x8_t*)(q_lds + r * RS + jc * 16) = o1;
        *(bf16x8_t*)(q_lds + r * RS + (jc + HC) * 16) = o2;
      }
    } else {
      for (int i = tid; i < BQ * DKC; i += NT) {
        const int r = i / DKC, c = i - r * DKC;
        bf16x8_t x = zero8;
        if (r < nq && c < DC) x = *(const bf16x8_t*)(a.q + (int64_t)(q0 + r) * a.ld + hoff + c * 8);
        *(bf16x8_t*)(q_lds + r * RS + c * 16) = x;
      }
    }
  }
  lstore_tile(0);
  store_ones_column(0);
  __syncthreads();
  bf16x8_t qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const bf16x8_t*)(q_lds + (wave * 32 + fr) * RS + (2 * ks + hf) * 16);
  __syncthreads();  // every wave holds its Q fragments: the Q region may now become K/V buffer 1
  store_ones_column(1);  // (ordered before the first read of buffer 1 by the barrier that ends iteration 0)

  f32x16_t oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[t][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const bool wave_active = wave * 32 < nq;
  const float sl2 = a.scale_log2e;

  int buf = 0;
  for (int kv0 = 0; kv0 < seg_len; kv0 += BKV, buf ^= 1) {
    const int nvalid = min(BKV, seg_len - kv0);
    const bool more = kv0 + BKV < seg_len;
    if (more) gload_tile(kv0 + BKV, min(BKV, seg_len - kv0 - BKV));
    if (wave_active) {
      const char* kd = k_buf(buf);
      const char* vd = v_buf(buf);
      f32x16_t sacc[2];
      bf16x8_t pf[2][2];
      score_tile<KS, RS>(sacc, kd, qf, nvalid, fr, hf);
      softmax_tile<DT, L_FROM_MFMA>(sacc, pf, oacc, m_run, l_run, sl2);
#pragma unroll
      for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) {
            const bf16x8_t vf = read_vt_frag(vd, t, kt * 2 + kk, lane);
            oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[kt][kk], oacc[t], 0, 0, 0);
          }
      }
    }
    if (more) lstore_tile(buf ^ 1);
    __syncthreads();
  }

  const int qi = wave * 32 + fr;
  write_output<D, DT, L_FROM_MFMA>(oacc, l_run, a.out + (int64_t)(q0 + min(qi, nq - 1)) * a.ldo + hoff, qi < nq, hf);
}

// Full attention without rotary (SigLIP): K and V tiles go global -> LDS directly (buffer_load ... lds: no
// staging registers, no LDS store instructions, no address arithmetic per tile) into a ring of NB tile buffers:
// three buffers requested two tiles ahead with two workgroups per CU, or two buffers requested one tile ahead with
// three workgroups per CU (what launch_attn selects).  A direct load fixes the LDS side -- the 64 lanes of a wave fill 1 KB of
// consecutive LDS -- so the padded row layout is produced on the global side: a tile is the flat sequence of
// 16-byte chunk slots (row, slot), lane l of load j owns slot j*64 + l and fetches chunk `slot % slots_per_row`
// of row `slot / slots_per_row`; lanes that own padding slots are switched off for the load, which leaves the
// padding as initialised once per buffer (zeros behind the K rows that the last k-step reads, the ones
// column of V that yields the softmax denominator).
typedef __attribute__((address_space(3))) void lds_void_t;

// Transposing LDS reads of the four V^T fragments (keys 16g .. 16g+15, g = 0..3) of dims 32*TT .. 32*TT+31, written in
// assembly (see the kernel for why); the caller waits for them with an explicit s_waitcnt.
template <int TT, int G>
CS_DEVICE void read_vt_pair_asm(i32x2_t& lo, i32x2_t& hi, uint32_t vbase) {
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(vbase), "n"(G * 16 * V_RS + TT * 64));
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(vbase), "n"(G * 16 * V_RS + TT * 64 + 8 * V_RS));
}
template <int TT>
CS_DEVICE void read_vt_block_asm(i32x2_t (&raw)[8], uint32_t vbase) {
  read_vt_pair_asm<TT, 0>(raw[0], raw[1], vbase);
  read_vt_pair_asm<TT, 1>(raw[2], raw[3], vbase);
  read_vt_pair_asm<TT, 2>(raw[4], raw[5], vbase);
  read_vt_pair_asm<TT, 3>(raw[6], raw[7], vbase);
}
template <bool LAST>
CS_DEVICE void pv_block(f32x16_t& o, i32x2_t (&raw)[8], const bf16x8_t (&pf)[2][2]) {
  if constexpr (LAST) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  else asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    i32x4_t both = {raw[2 * g][0], raw[2 * g][1], raw[2 * g + 1][0], raw[2 * g + 1][1]};
    asm volatile("" : "+v"(both));  // the registers hold the data only after the wait above
    o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, both), pf[g >> 1][g & 1], o, 0, 0, 0);
  }
}

template <int D, int NB = 3>
struct AttnDirectShape {
  static constexpr int KS = (D + 15) / 16, DKC = KS * 2, DC = D / 8;
  static constexpr int K_SLOTS = DKC | 1, V_SLOTS = V_RS / 16;      // 16-byte slots per tile row
  static constexpr int RS = K_SLOTS * 16;
  static constexpr int K_BYTES = BKV * RS, V_BYTES = BKV * V_RS, TILE_BYTES = K_BYTES + V_BYTES;
  static constexpr int K_LOADS = BKV * K_SLOTS / 64, V_LOADS = BKV * V_SLOTS / 64;   // BKV == 64: one load per slot column
  static constexpr int LOADS = K_LOADS + V_LOADS, PER_WAVE = (LOADS + 3) / 4;
  static constexpr int NBUF = NB, LDS = NBUF * TILE_BYTES;
  static constexpr int WGS_PER_CU = NB == 2 ? 3 : 2;
  static_assert(128 * RS <= (NBUF - 1) * TILE_BYTES, "the Q tile aliases the buffers behind the first");
  static_assert(WGS_PER_CU * LDS <= 160 * 1024, "workgroups per CU");
};

// ROPE_Q: the keys were rotated in place beforehand; the query rows are rotated here while they are staged (a
// query block is staged once, whereas every query block of a segment would rotate the segment's keys again).
template <int D, bool ROPE_Q = false, int NB = 3>
__global__ __launch_bounds__(256, (NB == 2 ? 3 : 2)) void attn_full_direct_kernel(const AttnArgs a) {
  constexpr int NT = 256, BQ = 128;
  static_assert(!ROPE_Q || D % 16 == 0, "rotary needs an even number of 16-byte chunks per half");
  using Shape = AttnDirectShape<D, NB>;
  constexpr int KS = Shape::KS, DT = (D + 31) / 32, DC = Shape::DC, DKC = Shape::DKC;
  constexpr int RS = Shape::RS, K_SLOTS = Shape::K_SLOTS, V_SLOTS = Shape::V_SLOTS;
  constexpr int K_BYTES = Shape::K_BYTES, TILE_BYTES = Shape::TILE_BYTES;
  constexpr int K_LOADS = Shape::K_LOADS, LOADS = Shape::LOADS, PER = Shape::PER_WAVE;
  static_assert(D % 8 == 0 && D <= 96 && BKV == 64, "head dim / tile");
  constexpr bool L_FROM_MFMA = (D % 32) != 0;   // see attn_full_kernel
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  auto k_buf = [&](int b) -> char* { return lds + b * TILE_BYTES; };
  auto v_buf = [&](int b) -> char* { return lds + b * TILE_BYTES + K_BYTES; };
  char* const q_lds = lds + TILE_BYTES;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int fr = lane & 31, hf = lane >> 5;
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;   // workgroup mapping: see attn_full_kernel
  const int cid = (j / a.chunk) * 8 + xcd;
  const int item = (cid % a.n_chunks_x) * a.chunk + j % a.chunk;
  const int head = cid / a.n_chunks_x;
  if (item >= a.n_work || head >= a.heads) return;
  const int seg_start = a.work[item * 4 + 0];
  const int seg_end = a.work[item * 4 + 1];
  const int q0 = a.work[item * 4 + 2];
  const int nq = a.work[item * 4 + 3];
  const int64_t hoff = (int64_t)head * D;
  const int seg_len = seg_end - seg_start;
  const int n_tiles = (seg_len + BKV - 1) / BKV;
  const bf16x8_t zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // ---- the wave's direct loads of a tile.  Load u of this wave is load number jl = min(4u + wave, LOADS-1) of the
  //      tile (the clamp makes a wave without a load of its own repeat the last one: every wave must issue the
  //      same number, because the waits count loads).  Byte offsets are relative to the segment's first row.
  const __amdgpu_buffer_rsrc_t rsrc_k =
      __builtin_amdgcn_make_buffer_rsrc((void*)(a.k + (int64_t)seg_start * a.ld + hoff), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_v =
      __builtin_amdgcn_make_buffer_rsrc((void*)(a.v + (int64_t)seg_start * a.ld + hoff), 0, -1, 0x00020000);
  const uint32_t row_bytes = (uint32_t)a.ld * 2u;
  int l_row[PER], l_chunk[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int jl = min(4 * u + wave, LOADS - 1);
    const bool is_k = jl < K_LOADS;
    const int slot = (is_k ? jl : jl - K_LOADS) * 64 + lane;
    const int per_row = is_k ? K_SLOTS : V_SLOTS;
    l_row[u] = slot / per_row;
    l_chunk[u] = slot - l_row[u] * per_row;   // >= DC: a padding slot, the lane sits the load out
  }
  auto issue_k = [&](char* dst, uint32_t off, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_k, (lds_void_t*)dst, 16, off, soff, 0, 0);
  };
  auto issue_v = [&](char* dst, uint32_t off, uint32_t soff) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_v, (lds_void_t*)dst, 16, off, soff, 0, 0);
  };
  auto issue_tile = [&](int t, int b) {
    const int nvalid = min(BKV, seg_len - t * BKV);
    const uint32_t soff = (uint32_t)(t * BKV) * row_bytes;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int jl = min(4 * u + wave, LOADS - 1);
      // rows past the segment end repeat the last valid row: as keys they are masked, and P = 0 times a finite V row is 0
      const uint32_t off = (uint32_t)min(l_row[u], nvalid - 1) * row_bytes + (uint32_t)l_chunk[u] * 16u;
      if (jl < K_LOADS) {   // uniform
        char* dst = k_buf(b) + jl * 1024;
        if (l_chunk[u] < DC) issue_k(dst, off, soff);
      } else {
        char* dst = v_buf(b) + (jl - K_LOADS) * 1024;
        if (l_chunk[u] < DC) issue_v(dst, off, soff);
      }
    }
  };
  auto init_padding = [&](int b) {
    if constexpr (DKC > DC) {
      for (int i = tid; i < BKV * (DKC - DC); i += NT) {
        const int r = i / (DKC - DC), c = DC + i % (DKC - DC);
        *(bf16x8_t*)(k_buf(b) + r * RS + c * 16) = zero8;
      }
    }
    if constexpr (L_FROM_MFMA) {
      bf16x8_t one = zero8;
      one[0] = f2bf(1.0f);
      for (int r = tid; r < BKV; r += NT) *(bf16x8_t*)(v_buf(b) + r * V_RS + DC * 16) = one;
    }
  };
  auto wait_loads = [&](auto pending_c) {   // at most `pending` of this wave's direct loads still in flight
    constexpr int N = decltype(pending_c)::value;
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
  };
  auto barrier = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  // ---- prologue: tile 0 requested, Q -> LDS -> fragments, then the Q region becomes buffers 1 and 2
  issue_tile(0, 0);
  init_padding(0);
  if constexpr (ROPE_Q) {
    constexpr int HC = DC / 2;   // chunks per half; D % 16 == 0, so there are no padding chunks (DKC == DC)
    for (int i = tid; i < BQ * HC; i += NT) {
      const int r = i / HC, jc = i - r * HC;
      bf16x8_t o1 = zero8, o2 = zero8;
      if (r < nq) {
        const int64_t g = q0 + r;
        const bf16_t* p = a.q + g * a.ld + hoff + jc * 8;
        const bf16x8_t x1 = *(const bf16x8_t*)p;
        const bf16x8_t x2 = *(const bf16x8_t*)(p + D / 2);
        const float* cs = a.cos_sin + g * D + jc * 8;
        const f32x4_t c0 = *(const f32x4_t*)cs, c1 = *(const f32x4_t*)(cs + 4);
        const f32x4_t s0 = *(const f32x4_t*)(cs + D / 2), s1 = *(const f32x4_t*)(cs + D / 2 + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float co = e < 4 ? c0[e] : c1[e - 4];
          const float si = e < 4 ? s0[e] : s1[e - 4];
          const float xa = bf2f(x1[e]), xb = bf2f(x2[e]);
          o1[e] = f2bf(rot_first(xa, xb, co, si));
          o2[e] = f2bf(rot_second(xa, xb, co, si));
        }
      }
      *(bf16x8_t*)(q_lds + r * RS + jc * 16) = o1;
      *(bf16x8_t*)(q_lds + r * RS + (jc + HC) * 16) = o2;
    }
  } else {
    for (int i = tid; i < BQ * DKC; i += NT) {
      const int r = i / DKC, c = i - r * DKC;
      bf16x8_t x = zero8;
      if (r < nq && c < DC) x = *(const bf16x8_t*)(a.q + (int64_t)(q0 + r) * a.ld + hoff + c * 8);
      *(bf16x8_t*)(q_lds + r * RS + c * 16) = x;
    }
  }
  __syncthreads();
  bf16x8_t qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const bf16x8_t*)(q_lds + (wave * 32 + fr) * RS + (2 * ks + hf) * 16);
  __syncthreads();
  init_padding(1);
  if constexpr (NB == 3) {
    init_padding(2);
    if (n_tiles > 1) issue_tile(1, 1);
  }

  f32x16_t oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[t][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const bool wave_active = wave * 32 < nq;
  const float sl2 = a.scale_log2e;

  int buf = 0, buf2 = 2;   // buffers of tile t and of tile t+2
  for (int t = 0; t < n_tiles; ++t) {
    // Tile t has landed when only the loads requested after it (tile t+1's) are in flight; the barrier then also
    // says that every wave is done with tile t-1, whose buffer the request for tile t+2 reuses.
    if constexpr (NB == 3) {
      if (t + 1 < n_tiles) wait_loads(std::integral_constant<int, PER>{});
      else wait_loads(std::integral_constant<int, 0>{});
      barrier();
      if (t + 2 < n_tiles) issue_tile(t + 2, buf2);
    } else {   // two buffers: tile t+1 travels while tile t is worked on (three workgroups per CU hide the rest)
      wait_loads(std::integral_constant<int, 0>{});
      barrier();
      if (t + 1 < n_tiles) issue_tile(t + 1, buf ^ 1);
    }
    const int nvalid = min(BKV, seg_len - t * BKV);
    if (wave_active) {
      const char* kd = k_buf(buf);
      const char* vd = v_buf(buf);
      f32x16_t sacc[2];
      bf16x8_t pf[2][2];
      score_tile<KS, RS>(sacc, kd, qf, nvalid, fr, hf);
      softmax_tile<DT, L_FROM_MFMA>(sacc, pf, oacc, m_run, l_run, sl2);
      // V^T fragments (see read_vt_frag for the addressing).  The transposing reads are written in assembly: as
      // an intrinsic, the compiler takes them for possible readers of the LDS bytes that the direct loads in
      // flight will write and puts a wait for ALL outstanding loads in front of them -- the tiles requested
      // ahead included.  The waits on the reads themselves are therefore explicit too: the reads of block
      // tt+1 are issued before the MFMAs of block tt, which wait until only those 8 are outstanding.
      {
        const int sg = lane & 15;
        const uint32_t vbase = (uint32_t)(uintptr_t)(lds_void_t*)vd + (uint32_t)((4 * hf + (sg >> 2)) * V_RS + (16 * ((lane >> 4) & 1) + 4 * (sg & 3)) * 2);
        i32x2_t vraw[2][8];   // [block parity][2 * fragment + half]
        read_vt_block_asm<0>(vraw[0], vbase);
        read_vt_block_asm<1>(vraw[1], vbase);
        pv_block<false>(oacc[0], vraw[0], pf);
        if constexpr (DT == 2) {
          pv_block<true>(oacc[1], vraw[1], pf);
        } else {
          static_assert(DT == 3, "head dims up to 96");
          read_vt_block_asm<2>(vraw[0], vbase);
          pv_block<false>(oacc[1], vraw[1], pf);
          pv_block<true>(oacc[DT - 1], vraw[0], pf);
        }
      }
    }
    if constexpr (NB == 3) {
      buf2 = buf;   // tile t+3 will reuse this iteration's buffer
      buf = buf == 2 ? 0 : buf + 1;
    } else {
      buf ^= 1;
    }
  }

  const int qi = wave * 32 + fr;
  write_output<D, DT, L_FROM_MFMA>(oacc, l_run, a.out + (int64_t)(q0 + min(qi, nq - 1)) * a.ldo + hoff, qi < nq, hf);
}


template <int D, bool ROPE_Q = false, int NB = 3>
int launch_attn_full_direct(const AttnArgs& a, dim3 grid, hipStream_t stream) {
  constexpr int lds = AttnDirectShape<D, NB>::LDS;
  static bool attr_set = false;
  auto kern = attn_full_direct_kernel<D, ROPE_Q, NB>;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return CS_ERR_LAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, a);
  return cs_launch_status();
}

template <int D>
int launch_attn(AttnArgs a, int n_work, int heads, int block_q, int max_seqlen, bool rope, bool keys_rotated,
                hipStream_t stream) {
  const dim3 grid(n_work, heads);
  a.n_work = n_work;
  a.heads = heads;
  a.chunk = min(32, max(1, (max_seqlen + 127) / 128));  // query blocks of the longest segment
  a.n_chunks_x = (n_work + a.chunk - 1) / a.chunk;
  const int n_chunks = a.n_chunks_x * heads;
  const dim3 grid_full(((n_chunks + 7) / 8) * 8 * a.chunk);
  // The direct-to-LDS kernel with two tile buffers and three workgroups per CU where its LDS allows (head dims up to
  // 80): the softmax keeps the vector unit as busy as the matrix cores, so a third wave per SIMD buys more overlap
  // than a third buffer of prefetch (measured: 4096 keys at d = 72 513 -> 444 us, 1024 keys at d = 80 87 -> 80 us).
  constexpr int RING_DEPTH = D <= 80 ? 2 : 3;
  if (keys_rotated) {
    // only the long-segment kernel has this form (short segments rotate q and k while staging, one workgroup each)
    if constexpr (D % 16 == 0) {
      if (block_q != 64 && rope && (int64_t)max_seqlen * a.ld * 2 < (int64_t)1 << 31)
        return launch_attn_full_direct<D, true, RING_DEPTH>(a, grid_full, stream);
    }
    return CS_ERR_UNSUPPORTED;
  }
  if (block_q == 64) {
    if (rope) {
      // two heads per workgroup when that still leaves several workgroups per CU
      const bool pair = heads % 2 == 0 && (int64_t)n_work * heads >= 2048;
      if constexpr (D % 16 == 0) {
        if (pair) hipLaunchKernelGGL((attn_kernel<D, 2, true, 2>), dim3(n_work, heads / 2), dim3(128), 0, stream, a);
        else hipLaunchKernelGGL((attn_kernel<D, 2, true, 1>), grid, dim3(128), 0, stream, a);
      } else {
        return CS_ERR_UNSUPPORTED;
      }
    } else {
      hipLaunchKernelGGL((attn_kernel<D, 2, false, 1>), grid, dim3(128), 0, stream, a);
    }
  } else {
    if (rope) {
      if constexpr (D % 16 == 0) hipLaunchKernelGGL((attn_full_kernel<D, true>), grid_full, dim3(256), 0, stream, a);
      else return CS_ERR_UNSUPPORTED;
    } else {
      // the direct-to-LDS kernel addresses a segment's K/V rows with 32-bit byte offsets
      if ((int64_t)max_seqlen * a.ld * 2 < (int64_t)1 << 31)
        return launch_attn_full_direct<D, false, RING_DEPTH>(a, grid_full, stream);
      hipLaunchKernelGGL((attn_full_kernel<D, false>), grid_full, dim3(256), 0, stream, a);
    }
  }
  return cs_launch_status();
}

}  // namespace

// Query rows per workgroup: 64 (2 waves) when no segment is longer than 64 rows (window attention),
// else 128 (4 waves).
extern "C" int cs_attn_block_q(int32_t max_seqlen) { return max_seqlen <= 64 ? 64 : 128; }

extern "C" int cs_attn_work_host(const int32_t* cu_seqlens_host, int32_t n_seg, int32_t block_q,
                                 int32_t* work_host, int32_t cap_items, int32_t* n_work) {
  if (!cu_seqlens_host || n_seg < 0 || block_q <= 0 || !work_host || !n_work) return CS_ERR_INVALID_ARG;
  int n = 0;
  for (int s = 0; s < n_seg; ++s) {
    const int b = cu_seqlens_host[s], e = cu_seqlens_host[s + 1];
    if (e < b) return CS_ERR_INVALID_ARG;
    for (int q = b; q < e; q += block_q) {
      if (n >= cap_items) return CS_ERR_TOO_LARGE;
      work_host[4 * n + 0] = b;
      work_host[4 * n + 1] = e;
      work_host[4 * n + 2] = q;
      work_host[4 * n + 3] = e - q < block_q ? e - q : block_q;
      ++n;
    }
  }
  *n_work = n;
  return CS_OK;
}

static int attn_varlen_entry(const void* q, const void* k, const void* v, int64_t ld, void* out, int64_t ldo,
                             const int32_t* work, int32_t n_work, int32_t heads, int32_t head_dim, float scale,
                             const float* cos_sin, int32_t max_seqlen, bool keys_rotated, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (keys_rotated && !cos_sin) return CS_ERR_INVALID_ARG;
  if (!q || !k || !v || !out || !work || n_work < 0 || heads <= 0 || heads > 65535 || head_dim <= 0 ||
      max_seqlen <= 0)
    return CS_ERR_INVALID_ARG;
  if (ld % 8 || ldo % 4 || head_dim % 8) return CS_ERR_INVALID_ARG;
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)cos_sin) & 15) return CS_ERR_INVALID_ARG;
  if ((uintptr_t)out & 7) return CS_ERR_INVALID_ARG;
  if (n_work == 0) return CS_OK;
  AttnArgs a;
  a.q = (const bf16_t*)q;
  a.k = (const bf16_t*)k;
  a.v = (const bf16_t*)v;
  a.ld = ld;
  a.out = (bf16_t*)out;
  a.ldo = ldo;
  a.work = work;
  a.cos_sin = cos_sin;
  a.scale_log2e = scale * 1.4426950408889634f;
  const int bq = cs_attn_block_q(max_seqlen);
  const bool rope = cos_sin != nullptr;
  switch (head_dim) {
    case 64: return launch_attn<64>(a, n_work, heads, bq, max_seqlen, rope, keys_rotated, stream);
    case 72: return launch_attn<72>(a, n_work, heads, bq, max_seqlen, rope, keys_rotated, stream);
    case 80: return launch_attn<80>(a, n_work, heads, bq, max_seqlen, rope, keys_rotated, stream);
    case 96: return launch_attn<96>(a, n_work, heads, bq, max_seqlen, rope, keys_rotated, stream);
    default: return CS_ERR_UNSUPPORTED;
  }
}

extern "C" int cs_attn_varlen(const void* q, const void* k, const void* v, int64_t ld, void* out, int64_t ldo,
                              const int32_t* work, int32_t n_work, int32_t heads, int32_t head_dim, float scale,
                              const float* cos_sin, int32_t max_seqlen, void* stream) {
  return attn_varlen_entry(q, k, v, ld, out, ldo, work, n_work, heads, head_dim, scale, cos_sin, max_seqlen, false, stream);
}

extern "C" int cs_attn_varlen_keys_rotated(const void* q, const void* k, const void* v, int64_t ld, void* out,
                                           int64_t ldo, const int32_t* work, int32_t n_work, int32_t heads,
                                           int32_t head_dim, float scale, const float* cos_sin, int32_t max_seqlen,
                                           void* stream) {
  return attn_varlen_entry(q, k, v, ld, out, ldo, work, n_work, heads, head_dim, scale, cos_sin, max_seqlen, true, stream);
}
