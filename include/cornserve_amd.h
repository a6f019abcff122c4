/*
 * cornserve_amd.h -- C ABI of the MI355X (gfx950) kernels behind the Eric encoder forward pass.
 *
 * The reference (cornserve-ai/cornserve) is pure Python; its encoder forward
 * (python/cornserve/task_executors/eric/models/{qwen2_5_vl,gemma3}.py, layers/{siglip,norm,linear,
 * attention,activations}.py) reaches device code only through torch / flash-attn / xformers calls.
 * Each entry point below replaces one of those call sites and cites it.  A reference-side binding is a
 * ctypes (or torch.library) stub: load libcornserve_amd.so, pass tensor.data_ptr() values, sizes and
 * torch.cuda.current_stream().cuda_stream.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the parameter name ends in _host;
 *   - matrices are row-major with an explicit leading dimension in ELEMENTS;
 *   - bf16 is the storage type of activations and weights (uint16 bit pattern of the upper half of an
 *     IEEE fp32, round-to-nearest-even); fp8 weights are OCP e4m3 (e4m3fn) bytes;
 *   - `stream` is a hipStream_t passed as void*; kernels are enqueued on it and the call returns
 *     without synchronising;
 *   - no entry point allocates or frees memory, and none takes ownership of a buffer;
 *   - the return value is a status code (0 = ok); nothing aborts the process.  The host wrapper maps
 *     CS_ERR_INVALID_ARG to ValueError and the rest to RuntimeError (reference error behaviour:
 *     qwen2_5_vl.py:420-421, gemma3.py:112-123).
 */
#ifndef CORNSERVE_AMD_H
#define CORNSERVE_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CS_OK 0
#define CS_ERR_INVALID_ARG 1
#define CS_ERR_UNSUPPORTED 2
#define CS_ERR_LAUNCH 3
#define CS_ERR_TOO_LARGE 4

/* ABI version of this header; cs_abi_version() returns the value the library was built with. */
#define CS_ABI_VERSION 7
int cs_abi_version(void);

/* ------------------------------------------------------------------------------------------------
 * GEMM:  C[M,N] = epilogue(A[M,K] . W[N,K]^T)     (bf16 in, fp32 accumulate on MFMA, bf16 out)
 * Replaces F.linear at linear.py:183 (ColumnParallelLinear) and linear.py:549 (RowParallelLinear),
 * the Conv3d patch embed at qwen2_5_vl.py:195-201 (a GEMM on the flat [L,1176] input), the merger
 * MLP at qwen2_5_vl.py:225-233, the SigLIP projections at siglip.py:121-125,142-143,155-163 and the
 * Gemma-3 projection matmul at gemma3.py:48.
 * ---------------------------------------------------------------------------------------------- */
enum CsEpilogue {
  CS_EPI_BIAS = 0,      /* y = acc (+ bias)                                                     */
  CS_EPI_RESIDUAL = 1,  /* y = bf16(acc + bias) + residual[m,n]         qwen2_5_vl.py:175,177
                           (with c_lo: y = acc + bias + residual, kept to 16 significant bits)  */
  CS_EPI_SWIGLU = 2,    /* W rows interleaved gate_j,up_j; y[m,j] = silu(g)*u; C is N/2 wide
                           qwen2_5_vl.py:143-148                                               */
  CS_EPI_GELU_ERF = 3,  /* y = gelu(acc + bias), erf form               qwen2_5_vl.py:220       */
  CS_EPI_GELU_TANH = 4, /* y = gelu(acc + bias), tanh form              siglip.py:155-163       */
  CS_EPI_QUICK_GELU = 5 /* y = x * sigmoid(1.702 x), x = acc + bias     layers/activations.py:9-12
                           (Qwen2-VL MLP, qwen2_vl.py:112-128)                                   */
};

typedef struct CsGemmArgs {
  const void* A;         /* bf16 [M,K], leading dimension lda                                    */
  int64_t lda;
  const void* W;         /* bf16 [N,K] (w_fp8 = 0) or e4m3 bytes [N,K] (w_fp8 = 1), ld = ldw      */
  int64_t ldw;
  const float* w_scale;  /* fp32 [N] per-output-channel scale; required when w_fp8, else NULL     */
  const void* bias;      /* bf16 [N] or NULL                                                     */
  const void* residual;  /* bf16 [M,N] (CS_EPI_RESIDUAL), leading dimension ldr                   */
  int64_t ldr;
  const void* pos;       /* optional bf16 [pos_period, N] addend indexed by (m % pos_period):     */
  int64_t ldpos;         /*   SigLIP learned position embedding, siglip.py:100                    */
  int32_t pos_period;
  void* C;               /* bf16 [M,N] (or [M,N/2] for CS_EPI_SWIGLU), leading dimension ldc      */
  int64_t ldc;
  const int32_t* a_rows; /* optional [M]: A row used for output row m (gather, qwen2_5_vl.py:438-440) */
  const int32_t* c_rows; /* optional [M]: C row written for output row m (scatter, :478-479)      */
  int32_t M, N, K;
  int32_t epilogue;      /* enum CsEpilogue                                                      */
  int32_t w_fp8;
  int32_t tiles_m, tiles_n; /* filled in by the library                                          */
  int32_t fast_epilogue;    /* filled in by the library                                          */
  /* RMSNorm folded into the neighbouring GEMMs (qwen2_5_vl.py:173-177: norm1 -> qkv, norm2 -> gate|up).
   * rsqrt(mean(x^2) + eps) is a per-row scalar, so  bf16(x*rstd) * w_norm . W^T  ==  rstd * (x . (W*w_norm)^T)
   * up to the rounding of the normalised activations: the caller folds w_norm into W's columns, passes the
   * residual stream itself as A, and the row scalar is applied to the fp32 accumulators.
   * a_row_sumsq: optional fp32 [M][CS_SUMSQ_PARTS]; the parts of row m add up to sum_k A[m,k]^2.  The
   *   epilogue becomes  y = acc * rsqrt(sum/K + norm_eps) (+ bias) ...   (CS_EPI_BIAS and CS_EPI_SWIGLU, bf16 W).
   * c_row_sumsq: optional fp32 [M][CS_SUMSQ_PARTS], indexed by OUTPUT row; part p receives the sum of squares
   *   of the rounded outputs C[m, 160p .. 160p+159], for the parts N covers (the caller zeroes the others once).
   *   CS_EPI_BIAS and CS_EPI_RESIDUAL, bf16 W, N <= 160 * CS_SUMSQ_PARTS.
   * Unsupported combinations return CS_ERR_UNSUPPORTED (nothing is launched).                      */
  const float* a_row_sumsq;
  float* c_row_sumsq;
  float norm_eps;
  /* LayerNorm folded the same way (nn.LayerNorm in front of qkv / fc1: siglip.py:333-345, qwen2_vl.py:277-291,
   * qwen3_vl.py:139-153).  With mean = sum/K, var = sumsq/K - mean^2, rstd = rsqrt(var + norm_eps):
   *   LN(x) . W^T + b  ==  rstd * (x . W'^T - mean * w_col_sum) + b'   with W' = W * w_ln (columns), b' = b + W . b_ln,
   *   w_col_sum[n] = sum_k W'[n,k]; the caller passes W', b' and w_col_sum.
   * a_row_sum:  optional fp32 [M][CS_SUMSQ_PARTS], parts of sum_k A[m,k]; needs a_row_sumsq and w_col_sum (fp32 [N]).
   *   CS_EPI_BIAS, CS_EPI_GELU_TANH, CS_EPI_QUICK_GELU, bf16 W.
   * c_row_sum:  optional, the sums of the rounded output rows in the layout of c_row_sumsq (which it needs);
   *   CS_EPI_RESIDUAL, bf16 W, N <= 160 * CS_SUMSQ_PARTS.                                           */
  const float* a_row_sum;
  float* c_row_sum;
  const float* w_col_sum;
  /* Residual stream with 16 significant bits (CS_EPI_RESIDUAL only).  The residual additions at qwen2_5_vl.py:175,177
   * (siglip.py:178,188) are the one place where a bf16 encoder accumulates rounding error with depth: 64 roundings of
   * the stream to 8 bits.  With these planes the stream is carried as a bf16 "hi" tensor (C / residual, which is what
   * every other kernel reads) plus a byte "lo" tensor with the next 8 mantissa bits as a signed correction:
   *   value = fp32 from bits  (hi << 16) + ((int8)lo << 8)
   * residual_lo: optional uint8 [M,N], leading dimension ldr; the addend is the joined value instead of bf16 residual.
   * c_lo:        optional uint8 [M,N], leading dimension ldc (rows scattered like C's); the sum acc + bias + addend is
   *              not rounded to bf16 on the way (neither is acc + bias) but split: 24 bits to nearest, the upper 16 of
   *              them rounded half-up to C, the rest to c_lo.  A zero-filled plane next to a bf16 tensor is a valid
   *              pair, so the stream can start from any bf16 tensor.  May alias residual_lo when C aliases residual. */
  const uint8_t* residual_lo;
  uint8_t* c_lo;
  /* Convolution with stride = kernel as a strided-gather GEMM (Conv2d patch embedding, siglip.py:30-36,94-95).  With
   * conv_patch > 0, A is not a matrix but NCHW pixels, bf16 [B, conv_c, conv_h, conv_w] (lda is ignored): output row m
   * is patch (b, py, px) in row-major patch order, M = B * (conv_h / patch) * (conv_w / patch), and element k =
   * (c, ky, kx) of its row is pixel [b, c, py*patch + ky, px*patch + kx]; k >= conv_c * patch^2 reads as zero, so K may
   * be that product rounded up to the multiple of 8 the kernel needs (W then carries zero columns).  patch and conv_w
   * must be even (pixel pairs are fetched as 4-byte words); pixels past the last whole patch are not read, as the
   * convolution drops them.  CS_EPI_BIAS (with or without the position addend), bf16 W, no a_rows.                  */
  int32_t conv_c, conv_h, conv_w, conv_patch;
  /* filled in by cs_qkv_window_attn (the rotary table and softmax scale of its fused epilogue)                      */
  const float* attn_cos_sin;
  float attn_scale_log2e;
  /* cs_qkv_window_attn only, set by the caller: windows of fewer than 64 rows (see there); NULL / 0 otherwise         */
  const int32_t* attn_win_start;
  int32_t attn_n_win;
  /* Optional hint for launches that leave compute units idle (at most 192 workgroups of the fast path's tile forms and
   * of cs_qkv_window_attn): prefetch_bytes bytes at prefetch (16-byte aligned) -- typically the weights of the NEXT
   * launch, which no kernel has touched since the previous forward pass -- are read once by up to 128 workgroups
   * started next to the computing ones, so that they sit in the last-level cache when the next launch asks for them
   * (a few-row launch is bound by operand latency, not by arithmetic).  Results are not affected; the hint is ignored
   * by launches that fill the chip and by the general kernel.  NULL / 0: no hint.  A prefetching workgroup moves
   * about 8 KB per microsecond and the launch ends when its last workgroup does: hint what the idle compute units
   * (256 minus the launch's tiles, at most 128) can read in the launch's own time -- 9 MB behind a 64-tile launch
   * of 20 K tiles costs nothing, 18 MB behind a 192-tile one doubles its duration.                                */
  const void* prefetch;
  int64_t prefetch_bytes;
} CsGemmArgs;
#define CS_SUMSQ_PARTS 8

/* Constraints: K % 8 == 0 (16 with fp8), lda/ldw % 8 == 0, N % 4 == 0, A and W 16-byte aligned. */
int cs_gemm(const CsGemmArgs* args, void* stream);

/* The RMSNorm-folded form of cs_gemm without a workspace: cs_row_sumsq on A followed by cs_gemm with a_row_sumsq, the
 * [M][CS_SUMSQ_PARTS] row sums living in a static device array of the library instead of a buffer of the caller's.
 * No counterpart in the reference (which allocates freely through torch): this entry point is for callers that cannot
 * allocate device memory -- code under HIP graph capture, serving loops and harnesses that forbid hipMalloc.  It
 * allocates and frees nothing.  args as for cs_gemm, with a_row_sumsq, a_row_sum and a_rows NULL and bf16 W; K is the
 * normalised width (<= 160 * CS_SUMSQ_PARTS); norm_eps as for cs_gemm.  M above CS_NOALLOC_MAX_ROWS (or K above that
 * width) returns CS_ERR_TOO_LARGE.  The folded form exists for K a multiple of 64 and at least 192, N a multiple of
 * 8, ldc a multiple of 8 with C 16-byte aligned, the epilogues CS_EPI_BIAS and CS_EPI_SWIGLU, and none of pos,
 * c_row_sumsq, c_row_sum, w_col_sum, w_scale, conv_patch, c_lo, residual_lo; anything else returns
 * CS_ERR_UNSUPPORTED (or CS_ERR_INVALID_ARG) BEFORE any kernel is enqueued.  Every GPU the library is used on holds
 * the array (CS_NOALLOC_MAX_ROWS * CS_SUMSQ_PARTS floats = 2 MiB) until the process ends; all calls on one GPU share
 * it, so calls that overlap on one GPU (different streams, or threads) race -- serialise them on one stream.
 * Under HIP graph capture: the first call on a device looks the array's address up (hipGetSymbolAddress) and the
 * first launch of every kernel form (tile shape x epilogue) sets that kernel's dynamic-LDS attribute
 * (hipFuncSetAttribute); neither is a stream operation, so make one call per shape and epilogue on each device
 * BEFORE capture begins -- later calls issue kernel launches only.                                                   */
#define CS_NOALLOC_MAX_ROWS 65536
int cs_gemm_rmsnorm_noalloc(const CsGemmArgs* args, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Normalisation (HBM-bound, one wavefront per row).
 * ---------------------------------------------------------------------------------------------- */
/* RMSNorm, norm.py:35-70: y = bf16(x * rsqrt(mean(x^2) + eps)) * w   (cast BEFORE the weight).
 * gemma = 1 selects GemmaRMSNorm, norm.py:90-113: y = bf16(x * rsqrt(..) * (1 + w)).              */
int cs_rmsnorm(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int32_t rows, int32_t H,
               float eps, int32_t gemma, void* stream);
/* Sum of squares of every row of x (bf16 [rows,H], H <= 160 * CS_SUMSQ_PARTS) in the layout of
 * CsGemmArgs.c_row_sumsq: out[m][p] = sum of x[m, 160p .. 160p+159]^2, parts beyond H are written as 0.
 * The variance term of RMSNorm (norm.py:35-70) for a GEMM launched with a_row_sumsq.               */
int cs_row_sumsq(const void* x, int64_t ldx, int32_t rows, int32_t H, float* out, void* stream);
/* The same with the plain row sums next to them (sum_out in the same layout): the statistics of LayerNorm for a
 * GEMM launched with a_row_sum.                                                                     */
int cs_row_stats(const void* x, int64_t ldx, int32_t rows, int32_t H, float* sumsq_out, float* sum_out, void* stream);
/* nn.LayerNorm with affine, siglip.py:173-175,333.                                                */
int cs_layernorm(const void* x, int64_t ldx, const void* w, const void* b, void* y, int64_t ldy,
                 int32_t rows, int32_t H, float eps, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Qwen2.5-VL index routines (integer, bit-exact).
 * ---------------------------------------------------------------------------------------------- */
/* Host routine.  From grid_thw_host[n_items][3] (t,h,w as int64) compute, exactly as
 * get_window_index + unique_consecutive (qwen2_5_vl.py:357-386,431-436) and the cu_seqlens
 * computation (:445-448):
 *   cu_window_host  int32, n_cu_window entries written (capacity cap_window)
 *   cu_full_host    int32, n_cu_full entries written   (capacity cap_full)
 *   item_meta_host  int32 [n_items][8]: t, gh = h/merge, gw = w/merge, first merged unit of the item,
 *                   ceil(gh/win), ceil(gw/win) (non-empty windows along h and w), first patch row of the
 *                   item, first merged unit of the item in the CALLER'S patch matrix (written equal to the
 *                   fourth entry; a caller that processes the items in another order than its patch matrix
 *                   holds them overwrites it, and src_rows of cs_vit_index then points into that matrix)
 * merge = spatial merge size (2), win = window side in merged units (window_size/merge/patch = 4).
 * Returns CS_ERR_TOO_LARGE if a capacity is too small.                                            */
int cs_vit_seqlens_host(const int64_t* grid_thw_host, int32_t n_items, int32_t merge, int32_t win,
                        int32_t* cu_window_host, int32_t cap_window, int32_t* n_cu_window,
                        int32_t* cu_full_host, int32_t cap_full, int32_t* n_cu_full,
                        int32_t* item_meta_host, int64_t* total_patches);

/* Device routine.  From item_meta (device copy of the array above) fill, for L = total patches and
 * U = L / merge^2 merged units:
 *   window_index  int32 [U]   qwen2_5_vl.py:357-386 (value = original unit at window-order position;
 *                             the reference holds the same values as int64)
 *   reverse_index int32 [U]   argsort(window_index), :478
 *   src_rows      int32 [L]   original patch row feeding window-order row m (units of merge^2 rows), :438-440,
 *                             counted from the item's eighth meta entry (its first unit in the caller's matrix)
 *   pos_ids       int32 [L,2] (h,w) of each patch in ORIGINAL order, rot_pos_emb :325-350
 *   cos_sin       fp32  [L, 2*rot_dim] window-order rotary table: cos(angles) | sin(angles) with
 *                 angles = [h*inv_freq | w*inv_freq], :251-259,352-354,441-443 and :26-29
 * inv_freq: fp32 [rot_dim/2] on device.  Any output pointer may be NULL to skip it.               */
int cs_vit_index(const int32_t* item_meta, int32_t n_items, int32_t max_units_per_item, int32_t merge,
                 int32_t win, const float* inv_freq, int32_t rot_dim, int32_t* window_index,
                 int32_t* reverse_index, int32_t* src_rows, int32_t* pos_ids, float* cos_sin, void* stream);

/* out[i, :] = in[rows[i], :] for row_bytes-wide rows (row_bytes % 4 == 0): the advanced-indexing
 * gathers at qwen2_5_vl.py:438-443 and :479.                                                     */
int cs_row_gather(const void* in, int64_t in_stride_bytes, const int32_t* rows, void* out,
                  int64_t out_stride_bytes, int32_t n_rows, int32_t row_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Rotary embedding, qwen2_5_vl.py:26-33,100-103 (flash_attn apply_rotary_emb, non-interleaved,
 * full head): for each row l, head h, j < d/2:
 *   o[j] = x[j]*cos[l,j] - x[j+d/2]*sin[l,j];  o[j+d/2] = x[j]*sin[l,j] + x[j+d/2]*cos[l,j]
 * fp32 math, one bf16 rounding.  In place on the q and k column blocks of a packed [L, 3*heads*d]
 * QKV buffer.  cos_sin is the [L, d] table written by cs_vit_index (cos | sin, d/2 each).        */
/* head_dim must be a multiple of 8 (72 for Qwen3-VL, qwen3_vl.py:218-219, takes an 8-byte-vector path).       */
int cs_rope_qk(void* qkv, int64_t ld, const float* cos_sin, int32_t L, int32_t heads, int32_t head_dim,
               void* stream);

/* Qwen3-VL learned position embedding, fast_pos_embed_interpolate at qwen3_vl.py:364-420: the side x side table
 * (bf16 [side*side, E]) bilinearly interpolated at linspace(0, side-1, h) x linspace(0, side-1, w) for every item
 * of item_meta (the records of cs_vit_seqlens_host: t, h/merge, w/merge, ..., first patch row), rows written in patch
 * order (merge x merge blocks, repeated per frame) to out (bf16 [L, ldo]).  Same operation order and rounding points
 * as the reference's tensor program (fp32 positions and weights, bf16 weights, bf16 products, one rounding of the
 * sum).                                                                                               */
int cs_pos_embed_interp(const void* table, int32_t side, int32_t E, const int32_t* item_meta, int32_t n_items,
                        int32_t max_units_per_item, int32_t merge, void* out, int64_t ldo, void* stream);

/* LLaVA-OneVision feature merge, llava_onevision.py:78-153 (`_merge_image_patch_embeddings`, strategy
 * "spatial_unpad": tiles arranged as one grid, padding cropped, grids above the token budget shrunk with
 * torch.nn.functional.interpolate(mode="bilinear"), one newline row behind every grid row) and :169-183
 * (`apply_pooling`: bilinear 2x pooling of video frames).  The caller expresses either as one record per output row:
 *   taps[r][4]  source rows (y0x0, y0x1, y1x0, y1x1) of src (bf16 [n_src_rows, lds]); frac[r][2] = (ly, lx)
 *   out[r] = (1-ly) * ((1-lx)*src[t0] + lx*src[t1]) + ly * ((1-lx)*src[t2] + lx*src[t3])   fp32, one bf16 rounding
 * and ly == lx == 0 copies src[t0] bit for bit.  A tap outside [0, n_src_rows) yields a zero row.  taps and frac are
 * device arrays; E % 8 == 0.                                                                            */
int cs_rows_bilinear(const void* src, int64_t lds, int32_t n_src_rows, const int32_t* taps, const float* frac,
                     int32_t n_rows, int32_t E, void* out, int64_t ldo, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Variable-length non-causal attention: replaces flash_attn_varlen_func (qwen2_5_vl.py:110-120)
 * and xformers memory_efficient_attention_forward (attention.py:51).
 * q, k, v: bf16, row l / head h at  base + l*ld + h*head_dim  (so a packed QKV buffer is passed as
 * three pointers with ld = 3*heads*head_dim); out: bf16 [L, heads*head_dim] with leading dimension
 * ldo.  cu_seqlens: int32 [n_seg+1] on device; work: int32 [n_work][4] = (segment start, segment
 * end, first query row, number of query rows <= block_q) built by cs_attn_work_host.  If cos_sin is
 * not NULL the rotary embedding above is applied to q and k as they are loaded (fused path).
 * scale = head_dim^-0.5.  Supported head_dim: multiples of 8 up to 96.                            */
int cs_attn_varlen(const void* q, const void* k, const void* v, int64_t ld, void* out, int64_t ldo,
                   const int32_t* work, int32_t n_work, int32_t heads, int32_t head_dim, float scale,
                   const float* cos_sin, int32_t max_seqlen, void* stream);
/* The same call for a caller that has ALREADY rotated the keys in place (cs_rope_qk on the k block, i.e. with the
 * k block's address and heads / 2): only the query rows are rotated here, with cos_sin (required), while a query
 * block is staged.  A segment's keys are then rotated once instead of once per query block, which is what the
 * fused path of cs_attn_varlen costs on long segments (the rotary of qwen2_5_vl.py:26-33,104-108 in front of full
 * attention).  Same bits as cs_attn_varlen with the same table.  Only for max_seqlen > 64 and head_dim % 16 == 0
 * (CS_ERR_UNSUPPORTED otherwise: short segments take cs_attn_varlen, which rotates each row once anyway).        */
int cs_attn_varlen_keys_rotated(const void* q, const void* k, const void* v, int64_t ld, void* out, int64_t ldo,
                                const int32_t* work, int32_t n_work, int32_t heads, int32_t head_dim, float scale,
                                const float* cos_sin, int32_t max_seqlen, void* stream);
/* QKV projection + rotary + window attention in ONE launch, for a sequence whose windows are all full: every segment of
 * cu_window_seqlens (qwen2_5_vl.py:357-386,431-436) is 64 rows starting at a multiple of 64 -- any batch of images whose
 * sides are multiples of 8 patches.  Replaces, for the window-attention blocks, the chain F.linear (qkv, linear.py:183)
 * -> split_qkv (:65-84) -> apply_rotary_pos_emb_vision (:26-33) -> flash_attn_varlen_func (:110-120): each workgroup
 * computes the q, k and v of ONE head for four windows (the GEMM of cs_gemm's direct-to-LDS kernel, one window per
 * wavefront), rotates q and k in fp32, and runs softmax(q k^T scale) v on the matrix cores without leaving registers;
 * the [L, 3*heads*head_dim] qkv tensor never exists.
 *   gemm->A, lda, K, M: the activations [M, K] (M a multiple of 64); a_row_sumsq / norm_eps as for cs_gemm (folded RMSNorm)
 *   gemm->W, ldw, bias: the qkv weight and bias PACKED per head, [heads * 256, K] and [heads * 256]: tile row
 *     rho = 32 (J/2) + 8 kq + 4 (J%2) + r of head h, for fragment J = 0..15, kq = 0..3, r = 0..3, holds
 *       J < 5:   q row h*80 + dim(kq, 4J + r)          with dim(kq, s) = 10 kq + s (s < 10), 40 + 10 kq + s - 10 (s >= 10)
 *       J < 10:  k row h*80 + dim(kq, 4(J-5) + r)
 *       J < 15:  v row h*80 + 16 (J-10) + 4 kq + r
 *       J = 15:  zeros
 *     (both halves of a rotary pair in one lane; eight consecutive slots of a lane = one MFMA operand)
 *   gemm->C, ldc: out [M, heads * 80] bf16;  gemm->N = heads * 256;  other fields zero
 *   cos_sin: the [M, 80] fp32 table of cs_vit_index;  scale = head_dim^-0.5;  head_dim must be 80.
 * Windows of fewer than 64 rows (the edge windows of an image whose sides are not multiples of 8 patches): with
 *   gemm->attn_win_start = the first attn_n_win + 1 entries of cu_window_seqlens on the device (int32; window w is rows
 *   attn_win_start[w] .. attn_win_start[w+1] - 1 of A, of cos_sin and of C; every count a multiple of 4 in 4 .. 64, the
 *   caller's to guarantee) every window takes a 64-row slot of its own: a workgroup loads a short window's last row in
 *   place of the missing ones, masks their keys in the softmax and does not store their queries.  M is then the number
 *   of real rows, attn_win_start[attn_n_win].  A window of 64 rows gives the same bits in both forms.
 * fp8 weights: gemm->w_fp8 = 1, W the e4m3 bytes of the same packed rows ([heads * 256, K], ldw % 16 == 0, zero bytes in
 *   the padding rows), gemm->w_scale fp32 [heads * 256] packed like the bias (16-byte aligned); no a_row_sumsq.
 * CS_ERR_UNSUPPORTED for any other shape (the caller then takes cs_gemm + cs_attn_varlen).                          */
int cs_qkv_window_attn(const CsGemmArgs* gemm, const float* cos_sin, float scale, int32_t heads, int32_t head_dim,
                       void* stream);

/* Host routine: expand cu_seqlens_host[n_seg+1] into query-block work items of at most block_q rows
 * (block_q = cs_attn_block_q(max_seqlen)).  Writes n_work items of 4 int32 into work_host.      */
int cs_attn_block_q(int32_t max_seqlen);
int cs_attn_work_host(const int32_t* cu_seqlens_host, int32_t n_seg, int32_t block_q, int32_t* work_host,
                      int32_t cap_items, int32_t* n_work);

/* ------------------------------------------------------------------------------------------------
 * SigLIP / Gemma-3 pieces.
 * ---------------------------------------------------------------------------------------------- */
/* Strided gather of non-overlapping patches (Conv2d k = s = patch, padding valid; siglip.py:30-36,
 * 94-95) from NCHW pixels [B,C,H,W] (bf16) into the GEMM operand [B*(H/p)*(W/p), ldo] with columns
 * ordered (c, ky, kx) and zero padding up to ldo.  H/p and W/p round down: pixels past the last whole
 * patch are dropped, as the convolution drops them (384 / 14 = 27 patches a side for LLaVA-OneVision's
 * tower).  patch and W must be even.                                                                */
int cs_patchify_nchw(const void* pixels, int32_t B, int32_t C, int32_t H, int32_t W, int32_t patch,
                     void* out, int64_t ldo, void* stream);
/* The step before the Qwen2.5-VL encoder, for callers that hand over resized uint8 frames instead of float
 * pixel_values (the reference runs the Hugging Face image processor on the CPU: ModalityProcessor,
 * qwen2_5_vl.py:488-512, called from router/processor.py:46-131, and ships 1176 floats per patch).
 * frames: uint8 [T,H,W,3] on the device, H and W multiples of patch*merge (the processor's resize is the caller's).
 * table:  fp32 [3][256] on the device: the processor's rescale + normalise applied to every byte value per
 *         channel, computed by the caller in the processor's own arithmetic.
 * out:    bf16 (or fp32 if out_fp32) [ceil(T/temporal)*(H/patch)*(W/patch), ldo], the processor's layout:
 *         rows (t, block row, block col, row in block, col in block) with merge x merge blocks, columns
 *         (channel, temporal, y, x); temporal slot tt of row group t shows frame min(t*temporal+tt, T-1).   */
int cs_qwen_patchify_u8(const void* frames, int32_t T, int32_t H, int32_t W, int32_t patch, int32_t merge,
                        int32_t temporal, const float* table, void* out, int64_t ldo, int32_t out_fp32,
                        void* stream);
/* Bicubic resampling of uint8 frames on the device, bit for bit Pillow's Image.resize(size, BICUBIC): the
 * resize the Hugging Face Qwen2-VL image processor (PIL backend) applies at its smart_resize target size
 * before rescale + normalise.  The reference runs it on the router's CPU (ModalityProcessor,
 * qwen2_5_vl.py:488-512, called from router/processor.py:46-131); with these two calls the router ships the
 * frames as decoded and the resize runs in front of cs_qwen_patchify_u8.
 * cs_resize_bicubic_taps_host (host only, no GPU call): the integer taps of one axis.  *ksize receives the taps
 *   per output position; with bounds == taps == NULL that is all it does (size query).  Otherwise bounds
 *   [out_size][2] receives (first input position, tap count) and taps [out_size][cap_ksize] the 22-bit
 *   fixed-point weights, zero past the count; cap_ksize >= *ksize.
 * cs_resize_u8_pass: one pass along the middle axis of src uint8 [outer, in_size, inner] -> dst
 *   [outer, out_size, inner], bounds / taps on the device, ksize = the row stride of taps (the cap_ksize above).
 *   Frames [T,H,W,3] -> [T,H2,W2,3] the way Pillow orders it: along x first (outer T*H, in W, out W2, inner 3)
 *   into a temporary, then along y (outer T, in H, out H2, inner W2*3); an axis whose size does not change is
 *   skipped.                                                                                         */
int cs_resize_bicubic_taps_host(int32_t in_size, int32_t out_size, int32_t* bounds, int32_t* taps,
                                int32_t cap_ksize, int32_t* ksize);
int cs_resize_u8_pass(const void* src, int64_t outer, int32_t in_size, int32_t out_size, int64_t inner,
                      const int32_t* bounds, const int32_t* taps, int32_t ksize, void* dst, void* stream);
/* Gemma3MultiModalProjector front half, gemma3.py:36-46: AvgPool2d(k) over the side x side token grid
 * followed by GemmaRMSNorm.  x: bf16 [B, side*side, H] -> y: bf16 [B, (side/k)^2, H].             */
int cs_avgpool_gemma_rmsnorm(const void* x, const void* w, void* y, int32_t B, int32_t side, int32_t k,
                             int32_t H, float eps, void* stream);

/* fp32 -> bf16 (round to nearest even) and the reverse, n elements: the `.to(dtype)` at
 * qwen2_5_vl.py:415-419.                                                                         */
int cs_cast_f32_bf16(const float* in, void* out, int64_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CORNSERVE_AMD_H */
