"""Thin PyTorch custom ops over the C ABI: torch supplies device memory and the stream, nothing else.

Every kernel entry point of libcornserve_amd.so is registered as an operator of the `cornserve_amd` namespace
(`torch.ops.cornserve_amd.gemm_`, `.attn_varlen_`, `.rmsnorm_`, ...: schema, a fake implementation for shape
propagation, and one implementation that validates its arguments and enqueues the HIP kernels on torch's current
stream through ctypes).  The functions of this module are the keyword-argument front ends the encoders call: they
allocate outputs with torch's caching allocator (so outputs stay IPC-exportable for the sidecar, reference:
sidecar/api.py:198-242) and dispatch through `torch.ops`, so the launches are visible to the dispatcher, the
profiler's operator records and tracing.  The operators that write into caller-provided tensors end in `_` and
return nothing; `gemm` also exists in a functional form.  There is no eager-PyTorch fallback in this module.
"""

from __future__ import annotations

import ctypes
import functools
import math
from dataclasses import dataclass

import numpy as np
import torch

from . import lib as _l
from .lib import (  # noqa: F401  (re-exported)
    EPI_BIAS,
    EPI_GELU_ERF,
    EPI_GELU_TANH,
    EPI_QUICK_GELU,
    EPI_RESIDUAL,
    EPI_SWIGLU,
)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def host_to_device(a: np.ndarray, device: torch.device) -> torch.Tensor:
    """Small host array -> device tensor through pinned memory, so that the copy is asynchronous and the host
    can keep enqueueing work (a copy from pageable memory waits for the stream)."""
    a = np.ascontiguousarray(a)
    if a.size == 0:
        return torch.from_numpy(a.copy()).to(device)
    staged = torch.empty(a.shape, dtype=torch.from_numpy(np.empty(0, dtype=a.dtype)).dtype, pin_memory=True)
    staged.numpy()[...] = a
    return staged.to(device, non_blocking=True)


def host_to_device_packed(arrays: list[np.ndarray], device: torch.device) -> list[torch.Tensor]:
    """Several small host arrays -> device tensors with ONE asynchronous copy: the arrays are laid end to end
    (256-byte aligned) in one pinned staging buffer and the results are views of one device buffer."""
    arrays = [np.ascontiguousarray(a) for a in arrays]
    offs, total = [], 0
    for a in arrays:
        offs.append(total)
        total += (a.nbytes + 255) // 256 * 256
    if total == 0:
        return [torch.from_numpy(a.copy()).to(device) for a in arrays]
    staged = torch.empty((total,), dtype=torch.uint8, pin_memory=True)
    host = staged.numpy()
    for a, o in zip(arrays, offs):
        host[o : o + a.nbytes] = a.reshape(-1).view(np.uint8)
    dev = staged.to(device, non_blocking=True)
    out = []
    for a, o in zip(arrays, offs):
        dt = torch.from_numpy(np.empty(0, dtype=a.dtype)).dtype
        out.append(dev[o : o + a.nbytes].view(dt).view(a.shape))
    return out


def cat_to_device(tensors: list[torch.Tensor], device: torch.device, dtype: torch.dtype) -> torch.Tensor:
    """`torch.cat(tensors).to(device, dtype)` (the reference's hand-over, qwen2_5_vl.py:415-419) without its two host
    passes when the tensors are floating-point HOST tensors: every item is converted to `dtype` straight into its rows
    of ONE pinned staging buffer (no concatenated fp32 copy; half the bytes cross PCIe when the source is fp32 and the
    target bf16; the conversion is the same round-to-nearest-even the device cast performs, so the result is
    bit-identical), followed by one asynchronous copy.  Anything else takes the plain route."""
    host = all(isinstance(t, torch.Tensor) and t.device.type == "cpu" and t.is_floating_point() and t.dim() >= 1
               for t in tensors)
    if not host or device.type != "cuda" or len({t.shape[1:] for t in tensors}) != 1 or sum(t.shape[0] for t in tensors) == 0:
        return torch.cat(tensors, dim=0).to(device=device, dtype=dtype)
    rows = sum(t.shape[0] for t in tensors)
    staged = torch.empty((rows, *tensors[0].shape[1:]), dtype=dtype, pin_memory=True)
    r = 0
    for t in tensors:
        staged[r : r + t.shape[0]].copy_(t)
        r += t.shape[0]
    return staged.to(device, non_blocking=True)


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _req(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if t.dim() >= 1 and t.stride(-1) != 1:
        raise ValueError(f"{name} must be contiguous in its last dimension")


# --------------------------------------------------------------------------------------------- GEMM
def gemm(
    a: torch.Tensor,
    w: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    epilogue: int = EPI_BIAS,
    residual: torch.Tensor | None = None,
    w_scale: torch.Tensor | None = None,
    pos: torch.Tensor | None = None,
    a_rows: torch.Tensor | None = None,
    c_rows: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    k: int | None = None,
    a_row_sumsq: torch.Tensor | None = None,
    c_row_sumsq: torch.Tensor | None = None,
    norm_eps: float = 0.0,
    a_row_sum: torch.Tensor | None = None,
    c_row_sum: torch.Tensor | None = None,
    w_col_sum: torch.Tensor | None = None,
    residual_lo: torch.Tensor | None = None,
    out_lo: torch.Tensor | None = None,
    conv_patch: int = 0,
    prefetch: torch.Tensor | None = None,
) -> torch.Tensor:
    """out[M,N] = epilogue(a[M,K] @ w[N,K]^T).  `w` is bf16, or float8_e4m3fn/uint8 with `w_scale`.

    `prefetch`: a contiguous tensor (the weights of the launch that follows) that a launch with few rows has its idle
    compute units read once, so that it sits in the last-level cache when the next launch asks for it; no effect on
    the result, ignored by launches that fill the chip.

    `conv_patch` > 0: `a` is NCHW pixels [B,C,H,W] (bf16, contiguous) and the product is the convolution with kernel =
    stride = conv_patch as a strided-gather GEMM: row m is patch (b, py, px), its K elements are the patch's pixels in
    (c, ky, kx) order, fetched from the image inside the kernel (no im2col buffer); `w` is the [N, C*patch*patch]
    kernel matrix, zero-padded along K to a multiple of 8.

    `a_row_sumsq` (fp32 [M, SUMSQ_PARTS]) scales row m of the product by rsqrt(sum(parts)/K + norm_eps): an
    RMSNorm of `a` whose weight the caller has folded into the columns of `w`.  `c_row_sumsq` (same layout,
    indexed by output row) receives the sums of squares of the output rows.  With `a_row_sum` (and `w_col_sum`,
    fp32 [N], the row sums of the folded weight) the fold is a LayerNorm's: rstd * (acc - mean * w_col_sum) + bias;
    `c_row_sum` receives the plain sums of the output rows.

    `out_lo` (uint8, shaped and strided like `out`; EPI_RESIDUAL only) carries the residual stream with 16
    significant bits: the sum is not rounded to bf16 but split into `out` (the leading 16 bits) and `out_lo` (the
    next 8 as a signed correction); `residual_lo` is the same plane of the addend (None: the addend is `residual`
    exactly).  A zero-filled plane next to any bf16 tensor is a valid pair.

    Dispatches to `torch.ops.cornserve_amd.gemm_` (or the functional `gemm` when nothing is written in place)."""
    if out is None and c_row_sumsq is None and c_row_sum is None and out_lo is None and residual_lo is None and prefetch is None:
        return torch.ops.cornserve_amd.gemm(a, w, bias, epilogue, residual, w_scale, pos, a_rows, c_rows, k,
                                            a_row_sumsq, norm_eps, a_row_sum, w_col_sum, conv_patch)
    if out is None:  # (with c_rows: a permutation of the M rows; anything else needs the caller's `out`)
        out = torch.empty((_gemm_rows(a, a_rows, conv_patch), w.shape[0] // 2 if epilogue == EPI_SWIGLU else w.shape[0]),
                          dtype=torch.bfloat16, device=a.device)
    torch.ops.cornserve_amd.gemm_(out, a, w, bias, epilogue, residual, w_scale, pos, a_rows, c_rows, k, a_row_sumsq,
                                  c_row_sumsq, norm_eps, a_row_sum, c_row_sum, w_col_sum, residual_lo, out_lo, conv_patch,
                                  prefetch)
    return out


def _set_prefetch(args, prefetch: torch.Tensor | None, device: torch.device) -> None:
    if prefetch is None:
        return
    if not prefetch.is_cuda or prefetch.device != device or not prefetch.is_contiguous() or prefetch.data_ptr() % 16:
        raise ValueError("prefetch must be a contiguous, 16-byte aligned tensor on the operands' device")
    args.prefetch, args.prefetch_bytes = prefetch.data_ptr(), prefetch.numel() * prefetch.element_size()


def _gemm_rows(a, a_rows, conv_patch) -> int:
    """Output rows of a product: A's rows, the gathered rows, or the patches of NCHW pixels."""
    if conv_patch:
        if a.dim() != 4 or conv_patch < 1:
            raise ValueError("with conv_patch, `a` must be NCHW pixels [B,C,H,W]")
        return a.shape[0] * (a.shape[2] // conv_patch) * (a.shape[3] // conv_patch)
    if a.dim() != 2:
        raise ValueError("gemm operands must be 2-D")
    return a.shape[0] if a_rows is None else a_rows.shape[0]


def _gemm_functional(a, w, bias, epilogue, residual, w_scale, pos, a_rows, c_rows, k, a_row_sumsq, norm_eps, a_row_sum,
                     w_col_sum, conv_patch=0):
    if w.dim() != 2:
        raise ValueError("gemm operands must be 2-D")
    M = _gemm_rows(a, a_rows, conv_patch)
    out = torch.empty((M, w.shape[0] // 2 if epilogue == EPI_SWIGLU else w.shape[0]), dtype=torch.bfloat16, device=a.device)
    _gemm_impl(out, a, w, bias, epilogue, residual, w_scale, pos, a_rows, c_rows, k, a_row_sumsq, None, norm_eps,
               a_row_sum, None, w_col_sum, None, None, conv_patch)
    return out


def _gemm_impl(out, a, w, bias, epilogue, residual, w_scale, pos, a_rows, c_rows, k, a_row_sumsq, c_row_sumsq, norm_eps,
               a_row_sum, c_row_sum, w_col_sum, residual_lo, out_lo, conv_patch=0, prefetch=None) -> None:
    """Implementation of cornserve_amd::gemm_: argument checks, then cs_gemm on the current stream."""
    lib = _l.load()
    _req(a, torch.bfloat16, "a")
    if w.dim() != 2:
        raise ValueError("gemm operands must be 2-D")
    conv = None
    if conv_patch:
        if a.dim() != 4 or not a.is_contiguous() or conv_patch < 2 or conv_patch % 2 or a.shape[3] % 2:
            raise ValueError("with conv_patch, `a` must be contiguous NCHW pixels with an even width and patch size")
        if a_rows is not None or k is not None or epilogue != EPI_BIAS:
            raise ValueError("the strided-gather product takes no a_rows / k and only the bias epilogue")
        conv = (a.shape[1], a.shape[2], a.shape[3], conv_patch)
        kreal = a.shape[1] * conv_patch * conv_patch
        if w.shape[1] != (kreal + 7) // 8 * 8:
            raise ValueError(f"w must have {(kreal + 7) // 8 * 8} columns (C*patch*patch = {kreal} rounded up to a multiple of 8)")
        a2d_rows, a2d_cols = _gemm_rows(a, None, conv_patch), w.shape[1]
    elif a.dim() != 2:
        raise ValueError("gemm operands must be 2-D")
    else:
        a2d_rows, a2d_cols = a.shape
    fp8 = w.dtype in (torch.float8_e4m3fn, torch.uint8)
    if not fp8:
        _req(w, torch.bfloat16, "w")
    elif w_scale is None:
        raise ValueError("fp8 weights need w_scale")
    for name, t in (("a_rows", a_rows), ("c_rows", c_rows)):
        if t is not None:
            _req(t, torch.int32, name)
            if t.dim() != 1 or not t.is_contiguous():
                raise ValueError(f"{name} must be a contiguous int32 vector")
    M = a2d_rows if a_rows is None else a_rows.shape[0]
    K = a2d_cols if k is None else k
    N = w.shape[0]
    if K > a2d_cols or K < 1:
        raise ValueError(f"k={K} exceeds the {a2d_cols} columns of a")
    if w.shape[1] < K:
        raise ValueError(f"w has {w.shape[1]} columns, need at least K={K}")
    if c_rows is not None and c_rows.shape[0] < M:
        raise ValueError(f"c_rows has {c_rows.shape[0]} entries for {M} output rows")
    n_out = N // 2 if epilogue == EPI_SWIGLU else N
    # Everything below reaches the kernel as a raw pointer: shapes, dtypes and devices are checked here, before
    # anything is enqueued, because an undersized or mistyped buffer would be an out-of-bounds device access.
    _req(out, torch.bfloat16, "out")
    if out.dim() != 2 or out.shape[1] < n_out or (c_rows is None and out.shape[0] < M):
        raise ValueError(f"out must be bf16 [>={M}, >={n_out}], got {tuple(out.shape)}")
    if bias is not None:
        _req(bias, torch.bfloat16, "bias")
        if bias.dim() != 1 or bias.shape[0] < N:
            raise ValueError(f"bias must be bf16 [{N}], got {tuple(bias.shape)}")
    if epilogue == EPI_RESIDUAL and residual is None:
        raise ValueError("EPI_RESIDUAL needs `residual`")
    if residual is not None:
        _req(residual, torch.bfloat16, "residual")
        if residual.dim() != 2 or residual.shape[0] < M or residual.shape[1] < N:
            raise ValueError(f"residual must be bf16 [>={M}, >={N}], got {tuple(residual.shape)}")
    if pos is not None:
        _req(pos, torch.bfloat16, "pos")
        if pos.dim() != 2 or pos.shape[0] < 1 or pos.shape[1] < N:
            raise ValueError(f"pos must be bf16 [period, >={N}], got {tuple(pos.shape)}")
    if w_scale is not None:
        _req(w_scale, torch.float32, "w_scale")
        if w_scale.dim() != 1 or w_scale.shape[0] < N or not w_scale.is_contiguous():
            raise ValueError(f"w_scale must be a contiguous fp32 [{N}] tensor")
    if residual_lo is not None or out_lo is not None:
        if epilogue != EPI_RESIDUAL or out_lo is None:
            raise ValueError("residual_lo / out_lo belong to EPI_RESIDUAL, and residual_lo needs out_lo")
        _req(out_lo, torch.uint8, "out_lo")
        if out_lo.shape != out.shape or out_lo.stride() != out.stride():
            raise ValueError("out_lo must have the shape and strides of out")
        if residual_lo is not None:
            _req(residual_lo, torch.uint8, "residual_lo")
            if residual_lo.shape != residual.shape or residual_lo.stride() != residual.stride():
                raise ValueError("residual_lo must have the shape and strides of residual")
    on = {t.device for t in (a, w, out, bias, residual, pos, w_scale, a_rows, c_rows, residual_lo, out_lo) if t is not None}
    if len(on) != 1:
        raise ValueError(f"gemm operands live on different devices: {sorted(map(str, on))}")
    args = _l.CsGemmArgs()
    args.A, args.lda = a.data_ptr(), (0 if conv else a.stride(0))
    if conv:
        args.conv_c, args.conv_h, args.conv_w, args.conv_patch = conv
    args.W, args.ldw = w.data_ptr(), w.stride(0)
    args.w_scale = _ptr(w_scale)
    args.bias = _ptr(bias)
    args.residual = _ptr(residual)
    args.ldr = residual.stride(0) if residual is not None else 0
    args.pos = _ptr(pos)
    args.ldpos = pos.stride(0) if pos is not None else 0
    args.pos_period = pos.shape[0] if pos is not None else 0
    args.C, args.ldc = out.data_ptr(), out.stride(0)
    args.a_rows = _ptr(a_rows)
    args.c_rows = _ptr(c_rows)
    args.M, args.N, args.K = M, N, K
    args.epilogue = epilogue
    args.w_fp8 = 1 if fp8 else 0
    for name, t in (("a_row_sumsq", a_row_sumsq), ("c_row_sumsq", c_row_sumsq), ("a_row_sum", a_row_sum),
                    ("c_row_sum", c_row_sum)):
        if t is not None:
            _req(t, torch.float32, name)
            if t.dim() != 2 or t.shape[1] != SUMSQ_PARTS or not t.is_contiguous() or t.shape[0] < M:
                raise ValueError(f"{name} must be a contiguous fp32 [>=M, {SUMSQ_PARTS}] tensor")
    args.a_row_sumsq = _ptr(a_row_sumsq)
    args.c_row_sumsq = _ptr(c_row_sumsq)
    args.norm_eps = norm_eps
    if w_col_sum is not None:
        _req(w_col_sum, torch.float32, "w_col_sum")
        if tuple(w_col_sum.shape) != (N,) or not w_col_sum.is_contiguous():
            raise ValueError(f"w_col_sum must be a contiguous fp32 [{N}] tensor")
    args.a_row_sum = _ptr(a_row_sum)
    args.c_row_sum = _ptr(c_row_sum)
    args.w_col_sum = _ptr(w_col_sum)
    args.residual_lo = _ptr(residual_lo)
    args.c_lo = _ptr(out_lo)
    _set_prefetch(args, prefetch, a.device)
    _l.check(lib.cs_gemm(ctypes.byref(args), _stream()), "cs_gemm")


# -------------------------------------------------------------------------------------------- norms
SUMSQ_PARTS = 8  # CS_SUMSQ_PARTS


def _rows_2d(t: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    _req(t, dtype, name)
    if t.dim() != 2:
        raise ValueError(f"{name} must be 2-D")


def _row_stats_impl(sumsq_out, sum_out, x) -> None:
    lib = _l.load()
    _rows_2d(x, torch.bfloat16, "x")
    for name, t in (("sumsq_out", sumsq_out), ("sum_out", sum_out)):
        if t is not None:
            _req(t, torch.float32, name)
            if tuple(t.shape) != (x.shape[0], SUMSQ_PARTS) or not t.is_contiguous() or t.device != x.device:
                raise ValueError(f"{name} must be a contiguous fp32 [rows, {SUMSQ_PARTS}] tensor on x's device")
    if sum_out is None:
        _l.check(lib.cs_row_sumsq(x.data_ptr(), x.stride(0), x.shape[0], x.shape[1], sumsq_out.data_ptr(), _stream()),
                 "cs_row_sumsq")
    else:
        _l.check(lib.cs_row_stats(x.data_ptr(), x.stride(0), x.shape[0], x.shape[1], sumsq_out.data_ptr(),
                                  sum_out.data_ptr(), _stream()), "cs_row_stats")


def row_stats(x: torch.Tensor, sumsq_out: torch.Tensor, sum_out: torch.Tensor) -> None:
    """Sums of squares and sums of the rows of `x`, each fp32 [rows, SUMSQ_PARTS] in parts of 160 columns."""
    torch.ops.cornserve_amd.row_stats_(sumsq_out, sum_out, x)


def row_sumsq(x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 [rows, SUMSQ_PARTS]: sums of squares of the rows of `x` in parts of 160 columns."""
    if out is None:
        if x.dim() != 2:
            raise ValueError("row_sumsq takes a 2-D tensor")
        out = torch.empty((x.shape[0], SUMSQ_PARTS), dtype=torch.float32, device=x.device)
    torch.ops.cornserve_amd.row_stats_(out, None, x)
    return out


def _norm_args(out, x, w, b) -> None:
    _rows_2d(x, torch.bfloat16, "x")
    _rows_2d(out, torch.bfloat16, "out")
    H = x.shape[1]
    if out.shape[0] < x.shape[0] or out.shape[1] < H or out.device != x.device:
        raise ValueError(f"out must be bf16 [>={x.shape[0]}, >={H}] on x's device")
    for name, t in (("w", w), ("b", b)):
        if t is not None:
            _req(t, torch.bfloat16, name)
            if t.dim() != 1 or t.shape[0] < H or t.device != x.device:
                raise ValueError(f"{name} must be bf16 [{H}] on x's device")


def _rmsnorm_impl(out, x, w, eps, gemma) -> None:
    lib = _l.load()
    _norm_args(out, x, w, None)
    _l.check(lib.cs_rmsnorm(x.data_ptr(), x.stride(0), w.data_ptr(), out.data_ptr(), out.stride(0), x.shape[0],
                            x.shape[1], eps, int(gemma), _stream()), "cs_rmsnorm")


def _layernorm_impl(out, x, w, b, eps) -> None:
    lib = _l.load()
    _norm_args(out, x, w, b)
    _l.check(lib.cs_layernorm(x.data_ptr(), x.stride(0), w.data_ptr(), b.data_ptr(), out.data_ptr(), out.stride(0),
                              x.shape[0], x.shape[1], eps, _stream()), "cs_layernorm")


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float, *, gemma: bool = False,
            out: torch.Tensor | None = None) -> torch.Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    if out is None:
        out = torch.empty_like(x2)
    torch.ops.cornserve_amd.rmsnorm_(out, x2, w, eps, gemma)
    return out.view(x.shape)


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float,
              out: torch.Tensor | None = None) -> torch.Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    if out is None:
        out = torch.empty_like(x2)
    torch.ops.cornserve_amd.layernorm_(out, x2, w, b, eps)
    return out.view(x.shape)


def _avgpool_gemma_rmsnorm_impl(out, x, w, side, k, eps) -> None:
    lib = _l.load()
    _req(x, torch.bfloat16, "x")
    _req(w, torch.bfloat16, "w")
    _req(out, torch.bfloat16, "out")
    if x.dim() != 3 or x.shape[1] != side * side or not x.is_contiguous() or k < 1 or side % k:
        raise ValueError("x must be contiguous [B, side*side, H] with side a multiple of k")
    B, _, H = x.shape
    if tuple(out.shape) != (B, (side // k) ** 2, H) or not out.is_contiguous() or w.dim() != 1 or w.shape[0] < H:
        raise ValueError("out must be contiguous [B, (side/k)^2, H] and w [H]")
    _l.check(lib.cs_avgpool_gemma_rmsnorm(x.data_ptr(), w.data_ptr(), out.data_ptr(), B, side, k, H, eps, _stream()),
             "cs_avgpool_gemma_rmsnorm")


def avgpool_gemma_rmsnorm(x: torch.Tensor, w: torch.Tensor, side: int, k: int, eps: float) -> torch.Tensor:
    """x [B, side*side, H] -> [B, (side/k)^2, H]: AvgPool2d(k) over the token grid, then GemmaRMSNorm."""
    if x.dim() != 3 or k < 1:
        raise ValueError("x must be contiguous [B, side*side, H]")
    out = torch.empty((x.shape[0], (side // k) ** 2, x.shape[2]), dtype=torch.bfloat16, device=x.device)
    torch.ops.cornserve_amd.avgpool_gemma_rmsnorm_(out, x, w, side, k, eps)
    return out


def _cast_impl(out, x) -> None:
    lib = _l.load()
    _req(x, torch.float32, "x")
    _req(out, torch.bfloat16, "out")
    if not x.is_contiguous() or not out.is_contiguous() or out.shape != x.shape or out.device != x.device:
        raise ValueError("x and out must be contiguous tensors of one shape on one device")
    _l.check(lib.cs_cast_f32_bf16(x.data_ptr(), out.data_ptr(), x.numel(), _stream()), "cs_cast_f32_bf16")


def cast_f32_bf16(x: torch.Tensor) -> torch.Tensor:
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    torch.ops.cornserve_amd.cast_f32_bf16_(out, x)
    return out


# -------------------------------------------------------------------------- Qwen2.5-VL index routines
@dataclass
class VitSeqlens:
    """Host-side result of cs_vit_seqlens_host (numpy arrays) for one batch of grids."""

    cu_window: np.ndarray   # int32 [n_windows + 1]
    cu_full: np.ndarray     # int32 [n_frames + 1]
    item_meta: np.ndarray   # int32 [n_items, 8]
    total_patches: int
    max_units_per_item: int


def vit_seqlens_host(grid_thw: np.ndarray, merge: int, win: int) -> VitSeqlens:
    lib = _l.load()
    g = np.ascontiguousarray(grid_thw, dtype=np.int64).reshape(-1, 3)
    n = g.shape[0]
    units = (g[:, 0] * (g[:, 1] // merge) * (g[:, 2] // merge)) if n else np.zeros(0, np.int64)
    frames = int(g[:, 0].sum()) if n else 0
    cap_w = int(units.sum()) + 2  # every window holds at least one merged unit
    cap_f = frames + 2
    cu_w = np.empty(cap_w, np.int32)
    cu_f = np.empty(cap_f, np.int32)
    meta = np.zeros((max(n, 1), 8), np.int32)
    n_w, n_f, total = ctypes.c_int32(0), ctypes.c_int32(0), ctypes.c_int64(0)
    _l.check(
        lib.cs_vit_seqlens_host(g.ctypes.data, n, merge, win, cu_w.ctypes.data, cap_w, ctypes.byref(n_w),
                                cu_f.ctypes.data, cap_f, ctypes.byref(n_f), meta.ctypes.data,
                                ctypes.byref(total)),
        "cs_vit_seqlens_host",
    )
    return VitSeqlens(cu_w[: n_w.value].copy(), cu_f[: n_f.value].copy(), meta[:n], int(total.value),
                      int(units.max()) if n else 0)


@dataclass
class VitIndex:
    window_index32: torch.Tensor  # int32 [U]
    reverse_index: torch.Tensor  # int32 [U]
    src_rows: torch.Tensor       # int32 [L]
    pos_ids: torch.Tensor | None  # int32 [L, 2]
    cos_sin: torch.Tensor        # fp32 [L, 2*rot_dim]

    @property
    def window_index(self) -> torch.Tensor:
        """int64 view of the permutation, the dtype the reference returns."""
        return self.window_index32.long()


def vit_index(item_meta: torch.Tensor, total_patches: int, max_units_per_item: int, merge: int, win: int,
              inv_freq: torch.Tensor, *, want_pos_ids: bool = False) -> VitIndex:
    _req(item_meta, torch.int32, "item_meta")
    _req(inv_freq, torch.float32, "inv_freq")
    dev = item_meta.device
    L = total_patches
    U = L // (merge * merge)
    rot_dim = 2 * inv_freq.numel()
    window_index = torch.empty(U, dtype=torch.int32, device=dev)
    reverse_index = torch.empty(U, dtype=torch.int32, device=dev)
    src_rows = torch.empty(L, dtype=torch.int32, device=dev)
    pos_ids = torch.empty((L, 2), dtype=torch.int32, device=dev) if want_pos_ids else None
    cos_sin = torch.empty((L, 2 * rot_dim), dtype=torch.float32, device=dev)
    torch.ops.cornserve_amd.vit_index_(window_index, reverse_index, src_rows, pos_ids, cos_sin, item_meta,
                                       max_units_per_item, merge, win, inv_freq)
    return VitIndex(window_index, reverse_index, src_rows, pos_ids, cos_sin)


def _vit_index_impl(window_index, reverse_index, src_rows, pos_ids, cos_sin, item_meta, max_units_per_item, merge, win,
                    inv_freq) -> None:
    lib = _l.load()
    _req(item_meta, torch.int32, "item_meta")
    _req(inv_freq, torch.float32, "inv_freq")
    if item_meta.dim() != 2 or item_meta.shape[1] != 8 or not item_meta.is_contiguous() or not inv_freq.is_contiguous():
        raise ValueError("item_meta must be contiguous int32 [n_items, 8] and inv_freq contiguous")
    rot_dim = 2 * inv_freq.numel()
    L, U = src_rows.shape[0], window_index.shape[0]
    for name, t, dt, shape in (("window_index", window_index, torch.int32, (U,)), ("reverse_index", reverse_index, torch.int32, (U,)),
                               ("src_rows", src_rows, torch.int32, (L,)), ("pos_ids", pos_ids, torch.int32, (L, 2)),
                               ("cos_sin", cos_sin, torch.float32, (L, 2 * rot_dim))):
        if t is not None:
            _req(t, dt, name)
            if tuple(t.shape) != shape or not t.is_contiguous() or t.device != item_meta.device:
                raise ValueError(f"{name} must be a contiguous {dt} {shape} tensor on item_meta's device")
    if U * merge * merge != L:
        raise ValueError("window_index and src_rows disagree about the number of patches")
    _l.check(
        lib.cs_vit_index(item_meta.data_ptr(), item_meta.shape[0], max_units_per_item, merge, win,
                         inv_freq.data_ptr(), rot_dim, window_index.data_ptr(), reverse_index.data_ptr(),
                         src_rows.data_ptr(), _ptr(pos_ids), cos_sin.data_ptr(), _stream()),
        "cs_vit_index",
    )


def pos_embed_interp(table: torch.Tensor, item_meta: torch.Tensor, total_patches: int, max_units_per_item: int,
                     merge: int) -> torch.Tensor:
    """Qwen3-VL position rows [total_patches, E] (bf16, patch order) interpolated from the learned side x side table."""
    if table.dim() != 2:
        raise ValueError("table must be a contiguous [side*side, E] tensor")
    out = torch.empty((total_patches, table.shape[1]), dtype=torch.bfloat16, device=table.device)
    torch.ops.cornserve_amd.pos_embed_interp_(out, table, item_meta, max_units_per_item, merge)
    return out


def _pos_embed_interp_impl(out, table, item_meta, max_units_per_item, merge) -> None:
    lib = _l.load()
    _req(table, torch.bfloat16, "table")
    _req(item_meta, torch.int32, "item_meta")
    _rows_2d(out, torch.bfloat16, "out")
    side = int(round(table.shape[0] ** 0.5))
    if table.dim() != 2 or side * side != table.shape[0] or not table.is_contiguous():
        raise ValueError("table must be a contiguous [side*side, E] tensor")
    if out.shape[1] < table.shape[1] or item_meta.dim() != 2 or item_meta.shape[1] != 8 or not item_meta.is_contiguous():
        raise ValueError("out must have the table's width and item_meta must be contiguous int32 [n_items, 8]")
    _l.check(
        lib.cs_pos_embed_interp(table.data_ptr(), side, table.shape[1], item_meta.data_ptr(), item_meta.shape[0],
                                max_units_per_item, merge, out.data_ptr(), out.stride(0), _stream()),
        "cs_pos_embed_interp",
    )


def rows_bilinear(src: torch.Tensor, taps: torch.Tensor, frac: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = bilinear mix of the four rows taps[r] of src with the fractions frac[r] = (ly, lx); (0, 0) copies
    row taps[r, 0].  src: bf16 [n, E] with contiguous rows, taps: int32 [R, 4], frac: fp32 [R, 2] (device tensors)."""
    if out is None:
        if src.dim() != 2 or taps.dim() != 2:
            raise ValueError("src must be 2-D with contiguous rows and taps [R, 4]")
        out = torch.empty((taps.shape[0], src.shape[1]), dtype=torch.bfloat16, device=src.device)
    torch.ops.cornserve_amd.rows_bilinear_(out, src, taps, frac)
    return out


def _rows_bilinear_impl(out, src, taps, frac) -> None:
    lib = _l.load()
    _req(src, torch.bfloat16, "src")
    _req(taps, torch.int32, "taps")
    _req(frac, torch.float32, "frac")
    if src.dim() != 2 or src.stride(1) != 1:
        raise ValueError("src must be 2-D with contiguous rows")
    R = taps.shape[0]
    if taps.shape != (R, 4) or frac.shape != (R, 2) or not taps.is_contiguous() or not frac.is_contiguous():
        raise ValueError("taps must be contiguous [R, 4] and frac contiguous [R, 2]")
    E = src.shape[1]
    _req(out, torch.bfloat16, "out")
    if out.shape != (R, E) or out.stride(1) != 1:
        raise ValueError("out must be [R, E] with contiguous rows")
    _l.check(
        lib.cs_rows_bilinear(src.data_ptr(), src.stride(0), src.shape[0], taps.data_ptr(), frac.data_ptr(), R, E,
                             out.data_ptr(), out.stride(0), _stream()),
        "cs_rows_bilinear",
    )


def row_gather(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """out[i] = x[rows[i]] for a 2-D tensor with contiguous rows."""
    if x.dim() != 2 or rows.dim() != 1:
        raise ValueError("x must be a 2-D device tensor with contiguous rows and rows a vector")
    out = torch.empty((rows.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    torch.ops.cornserve_amd.row_gather_(out, x, rows)
    return out


def _row_gather_impl(out, x, rows) -> None:
    lib = _l.load()
    _req(rows, torch.int32, "rows")
    if not x.is_cuda or x.dim() != 2 or x.stride(1) != 1:
        raise ValueError("x must be a 2-D device tensor with contiguous rows")
    es = x.element_size()
    if (not rows.is_contiguous() or out.dtype != x.dtype or out.device != x.device or out.dim() != 2 or out.stride(1) != 1
            or tuple(out.shape) != (rows.shape[0], x.shape[1]) or (x.shape[1] * es) % 4):
        raise ValueError("out must be [len(rows), x.shape[1]] of x's dtype on x's device, rows of whole 4-byte words")
    _l.check(
        lib.cs_row_gather(x.data_ptr(), x.stride(0) * es, rows.data_ptr(), out.data_ptr(), out.stride(0) * es,
                          rows.shape[0], x.shape[1] * es, _stream()),
        "cs_row_gather",
    )


def rope_qk_(qkv: torch.Tensor, cos_sin: torch.Tensor, heads: int, head_dim: int) -> torch.Tensor:
    """In-place rotary on the q and k blocks of a packed [L, 3*heads*head_dim] buffer."""
    torch.ops.cornserve_amd.rope_qk_(qkv, cos_sin, heads, head_dim)
    return qkv


def _rope_qk_impl(qkv, cos_sin, heads, head_dim) -> None:
    lib = _l.load()
    _rows_2d(qkv, torch.bfloat16, "qkv")
    _req(cos_sin, torch.float32, "cos_sin")
    if cos_sin.shape != (qkv.shape[0], head_dim) or not cos_sin.is_contiguous() or cos_sin.device != qkv.device:
        raise ValueError("cos_sin must be contiguous [L, head_dim] on qkv's device")
    if heads < 1 or qkv.shape[1] < 2 * heads * head_dim:
        raise ValueError(f"qkv rows hold {qkv.shape[1]} values, fewer than the q and k blocks of {heads} heads")
    _l.check(
        lib.cs_rope_qk(qkv.data_ptr(), qkv.stride(0), cos_sin.data_ptr(), qkv.shape[0], heads, head_dim, _stream()),
        "cs_rope_qk",
    )


# --------------------------------------------------------------------------------------- attention
@dataclass
class AttnPlan:
    """Device work list for one cu_seqlens: query blocks of one segment each."""

    work: torch.Tensor   # int32 [n_work, 4] on device
    n_work: int
    max_seqlen: int


def attn_work_host(cu_seqlens_host: np.ndarray) -> tuple[np.ndarray, int]:
    """Host half of attn_plan: the work list int32 [n_work, 4] (still on the host) and the longest segment."""
    lib = _l.load()
    cu = np.ascontiguousarray(cu_seqlens_host, dtype=np.int32)
    n_seg = cu.shape[0] - 1
    if n_seg <= 0:
        return np.zeros((0, 4), np.int32), 1
    lens = np.diff(cu)
    max_seqlen = int(lens.max())
    bq = lib.cs_attn_block_q(max_seqlen)
    cap = int(((lens + bq - 1) // bq).sum()) + 1
    work = np.empty((cap, 4), np.int32)
    n_work = ctypes.c_int32(0)
    _l.check(lib.cs_attn_work_host(cu.ctypes.data, n_seg, bq, work.ctypes.data, cap, ctypes.byref(n_work)),
             "cs_attn_work_host")
    return work[: n_work.value], max_seqlen


def attn_plan(cu_seqlens_host: np.ndarray, device: torch.device) -> AttnPlan:
    work, max_seqlen = attn_work_host(cu_seqlens_host)
    return AttnPlan(host_to_device(work, device), work.shape[0], max_seqlen)


def attn_varlen(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, plan: AttnPlan, heads: int, head_dim: int,
                scale: float, cos_sin: torch.Tensor | None = None, out: torch.Tensor | None = None,
                keys_rotated: bool = False) -> torch.Tensor:
    """q/k/v: [L, >= heads*head_dim] views sharing one row stride (e.g. thirds of a packed QKV buffer).
    `keys_rotated`: k already carries the rotary of `cos_sin`; only q is rotated (long segments only)."""
    if out is None:
        out = torch.empty((q.shape[0], heads * head_dim), dtype=torch.bfloat16, device=q.device)
    torch.ops.cornserve_amd.attn_varlen_(out, q, k, v, plan.work, plan.n_work, plan.max_seqlen, heads, head_dim, scale,
                                         cos_sin, keys_rotated)
    return out


def _attn_varlen_impl(out, q, k, v, work, n_work, max_seqlen, heads, head_dim, scale, cos_sin, keys_rotated) -> None:
    lib = _l.load()
    for name, t in (("q", q), ("k", k), ("v", v), ("out", out)):
        _rows_2d(t, torch.bfloat16, name)
        if t.shape[1] < heads * head_dim or t.device != q.device:
            raise ValueError(f"{name} must hold {heads} heads of {head_dim} values per row on q's device")
    if not (q.stride(0) == k.stride(0) == v.stride(0)):
        raise ValueError("q, k, v must share a row stride")
    L = q.shape[0]
    if k.shape[0] != L or v.shape[0] != L or out.shape[0] < L:
        raise ValueError("q, k, v and out must have one row per token")
    _req(work, torch.int32, "work")
    if work.dim() != 2 or work.shape[1] != 4 or not work.is_contiguous() or work.shape[0] < n_work or work.device != q.device:
        raise ValueError("work must be a contiguous int32 [>=n_work, 4] tensor on q's device")
    if cos_sin is not None:
        _req(cos_sin, torch.float32, "cos_sin")
        if cos_sin.shape != (L, head_dim) or not cos_sin.is_contiguous() or cos_sin.device != q.device:
            raise ValueError("cos_sin must be contiguous [L, head_dim] on q's device")
    entry = lib.cs_attn_varlen_keys_rotated if keys_rotated else lib.cs_attn_varlen
    _l.check(
        entry(q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
              work.data_ptr(), n_work, heads, head_dim, scale, _ptr(cos_sin), max_seqlen, _stream()),
        "cs_attn_varlen_keys_rotated" if keys_rotated else "cs_attn_varlen",
    )


def attn_varlen_rotary_(qkv: torch.Tensor, plan: AttnPlan, heads: int, head_dim: int, scale: float,
                        cos_sin: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """Rotary + attention over a packed [L, 3*heads*head_dim] buffer whose q and k the caller no longer needs.
    Segments of at most 64 rows (window attention) take the kernel that rotates while it stages q and k.  Longer
    segments rotate the keys in place once (every query block of a segment would otherwise rotate the segment's keys
    again) and take the kernel that streams K/V tiles straight into LDS and rotates its query rows while staging them;
    head shapes that kernel does not take rotate q and k in place and run without a table.  All routes give the same
    bits."""
    E = heads * head_dim
    q, k, v = qkv[:, :E], qkv[:, E : 2 * E], qkv[:, 2 * E :]
    if plan.max_seqlen <= 64:
        return attn_varlen(q, k, v, plan, heads, head_dim, scale, cos_sin=cos_sin, out=out)
    if heads % 2 == 0 and head_dim % 16 == 0 and plan.max_seqlen * qkv.stride(0) * 2 < 2**31:
        rope_qk_(qkv[:, E:], cos_sin, heads // 2, head_dim)   # the k block as two tensors of heads / 2 heads
        return attn_varlen(q, k, v, plan, heads, head_dim, scale, cos_sin=cos_sin, out=out, keys_rotated=True)
    rope_qk_(qkv, cos_sin, heads, head_dim)
    return attn_varlen(q, k, v, plan, heads, head_dim, scale, out=out)


@functools.lru_cache(maxsize=64)
def resize_bicubic_taps_host(in_size: int, out_size: int) -> tuple[np.ndarray, np.ndarray]:
    """Pillow's bicubic taps for one axis: (bounds int32 [out_size,2] = (first input position, tap count),
    taps int32 [out_size,ksize] in 22-bit fixed point).  Host arithmetic only; no GPU call."""
    lib = _l.load()
    ksize = ctypes.c_int32(0)
    _l.check(lib.cs_resize_bicubic_taps_host(in_size, out_size, None, None, 0, ctypes.byref(ksize)),
             "cs_resize_bicubic_taps_host")
    bounds = np.empty((out_size, 2), dtype=np.int32)
    taps = np.empty((out_size, ksize.value), dtype=np.int32)
    _l.check(lib.cs_resize_bicubic_taps_host(in_size, out_size, bounds.ctypes.data, taps.ctypes.data, ksize.value,
                                             ctypes.byref(ksize)), "cs_resize_bicubic_taps_host")
    bounds.setflags(write=False)
    taps.setflags(write=False)
    return bounds, taps


def resize_bicubic_u8(frames: torch.Tensor, out_h: int, out_w: int) -> torch.Tensor:
    """uint8 frames [T,H,W,C] on the device -> [T,out_h,out_w,C], bit for bit what Pillow's
    `Image.resize((out_w, out_h), BICUBIC)` makes of every frame: a pass along x, then one along y, an axis that keeps
    its size skipped (frames already at the target size come back as they are)."""
    _req(frames, torch.uint8, "frames")
    if frames.dim() != 4 or not frames.is_contiguous():
        raise ValueError("frames must be contiguous uint8 [T,H,W,C]")
    if out_h <= 0 or out_w <= 0:
        raise ValueError(f"target size must be positive, got {out_h}x{out_w}")
    T, H, W, C = frames.shape
    todo = [(axis, a, b) for axis, a, b in ((2, W, out_w), (1, H, out_h)) if a != b]
    if not todo:
        return frames
    for axis, a, b in todo:
        bounds, taps = _resize_taps_device(a, b, frames.device)
        shape = list(frames.shape)
        shape[axis] = b
        out = torch.empty(shape, dtype=torch.uint8, device=frames.device)
        torch.ops.cornserve_amd.resize_u8_pass_(out, frames, bounds, taps, axis)
        frames = out
    return frames


@functools.lru_cache(maxsize=256)
def _resize_taps_device(in_size: int, out_size: int, device: torch.device) -> list[torch.Tensor]:
    """The taps of one axis on the device, kept for the next frame of the same size (a few KB per size pair)."""
    return host_to_device_packed(list(resize_bicubic_taps_host(in_size, out_size)), device)


def _resize_u8_pass_impl(out, src, bounds, taps, axis) -> None:
    lib = _l.load()
    _req(src, torch.uint8, "src")
    _req(out, torch.uint8, "out")
    _req(bounds, torch.int32, "bounds")
    _req(taps, torch.int32, "taps")
    if src.dim() != out.dim() or not 0 <= axis < src.dim() or not src.is_contiguous() or not out.is_contiguous():
        raise ValueError("src and out must be contiguous tensors of the same rank")
    if any(a != b for i, (a, b) in enumerate(zip(src.shape, out.shape)) if i != axis):
        raise ValueError(f"out {tuple(out.shape)} must match src {tuple(src.shape)} except along axis {axis}")
    n_in, n_out = src.shape[axis], out.shape[axis]
    if (tuple(bounds.shape) != (n_out, 2) or taps.dim() != 2 or taps.shape[0] != n_out or not bounds.is_contiguous()
            or not taps.is_contiguous() or len({src.device, out.device, bounds.device, taps.device}) != 1):
        raise ValueError(f"bounds must be int32 [{n_out},2] and taps int32 [{n_out},ksize] on the frames' device")
    outer = math.prod(src.shape[:axis])
    inner = math.prod(src.shape[axis + 1:])
    if src.numel() == 0 or out.numel() == 0:
        raise ValueError("empty frames")
    _l.check(lib.cs_resize_u8_pass(src.data_ptr(), outer, n_in, n_out, inner, bounds.data_ptr(), taps.data_ptr(),
                                   taps.shape[1], out.data_ptr(), _stream()), "cs_resize_u8_pass")


def qwen_patchify_u8(frames: torch.Tensor, table: torch.Tensor, patch: int, merge: int, temporal: int, *,
                     out: torch.Tensor | None = None, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """uint8 frames [T,H,W,3] -> normalised patch rows [ceil(T/temporal)*(H/patch)*(W/patch), 3*temporal*patch^2]
    in the Qwen2-VL processor's layout; `table` is the fp32 [3,256] byte table.  `out` may be a row slice of a
    larger buffer."""
    if out is None:
        if frames.dim() != 4:
            raise ValueError("frames must be contiguous uint8 [T,H,W,3]")
        T, H, W, _ = frames.shape
        out = torch.empty((-(-T // temporal) * (H // patch) * (W // patch), 3 * temporal * patch * patch), dtype=dtype,
                          device=frames.device)
    torch.ops.cornserve_amd.qwen_patchify_u8_(out, frames, table, patch, merge, temporal)
    return out


def _qwen_patchify_u8_impl(out, frames, table, patch, merge, temporal) -> None:
    lib = _l.load()
    _req(frames, torch.uint8, "frames")
    _req(table, torch.float32, "table")
    if frames.dim() != 4 or frames.shape[-1] != 3 or not frames.is_contiguous():
        raise ValueError("frames must be contiguous uint8 [T,H,W,3]")
    if tuple(table.shape) != (3, 256) or not table.is_contiguous():
        raise ValueError("table must be contiguous fp32 [3,256]")
    T, H, W, _ = frames.shape
    if H % (patch * merge) or W % (patch * merge):
        raise ValueError(f"frame size {H}x{W} is not a multiple of patch*merge = {patch * merge}")
    rows, cols = -(-T // temporal) * (H // patch) * (W // patch), 3 * temporal * patch * patch
    if (not out.is_cuda or out.dtype not in (torch.bfloat16, torch.float32) or tuple(out.shape) != (rows, cols)
            or out.stride(1) != 1 or out.device != frames.device or table.device != frames.device):
        raise ValueError(f"out must be bf16 or fp32 [{rows},{cols}] on the frames' device")
    _l.check(lib.cs_qwen_patchify_u8(frames.data_ptr(), T, H, W, patch, merge, temporal, table.data_ptr(),
                                     out.data_ptr(), out.stride(0), int(out.dtype == torch.float32), _stream()),
             "cs_qwen_patchify_u8")


def patchify_nchw(pixels: torch.Tensor, patch: int, ldo: int) -> torch.Tensor:
    """[B,C,H,W] bf16 -> [B*(H//p)*(W//p), ldo] rows of (c,ky,kx)-ordered patch values, zero padded.  Pixels past the
    last whole patch are dropped, as a convolution with stride = kernel and no padding drops them."""
    if pixels.dim() != 4 or patch < 1:
        raise ValueError("pixels must be contiguous [B,C,H,W]")
    B, C, H, W = pixels.shape
    out = torch.empty((B * (H // patch) * (W // patch), ldo), dtype=torch.bfloat16, device=pixels.device)
    torch.ops.cornserve_amd.patchify_nchw_(out, pixels, patch)
    return out


def _patchify_nchw_impl(out, pixels, patch) -> None:
    lib = _l.load()
    _req(pixels, torch.bfloat16, "pixels")
    _rows_2d(out, torch.bfloat16, "out")
    if pixels.dim() != 4 or not pixels.is_contiguous() or patch < 1:
        raise ValueError("pixels must be contiguous [B,C,H,W]")
    B, C, H, W = pixels.shape
    if (out.shape[0] != B * (H // patch) * (W // patch) or out.shape[1] < C * patch * patch or not out.is_contiguous()
            or out.device != pixels.device):
        raise ValueError("out must be contiguous [B*(H//patch)*(W//patch), >= C*patch*patch] on the pixels' device")
    _l.check(lib.cs_patchify_nchw(pixels.data_ptr(), B, C, H, W, patch, out.data_ptr(), out.shape[1], _stream()),
             "cs_patchify_nchw")


# ------------------------------------------------- QKV projection + rotary + window attention in one launch
QKV_WATTN_HEAD_DIM = 80      # the head dim the fused kernel is written for (Qwen2.5-VL: 1280 / 16)
QKV_WATTN_TILE_ROWS = 256    # packed weight rows per head
QKV_WATTN_WINDOW = 64        # rows of every attention segment


@functools.lru_cache(maxsize=8)
def _qkv_window_attn_row_order(heads: int) -> torch.Tensor:
    """Row r of the packed [heads*256, K] weight of `qkv_window_attn` is row order[r] of the reference's qkv weight
    [3*heads*80, K] (q | k | v blocks, qwen2_5_vl.py:65-84), or -1 for a zero row.  Per head: tile row
    rho = 32 (J/2) + 8 kq + 4 (J%2) + r for fragment J, lane group kq, element r; q and k fragments (J < 5, J < 10) put
    both halves of every rotary pair into one lane group, the v fragments (J < 15) hold 16 consecutive head dims."""
    d, half = QKV_WATTN_HEAD_DIM, QKV_WATTN_HEAD_DIM // 2
    order = torch.full((heads, QKV_WATTN_TILE_ROWS), -1, dtype=torch.int64)
    for J in range(15):
        for kq in range(4):
            for r in range(4):
                rho = 32 * (J // 2) + 8 * kq + 4 * (J % 2) + r
                if J < 10:
                    s = 4 * (J % 5) + r
                    dim = 10 * kq + s if s < 10 else half + 10 * kq + (s - 10)
                    block = 0 if J < 5 else 1
                else:
                    dim = 16 * (J - 10) + 4 * kq + r
                    block = 2
                for h in range(heads):
                    order[h, rho] = block * heads * d + h * d + dim
    return order.reshape(-1)


def qkv_window_attn_row_order(heads: int) -> torch.Tensor:
    """Row order of the packed weight of `qkv_window_attn` (see `_qkv_window_attn_row_order`; computed once per head
    count)."""
    return _qkv_window_attn_row_order(int(heads)).clone()


def pack_qkv_window_attn(w: torch.Tensor, b: torch.Tensor, heads: int, w_scale: torch.Tensor | None = None):
    """The qkv weight [3*heads*80, K] and bias [3*heads*80] in the row order `qkv_window_attn` takes (done once, at load).
    fp8 weights (float8_e4m3fn or uint8 bytes, with `w_scale` fp32 [3*heads*80]): the bytes are reordered as they are,
    and the result has a third entry, the scales in the same order (1 for the padding rows, whose bytes are zero)."""
    if w.dim() != 2 or w.shape[0] != 3 * heads * QKV_WATTN_HEAD_DIM or b.shape != (w.shape[0],):
        raise ValueError(f"qkv weight must be [3*{heads}*{QKV_WATTN_HEAD_DIM}, K] with a matching bias")
    fp8 = w.dtype in (torch.float8_e4m3fn, torch.uint8)
    if fp8 != (w_scale is not None) or (fp8 and (w_scale.shape != (w.shape[0],) or w_scale.dtype != torch.float32)):
        raise ValueError("fp8 weights (float8_e4m3fn / uint8) come with an fp32 w_scale [3*heads*80]; bf16 weights without")
    order = qkv_window_attn_row_order(heads).to(w.device)
    keep = (order >= 0).unsqueeze(1)
    rows = order.clamp_min(0)
    wb = w.view(torch.uint8) if fp8 else w
    wp = torch.where(keep, wb[rows], torch.zeros((), dtype=wb.dtype, device=w.device)).contiguous()
    bp = torch.where(keep[:, 0], b[rows], torch.zeros((), dtype=b.dtype, device=b.device)).contiguous()
    if not fp8:
        return wp, bp
    sp = torch.where(keep[:, 0], w_scale[rows], torch.ones((), dtype=torch.float32, device=w.device)).contiguous()
    return wp, bp, sp


def unpack_qkv_window_attn(w_packed: torch.Tensor, b_packed: torch.Tensor, heads: int, w_scale: torch.Tensor | None = None):
    """The inverse of `pack_qkv_window_attn`: the plain [3*heads*80, K] weight, bias (and scales) back from the packed
    form, bit for bit (fp8 weights come back as uint8 bytes)."""
    order = qkv_window_attn_row_order(heads).to(w_packed.device)
    if w_packed.dim() != 2 or w_packed.shape[0] != order.numel() or b_packed.shape != (order.numel(),):
        raise ValueError(f"packed qkv weight must be [{heads}*{QKV_WATTN_TILE_ROWS}, K] with a matching bias")
    place = torch.empty(3 * heads * QKV_WATTN_HEAD_DIM, dtype=torch.int64, device=w_packed.device)
    packed_rows = torch.arange(order.numel(), device=w_packed.device)
    place[order[order >= 0]] = packed_rows[order >= 0]
    out = (w_packed[place].contiguous(), b_packed[place].contiguous())
    return out if w_scale is None else out + (w_scale[place].contiguous(),)


def qkv_window_attn(x: torch.Tensor, w_packed: torch.Tensor, b_packed: torch.Tensor, cos_sin: torch.Tensor, heads: int,
                    scale: float, *, a_row_sumsq: torch.Tensor | None = None, norm_eps: float = 0.0,
                    out: torch.Tensor | None = None, win_start: torch.Tensor | None = None,
                    w_scale: torch.Tensor | None = None, prefetch: torch.Tensor | None = None) -> torch.Tensor:
    """attention(rotary(x . Wq^T + bq), rotary(x . Wk^T + bk), x . Wv^T + bv) over windows of up to 64 rows, one launch.

    Replaces qkv Linear -> split -> rotary -> flash_attn_varlen_func (qwen2_5_vl.py:93-120).  Without `win_start` the
    attention segments are ALL 64 rows starting at multiples of 64; with it (int32 [windows + 1] on the device: the
    leading entries of cu_window_seqlens, ending at the number of rows of `x`) a window has 4 .. 64 rows, a multiple of
    4, which the caller guarantees.  `w_packed`, `b_packed` come from `pack_qkv_window_attn`; with `a_row_sumsq` the
    rows of `x` are RMS-normalised on the way (the norm weight folded into the packed weight's columns, as for
    `gemm`).  fp8 weights: `w_packed` uint8 with `w_scale` (both from `pack_qkv_window_attn`), no folded norm.
    `prefetch` as for `gemm`.
    Raises ValueError for shapes the kernel does not take."""
    if out is None:
        out = torch.empty((x.shape[0], heads * QKV_WATTN_HEAD_DIM), dtype=torch.bfloat16, device=x.device)
    torch.ops.cornserve_amd.qkv_window_attn_(out, x, w_packed, b_packed, cos_sin, heads, scale, a_row_sumsq, norm_eps,
                                              win_start, w_scale, prefetch)
    return out


def _qkv_window_attn_impl(out, x, w_packed, b_packed, cos_sin, heads, scale, a_row_sumsq, norm_eps, win_start=None,
                          w_scale=None, prefetch=None) -> None:
    lib = _l.load()
    _rows_2d(x, torch.bfloat16, "x")
    fp8 = w_scale is not None
    _rows_2d(w_packed, torch.uint8 if fp8 else torch.bfloat16, "w_packed")
    if fp8:
        _req(w_scale, torch.float32, "w_scale")
        if tuple(w_scale.shape) != (heads * QKV_WATTN_TILE_ROWS,) or not w_scale.is_contiguous():
            raise ValueError(f"w_scale must be a contiguous fp32 [{heads * QKV_WATTN_TILE_ROWS}] tensor")
        if a_row_sumsq is not None:
            raise ValueError("the folded norm (a_row_sumsq) does not exist for fp8 weights")
    _rows_2d(out, torch.bfloat16, "out")
    _req(b_packed, torch.bfloat16, "b_packed")
    _req(cos_sin, torch.float32, "cos_sin")
    M, K = x.shape
    d = QKV_WATTN_HEAD_DIM
    if heads < 1 or tuple(w_packed.shape) != (heads * QKV_WATTN_TILE_ROWS, K):
        raise ValueError(f"w_packed must be [{heads}*{QKV_WATTN_TILE_ROWS}, {K}], got {tuple(w_packed.shape)}")
    if tuple(b_packed.shape) != (heads * QKV_WATTN_TILE_ROWS,) or not b_packed.is_contiguous():
        raise ValueError(f"b_packed must be a contiguous [{heads * QKV_WATTN_TILE_ROWS}] tensor")
    if win_start is None:
        if M % QKV_WATTN_WINDOW:
            raise ValueError(f"the rows of x ({M}) must be a whole number of {QKV_WATTN_WINDOW}-row windows")
    else:
        _req(win_start, torch.int32, "win_start")
        n_win = win_start.numel() - 1
        if win_start.dim() != 1 or not win_start.is_contiguous() or n_win < 1 or not 4 * n_win <= M <= QKV_WATTN_WINDOW * n_win or M % 4:
            raise ValueError(f"win_start must be a contiguous int32 [windows + 1] tensor whose windows of 4 .. "
                             f"{QKV_WATTN_WINDOW} rows add up to the {M} rows of x")
    if tuple(cos_sin.shape) != (M, d) or not cos_sin.is_contiguous():
        raise ValueError(f"cos_sin must be a contiguous fp32 [{M}, {d}] table")
    if out.shape[0] < M or out.shape[1] < heads * d:
        raise ValueError(f"out must be bf16 [>={M}, >={heads * d}], got {tuple(out.shape)}")
    if a_row_sumsq is not None:
        _req(a_row_sumsq, torch.float32, "a_row_sumsq")
        if a_row_sumsq.dim() != 2 or a_row_sumsq.shape[1] != SUMSQ_PARTS or not a_row_sumsq.is_contiguous() or a_row_sumsq.shape[0] < M:
            raise ValueError(f"a_row_sumsq must be a contiguous fp32 [>=M, {SUMSQ_PARTS}] tensor")
    on = {t.device for t in (out, x, w_packed, b_packed, cos_sin, a_row_sumsq, win_start, w_scale) if t is not None}
    if len(on) != 1:
        raise ValueError(f"qkv_window_attn operands live on different devices: {sorted(map(str, on))}")
    args = _l.CsGemmArgs()
    args.A, args.lda = x.data_ptr(), x.stride(0)
    args.W, args.ldw = w_packed.data_ptr(), w_packed.stride(0)
    args.bias = b_packed.data_ptr()
    args.C, args.ldc = out.data_ptr(), out.stride(0)
    args.M, args.N, args.K = M, heads * QKV_WATTN_TILE_ROWS, K
    args.a_row_sumsq = _ptr(a_row_sumsq)
    args.norm_eps = norm_eps
    if win_start is not None:
        args.attn_win_start, args.attn_n_win = win_start.data_ptr(), win_start.numel() - 1
    if fp8:
        args.w_fp8, args.w_scale = 1, w_scale.data_ptr()
    _set_prefetch(args, prefetch, x.device)
    _l.check(lib.cs_qkv_window_attn(ctypes.byref(args), cos_sin.data_ptr(), scale, heads, d, _stream()), "cs_qkv_window_attn")


# ------------------------------------------------------------------------------- operator registration
# One operator per kernel entry point, in the `cornserve_amd` namespace.  Operators ending in `_` write into their
# leading tensor argument(s) and return nothing; every argument that reaches a kernel as a pointer is a Tensor of the
# schema, so the dispatcher sees it.  The implementation is registered for every backend key: it validates devices and
# dtypes itself and raises ValueError, the reference model API's error for bad input.
_LIBRARY = torch.library.Library("cornserve_amd", "DEF")
_OPERATORS: dict[str, tuple[str, object]] = {
    "gemm": ("(Tensor a, Tensor w, Tensor? bias, int epilogue, Tensor? residual, Tensor? w_scale, Tensor? pos, "
             "Tensor? a_rows, Tensor? c_rows, int? k, Tensor? a_row_sumsq, float norm_eps, Tensor? a_row_sum, "
             "Tensor? w_col_sum, int conv_patch=0) -> Tensor", _gemm_functional),
    "gemm_": ("(Tensor(a!) out, Tensor a, Tensor w, Tensor? bias, int epilogue, Tensor? residual, Tensor? w_scale, "
              "Tensor? pos, Tensor? a_rows, Tensor? c_rows, int? k, Tensor? a_row_sumsq, Tensor(b!)? c_row_sumsq, "
              "float norm_eps, Tensor? a_row_sum, Tensor(c!)? c_row_sum, Tensor? w_col_sum, Tensor? residual_lo, "
              "Tensor(d!)? out_lo, int conv_patch=0, Tensor? prefetch=None) -> ()", _gemm_impl),
    "row_stats_": ("(Tensor(a!) sumsq_out, Tensor(b!)? sum_out, Tensor x) -> ()", _row_stats_impl),
    "rmsnorm_": ("(Tensor(a!) out, Tensor x, Tensor w, float eps, bool gemma) -> ()", _rmsnorm_impl),
    "layernorm_": ("(Tensor(a!) out, Tensor x, Tensor w, Tensor b, float eps) -> ()", _layernorm_impl),
    "avgpool_gemma_rmsnorm_": ("(Tensor(a!) out, Tensor x, Tensor w, int side, int k, float eps) -> ()",
                               _avgpool_gemma_rmsnorm_impl),
    "cast_f32_bf16_": ("(Tensor(a!) out, Tensor x) -> ()", _cast_impl),
    "vit_index_": ("(Tensor(a!) window_index, Tensor(b!) reverse_index, Tensor(c!) src_rows, Tensor(d!)? pos_ids, "
                   "Tensor(e!) cos_sin, Tensor item_meta, int max_units_per_item, int merge, int win, Tensor inv_freq) -> ()",
                   _vit_index_impl),
    "pos_embed_interp_": ("(Tensor(a!) out, Tensor table, Tensor item_meta, int max_units_per_item, int merge) -> ()",
                          _pos_embed_interp_impl),
    "rows_bilinear_": ("(Tensor(a!) out, Tensor src, Tensor taps, Tensor frac) -> ()", _rows_bilinear_impl),
    "row_gather_": ("(Tensor(a!) out, Tensor x, Tensor rows) -> ()", _row_gather_impl),
    "rope_qk_": ("(Tensor(a!) qkv, Tensor cos_sin, int heads, int head_dim) -> ()", _rope_qk_impl),
    "attn_varlen_": ("(Tensor(a!) out, Tensor q, Tensor k, Tensor v, Tensor work, int n_work, int max_seqlen, int heads, "
                     "int head_dim, float scale, Tensor? cos_sin, bool keys_rotated) -> ()", _attn_varlen_impl),
    "qwen_patchify_u8_": ("(Tensor(a!) out, Tensor frames, Tensor table, int patch, int merge, int temporal) -> ()",
                          _qwen_patchify_u8_impl),
    "resize_u8_pass_": ("(Tensor(a!) out, Tensor src, Tensor bounds, Tensor taps, int axis) -> ()", _resize_u8_pass_impl),
    "patchify_nchw_": ("(Tensor(a!) out, Tensor pixels, int patch) -> ()", _patchify_nchw_impl),
    "qkv_window_attn_": ("(Tensor(a!) out, Tensor x, Tensor w_packed, Tensor b_packed, Tensor cos_sin, int heads, "
                         "float scale, Tensor? a_row_sumsq, float norm_eps, Tensor? win_start=None, Tensor? w_scale=None, "
                         "Tensor? prefetch=None) -> ()",
                         _qkv_window_attn_impl),
}


def _fake_gemm(a, w, bias, epilogue, residual, w_scale, pos, a_rows, c_rows, k, a_row_sumsq, norm_eps, a_row_sum, w_col_sum,
               conv_patch=0):
    M = _gemm_rows(a, a_rows, conv_patch)
    return a.new_empty((M, w.shape[0] // 2 if epilogue == EPI_SWIGLU else w.shape[0]), dtype=torch.bfloat16)


def _fake_nothing(*args, **kwargs) -> None:   # the in-place operators return nothing: shapes are their arguments'
    return None


for _name, (_schema, _impl) in _OPERATORS.items():
    _LIBRARY.define(_name + _schema)
    _LIBRARY.impl(_name, _impl, "CompositeExplicitAutograd")
    torch.library.register_fake(f"cornserve_amd::{_name}", _fake_gemm if _name == "gemm" else _fake_nothing, lib=_LIBRARY)
