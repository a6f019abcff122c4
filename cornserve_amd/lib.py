"""ctypes binding of libcornserve_amd.so (the C ABI declared in include/cornserve_amd.h).

The library is the product's only compute path: there is no CPU or eager-PyTorch fallback.  If the
shared object is missing or fails to load, `load()` raises and every op built on it fails loudly.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_float, c_int32, c_int64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libcornserve_amd.so"

CS_OK = 0
CS_ERR_INVALID_ARG = 1
CS_ERR_UNSUPPORTED = 2
CS_ERR_LAUNCH = 3
CS_ERR_TOO_LARGE = 4
ABI_VERSION = 7

EPI_BIAS, EPI_RESIDUAL, EPI_SWIGLU, EPI_GELU_ERF, EPI_GELU_TANH, EPI_QUICK_GELU = range(6)


class CsGemmArgs(ctypes.Structure):
    """Mirror of `struct CsGemmArgs` in include/cornserve_amd.h (field order and types must match)."""

    _fields_ = [
        ("A", c_void_p),
        ("lda", c_int64),
        ("W", c_void_p),
        ("ldw", c_int64),
        ("w_scale", c_void_p),
        ("bias", c_void_p),
        ("residual", c_void_p),
        ("ldr", c_int64),
        ("pos", c_void_p),
        ("ldpos", c_int64),
        ("pos_period", c_int32),
        ("C", c_void_p),
        ("ldc", c_int64),
        ("a_rows", c_void_p),
        ("c_rows", c_void_p),
        ("M", c_int32),
        ("N", c_int32),
        ("K", c_int32),
        ("epilogue", c_int32),
        ("w_fp8", c_int32),
        ("tiles_m", c_int32),
        ("tiles_n", c_int32),
        ("fast_epilogue", c_int32),
        ("a_row_sumsq", c_void_p),
        ("c_row_sumsq", c_void_p),
        ("norm_eps", ctypes.c_float),
        ("a_row_sum", c_void_p),
        ("c_row_sum", c_void_p),
        ("w_col_sum", c_void_p),
        ("residual_lo", c_void_p),
        ("c_lo", c_void_p),
        ("conv_c", c_int32),
        ("conv_h", c_int32),
        ("conv_w", c_int32),
        ("conv_patch", c_int32),
        ("attn_cos_sin", c_void_p),
        ("attn_scale_log2e", ctypes.c_float),
        ("attn_win_start", c_void_p),
        ("attn_n_win", c_int32),
        ("prefetch", c_void_p),
        ("prefetch_bytes", c_int64),
    ]


# name -> (argtypes); every entry point returns int.
_SIGNATURES: dict[str, list] = {
    "cs_abi_version": [],
    "cs_gemm": [POINTER(CsGemmArgs), c_void_p],
    "cs_gemm_rmsnorm_noalloc": [POINTER(CsGemmArgs), c_void_p],
    "cs_qkv_window_attn": [POINTER(CsGemmArgs), c_void_p, c_float, c_int32, c_int32, c_void_p],
    "cs_row_sumsq": [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p],
    "cs_row_stats": [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p],
    "cs_rmsnorm": [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_float, c_int32, c_void_p],
    "cs_layernorm": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_float, c_void_p],
    "cs_vit_seqlens_host": [
        c_void_p, c_int32, c_int32, c_int32,
        c_void_p, c_int32, POINTER(c_int32),
        c_void_p, c_int32, POINTER(c_int32),
        c_void_p, POINTER(c_int64),
    ],
    "cs_vit_index": [
        c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p, c_int32,
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
    ],
    "cs_row_gather": [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p],
    "cs_pos_embed_interp": [c_void_p, c_int32, c_int32, c_void_p, c_int32, c_int32, c_int32, c_void_p, c_int64, c_void_p],
    "cs_rows_bilinear": [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_int64, c_void_p],
    "cs_rope_qk": [c_void_p, c_int64, c_void_p, c_int32, c_int32, c_int32, c_void_p],
    "cs_attn_varlen": [
        c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
        c_void_p, c_int32, c_int32, c_int32, c_float, c_void_p, c_int32, c_void_p,
    ],
    "cs_attn_varlen_keys_rotated": [
        c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
        c_void_p, c_int32, c_int32, c_int32, c_float, c_void_p, c_int32, c_void_p,
    ],
    "cs_attn_block_q": [c_int32],
    "cs_attn_work_host": [c_void_p, c_int32, c_int32, c_void_p, c_int32, POINTER(c_int32)],
    "cs_qwen_patchify_u8": [c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_int64,
                            c_int32, c_void_p],
    "cs_resize_bicubic_taps_host": [c_int32, c_int32, c_void_p, c_void_p, c_int32, POINTER(c_int32)],
    "cs_resize_u8_pass": [c_void_p, c_int64, c_int32, c_int32, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p],
    "cs_patchify_nchw": [c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p, c_int64, c_void_p],
    "cs_avgpool_gemma_rmsnorm": [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_float, c_void_p],
    "cs_cast_f32_bf16": [c_void_p, c_void_p, c_int64, c_void_p],
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: ctypes.CDLL | None = None


class KernelLibraryError(RuntimeError):
    """The HIP kernel library is missing, stale, or reported a launch failure."""


def load() -> ctypes.CDLL:
    """Load the shared library once, bind prototypes, and check the ABI version."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise KernelLibraryError(
            f"{LIB_PATH} not found: build it with `python -m cornserve_amd.build` (hipcc, gfx950). "
            "There is no fallback path."
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, argtypes in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise KernelLibraryError(f"{LIB_PATH} does not export {name}; rebuild the library") from e
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    got = lib.cs_abi_version()
    if got != ABI_VERSION:
        raise KernelLibraryError(f"ABI version mismatch: library {got}, binding {ABI_VERSION}; rebuild")
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    """Map a C status code to the exception categories of the reference model API."""
    if status == CS_OK:
        return
    if status == CS_ERR_INVALID_ARG:
        raise ValueError(f"{what}: invalid argument")
    if status == CS_ERR_UNSUPPORTED:
        raise RuntimeError(f"{what}: unsupported configuration")
    if status == CS_ERR_TOO_LARGE:
        raise RuntimeError(f"{what}: problem exceeds a fixed capacity")
    raise KernelLibraryError(f"{what}: HIP launch failed (status {status})")
