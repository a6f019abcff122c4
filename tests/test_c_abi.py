"""C-ABI surface and host-side routines (CPU only; no kernel is launched here)."""

import ctypes
import json
import re
from pathlib import Path

import numpy as np
import pytest

from cornserve_amd import lib, ops
from oracle import vit_index as vi

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols() -> list[str]:
    text = (ROOT / "include" / "cornserve_amd.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\bint\s+(cs_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 14
    dll = ctypes.CDLL(str(lib.LIB_PATH))
    for n in names:
        assert hasattr(dll, n), f"{n} is declared in include/cornserve_amd.h but not exported"
    assert sorted(lib.EXPORTED_SYMBOLS) == names, "ctypes binding and header disagree"
    assert lib.load().cs_abi_version() == lib.ABI_VERSION


def test_gemm_args_struct_layout_matches_header():
    # 64-bit pointers / int64 / int32 fields in header order; sizeof must match the C struct (8-byte aligned)
    text = (ROOT / "include" / "cornserve_amd.h").read_text()
    body = re.search(r"typedef struct CsGemmArgs \{(.*?)\} CsGemmArgs;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        names = [n.strip().lstrip("*") for n in decl.split(",")]
        first = names[0].split()[-1].lstrip("*")
        fields += [first] + names[1:]
    assert fields == [f[0] for f in lib.CsGemmArgs._fields_]
    assert ctypes.sizeof(lib.CsGemmArgs) % 8 == 0


def test_status_mapping():
    lib.check(lib.CS_OK, "x")
    with pytest.raises(ValueError):
        lib.check(lib.CS_ERR_INVALID_ARG, "x")
    with pytest.raises(RuntimeError):
        lib.check(lib.CS_ERR_UNSUPPORTED, "x")
    with pytest.raises(lib.KernelLibraryError):
        lib.check(lib.CS_ERR_LAUNCH, "x")


def test_invalid_arguments_are_rejected_without_a_gpu():
    l = lib.load()
    assert l.cs_gemm(None, None) == lib.CS_ERR_INVALID_ARG
    args = lib.CsGemmArgs()
    assert l.cs_gemm(ctypes.byref(args), None) == lib.CS_ERR_INVALID_ARG
    assert l.cs_rmsnorm(None, 0, None, None, 0, 1, 8, 1e-6, 0, None) == lib.CS_ERR_INVALID_ARG
    assert l.cs_attn_varlen(None, None, None, 0, None, 0, None, 0, 16, 80, 0.1, None, 64, None) == lib.CS_ERR_INVALID_ARG
    assert l.cs_rope_qk(None, 0, None, 0, 16, 80, None) == lib.CS_ERR_INVALID_ARG
    # the entry point that allocates nothing refuses what its folded-norm GEMM cannot take before it touches the GPU
    # (fake, suitably aligned addresses: nothing is dereferenced on the way to the refusal)
    na = lib.CsGemmArgs()
    na.A, na.W, na.C = 0x1000, 0x2000, 0x3000
    na.lda = na.ldw = 1280
    na.ldc = na.N = 3840
    na.M, na.K, na.epilogue = 256, 1240, lib.EPI_BIAS
    assert l.cs_gemm_rmsnorm_noalloc(ctypes.byref(na), None) == lib.CS_ERR_UNSUPPORTED      # K not a multiple of 64
    na.K, na.epilogue = 1280, lib.EPI_RESIDUAL
    assert l.cs_gemm_rmsnorm_noalloc(ctypes.byref(na), None) == lib.CS_ERR_UNSUPPORTED      # no folded form of it
    na.epilogue, na.M = lib.EPI_BIAS, 65537
    assert l.cs_gemm_rmsnorm_noalloc(ctypes.byref(na), None) == lib.CS_ERR_TOO_LARGE
    # a prefetch hint must start on a 16-byte boundary and carry a size (and no size without an address)
    pa = lib.CsGemmArgs()
    pa.A, pa.W, pa.C = 0x1000, 0x2000, 0x3000
    pa.lda = pa.ldw = pa.K = 1280
    pa.ldc = pa.N = 3840
    pa.M, pa.epilogue = 256, lib.EPI_BIAS
    pa.prefetch, pa.prefetch_bytes = 0x4008, 4096
    assert l.cs_gemm(ctypes.byref(pa), None) == lib.CS_ERR_INVALID_ARG
    pa.prefetch, pa.prefetch_bytes = 0x4000, -1
    assert l.cs_gemm(ctypes.byref(pa), None) == lib.CS_ERR_INVALID_ARG
    pa.prefetch, pa.prefetch_bytes = None, 4096
    assert l.cs_gemm(ctypes.byref(pa), None) == lib.CS_ERR_INVALID_ARG
    g = np.array([[1, 3, 4]], np.int64)  # odd height cannot be merged 2x2
    with pytest.raises(ValueError):
        ops.vit_seqlens_host(g, 2, 4)


def test_seqlens_host_matches_oracle_and_golden(golden_dir):
    golden = json.loads((golden_dir / "index_golden.json").read_text())
    for name, rec in golden.items():
        sl = ops.vit_seqlens_host(np.array(rec["grids"]), 2, 4)
        assert sl.cu_window.dtype == np.int32
        assert sl.cu_window.tolist() == rec["cu_window_seqlens"], name
        assert sl.cu_full.tolist() == rec["cu_seqlens"], name
        assert sl.total_patches == rec["pos_ids_shape"][0], name
    rng = np.random.default_rng(0)
    for _ in range(50):
        n = int(rng.integers(1, 6))
        grids = [(int(rng.integers(1, 4)), int(rng.integers(1, 50)) * 2, int(rng.integers(1, 50)) * 2) for _ in range(n)]
        sl = ops.vit_seqlens_host(np.array(grids), 2, 4)
        _, cu = vi.get_window_index(grids)
        assert sl.cu_window.tolist() == cu.tolist()
        assert sl.cu_full.tolist() == vi.full_cu_seqlens(grids).tolist()
        units = np.array([t * (h // 2) * (w // 2) for t, h, w in grids])
        assert sl.item_meta[:, 3].tolist() == np.concatenate([[0], np.cumsum(units)[:-1]]).tolist()


def test_empty_batch():
    sl = ops.vit_seqlens_host(np.zeros((0, 3), np.int64), 2, 4)
    assert sl.cu_window.tolist() == [0] and sl.cu_full.tolist() == [0] and sl.total_patches == 0


def test_attention_work_list_host():
    l = lib.load()
    assert l.cs_attn_block_q(64) == 64 and l.cs_attn_block_q(65) == 128
    cu = np.array([0, 64, 64 + 300, 64 + 300 + 128], np.int32)
    work = np.empty((16, 4), np.int32)
    n = ctypes.c_int32(0)
    assert l.cs_attn_work_host(cu.ctypes.data, 3, 128, work.ctypes.data, 16, ctypes.byref(n)) == 0
    w = work[: n.value]
    assert w.tolist() == [[0, 64, 0, 64], [64, 364, 64, 128], [64, 364, 192, 128], [64, 364, 320, 44], [364, 492, 364, 128]]
    # every query row is covered exactly once and stays inside its segment
    cover = np.zeros(cu[-1], int)
    for s, e, q0, nq in w:
        assert s <= q0 and q0 + nq <= e
        cover[q0 : q0 + nq] += 1
    assert (cover == 1).all()
    assert l.cs_attn_work_host(cu.ctypes.data, 3, 128, work.ctypes.data, 2, ctypes.byref(n)) == lib.CS_ERR_TOO_LARGE


def test_resize_taps_host_matches_the_oracle_bit_for_bit():
    """cs_resize_bicubic_taps_host is host arithmetic (doubles, then 22-bit fixed point): no GPU needed."""
    from oracle import qwen_preprocess as qp

    for a, b in [(4000, 1344), (3000, 1008), (100, 250), (37, 37), (5, 3), (3, 300), (1080, 1092), (299, 28), (1, 7), (7, 1),
                 (9000, 28)]:
        bounds, taps = ops.resize_bicubic_taps_host(a, b)
        rb, rt = qp.pillow_bicubic_taps(a, b)
        assert bounds.dtype == np.int32 and taps.dtype == np.int32
        assert np.array_equal(bounds, rb) and np.array_equal(taps, rt), (a, b)
    dll = lib.load()
    k = ctypes.c_int32(0)
    assert dll.cs_resize_bicubic_taps_host(0, 5, None, None, 0, ctypes.byref(k)) == lib.CS_ERR_INVALID_ARG
    assert dll.cs_resize_bicubic_taps_host(10, 5, None, None, 0, ctypes.byref(k)) == 0 and k.value == 9
    small = np.zeros((5, 4), dtype=np.int32)
    b = np.zeros((5, 2), dtype=np.int32)
    assert dll.cs_resize_bicubic_taps_host(10, 5, b.ctypes.data, small.ctypes.data, 4, ctypes.byref(k)) == lib.CS_ERR_INVALID_ARG
    assert dll.cs_resize_u8_pass(None, 1, 4, 4, 3, None, None, 5, None, None) == lib.CS_ERR_INVALID_ARG
