"""Per-kernel parity on a real MI355X, through the C ABI, against the oracle's pieces.

Bars: integer/byte/index work bit-exact; floating point within the tolerances written at each check
(bf16 outputs: one or two bf16 roundings of slack, i.e. max |err| <= 2^-7 relative to the row scale).
"""

import json

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gemma3 as og
from oracle import qwen2_5_vl as oq
from oracle import vit_index as vi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def ops():
    from cornserve_amd import ops as _ops

    return _ops


def close(got: torch.Tensor, ref: torch.Tensor, rel: float, what: str = ""):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert not torch.isnan(got).any(), what
    err = (got - ref).abs().max().item()
    scale = ref.abs().max().item() + 1e-12
    assert err <= rel * scale, f"{what}: max err {err:.4g} vs scale {scale:.4g} (rel {err / scale:.4g} > {rel})"


def rnd(shape, std=1.0, seed=0, dev="cpu"):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).bfloat16().to(dev)


# ------------------------------------------------------------------------------------------- index
def test_vit_index_bit_exact(ops, dev, golden_dir):
    golden = json.loads((golden_dir / "index_golden.json").read_text())
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, 40, 2, dtype=torch.float) / 40))).to(dev)
    cases = {k: v["grids"] for k, v in golden.items()}
    rng = np.random.default_rng(3)
    cases["random"] = [(int(rng.integers(1, 4)), int(rng.integers(1, 40)) * 2, int(rng.integers(1, 40)) * 2) for _ in range(7)]
    for name, grids in cases.items():
        g = np.array(grids, np.int64)
        sl = ops.vit_seqlens_host(g, 2, 4)
        ix = ops.vit_index(torch.from_numpy(sl.item_meta).to(dev), sl.total_patches, sl.max_units_per_item, 2, 4,
                           inv_freq, want_pos_ids=True)
        wi, cu = vi.get_window_index(grids)
        assert ix.window_index.dtype == torch.int64
        assert np.array_equal(ix.window_index.cpu().numpy(), wi), name
        assert np.array_equal(ix.reverse_index.cpu().numpy(), np.argsort(wi)), name
        assert np.array_equal(ix.pos_ids.cpu().numpy(), vi.rot_pos_ids(grids)), name
        src = (wi[:, None] * 4 + np.arange(4)[None, :]).reshape(-1)
        assert np.array_equal(ix.src_rows.cpu().numpy(), src), name
        # rotary table: window-ordered angles [h*f | w*f] -> cos | sin, fp32
        ocfg = oq.QwenVisionConfig()
        ang = oq.rot_pos_emb(ocfg, g).reshape(-1, 4, 40)[torch.from_numpy(wi)].reshape(-1, 40)
        ref = torch.cat([ang.cos(), ang.sin()], dim=-1)
        assert (ix.cos_sin.cpu() - ref).abs().max().item() <= 2e-6, name  # fp32 cos/sin, angles < 100 rad


def test_row_gather_bit_exact(ops, dev):
    x = rnd((1000, 1280), dev=dev)
    rows = torch.randperm(1000, generator=torch.Generator().manual_seed(0)).int().to(dev)
    assert torch.equal(ops.row_gather(x, rows), x[rows.long()])
    xf = torch.randn(333, 40, device=dev)  # fp32 rows of 160 bytes (the rotary table)
    rows = torch.randint(0, 333, (500,), device=dev).int()
    assert torch.equal(ops.row_gather(xf, rows), xf[rows.long()])
    assert ops.row_gather(x, rows[:0]).shape == (0, 1280)


def test_cast_bit_exact(ops, dev):
    for n in (0, 1, 7, 8, 1176 * 333, 100003):
        x = torch.randn(n, device=dev) * 3
        assert torch.equal(ops.cast_f32_bf16(x), x.bfloat16())


def test_patchify_bit_exact(ops, dev):
    px = rnd((2, 3, 56, 84), dev=dev)
    got = ops.patchify_nchw(px, 14, 592)
    ref = px.view(2, 3, 4, 14, 6, 14).permute(0, 2, 4, 1, 3, 5).reshape(48, 588)
    assert torch.equal(got[:, :588], ref) and (got[:, 588:] == 0).all()


# ------------------------------------------------------------------------------------------- norms
@pytest.mark.parametrize("t,h,w,patch,merge,temporal", [
    (1, 448, 448, 14, 2, 2),    # one image of the benchmark's size
    (1, 28, 1344, 14, 2, 2),    # one block row
    (8, 336, 588, 14, 2, 2),    # config-5 style video
    (5, 56, 84, 14, 2, 2),      # odd frame count: the last frame fills the last group
    (7, 24, 36, 2, 3, 3),       # other patch / merge / temporal sizes
    (3, 64, 96, 16, 2, 2),      # patch 16
    (9, 28, 56, 14, 1, 3),      # patch 14 with another merge / temporal size
    (20, 28, 28, 14, 2, 10),    # temporal size beyond what the segment form stages: per-value form
])
def test_qwen_patchify_u8_bit_exact(ops, dev, t, h, w, patch, merge, temporal):
    from cornserve_amd.eric import frames as fr
    from oracle import qwen_preprocess as qp

    frames = np.random.default_rng(t * 1000 + h + w).integers(0, 256, (t, h, w, 3), dtype=np.uint8)
    for arithmetic in ("fused", "numpy"):
        table = fr.byte_table(arithmetic=arithmetic)
        ref, grid = qp.patchify_frames(frames, qp.normalization_table(arithmetic=arithmetic), patch, merge, temporal)
        got32 = ops.qwen_patchify_u8(torch.from_numpy(frames).to(dev), table.to(dev), patch, merge, temporal, dtype=torch.float32)
        assert got32.shape == ref.shape == (grid[0] * grid[1] * grid[2], 3 * temporal * patch * patch)
        assert np.array_equal(got32.cpu().numpy(), ref)
        got16 = ops.qwen_patchify_u8(torch.from_numpy(frames).to(dev), table.to(dev), patch, merge, temporal)
        assert torch.equal(got16.cpu(), torch.from_numpy(ref).bfloat16())   # the reference's .to(dtype), :415-419
    with pytest.raises(ValueError):
        ops.qwen_patchify_u8(torch.zeros((1, 30, 28, 3), dtype=torch.uint8, device=dev), table.to(dev), 14, 2, 2)


@pytest.mark.parametrize("heads,d", [(16, 80), (4, 64), (2, 96), (3, 80)])
def test_attn_rotary_in_place_route_equals_fused_route(ops, dev, heads, d):
    """Long segments: rotating the keys in place and the query rows while they are staged (or, for head shapes without
    that kernel, q and k in place) gives the bits of the kernel that rotates everything while staging (ragged segment
    lengths either side of the tile sizes)."""
    lens = [100, 1024, 65, 300, 128, 1, 777]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    L, E = int(cu[-1]), heads * d
    g = torch.Generator().manual_seed(heads * 100 + d)
    qkv = torch.randn((L, 3 * E), generator=g).bfloat16().to(dev)
    ang = torch.rand((L, d // 2), generator=g) * 6.2831853
    cs = torch.cat([ang.cos(), ang.sin()], dim=1).float().to(dev).contiguous()
    plan = ops.attn_plan(cu, dev)
    fused = ops.attn_varlen(qkv[:, :E], qkv[:, E:2 * E], qkv[:, 2 * E:], plan, heads, d, d ** -0.5, cos_sin=cs)
    buf = qkv.clone()
    got = ops.attn_varlen_rotary_(buf, plan, heads, d, d ** -0.5, cs)
    assert torch.equal(got, fused)
    # k rotated in place, v untouched; q only where the keys-rotated kernel does not apply (odd head count)
    assert not torch.equal(buf[:, E:2 * E], qkv[:, E:2 * E]) and torch.equal(buf[:, 2 * E:], qkv[:, 2 * E:])
    assert torch.equal(buf[:, :E], qkv[:, :E]) == (heads % 2 == 0)
    rot = qkv.clone()
    ops.rope_qk_(rot, cs, heads, d)
    assert torch.equal(buf[:, E:2 * E], rot[:, E:2 * E])   # the k block rotated as two half-size tensors = rotated as one
    short = ops.attn_plan(np.arange(0, 64 * 5 + 1, 64, dtype=np.int32), dev)   # window route: the buffer stays as it is
    buf = qkv[:320].clone()
    got = ops.attn_varlen_rotary_(buf, short, heads, d, d ** -0.5, cs[:320].contiguous())
    ref = ops.attn_varlen(qkv[:320, :E], qkv[:320, E:2 * E], qkv[:320, 2 * E:], short, heads, d, d ** -0.5, cos_sin=cs[:320].contiguous())
    assert torch.equal(got, ref) and torch.equal(buf, qkv[:320])


def test_resize_bicubic_u8_bit_exact(ops, dev):
    """GPU resize against the oracle's restatement of Pillow's bicubic (itself pinned against the package on the CPU)
    and, where the package is importable, against the package directly: random, black/white (clamping) and smooth
    frames; up- and down-scaling; one axis unchanged; both axes unchanged (returned as is); rows whose byte count is
    not a multiple of 4 (the byte-wise form of the pass); frames that do not start at a 4-byte boundary; along x every
    tap-count class of the staged kernel, several tiles of 256 positions, row groups with a remainder, and windows too
    wide for it (the general kernel)."""
    from oracle import qwen_preprocess as qp

    rng = np.random.default_rng(3)
    cases = [(1, 97, 64, 56, 140), (2, 600, 450, 196, 140), (1, 30, 45, 112, 168), (3, 37, 53, 37, 84), (1, 64, 64, 28, 64),
             (1, 33, 35, 31, 29), (1, 1080, 1920, 588, 1036), (1, 5, 7, 56, 56), (1, 1500, 20, 28, 28), (2, 40, 2100, 56, 28),
             (1, 19, 3000, 28, 420), (17, 50, 1300, 28, 300), (1, 64, 300, 64, 1100)]
    for i, (t, h, w, oh, ow) in enumerate(cases):
        if i % 3 == 1:
            frames = (rng.integers(0, 2, (t, h, w, 3)) * 255).astype(np.uint8)
        elif i % 3 == 2:
            frames = np.clip(np.cumsum(rng.integers(-9, 10, (t, h, w, 3)), axis=2) + 128, 0, 255).astype(np.uint8)
        else:
            frames = rng.integers(0, 256, (t, h, w, 3), dtype=np.uint8)
        ref = qp.pillow_bicubic_resize(frames, oh, ow)
        got = ops.resize_bicubic_u8(torch.from_numpy(frames).to(dev), oh, ow)
        assert got.shape == (t, oh, ow, 3) and got.dtype == torch.uint8
        assert np.array_equal(got.cpu().numpy(), ref), (t, h, w, oh, ow)
    try:
        from PIL import Image
    except ImportError:
        Image = None
    frames = rng.integers(0, 256, (1, 301, 517, 3), dtype=np.uint8)
    dbuf = torch.empty((frames.size + 3,), dtype=torch.uint8, device=dev)
    dbuf[3:] = torch.from_numpy(frames).to(dev).reshape(-1)
    got = ops.resize_bicubic_u8(dbuf[3:].view(1, 301, 517, 3), 308, 504).cpu().numpy()
    assert np.array_equal(got, qp.pillow_bicubic_resize(frames, 308, 504))
    if Image is not None:
        assert np.array_equal(got[0], np.asarray(Image.fromarray(frames[0]).resize((504, 308), resample=Image.Resampling.BICUBIC)))
    same = torch.from_numpy(frames).to(dev)
    assert ops.resize_bicubic_u8(same, 301, 517) is same
    grey = torch.from_numpy(frames[..., :1].copy()).to(dev)   # one channel: the pass takes any inner size
    assert np.array_equal(ops.resize_bicubic_u8(grey, 100, 90).cpu().numpy(), qp.pillow_bicubic_resize(frames[..., :1], 100, 90))
    with pytest.raises(ValueError):
        ops.resize_bicubic_u8(same[0], 28, 28)
    with pytest.raises(ValueError):
        ops.resize_bicubic_u8(same, 0, 28)
    with pytest.raises(ValueError):
        ops.resize_bicubic_u8(same.float(), 28, 28)


@pytest.mark.parametrize("patch", [14, 16])
def test_qwen_patchify_u8_unaligned_frames(ops, dev, patch):
    """Frames that start at any byte offset of a 4-byte word (a view into a larger buffer), last frame at the very end
    of the buffer."""
    from cornserve_amd.eric import frames as fr
    from oracle import qwen_preprocess as qp

    t, h, w = 3, 2 * patch * 2, 3 * patch * 2
    table = fr.byte_table(arithmetic="numpy")
    n = t * h * w * 3
    for lead in range(4):
        buf = np.random.default_rng(100 + lead).integers(0, 256, lead + n, dtype=np.uint8)
        frames = buf[lead:].reshape(t, h, w, 3)
        ref, _ = qp.patchify_frames(frames, qp.normalization_table(arithmetic="numpy"), patch, 2, 2)
        dbuf = torch.from_numpy(buf).to(dev)
        got = ops.qwen_patchify_u8(dbuf[lead:].view(t, h, w, 3), table.to(dev), patch, 2, 2, dtype=torch.float32)
        assert np.array_equal(got.cpu().numpy(), ref), lead


@pytest.mark.parametrize("rows,H", [(1, 1280), (1023, 1280), (64, 1152), (5, 64), (7, 5120)])
def test_rmsnorm(ops, dev, rows, H):
    x = rnd((rows, H), 2.0, 1, dev)
    w = (1 + 0.02 * torch.randn(H)).bfloat16().to(dev)
    ref = oq.rms_norm(x.cpu(), w.cpu(), 1e-6)
    close(ops.rmsnorm(x, w, 1e-6), ref, 2**-7, "rmsnorm")
    refg = og.gemma_rms_norm(x.cpu(), w.cpu(), 1e-6)
    close(ops.rmsnorm(x, w, 1e-6, gemma=True), refg, 2**-7, "gemma rmsnorm")


def test_rmsnorm_special_cases(ops, dev):
    x = torch.full((3, 1280), 3.0, dtype=torch.bfloat16, device=dev)
    w = torch.arange(1280, dtype=torch.float).bfloat16().to(dev)
    assert torch.equal(ops.rmsnorm(x, w, 0.0), w.expand(3, 1280))  # constant row -> exactly w


@pytest.mark.parametrize("rows,H", [(1, 1152), (777, 1152), (9, 1280)])
def test_layernorm(ops, dev, rows, H):
    x = rnd((rows, H), 2.0, 2, dev)
    w = (1 + 0.02 * torch.randn(H)).bfloat16().to(dev)
    b = (0.02 * torch.randn(H)).bfloat16().to(dev)
    ref = F.layer_norm(x.float().cpu(), (H,), w.float().cpu(), b.float().cpu(), 1e-6)
    close(ops.layernorm(x, w, b, 1e-6), ref, 2**-7, "layernorm")


def test_avgpool_gemma_rmsnorm(ops, dev):
    cfg = og.SiglipConfig(image_size=224, mm_tokens_per_image=16)
    x = rnd((2, 256, 1152), 1.0, 3, dev)
    w = (0.1 * torch.randn(1152)).bfloat16().to(dev)
    got = ops.avgpool_gemma_rmsnorm(x, w, 16, 4, 1e-6)
    xc = x.cpu()
    pooled = F.avg_pool2d(xc.transpose(1, 2).reshape(2, 1152, 16, 16), 4).flatten(2).transpose(1, 2)
    ref = og.gemma_rms_norm(pooled, w.cpu(), cfg.layer_norm_eps)
    close(got, ref, 2**-7, "avgpool+gemma rmsnorm")


# -------------------------------------------------------------------------------------------- GEMM
def lin_ref(a, w, bias):
    return a.float().cpu() @ w.float().cpu().t() + (bias.float().cpu() if bias is not None else 0.0)


@pytest.mark.parametrize("M,N,K", [(1, 1280, 1280), (255, 256, 64), (257, 260, 72), (1000, 1280, 1176),
                                   (300, 1152, 4304), (2048, 3840, 1280), (64, 3584, 5120), (130, 2560, 1152)])
def test_gemm_bias(ops, dev, M, N, K):
    a, w, b = rnd((M, K), 1.0, 1, dev), rnd((N, K), 0.02, 2, dev), rnd((N,), 0.02, 3, dev)
    close(ops.gemm(a, w, b), lin_ref(a, w, b), 2**-7, f"gemm {M}x{N}x{K}")
    close(ops.gemm(a, w, None), lin_ref(a, w, None), 2**-7, f"gemm nobias {M}x{N}x{K}")


def test_gemm_exact_small_integers(ops, dev):
    # products and sums of small integers are exact in bf16/fp32: any indexing mistake shows up bit-exactly
    g = torch.Generator().manual_seed(0)
    a = torch.randint(-3, 4, (300, 136), generator=g).bfloat16().to(dev)
    w = torch.randint(-3, 4, (200, 136), generator=g).bfloat16().to(dev)
    ref = (a.float() @ w.float().t())
    assert ref.abs().max() < 256  # representable in bf16
    assert torch.equal(ops.gemm(a, w, None).float(), ref)


def test_gemm_epilogues(ops, dev):
    M, N, K = 515, 1280, 1280
    a, w, b = rnd((M, K), 1.0, 1, dev), rnd((N, K), 0.05, 2, dev), rnd((N,), 0.02, 3, dev)
    res = rnd((M, N), 1.0, 4, dev)
    exact = lin_ref(a, w, b)
    base = exact.bfloat16().float()
    close(ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=res), base + res.float().cpu(), 2**-7, "residual")
    close(ops.gemm(a, w, b, epilogue=ops.EPI_GELU_ERF), F.gelu(exact), 2**-7, "gelu erf")
    close(ops.gemm(a, w, b, epilogue=ops.EPI_GELU_TANH), F.gelu(exact, approximate="tanh"), 2**-7, "gelu tanh")
    close(ops.gemm(a, w, b, epilogue=ops.EPI_QUICK_GELU), exact * torch.sigmoid(1.702 * exact), 2**-7, "quick gelu")
    # the general kernel's copy of the same epilogue (K = 72 is not a shape the fast kernel takes)
    a72, w72 = a[:, :72].contiguous(), w[:, :72].contiguous()
    base72 = lin_ref(a72, w72, b)
    close(ops.gemm(a72, w72, b, epilogue=ops.EPI_QUICK_GELU), base72 * torch.sigmoid(1.702 * base72), 2**-7, "quick gelu, general kernel")
    gate, up = exact[:, 0::2], exact[:, 1::2]
    close(ops.gemm(a, w, b, epilogue=ops.EPI_SWIGLU), F.silu(gate) * up, 2**-7, "swiglu")
    # in-place residual (out aliases residual), as the model uses it
    x = res.clone()
    ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=x, out=x)
    close(x, base + res.float().cpu(), 2**-7, "residual in place")
    pos = rnd((103, N), 1.0, 5, dev)
    idx = torch.arange(M) % 103
    close(ops.gemm(a, w, b, pos=pos), base + pos.float().cpu()[idx], 2**-7, "pos")


def test_both_gemm_kernels_round_their_epilogues_alike(ops, dev):
    """The direct-to-LDS kernel and the general kernel accumulate in different orders, so on random data their fp32
    sums differ in the last bits; on operands whose products and sums are exact (small integers over 8) the sums are
    equal, and then every fused epilogue -- SwiGLU included -- must give the same bits in either kernel: same rounding
    points, same activation code.  K = 192 takes the fast kernel; the same matrices with 8 zero columns appended
    (K = 200, a K tail) take the general one."""
    g = torch.Generator().manual_seed(5)
    M, N, K = 300, 512, 192
    a = torch.randint(-3, 4, (M, K), generator=g).bfloat16()
    w = (torch.randint(-3, 4, (N, K), generator=g).float() / 8).bfloat16()
    b = (torch.randint(-8, 9, (N,), generator=g).float() / 8).bfloat16().to(dev)
    res = (torch.randint(-64, 65, (M, N), generator=g).float() / 8).bfloat16().to(dev)
    pad = lambda t: torch.cat([t, torch.zeros((t.shape[0], 8), dtype=t.dtype)], dim=1).contiguous().to(dev)  # noqa: E731
    a_f, w_f, a_g, w_g = a.to(dev), w.to(dev), pad(a), pad(w)
    for epi in (ops.EPI_BIAS, ops.EPI_RESIDUAL, ops.EPI_SWIGLU, ops.EPI_GELU_ERF, ops.EPI_GELU_TANH, ops.EPI_QUICK_GELU):
        kw = dict(epilogue=epi, residual=res if epi == ops.EPI_RESIDUAL else None)
        fast, general = ops.gemm(a_f, w_f, b, **kw), ops.gemm(a_g, w_g, b, **kw)
        assert torch.equal(fast, general), f"epilogue {epi}"
    lo = torch.randint(0, 256, (M, N), generator=g, dtype=torch.uint8).to(dev)
    outs = []
    for aa, ww in ((a_f, w_f), (a_g, w_g)):
        o, ol = torch.empty_like(res), torch.empty_like(lo)
        ops.gemm(aa, ww, b, epilogue=ops.EPI_RESIDUAL, residual=res, residual_lo=lo, out=o, out_lo=ol)
        outs.append((o, ol))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


def test_kernels_are_registered_torch_operators(ops, dev):
    """Every kernel entry point is an operator of the `cornserve_amd` namespace with a schema that names what it
    mutates and a fake implementation (shape propagation without running a kernel); `torch.library.opcheck` checks both
    against real launches.  The front ends of `cornserve_amd.ops` dispatch through these operators."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    M, N, K, heads, d = 130, 256, 192, 2, 64
    a, w, b = rnd((M, K), 1.0, 1, dev), rnd((N, K), 0.05, 2, dev), rnd((N,), 0.02, 3, dev)
    res = rnd((M, N), 1.0, 4, dev)
    none14 = (None,) * 5
    functional = (a, w, b, ops.EPI_SWIGLU, None, None, None, None, None, None, None, 0.0, None, None)
    assert torch.equal(torch.ops.cornserve_amd.gemm(*functional), ops.gemm(a, w, b, epilogue=ops.EPI_SWIGLU))
    tests = ("test_schema", "test_faketensor")
    torch.library.opcheck(torch.ops.cornserve_amd.gemm.default, functional, test_utils=tests)
    ss = torch.zeros((M, 8), dtype=torch.float32, device=dev)
    lo = torch.zeros((M, N), dtype=torch.uint8, device=dev)
    inplace = (torch.empty_like(res), a, w, b, ops.EPI_RESIDUAL, res, None, None, None, None, None, None, ss, 0.0, None,
               None, None, lo.clone(), lo)
    torch.library.opcheck(torch.ops.cornserve_amd.gemm_.default, inplace, test_utils=tests)
    torch.library.opcheck(torch.ops.cornserve_amd.rmsnorm_.default, (torch.empty_like(a), a, rnd((K,), 1.0, 5, dev), 1e-6, False),
                          test_utils=tests)
    qkv = rnd((M, 3 * heads * d), 1.0, 6, dev)
    plan = ops.attn_plan(np.array([0, 70, M], np.int32), dev)
    E = heads * d
    torch.library.opcheck(torch.ops.cornserve_amd.attn_varlen_.default,
                          (torch.empty((M, E), dtype=torch.bfloat16, device=dev), qkv[:, :E], qkv[:, E:2 * E], qkv[:, 2 * E:],
                           plan.work, plan.n_work, plan.max_seqlen, heads, d, d ** -0.5, None, False), test_utils=tests)
    with FakeTensorMode():     # shapes propagate without a device launch
        fa = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
        fw = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
        out = torch.ops.cornserve_amd.gemm(fa, fw, None, ops.EPI_SWIGLU, *none14, None, None, 0.0, None, None)
        assert tuple(out.shape) == (M, N // 2) and out.dtype == torch.bfloat16
    for name in ("gemm", "gemm_", "attn_varlen_", "rmsnorm_", "layernorm_", "rope_qk_", "row_stats_", "vit_index_",
                 "row_gather_", "patchify_nchw_", "qwen_patchify_u8_", "avgpool_gemma_rmsnorm_", "rows_bilinear_",
                 "pos_embed_interp_", "cast_f32_bf16_"):
        assert hasattr(torch.ops.cornserve_amd, name), name


def _epilogue_ref(ops, epi, base, res):
    """fp32 reference of one fused epilogue on `base` = A.W^T + bias in fp32.  The residual epilogue rounds the linear
    layer's output before the addition (the reference's two bf16 operations); an activation takes the fp32 sum."""
    if epi == ops.EPI_BIAS:
        return base
    if epi == ops.EPI_RESIDUAL:
        return base.bfloat16().float() + res.float().cpu()
    if epi == ops.EPI_GELU_ERF:
        return F.gelu(base)
    if epi == ops.EPI_GELU_TANH:
        return F.gelu(base, approximate="tanh")
    if epi == ops.EPI_QUICK_GELU:
        return base * torch.sigmoid(1.702 * base)
    gate, up = base[:, 0::2], base[:, 1::2]
    return F.silu(gate) * up


# Shapes that reach every tile form and every schedule of the fast kernel: the 256x256 five-unit ring, the
# 256x160 / 256x128 / 128x192 three-stage rings (N = 1280; remainders of a column split), the shortest K the
# fast path takes (3 K tiles: the ring's tail iterations only) and 4, 5, 7 K tiles, row and column tails.
@pytest.mark.parametrize("M,N,K", [
    (8192, 3072, 192),    # 8 columns of 256x256 + 1024 columns of 256x128, 3 K tiles
    (8192, 2304, 256),    # 8 columns of 256x256 + 256 columns of 128x192, 4 K tiles
    (1000, 1280, 320),    # 256x160, row tail, 5 K tiles
    (300, 520, 448),      # 256x256 with row and column tails, 7 K tiles
    (8192, 1280, 192),    # 256x160, one tile per CU, 3 K tiles
    (1000, 6912, 256),    # few rows, many columns: the SwiGLU epilogue takes 256x128 over the whole width (216 workgroups)
    (2048, 3840, 192),    # 256x160 in one round of 192 workgroups
])
def test_gemm_fast_path_forms(ops, dev, M, N, K):
    a, w, b = rnd((M, K), 1.0, 11, dev), rnd((N, K), 0.05, 12, dev), rnd((N,), 0.02, 13, dev)
    res = rnd((M, N), 1.0, 14, dev)
    rows = torch.arange(0, M, max(1, M // 257))  # a sample of rows: the fp32 reference runs on the host
    rows = torch.cat([rows, torch.tensor([M - 1])])
    base = lin_ref(a[rows], w, b)
    for epi in (ops.EPI_BIAS, ops.EPI_RESIDUAL, ops.EPI_GELU_ERF, ops.EPI_GELU_TANH, ops.EPI_QUICK_GELU, ops.EPI_SWIGLU):
        got = ops.gemm(a, w, b, epilogue=epi, residual=res if epi == ops.EPI_RESIDUAL else None)
        close(got[rows], _epilogue_ref(ops, epi, base, res[rows]), 2**-7, f"{M}x{N}x{K} epilogue {epi}")
    # repeated launches give identical bits (fixed accumulation order, no races between the two launches of
    # a column split or between consecutive tiles of a persistent workgroup)
    first = ops.gemm(a, w, b)
    for _ in range(3):
        assert torch.equal(ops.gemm(a, w, b), first)
    # the tile form follows the row count; an output element's bits do not (same accumulation order in every form)
    for lo, hi in ((0, min(M, 256)), (M // 2, min(M, M // 2 + 100))):
        assert torch.equal(ops.gemm(a[lo:hi], w, b), first[lo:hi]), (lo, hi)
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(2)).int().to(dev)
    scat = ops.gemm(a, w, b, c_rows=perm)
    ref = torch.empty_like(first)
    ref[perm.long()] = first
    assert torch.equal(scat, ref)


def test_gemm_prefetch_hint_leaves_the_result_alone(ops, dev):
    """A launch with few tiles and a `prefetch` tensor starts extra workgroups that only read that tensor: the product
    has the bits it has without the hint, whatever the hinted size (odd, shorter than one 16-byte piece, many MB), on
    every tile form, and a launch that fills the chip ignores the hint."""
    hints = [torch.zeros(n, dtype=torch.uint8, device=dev) for n in (8, 16, 1000003, 24 << 20)]
    hints.append(rnd((3420, 1280), 0.05, 5, dev))
    for M, N, K in [(1000, 1280, 320), (300, 520, 448), (2100, 1280, 192), (8192, 1280, 192), (700, 2304, 256)]:
        a, w, b = rnd((M, K), 1.0, 11, dev), rnd((N, K), 0.05, 12, dev), rnd((N,), 0.02, 13, dev)
        res = rnd((M, N), 1.0, 14, dev)
        plain = ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=res)
        ss0 = torch.zeros((M, ops.SUMSQ_PARTS), device=dev) if N <= 1280 else None   # (parts past N's are not written)
        plain_ss = ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=res, c_row_sumsq=ss0) if ss0 is not None else None
        for h in hints:
            assert torch.equal(ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=res, prefetch=h), plain), (M, N, K, h.shape)
            if ss0 is not None:
                ss1 = torch.zeros_like(ss0)
                got = ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=res, c_row_sumsq=ss1, prefetch=h)
                assert torch.equal(got, plain_ss) and torch.equal(ss1, ss0)
    # fp8 weights (their own tile forms)
    a, b = rnd((520, 448), 1.0, 21, dev), rnd((640,), 0.02, 23, dev)
    wq = torch.randn(640, 448, generator=torch.Generator().manual_seed(22)) * 0.05
    sc = wq.abs().amax(dim=1) / 448.0
    q, sc = (wq / sc[:, None]).to(torch.float8_e4m3fn).to(dev), sc.to(dev)
    assert torch.equal(ops.gemm(a, q, b, w_scale=sc, prefetch=hints[2]), ops.gemm(a, q, b, w_scale=sc))
    # the hint has to be readable device memory in whole 16-byte pieces from its start
    with pytest.raises(ValueError):
        ops.gemm(a, q, b, w_scale=sc, prefetch=hints[2][1:])
    with pytest.raises(ValueError):
        ops.gemm(a, q, b, w_scale=sc, prefetch=hints[4][:, :64])
    with pytest.raises((ValueError, RuntimeError)):
        ops.gemm(a, q, b, w_scale=sc, prefetch=torch.zeros(64))


@pytest.mark.parametrize("M,N,K", [
    (8192, 3072, 192),    # 256x256 (three-stage ring with byte-wide W tiles) + 256x128 remainder, 3 K tiles
    (8192, 2304, 256),    # 256x256 + 128x192 remainder
    (1000, 1280, 320),    # 256x160: 10 W row blocks over 4 waves (two waves repeat the last block)
    (300, 520, 448),      # row and column tails
])
def test_gemm_fast_path_forms_fp8_weights(ops, dev, M, N, K):
    a, b = rnd((M, K), 1.0, 21, dev), rnd((N,), 0.02, 23, dev)
    res = rnd((M, N), 1.0, 24, dev)
    w = torch.randn(N, K, generator=torch.Generator().manual_seed(22)) * 0.05
    scale = w.abs().amax(dim=1) / 448.0
    q = (w / scale[:, None]).to(torch.float8_e4m3fn)
    wd = q.float() * scale[:, None]          # de-quantised fp32 weights: the comparator of the fp8 path
    rows = torch.cat([torch.arange(0, M, max(1, M // 257)), torch.tensor([M - 1])])
    base = a[rows].float().cpu() @ wd.t() + b.float().cpu()
    qd, sd = q.to(dev), scale.to(dev)
    for epi in (ops.EPI_BIAS, ops.EPI_RESIDUAL, ops.EPI_GELU_ERF, ops.EPI_GELU_TANH, ops.EPI_QUICK_GELU, ops.EPI_SWIGLU):
        got = ops.gemm(a, qd, b, w_scale=sd, epilogue=epi, residual=res if epi == ops.EPI_RESIDUAL else None)
        close(got[rows], _epilogue_ref(ops, epi, base, res[rows]), 2**-7, f"fp8 {M}x{N}x{K} epilogue {epi}")
    first = ops.gemm(a, qd, b, w_scale=sd)
    assert torch.equal(ops.gemm(a, qd, b, w_scale=sd), first)


def _sumsq_parts_ref(x: torch.Tensor) -> torch.Tensor:
    """fp32 [rows, 8]: sums of squares of 160-column blocks of x (zero where x has no such columns)."""
    rows, H = x.shape
    pad = torch.zeros((rows, 1280), dtype=torch.float32)
    pad[:, :H] = x.float().cpu()
    return (pad * pad).view(rows, 8, 160).sum(-1)


@pytest.mark.parametrize("rows,H", [(1, 1280), (1000, 1280), (77, 1152), (5, 64), (3, 160)])
def test_row_sumsq(ops, dev, rows, H):
    x = rnd((rows, H), 2.0, 31, dev)
    got = ops.row_sumsq(x)
    ref = _sumsq_parts_ref(x)
    assert got.shape == (rows, 8) and got.dtype == torch.float32
    torch.testing.assert_close(got.cpu(), ref, rtol=1e-5, atol=1e-6)
    assert (got.cpu()[:, (H + 159) // 160:] == 0).all()
    with pytest.raises(RuntimeError):
        ops.row_sumsq(rnd((4, 1288), 1.0, 1, dev))


# RMSNorm folded into the GEMMs on both sides of it: the producer (residual epilogue) emits the sums of squares
# of the rows it writes, the consumer scales its accumulators by rsqrt(mean square + eps).
@pytest.mark.parametrize("M,N,K", [(8192, 1280, 192), (1000, 1280, 320), (300, 1152, 448), (257, 168, 192)])
def test_gemm_emits_row_sums_of_squares(ops, dev, M, N, K):
    a, w, b = rnd((M, K), 1.0, 41, dev), rnd((N, K), 0.05, 42, dev), rnd((N,), 0.02, 43, dev)
    res = rnd((M, N), 1.0, 44, dev)
    for epi in (ops.EPI_RESIDUAL, ops.EPI_BIAS):
        kw = dict(epilogue=epi, residual=res if epi == ops.EPI_RESIDUAL else None)
        plain = ops.gemm(a, w, b, **kw)
        ss = torch.full((M, 8), 7.0, dtype=torch.float32, device=dev)
        got = ops.gemm(a, w, b, c_row_sumsq=ss, **kw)
        assert torch.equal(got, plain)                       # C itself is unchanged by the extra output
        ref = _sumsq_parts_ref(plain)                        # ... and the sums are those of the ROUNDED outputs
        parts = (N + 159) // 160
        torch.testing.assert_close(ss.cpu()[:, :parts], ref[:, :parts], rtol=1e-5, atol=1e-6)
        assert (ss.cpu()[:, parts:] == 7.0).all()            # parts beyond N are left to the caller
        ss2 = torch.zeros_like(ss)
        ops.gemm(a, w, b, c_row_sumsq=ss2, **kw)
        assert torch.equal(ss2[:, :parts], ss[:, :parts])    # fixed summation order: identical bits
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(3)).int().to(dev)
    ss = torch.zeros((M, 8), dtype=torch.float32, device=dev)
    scat = ops.gemm(a, w, b, c_rows=perm, c_row_sumsq=ss)
    torch.testing.assert_close(ss.cpu(), _sumsq_parts_ref(scat), rtol=1e-5, atol=1e-6)   # indexed by output row


@pytest.mark.parametrize("M,N,K", [(8192, 3072, 192), (8192, 2304, 256), (1000, 1280, 320), (300, 520, 448)])
def test_gemm_with_folded_rmsnorm(ops, dev, M, N, K):
    eps = 1e-6
    a, w, b = rnd((M, K), 3.0, 51, dev), rnd((N, K), 0.05, 52, dev), rnd((N,), 0.02, 53, dev)
    g = (1.0 + rnd((K,), 0.1, 54)).bfloat16()                           # the norm's weight
    wf = (w.float().cpu() * g.float()[None, :]).bfloat16().to(dev)     # folded into W's columns
    ss = ops.row_sumsq(a)
    rows = torch.cat([torch.arange(0, M, max(1, M // 257)), torch.tensor([M - 1])])
    af = a[rows].float().cpu()
    rstd = torch.rsqrt((af * af).mean(-1, keepdim=True) + eps)
    # closed form of the fused op in fp32 ...
    base = (af @ wf.float().cpu().t()) * rstd + b.float().cpu()
    # ... and the unfused reference sequence (norm.py:35-70 then F.linear): cast, multiply by the weight, cast
    n_ref = ((af * rstd).bfloat16().float() * g.float()).bfloat16()
    base_unfused = lin_ref(n_ref, w, b)
    for epi in (ops.EPI_BIAS, ops.EPI_SWIGLU):
        if epi == ops.EPI_SWIGLU and (N // 2) % 8:   # output rows the fast kernel's 16-byte stores cannot take
            with pytest.raises(RuntimeError):
                ops.gemm(a, wf, b, epilogue=epi, a_row_sumsq=ss, norm_eps=eps)
            continue
        got = ops.gemm(a, wf, b, epilogue=epi, a_row_sumsq=ss, norm_eps=eps)
        close(got[rows], _epilogue_ref(ops, epi, base, None), 2**-7, f"folded norm {M}x{N}x{K} epilogue {epi}")
        close(got[rows], _epilogue_ref(ops, epi, base_unfused, None), 2**-6, f"folded vs unfused {M}x{N}x{K} epilogue {epi}")
    # against the library's own unfused pair
    unfused = ops.gemm(ops.rmsnorm(a, g.to(dev), eps), w, b)
    close(ops.gemm(a, wf, b, a_row_sumsq=ss, norm_eps=eps), unfused.float().cpu(), 2**-6, "folded vs rmsnorm + gemm")
    # combinations that do not exist are refused, not silently computed without the norm
    with pytest.raises(RuntimeError):
        ops.gemm(a, wf, b, epilogue=ops.EPI_GELU_ERF, a_row_sumsq=ss, norm_eps=eps)
    with pytest.raises(RuntimeError):
        ops.gemm(a[:, :72].contiguous(), wf[:, :72].contiguous(), b, a_row_sumsq=ss, norm_eps=eps)   # K the fast kernel does not take


@pytest.mark.parametrize("M,N,K", [(8192, 3456, 1152), (1000, 1280, 320), (300, 520, 448)])
def test_gemm_with_folded_layernorm(ops, dev, M, N, K):
    eps = 1e-6
    a = (rnd((M, K), 2.0, 71).float() + 0.7).bfloat16().to(dev)          # rows with a non-zero mean
    w, b = rnd((N, K), 0.05, 72, dev), rnd((N,), 0.02, 73, dev)
    g, beta = (1.0 + rnd((K,), 0.1, 74)).bfloat16(), rnd((K,), 0.1, 75)
    wf = (w.float().cpu() * g.float()[None, :]).bfloat16()                # norm weight folded into W's columns
    bf = (b.float().cpu() + w.float().cpu() @ beta.float()).bfloat16()    # norm bias folded into the GEMM bias
    csum = wf.float().sum(dim=1).contiguous()
    ss = torch.empty((M, 8), dtype=torch.float32, device=dev)
    sm = torch.empty_like(ss)
    ops.row_stats(a, ss, sm)
    torch.testing.assert_close(sm.cpu().sum(1), a.float().cpu().sum(1), rtol=1e-5, atol=1e-3)
    rows = torch.cat([torch.arange(0, M, max(1, M // 257)), torch.tensor([M - 1])])
    af = a[rows].float().cpu()
    n_ref = F.layer_norm(af, (K,), g.float(), beta.float(), eps).bfloat16()     # the unfused reference sequence
    base = lin_ref(n_ref, w, b)
    for epi in (ops.EPI_BIAS, ops.EPI_GELU_TANH, ops.EPI_QUICK_GELU):
        got = ops.gemm(a, wf.to(dev), bf.to(dev), epilogue=epi, a_row_sumsq=ss, a_row_sum=sm, w_col_sum=csum.to(dev), norm_eps=eps)
        close(got[rows], _epilogue_ref(ops, epi, base, None), 2**-6, f"folded LayerNorm {M}x{N}x{K} epilogue {epi}")
    unfused = ops.gemm(ops.layernorm(a, g.to(dev), beta.bfloat16().to(dev), eps), w, b)
    fused = ops.gemm(a, wf.to(dev), bf.to(dev), a_row_sumsq=ss, a_row_sum=sm, w_col_sum=csum.to(dev), norm_eps=eps)
    close(fused, unfused.float().cpu(), 2**-6, "folded vs layernorm + gemm")
    with pytest.raises(RuntimeError):      # the mean term needs the column sums
        ops.gemm(a, wf.to(dev), bf.to(dev), a_row_sumsq=ss, a_row_sum=sm, norm_eps=eps)
    # producer side: a residual GEMM that also emits the sums of its output rows
    if N <= 1280:
        res = rnd((M, N), 1.0, 76, dev)
        a2 = rnd((M, K), 1.0, 77, dev)
        plain = ops.gemm(a2, w, b, epilogue=ops.EPI_RESIDUAL, residual=res)
        s2, m2 = torch.zeros((M, 8), dtype=torch.float32, device=dev), torch.zeros((M, 8), dtype=torch.float32, device=dev)
        got = ops.gemm(a2, w, b, epilogue=ops.EPI_RESIDUAL, residual=res, c_row_sumsq=s2, c_row_sum=m2)
        assert torch.equal(got, plain)
        torch.testing.assert_close(s2.cpu(), _sumsq_parts_ref(plain), rtol=1e-5, atol=1e-6)
        pad = torch.zeros((M, 1280))
        pad[:, :N] = plain.float().cpu()
        torch.testing.assert_close(m2.cpu(), pad.view(M, 8, 160).sum(-1), rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("offset", [64.0, -100.0])
def test_gemm_with_folded_layernorm_on_rows_with_a_large_common_offset(ops, dev, offset):
    """The folded LayerNorm forms the variance as sumsq/K - mean^2 from fp32 sums, and the mean term as
    acc - mean * colsum: both cancel when a row's mean is far larger than its spread (mean / std of 64 and 100 here,
    where two thirds of the bits of sumsq/K cancel).  Checked against LayerNorm + linear on the same bf16 rows (the
    reference's sequence, siglip.py:173-175 then F.linear) at the encoder tolerance."""
    M, N, K, eps = 1000, 1280, 1152, 1e-6
    a = (rnd((M, K), 1.0, 81).float() + offset).bfloat16().to(dev)
    w, b = rnd((N, K), 0.05, 82, dev), rnd((N,), 0.02, 83, dev)
    g, beta = (1.0 + rnd((K,), 0.1, 84)).bfloat16(), rnd((K,), 0.1, 85)
    wf = (w.float().cpu() * g.float()[None, :]).bfloat16()
    bf = (b.float().cpu() + (w.float().cpu() * beta.float()[None, :]).sum(1)).bfloat16()
    csum = wf.float().sum(dim=1).contiguous()
    ss = torch.empty((M, 8), dtype=torch.float32, device=dev)
    sm = torch.empty_like(ss)
    ops.row_stats(a, ss, sm)
    af = a.float().cpu()
    assert (af.mean(1).abs() / af.std(1)).min() > 50          # the case this test is about
    ref = lin_ref(F.layer_norm(af, (K,), g.float(), beta.float(), eps).bfloat16(), w, b)
    got = ops.gemm(a, wf.to(dev), bf.to(dev), a_row_sumsq=ss, a_row_sum=sm, w_col_sum=csum.to(dev), norm_eps=eps).float().cpu()
    cos = F.cosine_similarity(got.flatten(), ref.flatten(), dim=0).item()
    rel = ((got - ref).abs().max() / ref.abs().max()).item()
    assert cos >= 0.999 and rel <= 2e-2, (cos, rel)


def test_gemm_row_maps(ops, dev):
    M, N, K = 400, 512, 256
    a, w, b = rnd((M, K), 1.0, 1, dev), rnd((N, K), 0.05, 2, dev), rnd((N,), 0.02, 3, dev)
    plain = ops.gemm(a, w, b)
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(1)).int().to(dev)
    assert torch.equal(ops.gemm(a, w, b, a_rows=perm), plain[perm.long()])   # gather is bit-exact data movement
    scat = ops.gemm(a, w, b, c_rows=perm)
    ref = torch.empty_like(plain)
    ref[perm.long()] = plain
    assert torch.equal(scat, ref)


def test_gemm_linearity_at_full_size(ops, dev):
    # size-independent property at the benchmark's shape: f(a1 + a2) == f(a1) + f(a2) up to bf16 rounding
    M, N, K = 8192, 3840, 1280
    a1, a2, w = rnd((M, K), 1.0, 1, dev), rnd((M, K), 1.0, 2, dev), rnd((N, K), 0.02, 3, dev)
    s = (a1.float() + a2.float()).bfloat16()
    y = ops.gemm(s, w, None).float()
    y12 = ops.gemm(a1, w, None).float() + ops.gemm(a2, w, None).float()
    assert (y - y12).abs().max().item() <= 2**-5 * y.abs().max().item()
    # and a sampled check against the oracle's F.linear
    rows = torch.arange(0, M, 257, device=dev)
    close(y[rows], lin_ref(s[rows], w, None), 2**-7, "sampled rows")


def test_gemm_fp8_weights(ops, dev):
    M, N, K = 300, 1280, 1280
    a, b = rnd((M, K), 1.0, 1, dev), rnd((N,), 0.02, 3, dev)
    w = torch.randn(N, K, generator=torch.Generator().manual_seed(2)) * 0.02
    scale = w.abs().amax(dim=1) / 448.0
    q = (w / scale[:, None]).to(torch.float8_e4m3fn)
    ref = a.float().cpu() @ (q.float() * scale[:, None]).t() + b.float().cpu()
    got = ops.gemm(a, q.to(dev), b, w_scale=scale.to(dev))
    close(got, ref, 2**-7, "fp8 weights")
    # every finite e4m3 byte decodes exactly: one-hot activations read the weight matrix back
    bytes_ = torch.tensor([v for v in range(256) if (v & 0x7F) != 0x7F], dtype=torch.uint8)
    K2 = 256
    wq = torch.zeros((16, K2), dtype=torch.uint8)
    wq[:, : bytes_.numel()] = bytes_
    eye = torch.eye(K2).bfloat16().to(dev)
    dec = ops.gemm(eye, wq.view(torch.float8_e4m3fn).to(dev), None, w_scale=torch.ones(16, device=dev))
    assert torch.equal(dec.float().cpu(), wq.view(torch.float8_e4m3fn).float().t())


def test_gemm_rejects_bad_shapes(ops, dev):
    a, w = rnd((8, 60), dev=dev), rnd((8, 60), dev=dev)
    with pytest.raises(ValueError):
        ops.gemm(a, w, None)   # K not a multiple of 8
    with pytest.raises(ValueError):
        ops.gemm(a.float(), w, None)


def test_gemm_rejects_mistyped_or_undersized_buffers(ops, dev):
    """Every buffer reaches the kernel as a raw pointer, so the wrapper refuses what the kernel would read or write
    out of bounds -- before anything is enqueued."""
    M, N, K = 64, 128, 64
    a, w, b = rnd((M, K), dev=dev), rnd((N, K), dev=dev), rnd((N,), dev=dev)
    res = rnd((M, N), dev=dev)
    rows64 = torch.arange(M, device=dev)                       # int64, as get_window_index returns it
    bad = [
        dict(a_rows=rows64),
        dict(c_rows=rows64),
        dict(c_rows=torch.arange(M - 1, device=dev, dtype=torch.int32)),
        dict(out=torch.empty((M, N), dtype=torch.float16, device=dev)),
        dict(out=torch.empty((M - 1, N), dtype=torch.bfloat16, device=dev)),
        dict(out=torch.empty((M, N - 8), dtype=torch.bfloat16, device=dev)),
        dict(out=torch.empty((M, N), dtype=torch.bfloat16)),   # host tensor
        dict(k=K + 8),
        dict(epilogue=ops.EPI_RESIDUAL),                          # no residual
        dict(epilogue=ops.EPI_RESIDUAL, residual=res[:, : N - 8]),
        dict(epilogue=ops.EPI_RESIDUAL, residual=res[: M - 1]),
        dict(epilogue=ops.EPI_RESIDUAL, residual=res.float()),
        dict(pos=rnd((4, N - 8), dev=dev)),
        dict(pos=rnd((4, N), dev=dev).float()),
        dict(out_lo=torch.zeros((M, N), dtype=torch.uint8, device=dev)),   # not the residual epilogue
        dict(epilogue=ops.EPI_RESIDUAL, residual=res, residual_lo=torch.zeros((M, N), dtype=torch.uint8, device=dev)),
        dict(epilogue=ops.EPI_RESIDUAL, residual=res, out=torch.empty_like(res),
             out_lo=torch.zeros((M, N), dtype=torch.int8, device=dev)),
        dict(epilogue=ops.EPI_RESIDUAL, residual=res, out=torch.empty_like(res),
             out_lo=torch.zeros((M, N + 8), dtype=torch.uint8, device=dev)),
    ]
    for kw in bad:
        with pytest.raises(ValueError):
            ops.gemm(a, w, b, **kw)
    for bias in (b.float(), b[: N - 8], b[None]):
        with pytest.raises(ValueError):
            ops.gemm(a, w, bias)
    with pytest.raises(ValueError):
        ops.gemm(a, w.to(torch.float8_e4m3fn), b, w_scale=torch.ones(N - 1, device=dev))
    torch.cuda.synchronize()
    assert torch.isfinite(ops.gemm(a, w, b).float()).all()    # the device is still healthy


def _join24(hi: torch.Tensor, lo: torch.Tensor) -> torch.Tensor:
    """The value a (bf16 plane, byte plane) pair stands for: fp32 from the bits (hi << 16) + (int8(lo) << 8)."""
    h = hi.cpu().view(torch.int16).to(torch.int32) << 16
    l = lo.cpu().view(torch.int8).to(torch.int32) << 8
    return (h + l).view(torch.float32)


# The residual stream with 16 significant bits, in every kernel that has the residual epilogue: the 160-column forms
# that also emit row sums (as the encoder blocks call them), the plain fast forms, fp8 weights, the general kernel.
@pytest.mark.parametrize("M,N,K,form", [
    (8192, 1280, 192, "sumsq"), (1000, 1280, 320, "sumsq"), (300, 1152, 448, "stats"), (8192, 2304, 256, "plain"),
    (300, 520, 448, "plain"), (777, 1280, 256, "fp8"), (515, 1280, 72, "general"),
])
def test_gemm_split_residual(ops, dev, M, N, K, form):
    a, b = rnd((M, K), 1.0, 51, dev), rnd((N,), 0.02, 53, dev)
    w = rnd((N, K), 0.05, 52, dev)
    kw, wf = {}, w.float().cpu()
    if form == "fp8":
        q, s = w.to(torch.float8_e4m3fn), torch.full((N,), 0.5, device=dev)
        wf, w, kw = q.float().cpu() * 0.5, q, dict(w_scale=s)
    res = rnd((M, N), 3.0, 54, dev)
    res_lo = torch.randint(0, 256, (M, N), generator=torch.Generator().manual_seed(55), dtype=torch.uint8).to(dev)
    ss = torch.zeros((M, 8), dtype=torch.float32, device=dev)
    sm = torch.zeros_like(ss)
    if form == "sumsq":
        kw["c_row_sumsq"] = ss
    if form == "stats":
        kw.update(c_row_sumsq=ss, c_row_sum=sm)
    rows = torch.cat([torch.arange(0, M, max(1, M // 199)), torch.tensor([M - 1])])
    exact = a.float().cpu()[rows] @ wf.t() + b.float().cpu()             # fp32, no rounding anywhere
    for lo_in in (res_lo, None):
        out, out_lo = torch.empty_like(res), torch.full((M, N), 0xAB, dtype=torch.uint8, device=dev)
        ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=res, residual_lo=lo_in, out=out, out_lo=out_lo, **kw)
        addend = _join24(res, lo_in) if lo_in is not None else res.float().cpu()
        want = exact + addend[rows]
        got = _join24(out, out_lo)[rows]
        # 2^-17 of the value from the split, plus the accumulation-order noise of an fp32 dot product
        assert (got - want).abs().max().item() <= want.abs().max().item() * 2.0**-16, (form, (got - want).abs().max().item())
        # the bf16 plane alone is the value rounded to bf16 (half an ulp; a bf16 ulp is at most 2^-7 of the value)
        assert ((out.float().cpu()[rows] - got).abs() <= got.abs() * 2.0**-8 + 1e-30).all()
        if form in ("sumsq", "stats"):
            parts = (N + 159) // 160
            torch.testing.assert_close(ss.cpu()[:, :parts], _sumsq_parts_ref(out)[:, :parts], rtol=1e-5, atol=1e-6)
    # a zero byte plane is "the bf16 value exactly": the addend equals the plain residual
    assert torch.equal(_join24(res, torch.zeros_like(res_lo)), res.float().cpu())
    # in place, 64 times: the stream follows the exact sum to 16 bits where a bf16 stream drifts by 2^-9 per addition
    x, x_lo = res.clone(), torch.zeros_like(res_lo)
    xb = res.clone()
    for _ in range(64):
        ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=x, residual_lo=x_lo, out=x, out_lo=x_lo, **kw)
        ops.gemm(a, w, b, epilogue=ops.EPI_RESIDUAL, residual=xb, out=xb, **kw)
    want = res.float().cpu()[rows] + 64.0 * exact
    err_split = (_join24(x, x_lo)[rows] - want).abs().max().item()
    err_bf16 = (xb.float().cpu()[rows] - want).abs().max().item()
    top = want.abs().max().item()
    assert err_split <= 64 * top * 2.0**-16 and err_split < err_bf16 / 16, (err_split, err_bf16, top)


# --------------------------------------------------------------------------------------- attention
def attn_ref(qkv, cu, nh, d, cos_sin=None):
    L = qkv.shape[0]
    q, k, v = (t.reshape(L, nh, d) for t in qkv.cpu().chunk(3, dim=-1))
    if cos_sin is not None:
        ang = cos_sin
        q, k = oq.apply_rotary(q, ang), oq.apply_rotary(k, ang)
    return oq.varlen_attention(q, k, v, cu, d**-0.5).reshape(L, nh * d)


@pytest.mark.parametrize("d,cu", [
    (80, [0, 64, 128, 176, 192, 256]),      # windows, ragged edges (48 and 16 rows)
    (80, [0, 1024, 1324]),                  # full segments, partial last tile
    (80, [0, 1, 3, 70, 200]),               # tiny segments
    (72, [0, 500, 1000]),                   # SigLIP head dim (zero padded in LDS)
    (72, [0, 64]),
    (64, [0, 130]),
    (96, [0, 200, 265]),
    (72, [0, 4096]),                        # one SigLIP image: 64 key tiles through the three-buffer ring
    (72, [0, 65, 129, 322]),                # one, two and three key tiles
    (72, [0, 729, 1458, 2187]),             # LLaVA-OneVision tiles: 27 x 27 tokens each
])
def test_attention(ops, dev, d, cu):
    nh, L = 16, cu[-1]
    qkv = rnd((L, 3 * nh * d), 1.0, 7, dev)
    plan = ops.attn_plan(np.array(cu, np.int32), dev)
    H = nh * d
    got = ops.attn_varlen(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], plan, nh, d, d**-0.5)
    close(got, attn_ref(qkv, cu, nh, d), 2**-6, f"attention d={d} cu={cu}")


@pytest.mark.parametrize("d,rotary", [(72, False), (80, True), (80, False), (64, False)])
def test_attention_wide_score_range(ops, dev, d, rotary):
    """Scores spread over many powers of two, with the largest keys LAST in each segment: the kernels keep a
    reference maximum that is only raised when a score exceeds it by 2^6, so this walks through both the raised
    and the not-raised case in every tile position, and through P values well above 1."""
    nh, cu = 16, [0, 700, 1000]
    L = cu[-1]
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn((L, 3 * nh * d), generator=g)
    ramp = torch.linspace(0.2, 4.0, L)[:, None]
    qkv[:, nh * d:2 * nh * d] *= ramp                  # key magnitude grows along the sequence
    qkv[:, :nh * d] *= 3.0
    qkv = qkv.bfloat16().to(dev)
    H = nh * d
    plan = ops.attn_plan(np.array(cu, np.int32), dev)
    cs = None
    ang = None
    if rotary:
        ang = torch.rand((L, d // 2), generator=g) * 6.0
        cs = torch.cat([ang.cos(), ang.sin()], dim=1).float().contiguous().to(dev)
    got = ops.attn_varlen(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], plan, nh, d, d**-0.5, cs)
    assert torch.isfinite(got.float()).all()
    close(got, attn_ref(qkv, cu, nh, d, ang), 2**-6, f"wide score range d={d} rotary={rotary}")


@pytest.mark.parametrize("d,rotary", [(72, False), (80, True), (80, False), (64, False)])
def test_attention_short_segment_same_bits_in_either_kernel(ops, dev, d, rotary):
    """A segment of at most 64 rows takes the 64-row kernel when it is the batch's longest and the 128-row kernels
    when a longer segment is in the batch: the result must not depend on that."""
    nh = 16
    cu_short, cu_both = [0, 40, 104], [0, 40, 104, 404]
    L = cu_both[-1]
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn((L, 3 * nh * d), generator=g).bfloat16().to(dev)
    cs = None
    if rotary:
        ang = torch.rand((L, d // 2), generator=g) * 6.0
        cs = torch.cat([ang.cos(), ang.sin()], dim=1).float().contiguous().to(dev)
    H = nh * d
    both = ops.attn_varlen(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], ops.attn_plan(np.array(cu_both, np.int32), dev), nh, d, d**-0.5, cs)
    short = ops.attn_varlen(qkv[:104, :H], qkv[:104, H:2 * H], qkv[:104, 2 * H:], ops.attn_plan(np.array(cu_short, np.int32), dev),
                            nh, d, d**-0.5, None if cs is None else cs[:104].contiguous())
    assert torch.equal(both[:104], short)


def test_rotary_head_dim_72(ops, dev):
    """Qwen3-VL: head dim 72, rotary halves of 36 (the 8-byte-vector path of the in-place kernel)."""
    nh, d, L = 16, 72, 333
    qkv = rnd((L, 3 * nh * d), 1.0, 61, dev)
    ang = torch.rand((L, d // 2), generator=torch.Generator().manual_seed(62)) * 6.0
    cs = torch.cat([ang.cos(), ang.sin()], dim=1).float().contiguous().to(dev)
    H = nh * d
    out = ops.rope_qk_(qkv.clone(), cs, nh, d)
    close(out[:, :H], oq.apply_rotary(qkv[:, :H].cpu().reshape(L, nh, d), ang).reshape(L, H), 2**-8, "rope q d=72")
    close(out[:, H:2 * H], oq.apply_rotary(qkv[:, H:2 * H].cpu().reshape(L, nh, d), ang).reshape(L, H), 2**-8, "rope k d=72")
    assert torch.equal(out[:, 2 * H:], qkv[:, 2 * H:])


@pytest.mark.parametrize("grids", [[(1, 12, 20)], [(2, 8, 8), (1, 48, 48), (1, 2, 2), (3, 6, 90)]])
def test_pos_embed_interp(ops, dev, grids):
    from oracle import qwen3_vl as o3

    side, E = 48, 1152
    table = rnd((side * side, E), 0.02, 63)
    g = np.array(grids, np.int64)
    ref = o3.pos_embed_interpolate(table, g, 2)                   # bf16 table: the reference's rounding points
    sl = ops.vit_seqlens_host(g, 2, 1 << 20)
    meta = torch.from_numpy(sl.item_meta).to(dev)
    got = ops.pos_embed_interp(table.to(dev), meta, sl.total_patches, sl.max_units_per_item, 2)
    assert got.shape == ref.shape and got.dtype == torch.bfloat16
    # identical operation order; a last-bit difference of an fp32 linspace position can move a bf16 weight
    diff = (got.float().cpu() - ref.float()).abs()
    assert diff.max().item() <= 2**-7 * ref.float().abs().max().item()
    assert (diff > 0).float().mean().item() < 0.02


def test_attention_fused_rotary_and_standalone_rotary(ops, dev):
    nh, d, cu = 16, 80, [0, 64, 128, 1024 + 128, 1024 + 128 + 37]
    L = cu[-1]
    qkv = rnd((L, 3 * nh * d), 1.0, 8, dev)
    ang = torch.rand(L, 40, generator=torch.Generator().manual_seed(1)) * 60
    cs = torch.cat([ang.cos(), ang.sin()], -1).contiguous().to(dev)
    plan = ops.attn_plan(np.array(cu, np.int32), dev)
    H = nh * d
    ref = attn_ref(qkv, cu, nh, d, ang)
    got = ops.attn_varlen(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], plan, nh, d, d**-0.5, cos_sin=cs)
    close(got, ref, 2**-6, "fused rotary attention")
    # standalone rotary kernel: same rounding as the oracle (fp32 math, one bf16 rounding) -> near bit-exact
    q2 = qkv.clone()
    ops.rope_qk_(q2, cs, nh, d)
    qr = oq.apply_rotary(qkv[:, :H].cpu().reshape(L, nh, d), ang).reshape(L, H)
    kr = oq.apply_rotary(qkv[:, H:2 * H].cpu().reshape(L, nh, d), ang).reshape(L, H)
    close(q2[:, :H], qr, 2**-8, "rope q")
    close(q2[:, H:2 * H], kr, 2**-8, "rope k")
    assert torch.equal(q2[:, 2 * H:], qkv[:, 2 * H:])
    got2 = ops.attn_varlen(q2[:, :H], q2[:, H:2 * H], q2[:, 2 * H:], plan, nh, d, d**-0.5)
    close(got2, ref, 2**-6, "rotary then attention")


def test_attention_invariants_at_full_size(ops, dev):
    nh, d, L = 16, 80, 8192
    H = nh * d
    qkv = rnd((L, 3 * H), 1.0, 9, dev)
    for seg in (64, 1024):
        cu = np.arange(0, L + 1, seg, dtype=np.int32)
        plan = ops.attn_plan(cu, dev)
        base = ops.attn_varlen(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], plan, nh, d, d**-0.5)
        # segments are independent: perturbing segment 0 leaves every other segment bit-identical
        q2 = qkv.clone()
        q2[:seg] += 1.0
        pert = ops.attn_varlen(q2[:, :H], q2[:, H:2 * H], q2[:, 2 * H:], plan, nh, d, d**-0.5)
        assert torch.equal(pert[seg:], base[seg:]) and not torch.equal(pert[:seg], base[:seg])
        # uniform V -> output equals V
        q3 = qkv.clone()
        q3[:, 2 * H:] = 0.75
        out = ops.attn_varlen(q3[:, :H], q3[:, H:2 * H], q3[:, 2 * H:], plan, nh, d, d**-0.5)
        assert (out.float() - 0.75).abs().max().item() <= 2**-8
        # sampled segments against the oracle
        s0 = (L // seg - 1) * seg
        ref = attn_ref(qkv[s0:], [0, seg], nh, d)
        close(base[s0:], ref, 2**-6, f"last segment of {seg}")
    # one-token segments return V exactly
    cu = np.arange(0, 257, dtype=np.int32)
    plan = ops.attn_plan(cu, dev)
    out = ops.attn_varlen(qkv[:256, :H], qkv[:256, H:2 * H], qkv[:256, 2 * H:], plan, nh, d, d**-0.5)
    assert torch.equal(out, qkv[:256, 2 * H:])


# ------------------------------------------------------------------------------- weighted row gather
def test_rows_bilinear_bit_exact(ops, dev):
    """cs_rows_bilinear against the same formula in numpy fp32 (no fused multiply-add on either side): identical bits.
    Copy rows (both fractions zero) keep the source bits, signed zeros and infinities included."""
    n_src, E, R = 300, 3584, 1000
    src = rnd((n_src, E), 1.0, 71)
    src[5, :8] = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 1.0, -1.0, 3.0e38, -3.0e38]).bfloat16()
    rng = np.random.default_rng(5)
    taps = rng.integers(0, n_src, size=(R, 4)).astype(np.int32)
    taps[taps == 5] = 6        # row 5 (special values) is only ever copied
    frac = rng.random((R, 2)).astype(np.float32)
    frac[::7] = 0.0            # copies
    taps[0] = 5                # the row with the special values
    frac[3, 0] = 0.0           # one fraction zero is still an interpolation
    taps[11] = [0, n_src, 1, 2]        # a tap past the source: zero row, no stray read
    taps[12] = [-1, 0, 1, 2]
    frac[11] = frac[12] = 0.5
    got = ops.rows_bilinear(src.to(dev), torch.from_numpy(taps).to(dev), torch.from_numpy(frac).to(dev)).cpu()
    s32 = src.float().numpy()
    ok = ((taps >= 0) & (taps < n_src)).all(axis=1)
    t = np.where(ok[:, None], taps, 0)
    a = [s32[t[:, k]] for k in range(4)]
    ly, lx = frac[:, 0:1], frac[:, 1:2]
    hy, hx = np.float32(1) - ly, np.float32(1) - lx
    with np.errstate(all="ignore"):
        ref = hy * (hx * a[0] + lx * a[1]) + ly * (hx * a[2] + lx * a[3])
    copy = (frac == 0).all(axis=1)
    ref[copy] = a[0][copy]
    ref[~ok] = 0.0
    ref = torch.from_numpy(ref).bfloat16()
    assert got.dtype == torch.bfloat16 and got.shape == (R, E)
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
    assert torch.equal(got[0].view(torch.int16), src[5].view(torch.int16))
    # strided source and destination rows
    wide = torch.zeros((n_src, E + 64), dtype=torch.bfloat16, device=dev)
    wide[:, :E] = src.to(dev)
    out = torch.full((R, E + 8), 7.0, dtype=torch.bfloat16, device=dev)
    ops.rows_bilinear(wide[:, :E], torch.from_numpy(taps).to(dev), torch.from_numpy(frac).to(dev), out=out[:, :E])
    assert torch.equal(out[:, :E].cpu().view(torch.int16), ref.view(torch.int16)) and bool((out[:, E:] == 7.0).all())
    empty = ops.rows_bilinear(src.to(dev), torch.zeros((0, 4), dtype=torch.int32, device=dev),
                              torch.zeros((0, 2), dtype=torch.float32, device=dev))
    assert empty.shape == (0, E)
    with pytest.raises(ValueError):
        ops.rows_bilinear(src.to(dev), torch.zeros((4, 3), dtype=torch.int32, device=dev),
                          torch.zeros((4, 2), dtype=torch.float32, device=dev))
    with pytest.raises(ValueError, match="invalid argument"):      # rows of 3580 values: not whole 16-byte vectors
        ops.rows_bilinear(src.to(dev)[:, :E - 4], torch.zeros((4, 4), dtype=torch.int32, device=dev),
                          torch.zeros((4, 2), dtype=torch.float32, device=dev))


@pytest.mark.parametrize("B,C,H,W,patch,N", [(2, 3, 896, 896, 14, 1152), (3, 3, 384, 384, 14, 1152), (5, 3, 56, 84, 14, 64),
                                               (2, 1, 48, 32, 16, 40), (1, 3, 30, 44, 6, 24)])
def test_gemm_strided_gather_convolution(ops, dev, B, C, H, W, patch, N):
    """Conv2d with kernel = stride = patch (siglip.py:30-36) as a GEMM whose activation operand is gathered from the
    NCHW image inside the kernel: against torch's convolution, and bit for bit against the same GEMM on patches
    materialised by cs_patchify_nchw (same K order, same kernel, so the same accumulation order).  384 / 14 and
    30 / 6 leave pixels past the last whole patch, which neither form reads."""
    g = torch.Generator().manual_seed(61)
    px = (torch.rand((B, C, H, W), generator=g) * 2 - 1).bfloat16()
    wt = (torch.randn((N, C, patch, patch), generator=g) * 0.05).bfloat16()
    bias = (torch.randn((N,), generator=g) * 0.02).bfloat16()
    kraw = C * patch * patch
    kp = (kraw + 7) // 8 * 8
    w2 = torch.zeros((N, kp), dtype=torch.bfloat16)
    w2[:, :kraw] = wt.reshape(N, kraw)
    hp, wp = H // patch, W // patch
    pos = (torch.randn((hp * wp, N), generator=g) * 0.1).bfloat16()
    dpx, dw, db, dpos = px.to(dev), w2.to(dev), bias.to(dev), pos.to(dev)
    got = ops.gemm(dpx, dw, db, conv_patch=patch)
    assert got.shape == (B * hp * wp, N)
    ref = F.conv2d(px.float(), wt.float(), bias.float(), stride=patch).flatten(2).transpose(1, 2).reshape(-1, N)
    close(got, ref, 2**-7, "strided-gather GEMM vs conv2d")
    mat = ops.gemm(ops.patchify_nchw(dpx, patch, kp), dw, db)
    assert torch.equal(got, mat)
    with_pos = ops.gemm(dpx, dw, db, pos=dpos, conv_patch=patch)
    assert torch.equal(with_pos, ops.gemm(ops.patchify_nchw(dpx, patch, kp), dw, db, pos=dpos))
    out = torch.empty_like(got)
    assert torch.equal(ops.gemm(dpx, dw, db, conv_patch=patch, out=out), got)
    for bad in (dict(conv_patch=patch + 1), dict(conv_patch=patch, epilogue=ops.EPI_GELU_TANH),
                dict(conv_patch=patch, a_rows=torch.zeros(4, dtype=torch.int32, device=dev))):
        with pytest.raises(ValueError):
            ops.gemm(dpx, dw, db, **bad)
    with pytest.raises(ValueError):
        ops.gemm(dpx, dw[:, : kp - 8].contiguous(), db, conv_patch=patch)


def test_patchify_nchw_drops_the_partial_patches(ops, dev):
    """384 = 27 * 14 + 6: a convolution with stride = kernel and no padding ignores the last 6 rows and columns."""
    px = rnd((3, 3, 384, 384), 1.0, 72)
    got = ops.patchify_nchw(px.to(dev), 14, 592).cpu()
    ref = F.unfold(px.float()[:, :, :378, :378], kernel_size=14, stride=14).transpose(1, 2).reshape(3 * 729, 588)
    assert got.shape == (3 * 729, 592)
    assert torch.equal(got[:, :588].float(), ref) and not got[:, 588:].any()


@pytest.mark.parametrize("B,C,H,W,patch,ldo", [
    (2, 3, 896, 896, 14, 592),    # config-3 tiles: 64 patches per row, eight runs of eight
    (1, 3, 70, 154, 14, 590),     # 11 patches per row (last run has three), rows that are not whole 16-byte vectors
    (2, 3, 64, 176, 16, 768),     # patch 16, no padding columns
    (1, 5, 30, 50, 10, 504),      # any even patch size, five channels, partial patches dropped
    (1, 3, 12, 36, 6, 110),       # narrow stores with padding
    (1, 40, 56, 56, 28, 31360),   # eight patches' row segments exceed the LDS budget: fewer patches per workgroup
])
def test_patchify_nchw_shapes(ops, dev, B, C, H, W, patch, ldo):
    px = rnd((B, C, H, W), 1.0, 73)
    got = ops.patchify_nchw(px.to(dev), patch, ldo).cpu()
    gh, gw, K = H // patch, W // patch, C * patch * patch
    ref = F.unfold(px.float()[:, :, :gh * patch, :gw * patch], kernel_size=patch, stride=patch)
    ref = ref.transpose(1, 2).reshape(B * gh * gw, K)
    assert got.shape == (B * gh * gw, ldo)
    assert torch.equal(got[:, :K].float(), ref) and not got[:, K:].any()


def test_gemm_random_shapes_epilogues_and_folds(ops, dev):
    """A seeded sweep over row counts either side of every tile height (1 .. 5000), widths, depths, epilogues and the
    folded-norm forms, against fp32 torch arithmetic with the reference's rounding points."""
    rng = np.random.default_rng(11)
    rbf = lambda x: x.bfloat16().float()
    ran = folded = 0
    for it in range(90):
        M = int(rng.choice([1, 7, 64, 100, 127, 128, 129, 255, 256, 257, 300, 511, 513, 1000, 1024, 1500, 2048, 3000, 4096, 4100, 5000]))
        N = int(rng.choice([8, 64, 160, 168, 320, 520, 640, 1152, 1280, 1288, 2304, 3456, 3840]))
        K = int(rng.choice([64, 128, 192, 200, 256, 320, 448, 1152, 1176, 1280]))
        epi = int(rng.choice([ops.EPI_BIAS, ops.EPI_RESIDUAL, ops.EPI_SWIGLU, ops.EPI_GELU_ERF, ops.EPI_GELU_TANH, ops.EPI_QUICK_GELU]))
        fold = int(rng.choice([0, 0, 1, 2, 3]))
        if epi == ops.EPI_SWIGLU and (N // 2) % 8:
            continue
        a, w, b = rnd((M, K), 1.0, it, dev), rnd((N, K), 0.05, it + 1000, dev), rnd((N,), 0.05, it + 2000, dev)
        res = rnd((M, N), 1.0, it + 3000, dev) if epi == ops.EPI_RESIDUAL else None
        af, wf = a.float().cpu(), w.float().cpu()
        acc = af @ wf.t()
        eps, kw = 1e-6, {}
        fast = K % 64 == 0 and K >= 192
        if fold == 1 and epi in (ops.EPI_BIAS, ops.EPI_SWIGLU) and fast:
            ss = torch.zeros((M, ops.SUMSQ_PARTS), dtype=torch.float32, device=dev)
            ops.row_sumsq(a, ss)
            kw = dict(a_row_sumsq=ss, norm_eps=eps)
            acc = acc * torch.rsqrt((af * af).sum(1, keepdim=True) / K + eps)
        elif fold == 2 and epi in (ops.EPI_RESIDUAL, ops.EPI_BIAS) and fast and N <= 1280:
            kw = dict(c_row_sumsq=torch.zeros((M, ops.SUMSQ_PARTS), dtype=torch.float32, device=dev))
        elif fold == 3 and epi in (ops.EPI_BIAS, ops.EPI_GELU_TANH, ops.EPI_QUICK_GELU) and fast:
            ss = torch.zeros((M, ops.SUMSQ_PARTS), dtype=torch.float32, device=dev)
            sm = torch.zeros_like(ss)
            ops.row_stats(a, ss, sm)
            kw = dict(a_row_sumsq=ss, a_row_sum=sm, w_col_sum=wf.sum(1).to(dev), norm_eps=eps)
            mean = af.mean(1, keepdim=True)
            var = ((af * af).mean(1, keepdim=True) - mean * mean).clamp_min(0)
            acc = torch.rsqrt(var + eps) * (acc - mean * wf.sum(1)[None, :])
        folded += bool(kw)
        got = ops.gemm(a, w, b, epilogue=epi, residual=res, **kw).float().cpu()
        v = acc + b.float().cpu()
        if epi == ops.EPI_RESIDUAL:
            ref = rbf(v) + res.float().cpu()
        elif epi == ops.EPI_SWIGLU:
            ref = F.silu(rbf(v[:, 0::2])) * rbf(v[:, 1::2])
        elif epi == ops.EPI_GELU_ERF:
            ref = F.gelu(rbf(v))
        elif epi == ops.EPI_GELU_TANH:
            ref = F.gelu(rbf(v), approximate="tanh")
        elif epi == ops.EPI_QUICK_GELU:
            ref = rbf(v) * torch.sigmoid(1.702 * rbf(v))
        else:
            ref = v
        close(got, ref, 2**-6, f"gemm {M}x{N}x{K} epilogue {epi} fold {fold}")
        if "c_row_sumsq" in kw:
            close(kw["c_row_sumsq"].sum(1), (got * got).sum(1), 1e-3, f"row sums of squares {M}x{N}x{K}")
        ran += 1
    assert ran >= 70 and folded >= 10


def test_attention_random_segments(ops, dev):
    """A seeded sweep over head dims, segment-length mixes (1 .. 3000 rows, lengths either side of the 64-key tile and
    the 64/128-row query blocks) and rotary on/off, against fp32 softmax attention."""
    rng = np.random.default_rng(17)
    for it in range(24):
        d = int(rng.choice([64, 72, 80, 96]))
        nh = int(rng.choice([2, 4, 16]))
        kind = it % 4
        if kind == 0:      # many short segments (the window kernel)
            lens = rng.integers(1, 65, size=int(rng.integers(3, 40))).tolist()
        elif kind == 1:    # a few long ones (the full kernels)
            lens = rng.integers(100, 3000, size=int(rng.integers(1, 4))).tolist()
        elif kind == 2:    # lengths at the tile edges
            lens = [int(x) for x in rng.choice([63, 64, 65, 127, 128, 129, 191, 192, 193, 256, 729], size=5)]
        else:              # short and long mixed
            lens = rng.integers(1, 700, size=int(rng.integers(2, 10))).tolist()
        cu = [0] + np.cumsum(lens).tolist()
        L, H = cu[-1], nh * d
        qkv = rnd((L, 3 * H), 1.0, 100 + it, dev)
        rotary = bool(rng.integers(0, 2)) and d % 16 == 0
        ang = cs = None
        if rotary:
            ang = torch.rand(L, d // 2, generator=torch.Generator().manual_seed(it)) * 50
            cs = torch.cat([ang.cos(), ang.sin()], -1).contiguous().to(dev)
        plan = ops.attn_plan(np.array(cu, np.int32), dev)
        got = ops.attn_varlen(qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:], plan, nh, d, d**-0.5, cs)
        close(got, attn_ref(qkv, cu, nh, d, ang), 2**-6, f"attention d={d} heads={nh} lens={lens[:8]} rotary={rotary}")


# ------------------------------------------------ QKV projection + rotary + window attention in one launch
@pytest.mark.gpu
@pytest.mark.parametrize("M,K,heads,fold", [(256, 192, 1, False), (512, 1280, 16, False), (8192, 1280, 16, True),
                                            (320, 256, 3, True), (64, 1280, 2, False)])
def test_qkv_window_attn_against_fp32_and_the_unfused_chain(ops, dev, M, K, heads, fold):
    d = 80
    x = rnd((M, K), 1.0, 11, dev)
    w = rnd((3 * heads * d, K), K**-0.5, 12, dev)
    b = rnd((3 * heads * d,), 0.5, 13, dev)
    g = torch.Generator().manual_seed(14)
    ang = torch.rand((M, d // 2), generator=g) * 6.0
    cs = torch.cat([ang.cos(), ang.sin()], dim=1).float().contiguous().to(dev)
    eps = 1e-6
    sums = ops.row_sumsq(x) if fold else None
    wp, bp = ops.pack_qkv_window_attn(w, b, heads)
    got = ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5, a_row_sumsq=sums, norm_eps=eps)
    # fp32 restatement: (normalised) rows . W^T + b, rotary, softmax attention inside windows of 64 rows
    xf = x.float().cpu()
    if fold:
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    qkv = xf @ w.float().cpu().T + b.float().cpu()
    cu = list(range(0, M + 1, 64))
    ref = attn_ref(qkv, cu, heads, d, ang)
    close(got, ref, 2**-6, f"fused qkv + window attention M={M} K={K} heads={heads} fold={fold}")
    # the chain it replaces (bf16 qkv tensor in between) sits within the same distance of the fp32 result
    qkv_dev = ops.gemm(x, w, b, a_row_sumsq=sums, norm_eps=eps)
    H = heads * d
    plan = ops.attn_plan(np.array(cu, np.int32), dev)
    chain = ops.attn_varlen(qkv_dev[:, :H], qkv_dev[:, H:2 * H], qkv_dev[:, 2 * H:], plan, heads, d, d**-0.5, cs)
    close(chain, ref, 2**-6, "unfused chain")
    err_fused = (got.float().cpu() - ref).abs().max().item()
    err_chain = (chain.float().cpu() - ref).abs().max().item()
    assert err_fused <= 1.5 * err_chain + 1e-3, (err_fused, err_chain)


@pytest.mark.gpu
@pytest.mark.parametrize("fold", [True, False])
def test_qkv_window_attn_windows_of_fewer_than_64_rows(ops, dev, fold):
    """Windows of 4 .. 64 rows, one 64-row slot each: against the fp32 restatement and the unfused chain on the same
    segments, every row count a window can have (4 r c for r, c in 1..4) among them, a number of windows that is not a
    multiple of the four a workgroup takes; a window of 64 rows comes out with the bits of the whole-window form; rows
    past the last window's end are not written."""
    d, heads, K = 80, 4, 1280
    counts = [64, 48, 36, 64, 16, 4, 8, 12, 24, 32, 64, 64, 16, 48, 64, 36, 4]
    cu = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    M = int(cu[-1])
    x = rnd((M, K), 1.0, 21, dev)
    w = rnd((3 * heads * d, K), K**-0.5, 22, dev)
    b = rnd((3 * heads * d,), 0.5, 23, dev)
    g = torch.Generator().manual_seed(24)
    ang = torch.rand((M, d // 2), generator=g) * 6.0
    cs = torch.cat([ang.cos(), ang.sin()], dim=1).float().contiguous().to(dev)
    eps = 1e-6
    sums = ops.row_sumsq(x) if fold else None
    wp, bp = ops.pack_qkv_window_attn(w, b, heads)
    out = torch.full((M + 8, heads * d), 7.0, dtype=torch.bfloat16, device=dev)
    ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5, a_row_sumsq=sums, norm_eps=eps, out=out[:M],
                        win_start=torch.from_numpy(cu).to(dev))
    assert torch.all(out[M:] == 7.0)
    got = out[:M]
    xf = x.float().cpu()
    if fold:
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    qkv = xf @ w.float().cpu().T + b.float().cpu()
    ref = attn_ref(qkv, cu.tolist(), heads, d, ang)
    close(got, ref, 2**-6, f"fused qkv + ragged window attention fold={fold}")
    qkv_dev = ops.gemm(x, w, b, a_row_sumsq=sums, norm_eps=eps)
    H = heads * d
    plan = ops.attn_plan(cu, dev)
    chain = ops.attn_varlen(qkv_dev[:, :H], qkv_dev[:, H:2 * H], qkv_dev[:, 2 * H:], plan, heads, d, d**-0.5, cs)
    err_fused = (got.float().cpu() - ref).abs().max().item()
    err_chain = (chain.float().cpu() - ref).abs().max().item()
    assert err_fused <= 1.5 * err_chain + 1e-3, (err_fused, err_chain)
    # whole windows: the two forms of the launch give the same bits (what lets one batch hold both kinds of item)
    for w0 in [i for i, c in enumerate(counts) if c == 64]:
        lo = int(cu[w0])
        alone = ops.qkv_window_attn(x[lo:lo + 64], wp, bp, cs[lo:lo + 64].contiguous(), heads, d**-0.5,
                                    a_row_sumsq=None if sums is None else sums[lo:lo + 64].contiguous(), norm_eps=eps)
        assert torch.equal(alone, got[lo:lo + 64]), w0
    whole_cu = torch.arange(0, 64 * 6 + 1, 64, dtype=torch.int32, device=dev)
    xs, css = x[:384], cs[:384].contiguous()
    ss = None if sums is None else sums[:384].contiguous()
    a = ops.qkv_window_attn(xs, wp, bp, css, heads, d**-0.5, a_row_sumsq=ss, norm_eps=eps)
    r = ops.qkv_window_attn(xs, wp, bp, css, heads, d**-0.5, a_row_sumsq=ss, norm_eps=eps, win_start=whole_cu)
    assert torch.equal(a, r)
    # a prefetch hint (extra workgroups that only read it) changes no bit of either form
    hint = rnd((3420, 1280), 0.05, 25, dev)
    assert torch.equal(ops.qkv_window_attn(xs, wp, bp, css, heads, d**-0.5, a_row_sumsq=ss, norm_eps=eps, prefetch=hint), a)
    assert torch.equal(ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5, a_row_sumsq=sums, norm_eps=eps,
                                           win_start=torch.from_numpy(cu).to(dev), prefetch=hint), got)
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5, win_start=torch.from_numpy(cu[:3].copy()).to(dev))   # 2 windows cannot hold M rows
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5, win_start=torch.from_numpy(cu.astype(np.int64)).to(dev))


@pytest.mark.gpu
def test_qkv_window_attn_fp8_weights(ops, dev):
    """The one launch with e4m3 weights and per-output-channel scales (the bytes and scales of the plain fp8 GEMM,
    reordered): whole windows and short ones against the fp32 restatement on the de-quantised weights, and no further
    from it than the unfused fp8 chain."""
    from cornserve_amd.eric.models.qwen2_5_vl import quantize_fp8_rows

    d, heads, K = 80, 4, 1280
    w = rnd((3 * heads * d, K), K**-0.5, 32, dev)
    b = rnd((3 * heads * d,), 0.5, 33, dev)
    q, sc = quantize_fp8_rows(w)
    w_deq = q.float().cpu() * sc.float().cpu()[:, None]
    wp, bp, sp = ops.pack_qkv_window_attn(q, b, heads, w_scale=sc)
    assert wp.dtype == torch.uint8 and sp.dtype == torch.float32 and sp.shape == (heads * 256,)
    for counts in ([64] * 9, [64, 48, 36, 16, 4, 64, 24, 32, 12, 8]):
        cu = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
        M = int(cu[-1])
        x = rnd((M, K), 1.0, 31, dev)
        g = torch.Generator().manual_seed(34)
        ang = torch.rand((M, d // 2), generator=g) * 6.0
        cs = torch.cat([ang.cos(), ang.sin()], dim=1).float().contiguous().to(dev)
        ragged = any(c != 64 for c in counts)
        got = ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5, w_scale=sp,
                                  win_start=torch.from_numpy(cu).to(dev) if ragged else None)
        qkv = x.float().cpu() @ w_deq.T + b.float().cpu()
        ref = attn_ref(qkv, cu.tolist(), heads, d, ang)
        close(got, ref, 2**-6, f"fused fp8 qkv + window attention, ragged={ragged}")
        qkv_dev = ops.gemm(x, q, b, w_scale=sc)
        H = heads * d
        chain = ops.attn_varlen(qkv_dev[:, :H], qkv_dev[:, H:2 * H], qkv_dev[:, 2 * H:], ops.attn_plan(cu, dev), heads, d,
                                d**-0.5, cs)
        err_fused = (got.float().cpu() - ref).abs().max().item()
        err_chain = (chain.float().cpu() - ref).abs().max().item()
        assert err_fused <= 1.5 * err_chain + 1e-3, (err_fused, err_chain)
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5)                      # fp8 bytes without their scales
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x, wp, bp, cs, heads, d**-0.5, w_scale=sp, a_row_sumsq=ops.row_sumsq(x))
    with pytest.raises(ValueError):
        ops.pack_qkv_window_attn(q, b, heads)


@pytest.mark.gpu
def test_qkv_window_attn_rejects_what_the_kernel_does_not_take(ops, dev):
    d, heads, K = 80, 2, 192
    x = rnd((128, K), 1.0, 1, dev)
    w = rnd((3 * heads * d, K), 0.1, 2, dev)
    b = rnd((3 * heads * d,), 0.1, 3, dev)
    wp, bp = ops.pack_qkv_window_attn(w, b, heads)
    cs = torch.zeros((128, d), device=dev)
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x[:100], wp, bp, cs[:100], heads, d**-0.5)            # not whole windows
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x, wp[:256], bp, cs, heads, d**-0.5)                  # weight not packed per head
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x, wp, bp, cs[:, :40].contiguous(), heads, d**-0.5)   # table of another head dim
    with pytest.raises(ValueError):
        ops.qkv_window_attn(x, wp, bp, cs.double(), heads, d**-0.5)
    with pytest.raises(ValueError):
        ops.pack_qkv_window_attn(w[:100], b[:100], heads)
