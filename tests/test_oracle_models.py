"""Pins oracle/qwen2_5_vl.py and oracle/gemma3.py (CPU only).

  * committed golden samples written from the Hugging Face implementations (the reference's own test oracle)
    on the same seeded weights and inputs -- an fp32-vs-fp32 comparison, so the tolerance is tight;
  * closed forms / special cases of the pieces: rotary at angle 0 is the identity and preserves the norm of
    each (j, j+d/2) pair; a one-token segment returns V; uniform V returns V; segments are independent;
    RMSNorm of a constant row; conv-as-linear identity for the patch embed.
"""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests import synth
from oracle import gemma3 as og
from oracle import qwen2_5_vl as oq


def test_qwen_cfg1_against_golden(golden_dir):
    gold = np.load(golden_dir / "qwen2_5_vl_cfg1.npz")
    cfg = synth.qwen_vision_config(depth=4, fullatt_block_indexes=(3,))
    ocfg = oq.QwenVisionConfig(depth=4, fullatt_block_indexes=[3])
    sd = synth.qwen_state_dict(cfg, seed=int(gold["seed"]))
    px, grid = synth.qwen_inputs([(1, 32, 32)], seed=int(gold["seed"]))
    out = oq.forward(sd, ocfg, px, grid, dtype=torch.float32)
    assert len(out) == 1 and out[0].shape == (256, 3584)
    o = out[0].numpy()
    scale = np.abs(gold["sample"]).max()
    assert np.abs(o[:, ::16] - gold["sample"]).max() <= 2e-4 * scale
    assert np.allclose(np.linalg.norm(o.astype(np.float64), axis=1), gold["row_l2"], rtol=1e-4)
    assert abs(np.abs(o.astype(np.float64)).sum() - float(gold["abs_total"])) <= 1e-4 * float(gold["abs_total"])


def test_gemma3_small_against_golden(golden_dir):
    gold = np.load(golden_dir / "gemma3_small.npz")
    cfg = synth.gemma3_config(num_hidden_layers=2, image_size=224, text_hidden=640, mm_tokens_per_image=16)
    ocfg = og.SiglipConfig(num_hidden_layers=2, image_size=224, mm_tokens_per_image=16, text_hidden_size=640)
    sd = synth.gemma3_state_dict(cfg, seed=int(gold["seed"]))
    px, crops = synth.gemma3_inputs(2, 224, seed=int(gold["seed"]))
    feats = og.vision_tower(sd, ocfg, torch.cat(px))
    fs = gold["feats_sample"]
    assert np.abs(feats.numpy()[:, ::8, ::8] - fs).max() <= 2e-4 * np.abs(fs).max()
    out = og.forward(sd, ocfg, px, crops)
    assert len(out) == 2 and out[0].shape == (16, 640)
    got = torch.stack(out).numpy()
    assert np.abs(got - gold["out"]).max() <= 2e-4 * np.abs(gold["out"]).max()


def test_rotary_special_cases():
    torch.manual_seed(0)
    t = torch.randn(7, 3, 80)
    assert torch.equal(oq.apply_rotary(t, torch.zeros(7, 40)), t)
    fr = torch.rand(7, 40) * 6
    r = oq.apply_rotary(t, fr)
    n0 = t[..., :40] ** 2 + t[..., 40:] ** 2
    n1 = r[..., :40] ** 2 + r[..., 40:] ** 2
    assert torch.allclose(n0, n1, atol=1e-5)
    # quarter turn: (x1, x2) -> (-x2, x1)
    q = oq.apply_rotary(t, torch.full((7, 40), np.pi / 2))
    assert torch.allclose(q[..., :40], -t[..., 40:], atol=1e-6) and torch.allclose(q[..., 40:], t[..., :40], atol=1e-6)


def test_attention_special_cases():
    torch.manual_seed(0)
    q, k, v = torch.randn(3, 10, 4, 16).unbind(0)
    one = oq.varlen_attention(q, k, v, list(range(11)), 0.25)
    assert torch.allclose(one, v, atol=1e-6)  # one-token segments return V
    vu = torch.ones(10, 4, 16) * 3.0
    assert torch.allclose(oq.varlen_attention(q, k, vu, [0, 4, 10], 0.25), vu, atol=1e-6)
    base = oq.varlen_attention(q, k, v, [0, 4, 10], 0.25)
    k2, v2 = k.clone(), v.clone()
    k2[4:] += 1.0
    v2[4:] -= 2.0
    pert = oq.varlen_attention(q, k2, v2, [0, 4, 10], 0.25)
    assert torch.equal(pert[:4], base[:4]) and not torch.allclose(pert[4:], base[4:])
    # against the library routine
    ref = F.scaled_dot_product_attention(q[:4].transpose(0, 1), k[:4].transpose(0, 1), v[:4].transpose(0, 1), scale=0.25)
    assert torch.allclose(base[:4], ref.transpose(0, 1), atol=1e-6)


def test_norms():
    x = torch.full((2, 8), 3.0)
    w = torch.arange(8, dtype=torch.float)
    assert torch.allclose(oq.rms_norm(x, w, 0.0), w.expand(2, 8))
    assert torch.allclose(og.gemma_rms_norm(x, w, 0.0), (1 + w).expand(2, 8))
    y = torch.randn(5, 32)
    assert torch.allclose(oq.rms_norm(y, torch.ones(32), 1e-6), F.rms_norm(y, (32,), eps=1e-6), atol=1e-6)


def test_patch_embed_is_a_linear_map():
    cfg = synth.qwen_vision_config(depth=0)
    w = synth.normal(3, "w", (1280, 3, 2, 14, 14), 0.02)
    x = synth.normal(3, "x", (16, 1176))
    conv = F.conv3d(x.view(16, 3, 2, 14, 14), w, stride=(2, 14, 14)).view(16, 1280)
    assert torch.allclose(conv, x @ w.view(1280, -1).t(), atol=1e-5)
    assert cfg.vision_config.hidden_size == 1280


def test_bf16_stepwise_close_to_fp32():
    cfg = synth.qwen_vision_config(depth=2, fullatt_block_indexes=(1,))
    ocfg = oq.QwenVisionConfig(depth=2, fullatt_block_indexes=[1])
    sd = synth.qwen_state_dict(cfg, seed=5)
    px, grid = synth.qwen_inputs([(1, 8, 12)], seed=5)
    a = oq.forward(sd, ocfg, px, grid, dtype=torch.float32)[0]
    b = oq.forward(sd, ocfg, px, grid, dtype=torch.bfloat16)[0].float()
    cos = F.cosine_similarity(a.flatten(), b.flatten(), dim=0).item()
    assert cos > 0.999


# ------------------------------------------------------------------------------------------ Qwen2-VL
def _qwen2_small(depth=2, seed=3):
    from oracle import qwen2_vl as o2

    cfg = synth.qwen2_vision_config(depth=depth)
    return o2, cfg, o2.Qwen2VisionConfig(depth=depth), synth.qwen2_state_dict(cfg, seed=seed)


def test_qwen2_vl_against_golden(golden_dir):
    gold = np.load(golden_dir / "qwen2_vl_small.npz")
    o2, cfg, ocfg, sd = _qwen2_small(seed=int(gold["seed"]))
    px, grid = synth.qwen_inputs([(1, 16, 16), (2, 8, 12)], seed=int(gold["seed"]))
    out = o2.forward(sd, ocfg, px, grid, dtype=torch.float32)
    assert [tuple(o.shape) for o in out] == [(64, 3584), (48, 3584)]
    o = torch.cat(out).numpy()
    assert np.abs(o[:, ::8] - gold["sample"]).max() <= 2e-4 * np.abs(gold["sample"]).max()
    assert np.allclose(np.linalg.norm(o.astype(np.float64), axis=1), gold["row_l2"], rtol=1e-4)
    assert abs(o.astype(np.float64).sum() - float(gold["total"])) <= 1e-4 * np.abs(o.astype(np.float64)).sum()


def test_qwen2_vl_live_against_hugging_face():
    """The same comparison against the installed third-party implementation on another shape (a ragged image and a
    three-frame-group video), when it is importable."""
    cm = pytest.importorskip("transformers.models.qwen2_vl.configuration_qwen2_vl")
    mm = pytest.importorskip("transformers.models.qwen2_vl.modeling_qwen2_vl")
    o2, cfg, ocfg, sd = _qwen2_small(depth=1, seed=8)
    vc = cfg.vision_config
    hf_cfg = cm.Qwen2VLVisionConfig(depth=1, embed_dim=vc.embed_dim, hidden_size=vc.hidden_size, num_heads=vc.num_heads,
                                    mlp_ratio=int(vc.mlp_ratio), patch_size=14, spatial_merge_size=2, temporal_patch_size=2,
                                    hidden_act="quick_gelu")
    hf_cfg._attn_implementation = "sdpa"
    model = mm.Qwen2VisionTransformerPretrainedModel(hf_cfg).float().eval()
    inc = model.load_state_dict(sd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys
    px, grid = synth.qwen_inputs([(1, 6, 10), (3, 4, 4)], seed=8)
    with torch.no_grad():
        ref = model(torch.cat(px), grid_thw=torch.cat(grid))
    ref = ref.pooler_output if hasattr(ref, "pooler_output") else ref
    got = torch.cat(o2.forward(sd, ocfg, px, grid, dtype=torch.float32))
    assert got.shape == ref.shape == ((60 + 48) // 4, 3584)
    assert (got - ref).abs().max().item() <= 2e-4 * ref.abs().max().item()


def test_qwen2_vl_pieces():
    from oracle import qwen2_vl as o2

    x = torch.linspace(-6, 6, 25)
    assert torch.allclose(o2.quick_gelu(x), x / (1 + torch.exp(-1.702 * x)), atol=1e-6)
    assert o2.quick_gelu(torch.tensor(0.0)).item() == 0.0 and abs(o2.quick_gelu(torch.tensor(20.0)).item() - 20.0) < 1e-5
    # rotary angles: position (h, w) times inv_freq, h-half then w-half, rows in 2x2-block-major order
    cfg = o2.Qwen2VisionConfig()
    ang = o2.rotary_angles(cfg, np.array([[1, 4, 4]]))
    inv = 1.0 / (10000.0 ** (torch.arange(0, 40, 2, dtype=torch.float) / 40))
    assert ang.shape == (16, 40)
    assert torch.equal(ang[0], torch.zeros(40))                                  # patch (0,0)
    assert torch.allclose(ang[1], torch.cat([torch.zeros(20), inv]))             # patch (0,1)
    assert torch.allclose(ang[2], torch.cat([inv, torch.zeros(20)]))             # patch (1,0)
    assert torch.allclose(ang[4], torch.cat([torch.zeros(20), 2 * inv]))         # next block: patch (0,2)
    # items are independent and frames of a video do not attend to each other
    o2_, cfg_s, ocfg, sd = _qwen2_small(depth=1, seed=9)
    px, grid = synth.qwen_inputs([(2, 4, 4), (1, 4, 6)], seed=9)
    both = o2.forward(sd, ocfg, px, grid)
    alone = o2.forward(sd, ocfg, px[1:], grid[1:])
    assert torch.allclose(both[1], alone[0], atol=1e-6)
    px2 = [px[0].clone(), px[1]]
    px2[0][16:] += 1.0                                                           # change the second frame group only
    pert = o2.forward(sd, ocfg, px2, grid)
    assert torch.equal(pert[0][:4], both[0][:4]) and not torch.allclose(pert[0][4:], both[0][4:])


# ------------------------------------------------------------------------------------------ Qwen3-VL
def _qwen3_small(depth=3, deepstack=(0, 2), out=1024, seed=6):
    from oracle import qwen3_vl as o3

    cfg = synth.qwen3_vision_config(depth=depth, deepstack_visual_indexes=deepstack, out_hidden_size=out)
    ocfg = o3.Qwen3VisionConfig(depth=depth, deepstack_visual_indexes=list(deepstack), out_hidden_size=out)
    return o3, cfg, ocfg, synth.qwen3_state_dict(cfg, seed=seed)


def test_qwen3_vl_against_golden(golden_dir):
    gold = np.load(golden_dir / "qwen3_vl_small.npz")
    o3, cfg, ocfg, sd = _qwen3_small(seed=int(gold["seed"]))
    px, grid = synth.qwen3_inputs([(1, 12, 20), (2, 8, 8)], seed=int(gold["seed"]))
    out = o3.forward(sd, ocfg, px, grid, dtype=torch.float32)
    assert [tuple(o.shape) for o in out] == [(60, 3072), (32, 3072)]      # main + two deepstack blocks of 1024
    o = torch.cat(out).numpy()
    assert np.abs(o[:, ::4] - gold["sample"]).max() <= 2e-4 * np.abs(gold["sample"]).max()
    assert np.allclose(np.linalg.norm(o.astype(np.float64), axis=1), gold["row_l2"], rtol=1e-4)


def test_qwen3_vl_live_against_hugging_face():
    pytest.importorskip("transformers.models.qwen3_vl.modeling_qwen3_vl")
    import sys
    from pathlib import Path
    sys.path.insert(0, str(Path(__file__).parent / "golden"))
    import make_golden

    o3, cfg, ocfg, sd = _qwen3_small(depth=2, deepstack=(1,), out=512, seed=10)
    px, grid = synth.qwen3_inputs([(1, 6, 10), (3, 4, 4)], seed=10)
    ref = make_golden.hf_qwen3_forward(cfg, sd, px, grid)
    got = torch.cat(o3.forward(sd, ocfg, px, grid, dtype=torch.float32))
    assert got.shape == ref.shape == ((60 + 48) // 4, 1024)
    assert (got - ref).abs().max().item() <= 2e-4 * ref.abs().max().item()


def test_qwen3_vl_position_interpolation_closed_forms():
    from oracle import qwen3_vl as o3

    side, E = 6, 8
    table = torch.arange(side * side * E, dtype=torch.float32).reshape(side * side, E)
    # a grid of the table's own size samples it exactly; rows come out in 2x2-block-major order
    got = o3.pos_embed_interpolate(table, np.array([[1, side, side]]), merge=2)
    order = [(by * 2 + my) * side + bx * 2 + mx for by in range(3) for bx in range(3) for my in range(2) for mx in range(2)]
    assert torch.equal(got, table[order])
    # two points per side: the four corners
    got = o3.pos_embed_interpolate(table, np.array([[1, 2, 2]]), merge=2)
    assert torch.equal(got, table[[0, side - 1, side * (side - 1), side * side - 1]])
    # a linear table is reproduced by bilinear interpolation at any resolution
    yy, xx = torch.meshgrid(torch.arange(side, dtype=torch.float32), torch.arange(side, dtype=torch.float32), indexing="ij")
    lin = (3.0 * yy + 0.5 * xx).reshape(-1, 1).repeat(1, E)
    got = o3.pos_embed_interpolate(lin, np.array([[2, 4, 10]]), merge=2)
    hs, ws = torch.linspace(0, side - 1, 4), torch.linspace(0, side - 1, 10)
    want = [3.0 * hs[by * 2 + my] + 0.5 * ws[bx * 2 + mx] for by in range(2) for bx in range(5) for my in range(2) for mx in range(2)]
    assert got.shape == (80, E) and torch.allclose(got[:40, 0], torch.stack(want), atol=1e-5)
    assert torch.equal(got[:40], got[40:])                       # repeated per frame


# ---------------------------------------------------------------------------------------------------------
# LLaVA-OneVision (oracle/llava_onevision.py)
# ---------------------------------------------------------------------------------------------------------
def _llava_small():
    from oracle import llava_onevision as ol

    cfg = synth.llava_ov_config(num_hidden_layers=2, image_size=70, text_hidden=256, max_grid=4)
    ocfg = ol.LlavaOneVisionConfig(vision=og.SiglipConfig(num_hidden_layers=2, image_size=70), text_hidden_size=256,
                                   image_grid_pinpoints=cfg.image_grid_pinpoints)
    return ol, cfg, ocfg


def test_llava_onevision_small_against_golden(golden_dir):
    """Five images (one tile grid each of 1x1, 2x4, 4x4 shrunk, 4x4 cropped and shrunk, 4x2 cropped) and two videos."""
    ol, cfg, ocfg = _llava_small()
    gold = np.load(golden_dir / "llava_onevision_small.npz")
    seed = int(gold["seed"])
    sd = synth.llava_ov_state_dict(cfg, seed=seed)
    sizes = [(70, 70), (100, 260), (280, 280), (211, 277), (277, 90)]
    px, szs = synth.llava_ov_image_inputs(cfg, sizes, seed=seed)
    out = ol.forward_images(sd, ocfg, px, szs)
    assert [tuple(o.shape) for o in out] == [(55, 256), (193, 256), (265, 256), (246, 256), (165, 256)]
    for i, o in enumerate(out):
        g = gold[f"image{i}"]
        assert np.abs(o.numpy() - g).max() <= 2e-4 * np.abs(g).max(), i
    vids = ol.forward_videos(sd, ocfg, synth.llava_ov_video_inputs(cfg, [2, 3], seed=seed))
    assert [tuple(v.shape) for v in vids] == [(1, 19, 256), (1, 28, 256)]
    for i, v in enumerate(vids):
        g = gold[f"video{i}"]
        assert np.abs(v.numpy() - g).max() <= 2e-4 * np.abs(g).max(), i
    with pytest.raises(RuntimeError, match="one frame"):
        ol.forward_videos(sd, ocfg, synth.llava_ov_video_inputs(cfg, [1], seed=seed))


def test_llava_onevision_geometry_against_installed_package():
    """select_best_resolution / get_anyres_image_grid_shape / unpad_image as the third-party package computes them."""
    m = pytest.importorskip("transformers.models.llava_onevision.modeling_llava_onevision")
    ol, cfg, _ = _llava_small()
    pins = [[384 * i, 384 * j] for i in range(1, 7) for j in range(1, 7)]
    rng = np.random.default_rng(3)
    sizes = [(int(h), int(w)) for h, w in rng.integers(20, 3000, size=(300, 2))]
    sizes += [(384, 384), (385, 384), (2304, 2304), (768, 383), (1, 200), (199, 1), (1000, 1001)]
    for h, w in sizes:
        th, tw = ol.anyres_grid_shape((h, w), pins, 384)
        assert (th, tw) == tuple(m.get_anyres_image_grid_shape((h, w), pins, 384)), (h, w)
        ch, cw = th * 27, tw * 27
        marks = torch.arange(ch * cw, dtype=torch.float32).view(1, ch, cw)
        kept = m.unpad_image(marks, (h, w))
        y0, y1, x0, x1 = ol.unpad_bounds(ch, cw, h, w)
        assert torch.equal(kept, marks[:, y0:y1, x0:x1]), (h, w)


def test_llava_onevision_bilinear_resize_is_torch_interpolate():
    from oracle import llava_onevision as ol

    torch.manual_seed(0)
    for (h, w), (oh, ow) in [((27, 27), (14, 14)), ((108, 81), (93, 70)), ((5, 9), (5, 4)), ((20, 20), (17, 17)),
                             ((162, 54), (141, 47)), ((3, 3), (7, 5))]:
        x = torch.randn(6, h, w)
        ref = F.interpolate(x[None], [oh, ow], mode="bilinear")[0]
        got = ol.bilinear_resize(x, oh, ow)
        assert torch.allclose(got, ref, rtol=0, atol=2e-5), ((h, w), (oh, ow), (got - ref).abs().max())  # fp32 rounding
    # a resize to the same size is the identity; a constant stays constant
    x = torch.randn(3, 9, 11)
    assert torch.equal(ol.bilinear_resize(x, 9, 11), x)
    c = torch.full((2, 8, 8), 1.25)
    assert torch.equal(ol.bilinear_resize(c, 5, 3), torch.full((2, 5, 3), 1.25))


def test_llava_onevision_merge_special_cases():
    """A single tile is the tile plus one newline; a 1x1 grid of a square image is the tile, then the tile again with a
    newline behind each of its rows; the newline count equals the number of grid rows kept."""
    ol, cfg, ocfg = _llava_small()
    torch.manual_seed(1)
    nl = torch.randn(8)
    one = torch.randn(1, 25, 8)
    out = ol.merge_image(ocfg, one, (70, 70), nl)
    assert torch.equal(out[:25], one[0]) and torch.equal(out[25], nl) and out.shape[0] == 26
    two = torch.randn(2, 25, 8)
    out = ol.merge_image(ocfg, two, (70, 70), nl)
    assert out.shape[0] == 25 + 5 * 6
    assert torch.equal(out[:25], two[0])
    rows = out[25:].view(5, 6, 8)
    assert torch.equal(rows[:, :5].reshape(25, 8), two[1]) and torch.equal(rows[:, 5], nl.expand(5, 8))
    # a wide image in a 2x4 grid: rows cropped symmetrically, every kept row ends with the newline
    tiles = torch.randn(9, 25, 8)
    out = ol.merge_image(ocfg, tiles, (100, 260), nl)
    kept = (out.shape[0] - 25) // 21
    assert (out.shape[0] - 25) % 21 == 0 and 0 < kept <= 10
    assert torch.equal(out[25:].view(kept, 21, 8)[:, 20], nl.expand(kept, 8))
    with pytest.raises(ValueError, match="not consistent"):
        ol.merge_image(ocfg, torch.randn(2, 24, 8), (70, 70), nl)


def test_distance_measures_known_answers():
    """oracle.metrics.distances on cases with closed-form answers (a wrong normaliser, a missed row or an fp32
    reduction would fail one of them)."""
    from oracle.metrics import distances

    ref = torch.tensor([[3.0, 4.0], [0.0, 2.0], [1.0, 0.0]])
    d = distances(ref.clone(), ref)
    assert d == {"cosine": 1.0, "max_rel_err": 0.0, "min_row_cosine": 1.0, "max_row_rel_l2": 0.0}
    got = ref.clone()
    got[1] = torch.tensor([2.0, 0.0])                    # one row rotated by 90 degrees, same norm
    d = distances(got, ref)
    assert abs(d["min_row_cosine"]) < 1e-15 and abs(d["max_row_rel_l2"] - 2**0.5) < 1e-12
    assert abs(d["max_rel_err"] - 2.0 / 4.0) < 1e-15     # |err| max 2 against the largest reference magnitude 4
    assert abs(d["cosine"] - 26.0 / 30.0) < 1e-12        # (25 + 0 + 1) / (sqrt(30) sqrt(30))
    big = torch.full((4000, 2000), 1.0 + 2.0**-12)       # an fp32 dot product of 8M equal terms drifts above 1
    c = distances(big, big)["cosine"]
    assert c <= 1.0 and 1.0 - c < 1e-12
    with pytest.raises(ValueError):
        distances(ref, ref[:2])


def test_oracle_linear_in_a_second_summation_order():
    """`linear_mode="fp32_accumulate"` is the same network: identical in fp32, and in bf16 within the rounding noise of
    one shallow pass (the two modes differ in the order of the fp32 accumulation only)."""
    cfg = synth.qwen_vision_config(depth=2, fullatt_block_indexes=(1,))
    sd = synth.qwen_state_dict(cfg, seed=3)
    ocfg = oq.QwenVisionConfig(depth=2, fullatt_block_indexes=[1])
    px, grid = synth.qwen_inputs([(1, 8, 12)], seed=3)
    a = oq.forward(sd, ocfg, px, grid, dtype=torch.float32)[0]
    b = oq.forward(sd, ocfg, px, grid, dtype=torch.float32, linear_mode="fp32_accumulate")[0]
    assert torch.equal(a, b)
    a16 = oq.forward(sd, ocfg, px, grid, dtype=torch.bfloat16)[0].float()
    b16 = oq.forward(sd, ocfg, px, grid, dtype=torch.bfloat16, linear_mode="fp32_accumulate")[0].float()
    assert (a16 - b16).abs().max() <= 1e-2 * a.abs().max() and (b16 - a).abs().max() <= 1e-2 * a.abs().max()
    with pytest.raises(ValueError):
        oq.forward(sd, ocfg, px, grid, linear_mode="other")
