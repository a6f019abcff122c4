"""Writes the golden fixtures in this directory.  Run once, in a container that has `transformers`:

    python tests/golden/make_golden.py

Source of truth: the third-party Hugging Face implementations of the same networks, which are what the
reference's own tests compare Eric against (python/tests/task_executors/eric/models/test_qwen2_5_vl.py:
63-105, test_gemma3.py:73-97).  The reference package itself is not imported (it needs Python >= 3.11,
flash-attn and xformers).  Models are built from local config objects with the seeded synthetic weights
of cornserve_amd.synth, fp32, CPU, eager/sdpa attention.  Outputs:

    index_golden.json        window_index / cu_window_seqlens / cu_seqlens / position ids from
                             transformers.vision_utils for the benchmark grids and a set of ragged grids
                             (full arrays for small grids, sha256 + head for large ones)
    qwen2_5_vl_cfg1.npz      config 1 (4 blocks, one 448x448 image): every 16th column of the [256,3584]
                             output, per-row L2 norms, sum and abs-sum
    qwen2_vl_small.npz       2-block Qwen2-VL tower (width 1280), an image (1,16,16) and a video (2,8,12): every 8th
                             column of the [112,3584] output, per-row L2 norms, sum
    qwen3_vl_small.npz       3-block Qwen3-VL tower (width 1152, deepstack after blocks 0 and 2, output width 1024), an
                             image (1,12,20) and a video (2,8,8): every 4th column of the [92,3072] output, row norms, sum
    gemma3_small.npz         2-layer SigLIP (224x224, 256 tokens) + projector to 16 tokens x 640: full output
"""

from __future__ import annotations

import hashlib
import json
import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))

from tests import synth  # noqa: E402

INDEX_GRIDS = {
    "cfg1": [(1, 32, 32)],
    "cfg2": [(1, 32, 32)] * 8,
    "cfg5": [(8, 24, 42)] * 2,
    "cfg4_ragged16": synth.ragged_grids(16, seed=4),
    "tiny_mixed": [(1, 4, 4), (2, 6, 10), (1, 18, 14), (3, 2, 2), (1, 8, 16), (1, 10, 6)],
    "edge_exact_multiple": [(1, 8, 8), (1, 16, 24), (2, 8, 40)],
    "edge_single_unit": [(1, 2, 2), (1, 2, 34), (1, 34, 2)],
}


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def make_index() -> None:
    from transformers import vision_utils as vu

    out = {}
    for name, grids in INDEX_GRIDS.items():
        g = torch.tensor(grids, dtype=torch.int64)
        wi, cu_w = vu.get_vision_window_index(g, spatial_merge_size=2, window_size=112, patch_size=14)
        pos = vu.get_vision_position_ids(g, 2)
        cu_f = vu.get_vision_cu_seqlens(g)
        wi, cu_w, pos, cu_f = (np.asarray(t.cpu()) for t in (wi, cu_w, pos, cu_f))
        rec = {
            "grids": [list(x) for x in grids],
            "window_index_len": int(wi.shape[0]),
            "window_index_sha256_int64": sha(wi.astype(np.int64)),
            "cu_window_seqlens": cu_w.astype(np.int64).tolist(),
            "cu_seqlens": cu_f.astype(np.int64).tolist(),
            "pos_ids_shape": list(pos.shape),
            "pos_ids_sha256_int64": sha(pos.astype(np.int64)),
        }
        if wi.shape[0] <= 4096:
            rec["window_index"] = wi.astype(np.int64).tolist()
        else:
            rec["window_index_head"] = wi[:64].astype(np.int64).tolist()
        if pos.shape[0] <= 2048:
            rec["pos_ids"] = pos.astype(np.int64).tolist()
        out[name] = rec
    (HERE / "index_golden.json").write_text(json.dumps(out))
    print("index_golden.json", {k: v["window_index_len"] for k, v in out.items()})


def make_qwen_cfg1() -> None:
    from transformers.models.qwen2_5_vl.configuration_qwen2_5_vl import Qwen2_5_VLVisionConfig
    from transformers.models.qwen2_5_vl.modeling_qwen2_5_vl import Qwen2_5_VisionTransformerPretrainedModel

    cfg = synth.qwen_vision_config(depth=4, fullatt_block_indexes=(3,))
    vc = cfg.vision_config
    hf_cfg = Qwen2_5_VLVisionConfig(
        depth=vc.depth, hidden_size=vc.hidden_size, intermediate_size=vc.intermediate_size, num_heads=vc.num_heads,
        out_hidden_size=vc.out_hidden_size, fullatt_block_indexes=list(vc.fullatt_block_indexes),
        window_size=vc.window_size, patch_size=vc.patch_size, spatial_merge_size=vc.spatial_merge_size,
        temporal_patch_size=vc.temporal_patch_size, hidden_act="silu",
    )
    hf_cfg._attn_implementation = "sdpa"
    model = Qwen2_5_VisionTransformerPretrainedModel(hf_cfg).float().eval()
    sd = synth.qwen_state_dict(cfg, seed=1)
    inc = model.load_state_dict(sd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys, inc
    px, grid = synth.qwen_inputs([(1, 32, 32)], seed=1)
    with torch.no_grad():
        out = model(px[0], grid_thw=grid[0]).pooler_output.float().numpy()
    assert out.shape == (256, 3584)
    np.savez_compressed(
        HERE / "qwen2_5_vl_cfg1.npz",
        sample=out[:, ::16].astype(np.float32),
        row_l2=np.linalg.norm(out.astype(np.float64), axis=1).astype(np.float32),
        total=np.float64(out.astype(np.float64).sum()),
        abs_total=np.float64(np.abs(out.astype(np.float64)).sum()),
        seed=np.int64(1),
    )
    print("qwen2_5_vl_cfg1.npz", out.shape, float(np.abs(out).mean()))


def make_qwen2_vl_small() -> None:
    from transformers.models.qwen2_vl.configuration_qwen2_vl import Qwen2VLVisionConfig
    from transformers.models.qwen2_vl.modeling_qwen2_vl import Qwen2VisionTransformerPretrainedModel

    cfg = synth.qwen2_vision_config(depth=2)
    vc = cfg.vision_config
    hf_cfg = Qwen2VLVisionConfig(depth=vc.depth, embed_dim=vc.embed_dim, hidden_size=vc.hidden_size, num_heads=vc.num_heads,
                                 mlp_ratio=int(vc.mlp_ratio), patch_size=vc.patch_size, spatial_merge_size=vc.spatial_merge_size,
                                 temporal_patch_size=vc.temporal_patch_size, hidden_act="quick_gelu")
    hf_cfg._attn_implementation = "sdpa"
    model = Qwen2VisionTransformerPretrainedModel(hf_cfg).float().eval()
    sd = synth.qwen2_state_dict(cfg, seed=3)
    inc = model.load_state_dict(sd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys, inc
    grids = [(1, 16, 16), (2, 8, 12)]
    px, grid = synth.qwen_inputs(grids, seed=3)
    with torch.no_grad():
        out = model(torch.cat(px), grid_thw=torch.cat(grid))
    out = (out.pooler_output if hasattr(out, "pooler_output") else out).float().numpy()
    assert out.shape == ((256 + 192) // 4, 3584), out.shape
    np.savez_compressed(HERE / "qwen2_vl_small.npz", sample=out[:, ::8].astype(np.float32),
                        row_l2=np.linalg.norm(out.astype(np.float64), axis=1).astype(np.float32),
                        total=np.float64(out.astype(np.float64).sum()), seed=np.int64(3))
    print("qwen2_vl_small.npz", out.shape, float(np.abs(out).mean()))


def _hf_qwen3(cfg):
    from transformers.models.qwen3_vl.configuration_qwen3_vl import Qwen3VLVisionConfig
    from transformers.models.qwen3_vl.modeling_qwen3_vl import Qwen3VLVisionModel

    vc = cfg.vision_config
    hf_cfg = Qwen3VLVisionConfig(depth=vc.depth, hidden_size=vc.hidden_size, hidden_act=vc.hidden_act,
                                 intermediate_size=vc.intermediate_size, num_heads=vc.num_heads, in_channels=vc.in_channels,
                                 patch_size=vc.patch_size, spatial_merge_size=vc.spatial_merge_size,
                                 temporal_patch_size=vc.temporal_patch_size, out_hidden_size=vc.out_hidden_size,
                                 num_position_embeddings=vc.num_position_embeddings,
                                 deepstack_visual_indexes=list(vc.deepstack_visual_indexes))
    hf_cfg._attn_implementation = "sdpa"
    return Qwen3VLVisionModel(hf_cfg).float().eval()


def hf_qwen3_forward(cfg, sd, px, grid) -> torch.Tensor:
    """[L/4, out * (1 + n_deepstack)]: the main output with the deepstack features behind it, as the reference
    concatenates them (eric/models/qwen3_vl.py:300-311)."""
    model = _hf_qwen3(cfg)
    inc = model.load_state_dict(sd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys, inc
    with torch.no_grad():
        out = model(torch.cat(px), grid_thw=torch.cat(grid))
    return torch.cat([out.pooler_output, *out.deepstack_features], dim=1).float()


def make_qwen3_vl_small() -> None:
    cfg = synth.qwen3_vision_config(depth=3, deepstack_visual_indexes=(0, 2), out_hidden_size=1024)
    sd = synth.qwen3_state_dict(cfg, seed=6)
    px, grid = synth.qwen3_inputs([(1, 12, 20), (2, 8, 8)], seed=6)
    out = hf_qwen3_forward(cfg, sd, px, grid).numpy()
    assert out.shape == ((240 + 128) // 4, 3 * 1024), out.shape
    np.savez_compressed(HERE / "qwen3_vl_small.npz", sample=out[:, ::4].astype(np.float32),
                        row_l2=np.linalg.norm(out.astype(np.float64), axis=1).astype(np.float32),
                        total=np.float64(out.astype(np.float64).sum()), seed=np.int64(6))
    print("qwen3_vl_small.npz", out.shape, float(np.abs(out).mean()))


def make_gemma3_small() -> None:
    from transformers.models.gemma3.configuration_gemma3 import Gemma3Config, Gemma3TextConfig
    from transformers.models.gemma3.modeling_gemma3 import Gemma3MultiModalProjector
    from transformers.models.siglip.configuration_siglip import SiglipVisionConfig
    from transformers.models.siglip.modeling_siglip import SiglipVisionModel

    cfg = synth.gemma3_config(num_hidden_layers=2, image_size=224, text_hidden=640, mm_tokens_per_image=16)
    vc = cfg.vision_config
    hf_vc = SiglipVisionConfig(
        hidden_size=vc.hidden_size, intermediate_size=vc.intermediate_size, num_hidden_layers=vc.num_hidden_layers,
        num_attention_heads=vc.num_attention_heads, image_size=vc.image_size, patch_size=vc.patch_size,
        hidden_act=vc.hidden_act, layer_norm_eps=vc.layer_norm_eps, vision_use_head=False,
    )
    hf_vc._attn_implementation = "sdpa"
    tower = SiglipVisionModel(hf_vc).float().eval()
    g3 = Gemma3Config(vision_config=hf_vc, text_config=Gemma3TextConfig(hidden_size=640), mm_tokens_per_image=16)
    proj = Gemma3MultiModalProjector(g3).float().eval()
    sd = synth.gemma3_state_dict(cfg, seed=2)
    # HF's SiglipVisionModel in this version is flat (no `vision_model.` level).
    tower_keys = set(tower.state_dict().keys())
    prefix = "vision_tower.vision_model." if not any(k.startswith("vision_model.") for k in tower_keys) else "vision_tower."
    tsd = {k[len(prefix):]: v for k, v in sd.items() if k.startswith("vision_tower.")}
    inc = tower.load_state_dict(tsd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys, inc
    psd = {k[len("multi_modal_projector."):]: v for k, v in sd.items() if k.startswith("multi_modal_projector.")}
    inc = proj.load_state_dict(psd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys, inc
    px, _ = synth.gemma3_inputs(2, 224, seed=2)
    with torch.no_grad():
        feats = tower(pixel_values=torch.cat(px)).last_hidden_state
        out = proj(feats).float().numpy()
    assert out.shape == (2, 16, 640), out.shape
    np.savez_compressed(HERE / "gemma3_small.npz", out=out.astype(np.float32),
                        feats_sample=feats.float().numpy()[:, ::8, ::8].astype(np.float32), seed=np.int64(2))
    print("gemma3_small.npz", out.shape, float(np.abs(out).mean()))


def _hf_llava_onevision(cfg):
    """The installed Hugging Face LlavaOnevisionModel with `cfg`'s vision tower and a minimal language model (unused)."""
    from transformers.models.llava_onevision.configuration_llava_onevision import LlavaOnevisionConfig
    from transformers.models.llava_onevision.modeling_llava_onevision import LlavaOnevisionModel
    from transformers.models.qwen2.configuration_qwen2 import Qwen2Config
    from transformers.models.siglip.configuration_siglip import SiglipVisionConfig

    vc = cfg.vision_config
    hf_vc = SiglipVisionConfig(
        hidden_size=vc.hidden_size, intermediate_size=vc.intermediate_size, num_hidden_layers=vc.num_hidden_layers,
        num_attention_heads=vc.num_attention_heads, image_size=vc.image_size, patch_size=vc.patch_size,
        hidden_act=vc.hidden_act, layer_norm_eps=vc.layer_norm_eps, vision_use_head=False,
    )
    text = Qwen2Config(hidden_size=cfg.text_config.hidden_size, intermediate_size=64, num_hidden_layers=1,
                       num_attention_heads=2, num_key_value_heads=2, vocab_size=64)
    hf_cfg = LlavaOnevisionConfig(
        vision_config=hf_vc, text_config=text, vision_feature_layer=cfg.vision_feature_layer,
        vision_feature_select_strategy=cfg.vision_feature_select_strategy, projector_hidden_act=cfg.projector_hidden_act,
        image_grid_pinpoints=cfg.image_grid_pinpoints, vision_aspect_ratio=cfg.vision_aspect_ratio,
        multimodal_projector_bias=cfg.multimodal_projector_bias,
    )
    hf_cfg._attn_implementation = "sdpa"
    return LlavaOnevisionModel(hf_cfg).float().eval()


def hf_llava_onevision_forward(cfg, sd, px, sizes, videos):
    """(per-image sequences, per-video sequences) from the Hugging Face implementation."""
    model = _hf_llava_onevision(cfg)
    own = model.state_dict()
    flat_tower = not any(k.startswith("vision_tower.vision_model.") for k in own)
    mapped = {}
    for k, v in sd.items():
        if flat_tower and k.startswith("vision_tower.vision_model."):
            k = "vision_tower." + k[len("vision_tower.vision_model."):]
        mapped[k] = v
    inc = model.load_state_dict(mapped, strict=False)
    bad = [k for k in inc.missing_keys if not k.startswith("language_model.") and "post_layernorm" not in k
           and ".head." not in k]
    assert not bad and not inc.unexpected_keys, (bad, inc.unexpected_keys)
    S = cfg.vision_config.image_size
    with torch.no_grad():
        # images: padded to the largest tile count, as the Hugging Face processor batches them
        most = max(p.shape[0] for p in px)
        batch = torch.zeros(len(px), most, 3, S, S)
        for i, p in enumerate(px):
            batch[i, : p.shape[0]] = p
        image_sizes = torch.stack(sizes)
        out = model.get_image_features(pixel_values=batch, image_sizes=image_sizes)
        feats = out.pooler_output if hasattr(out, "pooler_output") else out
        feats = [f[: p.shape[0]] for f, p in zip(feats, px)] if isinstance(feats, (list, tuple)) and feats[0].dim() == 3 else feats
        if isinstance(feats, (list, tuple)) and feats[0].dim() == 3:
            images, _ = model.pack_image_features(list(feats), image_sizes, image_newline=model.image_newline,
                                                  vision_aspect_ratio=cfg.vision_aspect_ratio)
        else:  # this version already packs inside get_image_features
            images = list(feats)
        vids = []
        for v in videos:
            vo = model.get_video_features(pixel_values=v[None])
            vf = vo.pooler_output if hasattr(vo, "pooler_output") else vo
            vf = vf.reshape(1, -1, vf.shape[-1])
            vids.append(torch.cat([vf, model.image_newline[None, None, :]], dim=1))
    return [t.float() for t in images], [t.float() for t in vids]


LLAVA_OV_SMALL_SIZES = [(70, 70), (100, 260), (280, 280), (211, 277), (277, 90)]
LLAVA_OV_SMALL_FRAMES = [2, 3]


def llava_onevision_small_case():
    cfg = synth.llava_ov_config(num_hidden_layers=2, image_size=70, text_hidden=256, max_grid=4)
    sd = synth.llava_ov_state_dict(cfg, seed=5)
    px, sizes = synth.llava_ov_image_inputs(cfg, LLAVA_OV_SMALL_SIZES, seed=5)
    videos = synth.llava_ov_video_inputs(cfg, LLAVA_OV_SMALL_FRAMES, seed=5)
    return cfg, sd, px, sizes, videos


def make_llava_onevision_small() -> None:
    cfg, sd, px, sizes, videos = llava_onevision_small_case()
    images, vids = hf_llava_onevision_forward(cfg, sd, px, sizes, videos)
    arrays = {f"image{i}": t.numpy().astype(np.float32) for i, t in enumerate(images)}
    arrays.update({f"video{i}": t.numpy().astype(np.float32) for i, t in enumerate(vids)})
    np.savez_compressed(HERE / "llava_onevision_small.npz", seed=np.int64(5), **arrays)
    print("llava_onevision_small.npz", [a.shape for a in arrays.values()])


if __name__ == "__main__":
    make_index()
    make_qwen_cfg1()
    make_qwen2_vl_small()
    make_qwen3_vl_small()
    make_gemma3_small()
    make_llava_onevision_small()
