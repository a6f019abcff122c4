"""Host-side mirror of the Eric model interface (CPU only): names, registry, error behaviour."""

import importlib

import numpy as np
import pytest
import torch

from tests import synth
from cornserve_amd.eric.api import Modality
from cornserve_amd.eric.models import base, registry
from cornserve_amd.eric.models.gemma3 import Gemma3VisionEncoder
from cornserve_amd.eric.models.qwen2_5_vl import Qwen2_5_VisionTransformer


def test_registry_resolves_like_the_reference_loader():
    for model_type in registry.MODEL_REGISTRY:
        entry = registry.MODEL_REGISTRY[model_type]
        module = importlib.import_module(f"cornserve_amd.eric.models.{entry.module}")
        cls = getattr(module, entry.class_name)
        assert issubclass(cls, base.EricModel)
        assert issubclass(module.ModalityProcessor, base.BaseModalityProcessor)
    with pytest.raises(ValueError):
        registry.RegistryEntry("m", "C", "adapter", registry.ViTResolutionType.FIXED,
                               registry.WeightInfo(required_prefixes=["x."]), {})


def test_qwen_state_dict_names_and_properties():
    cfg = synth.qwen_vision_config(depth=2, fullatt_block_indexes=(1,))
    with torch.device("meta"):
        model = Qwen2_5_VisionTransformer(cfg)
    names = set(model.state_dict().keys())
    assert names == set(synth.qwen_state_dict(cfg).keys())
    expect = {"patch_embed.proj.weight", "blocks.0.norm1.weight", "blocks.1.attn.qkv.bias", "blocks.0.mlp.down_proj.weight",
              "merger.ln_q.weight", "merger.mlp.0.weight", "merger.mlp.2.bias"}
    assert expect <= names
    assert model.state_dict()["patch_embed.proj.weight"].shape == (1280, 3, 2, 14, 14)
    assert model.chunk_shape == (1, 3584)
    assert model.device.type == "meta"


def test_qwen_loads_checkpoint_names_strictly():
    cfg = synth.qwen_vision_config(depth=1, fullatt_block_indexes=(0,))
    model = Qwen2_5_VisionTransformer(cfg)
    sd = synth.qwen_state_dict(cfg, seed=0)
    inc = model.load_state_dict(sd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys
    assert torch.equal(model.blocks[0].attn.qkv.weight, sd["blocks.0.attn.qkv.weight"])


def test_qwen_errors():
    cfg = synth.qwen_vision_config(depth=1, fullatt_block_indexes=(0,))
    model = Qwen2_5_VisionTransformer(cfg)
    with pytest.raises(ValueError, match="Unsupported modality"):
        model(Modality.AUDIO, "", {})
    px, grid = synth.qwen_inputs([(1, 4, 4)])
    # fp32 on the CPU: the kernels have no CPU path and must say so instead of silently falling back
    with pytest.raises(RuntimeError, match="no CPU path"):
        model(Modality.IMAGE, "", {"pixel_values": px, "image_grid_thw": grid})
    with pytest.raises(ValueError):
        Qwen2_5_VisionTransformer(cfg, weight_format="int4")


def test_gemma3_names_adapters_and_errors():
    cfg = synth.gemma3_config(num_hidden_layers=1, image_size=56, text_hidden=64, mm_tokens_per_image=4)
    model = Gemma3VisionEncoder(cfg)
    sd = synth.gemma3_state_dict(cfg, seed=0)
    synth.load_gemma3(model, sd, adapter_name="google/gemma-3-4b-it")
    assert model.chunk_shape == (1, 4, 256)
    assert set(model.state_dict().keys()) == {k for k in sd if k.startswith("vision_tower.")}
    adapter = model.multi_modal_projector.adapters["google/gemma-3-4b-it"]
    assert set(adapter.state_dict().keys()) == {"mm_input_projection_weight", "mm_soft_emb_norm.weight"}
    px, crops = synth.gemma3_inputs(1, 56)
    with pytest.raises(ValueError, match="Unsupported modality"):
        model(Modality.VIDEO, "google/gemma-3-4b-it", {"pixel_values": px, "num_crops": crops})
    with pytest.raises(ValueError, match="Adapter name"):
        model(Modality.IMAGE, None, {"pixel_values": px, "num_crops": crops})
    with pytest.raises(AssertionError):
        model(Modality.IMAGE, "google/gemma-3-4b-it", {"pixel_values": [torch.zeros(1, 3, 28, 28)], "num_crops": crops})
    with pytest.raises(ValueError, match="not found"):
        model.multi_modal_projector("nope", torch.zeros(1))


def test_modality_is_a_str_enum():
    assert Modality.IMAGE == "image" and str(Modality.VIDEO) == "video" and Modality("audio") is Modality.AUDIO


# ------------------------------------------------------------------ uint8-frame input format (host side)
def test_frame_processor_resize_and_table_match_the_hf_pil_processor():
    """FrameModalityProcessor's resize + the byte table + the oracle's layout reproduce the Hugging Face PIL
    processor's pixel_values bit for bit on images that DO need resampling."""
    import numpy as np
    pytest.importorskip("PIL")
    mod = pytest.importorskip("transformers.models.qwen2_vl.image_processing_pil_qwen2_vl")
    from cornserve_amd.eric import frames as fr
    from cornserve_amd.eric.api import Modality
    from cornserve_amd.eric.models.qwen2_5_vl import FrameModalityProcessor
    from oracle import qwen_preprocess as qp

    hf = mod.Qwen2VLImageProcessorPil()
    proc = FrameModalityProcessor("unused")
    rng = np.random.default_rng(5)
    for h, w in [(50, 70), (33, 200), (448, 448), (301, 517)]:
        img = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
        ref = hf(images=[img], return_tensors="np")
        out = proc.process(Modality.IMAGE, img)["pixel_frames"]
        assert out.dtype == torch.uint8 and out.shape[0] == 1 and out.shape[3] == 3
        assert tuple(out.shape[1:3]) == fr.target_size(h, w) == qp.smart_resize(h, w)
        table = fr.byte_table(arithmetic="numpy").numpy()
        assert np.array_equal(table, qp.normalization_table(arithmetic="numpy"))
        px, grid = qp.patchify_frames(out.numpy(), table)
        assert grid == tuple(ref["image_grid_thw"][0]) and np.array_equal(px, ref["pixel_values"])
    assert np.array_equal(fr.byte_table(arithmetic="fused").numpy(), qp.normalization_table(arithmetic="fused"))
    raw = FrameModalityProcessor("unused", min_pixels=3136, max_pixels=200704, resize_on="gpu")
    img = rng.integers(0, 256, (301, 517, 3), dtype=np.uint8)
    out = raw.process(Modality.IMAGE, img)
    assert torch.equal(out["raw_frames"], torch.from_numpy(img[None])) and out["raw_frames_budget"].tolist() == [3136, 200704]
    out = raw.process(Modality.VIDEO, np.stack([img, img]))
    assert out["raw_frames_videos"].shape == (2, 301, 517, 3)
    with pytest.raises(ValueError):
        raw.process(Modality.IMAGE, np.zeros((1, 500, 3), np.uint8))   # aspect ratio beyond the processor's limit
    with pytest.raises(ValueError):
        FrameModalityProcessor("unused", resize_on="host")
    with pytest.raises(ValueError):
        fr.resize_frames(np.zeros((4, 4), np.uint8))
    with pytest.raises(ValueError):
        fr.target_size(1, 500)


def test_qwen2_vl_class_surface():
    from tests import synth
    from cornserve_amd.eric.models.qwen2_vl import Qwen2VisionTransformer
    from cornserve_amd.eric.models.registry import MODEL_REGISTRY

    cfg = synth.qwen2_vision_config(depth=2)
    model = Qwen2VisionTransformer(cfg)
    sd = synth.qwen2_state_dict(cfg, seed=0)
    inc = model.load_state_dict(sd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys          # the checkpoint's names, nothing else
    assert model.chunk_shape == (1, 3584) and model.dtype == torch.float32 and model.device.type == "cpu"
    entry = MODEL_REGISTRY["qwen2_vl"]
    assert entry.module == "qwen2_vl" and entry.class_name == "Qwen2VisionTransformer" and entry.weight.required_prefixes == ["visual."]
    with pytest.raises(RuntimeError):                                # no CPU path
        model._ensure_packed()
    with pytest.raises(ValueError):
        Qwen2VisionTransformer(cfg, weight_format="int4")


def test_qwen3_vl_class_surface():
    from tests import synth
    from cornserve_amd.eric.models.qwen3_vl import Qwen3_VisionTransformer
    from cornserve_amd.eric.models.registry import MODEL_REGISTRY

    cfg = synth.qwen3_vision_config(depth=2, deepstack_visual_indexes=(0,))
    model = Qwen3_VisionTransformer(cfg)
    sd = synth.qwen3_state_dict(cfg, seed=0)          # Conv3d-shaped patch weight, as in the checkpoint
    inc = model.load_state_dict(sd, strict=False)
    assert not inc.missing_keys and not inc.unexpected_keys
    assert model.patch_embed.proj.weight.shape == (1152, 1536)
    assert model.chunk_shape == (1, 4096 * 2)
    for key in ("qwen3_vl", "qwen3_vl_moe"):
        entry = MODEL_REGISTRY[key]
        assert entry.module == "qwen3_vl" and entry.class_name == "Qwen3_VisionTransformer"
        assert entry.weight.required_prefixes == ["model.visual."]
    with pytest.raises(RuntimeError):
        model._ensure_packed()
    bad = synth.qwen3_vision_config(depth=1)
    bad.vision_config.hidden_act = "relu6"
    with pytest.raises(NotImplementedError):
        Qwen3_VisionTransformer(bad)


def test_worker_hands_embeddings_to_the_mock_sidecar(tmp_path, monkeypatch):
    """Host logic of the hand-off (the reference's Worker.execute_model + the sidecar client's mock mode)."""
    from cornserve_amd.eric.api import Modality
    from cornserve_amd.eric.worker import MockSidecar, Worker, WorkerBatch

    class FakeModel:
        def __call__(self, modality, adapter_name, batch):
            return [x.float() * 2 for x in batch["pixel_values"]]

    mapping = {"a-0": str(tmp_path / "a.pt"), "b-1": str(tmp_path / "b.pt")}
    monkeypatch.setenv("CORNSERVE_MOCK_SIDECAR", "1")
    monkeypatch.setenv("CORNSERVE_MOCK_SIDECAR_MAPPING", __import__("json").dumps(mapping))
    worker = Worker(FakeModel())
    assert isinstance(worker.sender_sidecar_client, MockSidecar)
    xs = [torch.arange(6.0).reshape(2, 3), torch.ones(1, 3), torch.zeros(4, 3)]
    batch = WorkerBatch(modality=Modality.IMAGE, adapter_name="", request_ids=["r", "r", "s"], data_ids=["a", "b", "c"],
                        chunk_ids=[0, 1, 0], num_chunks=[1, 2, 1], receiver_ranks=[[[1]], [[2, 3]], None],
                        data={"pixel_values": xs})
    out = worker.execute_model(batch)
    assert len(out) == 3
    assert torch.equal(torch.load(tmp_path / "a.pt", weights_only=True), xs[0] * 2)
    assert torch.equal(torch.load(tmp_path / "b.pt", weights_only=True), xs[1] * 2)
    assert not (tmp_path / "c.pt").exists()                          # no receiver: nothing sent
    batch.data_ids[0] = "zzz"
    with pytest.raises(ValueError):                                  # key not in the mapping
        worker.execute_model(batch)
    batch.chunk_ids = [0]
    with pytest.raises(ValueError):
        worker.execute_model(batch)
    MockSidecar({"j-0": tmp_path / "j.json"}).send({"k": 1}, "j", [[0]])
    assert (tmp_path / "j.json").read_text() == '{"k": 1}'


# ------------------------------------------------------------------ loading from a local checkpoint directory
def _ns_to_dict(o):
    from types import SimpleNamespace
    if isinstance(o, SimpleNamespace):
        return {k: _ns_to_dict(v) for k, v in vars(o).items()}
    return o


def _write_checkpoint(directory, config, tensors: dict, shards: int = 2, with_index: bool = True):
    import json
    from safetensors.torch import save_file

    directory.mkdir(parents=True, exist_ok=True)
    cfg = _ns_to_dict(config)
    cfg.setdefault("dtype", "float32")
    (directory / "config.json").write_text(json.dumps(cfg))
    names = sorted(tensors)
    weight_map = {}
    for s in range(shards):
        part = {n: tensors[n].contiguous() for n in names[s::shards]}
        fname = f"model-{s + 1:05d}-of-{shards:05d}.safetensors"
        save_file(part, str(directory / fname))
        weight_map.update({n: fname for n in part})
    if with_index:
        (directory / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))


def test_load_model_from_local_checkpoint(tmp_path):
    from tests import synth
    from cornserve_amd.eric.loader import load_model
    from cornserve_amd.eric.models.gemma3 import Gemma3VisionEncoder
    from cornserve_amd.eric.models.qwen2_5_vl import Qwen2_5_VisionTransformer

    cpu = torch.device("cpu")
    # Qwen2.5-VL: `visual.` weights among language-model weights, two shards with an index
    cfg = synth.qwen_vision_config(depth=2, fullatt_block_indexes=(1,))
    sd = synth.qwen_state_dict(cfg, seed=3)
    ckpt = {"visual." + k: v for k, v in sd.items()}
    ckpt.update({"model.layers.0.mlp.up_proj.weight": torch.zeros(4, 4), "lm_head.weight": torch.ones(2, 2)})
    _write_checkpoint(tmp_path / "qwen", cfg, ckpt)
    model = load_model(tmp_path / "qwen", torch_device=cpu)
    assert isinstance(model, Qwen2_5_VisionTransformer) and not model.training and model.dtype == torch.float32
    assert torch.equal(model.blocks[1].attn.qkv.weight, sd["blocks.1.attn.qkv.weight"])
    assert load_model(tmp_path / "qwen", torch_device=cpu, torch_dtype=torch.bfloat16).dtype == torch.bfloat16
    assert load_model(tmp_path / "qwen", torch_device=cpu, weight_format="fp8_e4m3").weight_format == "fp8_e4m3"
    # a missing weight and an unexpected one are errors, as in the reference
    bad = dict(ckpt)
    del bad["visual.merger.ln_q.weight"]
    _write_checkpoint(tmp_path / "qwen_missing", cfg, bad, shards=1, with_index=False)
    with pytest.raises(ValueError, match="Missing weights"):
        load_model(tmp_path / "qwen_missing", torch_device=cpu)
    bad = dict(ckpt)
    bad["visual.extra.weight"] = torch.zeros(1)
    _write_checkpoint(tmp_path / "qwen_extra", cfg, bad, shards=1, with_index=False)
    with pytest.raises(ValueError, match="Unexpected weights"):
        load_model(tmp_path / "qwen_extra", torch_device=cpu)
    with pytest.raises(FileNotFoundError):
        load_model(tmp_path / "nowhere", torch_device=cpu)
    unknown = synth.qwen_vision_config(depth=1)
    unknown.model_type = "no_such_model"
    _write_checkpoint(tmp_path / "unknown", unknown, {"visual.x": torch.zeros(1)}, shards=1)
    with pytest.raises(KeyError):
        load_model(tmp_path / "unknown", torch_device=cpu)

    # Gemma-3: tower weights into the model (post_layernorm ignored), projector weights into an adapter per directory
    gcfg = synth.gemma3_config(num_hidden_layers=1, image_size=56, text_hidden=64, mm_tokens_per_image=4)
    gsd = synth.gemma3_state_dict(gcfg, seed=4)
    gsd["language_model.embed.weight"] = torch.zeros(3, 3)
    _write_checkpoint(tmp_path / "gemma", gcfg, gsd)
    other = {k: v + 1 for k, v in gsd.items() if k.startswith("multi_modal_projector.")}
    _write_checkpoint(tmp_path / "gemma_ft", gcfg, other, shards=1, with_index=False)
    g = load_model(tmp_path / "gemma", adapter_model_dirs=[tmp_path / "gemma_ft"], torch_device=cpu)
    assert isinstance(g, Gemma3VisionEncoder)
    adapters = g.multi_modal_projector.adapters
    assert list(adapters) == [str(tmp_path / "gemma"), str(tmp_path / "gemma_ft")]
    w0 = adapters[str(tmp_path / "gemma")].mm_input_projection_weight
    w1 = adapters[str(tmp_path / "gemma_ft")].mm_input_projection_weight
    assert torch.equal(w0, gsd["multi_modal_projector.mm_input_projection_weight"]) and torch.equal(w1, w0 + 1)


def test_llava_onevision_names_plans_and_errors():
    from cornserve_amd.eric.models import llava_onevision as lv
    from oracle import gemma3 as og
    from oracle import llava_onevision as ol

    cfg = synth.llava_ov_config(num_hidden_layers=2, image_size=70, text_hidden=64, max_grid=4)
    model = lv.LlavaOneVisionEncoder(cfg)
    sd = synth.llava_ov_state_dict(cfg, seed=0)
    assert set(model.state_dict().keys()) == set(sd)        # no post_layernorm: the tower stops at the feature layer
    model.load_state_dict(sd)
    assert model.chunk_shape == (1, 64) and model.dtype == torch.float32
    cfg2 = synth.llava_ov_config(num_hidden_layers=3, image_size=70, text_hidden=64)
    cfg2.vision_feature_layer = -2
    assert len(lv.LlavaOneVisionEncoder(cfg2).vision_tower.vision_model.encoder.layers) == 2
    cfg2.vision_feature_layer = [1, -1]
    assert len(lv.LlavaOneVisionEncoder(cfg2).vision_tower.vision_model.encoder.layers) == 3
    cfg2.vision_feature_layer = "last"
    with pytest.raises(TypeError):
        lv.LlavaOneVisionEncoder(cfg2)

    # the gather records, applied on the host, are the reference's merge (restated by the oracle) bit for bit
    ocfg = ol.LlavaOneVisionConfig(vision=og.SiglipConfig(num_hidden_layers=2, image_size=70), text_hidden_size=64,
                                   image_grid_pinpoints=cfg.image_grid_pinpoints)

    def apply(src, taps, frac):
        a = [src[taps[:, k]].astype(np.float32) for k in range(4)]
        ly, lx = frac[:, 0:1], frac[:, 1:2]
        hy, hx = np.float32(1) - ly, np.float32(1) - lx
        return hy * (hx * a[0] + lx * a[1]) + ly * (hx * a[2] + lx * a[3])

    rng = np.random.default_rng(0)
    sizes = [(70, 70), (100, 260), (280, 280), (211, 277), (280, 140), (50, 300), (277, 90), (139, 141), (33, 280)]
    sizes += [(int(h), int(w)) for h, w in rng.integers(10, 600, size=(40, 2)) if max(h, w) / min(h, w) < 20]
    shrunk = 0
    for h, w in sizes:
        th, tw = lv.anyres_grid_shape((h, w), cfg.image_grid_pinpoints, 70)
        n = 1 + th * tw
        feats = rng.standard_normal((7 + n * 25 + 1, 8)).astype(np.float32)    # 7 rows of another item in front
        taps, frac = lv.image_merge_plan(n, (h, w), 7, 7 + n * 25, 5, cfg.image_grid_pinpoints, 70)
        assert taps.min() >= 7 and taps.max() <= 7 + n * 25
        ref = ol.merge_image(ocfg, torch.from_numpy(feats[7:-1]).view(n, 25, 8), (h, w), torch.from_numpy(feats[-1]))
        assert np.array_equal(apply(feats, taps, frac), ref.numpy()), (h, w)
        shrunk += bool((frac != 0).any())
    assert shrunk >= 5
    # padded tile lists (more tiles than the grid needs) use the leading ones; too few are an error
    taps_a, _ = lv.image_merge_plan(9, (100, 260), 0, 500, 5, cfg.image_grid_pinpoints, 70)
    taps_b, _ = lv.image_merge_plan(12, (100, 260), 0, 500, 5, cfg.image_grid_pinpoints, 70)
    assert np.array_equal(taps_a, taps_b)
    with pytest.raises(RuntimeError, match="needs 8 tiles"):
        lv.image_merge_plan(5, (100, 260), 0, 500, 5, cfg.image_grid_pinpoints, 70)
    taps, frac = lv.image_merge_plan(1, (70, 70), 3, 99, 5, cfg.image_grid_pinpoints, 70)
    assert taps[:, 0].tolist() == list(range(3, 28)) + [99] and not frac.any()
    with pytest.raises(ValueError, match="not consistent"):
        lv.image_merge_plan(2, (70, 70), 0, 48, 5, cfg.image_grid_pinpoints, 70, tokens_per_tile=24)

    feats = rng.standard_normal((3 * 25 + 1, 8)).astype(np.float32)
    taps, frac = lv.video_pool_plan(3, 0, 75, 5)
    ref = ol.pool_video(ocfg, torch.from_numpy(feats[:-1]).view(3, 25, 8), torch.from_numpy(feats[-1]))
    assert np.array_equal(apply(feats, taps, frac), ref[0].numpy())

    px, szs = synth.llava_ov_image_inputs(cfg, [(70, 70)])
    with pytest.raises(ValueError, match="Unsupported modality"):
        model(Modality.AUDIO, "", {"pixel_values": px, "image_sizes": szs})
    with pytest.raises(AssertionError):
        model(Modality.IMAGE, "", {"pixel_values": [torch.zeros(2, 3, 56, 56)], "image_sizes": szs})
    with pytest.raises(AssertionError):
        model(Modality.IMAGE, "", {"pixel_values": px, "image_sizes": szs + szs})
    with pytest.raises(RuntimeError, match="one frame"):
        model(Modality.VIDEO, "", {"pixel_values_videos": synth.llava_ov_video_inputs(cfg, [1])})
    with pytest.raises(RuntimeError, match="no CPU path"):     # the kernels are the only implementation
        model(Modality.IMAGE, "", {"pixel_values": px, "image_sizes": szs})


def test_load_llava_onevision_from_local_checkpoint(tmp_path):
    from cornserve_amd.eric.loader import load_model
    from cornserve_amd.eric.models.llava_onevision import LlavaOneVisionEncoder

    cfg = synth.llava_ov_config(num_hidden_layers=2, image_size=70, text_hidden=64, max_grid=2)
    sd = synth.llava_ov_state_dict(cfg, seed=6)
    ckpt = dict(sd)
    ckpt["language_model.embed.weight"] = torch.zeros(3, 3)
    ckpt["vision_tower.vision_model.post_layernorm.weight"] = torch.ones(1152)    # in the checkpoint, not in the model
    ckpt["vision_tower.vision_model.post_layernorm.bias"] = torch.zeros(1152)
    _write_checkpoint(tmp_path / "llava", cfg, ckpt)
    model = load_model(tmp_path / "llava", torch_device=torch.device("cpu"))
    assert isinstance(model, LlavaOneVisionEncoder) and not model.training
    assert torch.equal(model.image_newline, sd["image_newline"])
    assert torch.equal(model.multi_modal_projector.linear_2.weight, sd["multi_modal_projector.linear_2.weight"])
    assert model.config.image_grid_pinpoints == cfg.image_grid_pinpoints


def test_scheduler_batches_like_the_reference_and_bounds_patches():
    from cornserve_amd.eric import scheduler as sc

    def item(i, modality=Modality.IMAGE, model="m", grid=(1, 4, 4)):
        return sc.ProcessedEmbeddingData(id=f"d{i}", modality=modality, model_id=model,
                                         data={"pixel_values": torch.zeros(grid[0] * grid[1] * grid[2], 8),
                                               "image_grid_thw": torch.tensor([grid])},
                                         receiver_sidecar_ranks=[[i]])

    s = sc.Scheduler()
    assert not s.has_waiting_requests()
    s.enqueue(sc.EngineEnqueueRequest("r0", [item(0), item(1)]))
    s.enqueue(sc.EngineEnqueueRequest("r1", [item(2), item(3, Modality.VIDEO), item(4)]))
    s.enqueue(sc.EngineEnqueueRequest("r2", [item(5, model="other")]))
    b = s.schedule()                                    # every image at the head, up to the modality change
    assert (b.modality, b.adapter_name, b.request_ids, b.data_ids) == (Modality.IMAGE, "m", ["r0", "r0", "r1"], ["d0", "d1", "d2"])
    assert b.chunk_ids == [0, 0, 0] and b.num_chunks == [1, 1, 1] and b.receiver_ranks == [[[0]], [[1]], [[2]]]
    assert len(b.data["pixel_values"]) == 3 and len(b) == 3
    wb = b.to_worker_batch()
    assert type(wb).__name__ == "WorkerBatch" and wb.data is b.data
    assert s.process_batch_result(b.request_ids, b.data_ids) == ["r0"]
    b = s.schedule()
    assert (b.modality, b.data_ids) == (Modality.VIDEO, ["d3"])
    assert s.process_batch_result(["r1"], ["d3"]) == []
    b = s.schedule()                                    # the adapter changes behind d4
    assert b.data_ids == ["d4"] and s.process_batch_result(["r1"], ["d4"]) == ["r1"]
    b = s.schedule()
    assert b.adapter_name == "other" and s.process_batch_result(["r2"], ["d5"]) == ["r2"]
    assert not s.has_waiting_requests()
    with pytest.raises(ValueError, match="different modalities"):
        b.add_data("r9", [item(9, Modality.VIDEO)], [0], [1])

    s = sc.Scheduler(max_batch_size=2)
    s.enqueue(sc.EngineEnqueueRequest("r0", [item(i) for i in range(5)]))
    assert s.schedule().data_ids == ["d0", "d1"]

    # patch budget: 16 + 16 fit into 40, the third item does not; an item above the budget still runs, alone
    s = sc.Scheduler(max_batch_patches=40)
    s.enqueue(sc.EngineEnqueueRequest("r0", [item(0), item(1), item(2), item(3, grid=(2, 8, 8)), item(4)]))
    b = s.schedule()
    assert b.data_ids == ["d0", "d1"]
    s.process_batch_result(b.request_ids, b.data_ids)
    assert s.schedule().data_ids == ["d2"]               # 16 + 128 > 40
    s.process_batch_result(["r0"], ["d2"])
    assert s.schedule().data_ids == ["d3"]
    with pytest.raises(ValueError):
        sc.Scheduler(max_batch_patches=0)
    # items handed out are in flight: a second schedule() before the result is reported takes the NEXT items, so a
    # caller can prepare batch k+1 (upload it) while batch k runs; nothing is handed out twice
    s = sc.Scheduler(max_batch_size=2)
    s.enqueue(sc.EngineEnqueueRequest("r0", [item(i) for i in range(3)]))
    s.enqueue(sc.EngineEnqueueRequest("r1", [item(3, Modality.VIDEO), item(4)]))
    b0, b1 = s.schedule(), s.schedule()
    assert b0.data_ids == ["d0", "d1"] and b1.data_ids == ["d2"]          # d3 is another modality
    b2 = s.schedule()
    assert (b2.modality, b2.data_ids) == (Modality.VIDEO, ["d3"]) and s.has_schedulable_items()
    assert s.schedule().data_ids == ["d4"] and not s.has_schedulable_items() and s.has_waiting_requests()
    with pytest.raises(RuntimeError, match="nothing to schedule"):
        s.schedule()
    assert s.process_batch_result(b1.request_ids, b1.data_ids) == []       # results may come back in any order
    assert s.process_batch_result(b0.request_ids, b0.data_ids) == ["r0"]
    with pytest.raises(KeyError):
        s.process_batch_result(["r0"], ["d0"])                             # reported twice
    with pytest.raises(KeyError):
        s.process_batch_result(["r1", "r1"], ["d4", "nope"])               # a bad pair behind a good one ...
    with pytest.raises(KeyError):
        s.process_batch_result(["r1", "r1"], ["d4", "d4"])
    assert s.has_waiting_requests()                                        # ... leaves d4 queued: nothing was changed
    assert s.process_batch_result(["r1", "r1"], ["d4", "d3"]) == ["r1"] and not s.has_waiting_requests()
    with pytest.raises(ValueError):
        s.enqueue(sc.EngineEnqueueRequest("r5", []))
    s.enqueue(sc.EngineEnqueueRequest("r6", [item(0)]))
    with pytest.raises(ValueError, match="already queued"):
        s.enqueue(sc.EngineEnqueueRequest("r6", [item(1)]))
    # the upload event of a batch sent ahead travels with the conversion
    b = s.schedule()
    b._uploaded = marker = object()
    assert b.to_worker_batch()._uploaded is marker
    tiles = sc.ProcessedEmbeddingData("t", Modality.IMAGE, "m", {"pixel_values": torch.zeros(3, 3, 28, 42)})
    assert sc.patch_count(tiles) == 3 * 2 * 3 and sc.patch_count(item(0, grid=(2, 4, 6))) == 48


def test_qkv_window_attn_row_order_is_a_permutation_with_padding():
    from cornserve_amd import ops as o
    heads = 3
    order = o.qkv_window_attn_row_order(heads)
    assert order.shape == (heads * 256,)
    used = order[order >= 0]
    assert sorted(used.tolist()) == list(range(3 * heads * 80))      # every qkv row exactly once
    pad = [32 * 7 + 8 * kq + 4 + r for kq in range(4) for r in range(4)]
    assert (order.reshape(heads, 256)[:, pad] == -1).all()           # fragment 15 of every head is padding
    # both halves of a rotary pair sit in the same lane group of the same head: dims d and d + 40
    per_head = order.reshape(heads, 256)[1]
    pos = {int(r): i for i, r in enumerate(per_head.tolist()) if r >= 0}
    for d in range(40):
        a, b = pos[80 + d], pos[80 + d + 40]      # q rows of head 1
        assert (a % 32) // 8 == (b % 32) // 8


def test_qkv_window_attn_pack_and_unpack_are_inverse():
    """The per-head packed qkv weight (the only copy a window block keeps) gives back the plain rows bit for bit."""
    from cornserve_amd import ops

    heads, K = 3, 64
    g = torch.Generator().manual_seed(3)
    w = torch.randn((3 * heads * 80, K), generator=g).to(torch.bfloat16)
    b = torch.randn((3 * heads * 80,), generator=g).to(torch.bfloat16)
    wp, bp = ops.pack_qkv_window_attn(w, b, heads)
    assert wp.shape == (heads * 256, K) and int((wp.float().abs().sum(1) == 0).sum()) >= heads * 16   # 16 zero rows per head
    w2, b2 = ops.unpack_qkv_window_attn(wp, bp, heads)
    assert torch.equal(w2, w) and torch.equal(b2, b)
    q = torch.randint(0, 256, (3 * heads * 80, K), generator=g, dtype=torch.uint8)
    sc = torch.rand((3 * heads * 80,), generator=g) + 0.5
    qp, bp, sp = ops.pack_qkv_window_attn(q, b, heads, w_scale=sc)
    q2, b2, s2 = ops.unpack_qkv_window_attn(qp, bp, heads, w_scale=sp)
    assert torch.equal(q2, q) and torch.equal(b2, b) and torch.equal(s2, sc)
    with pytest.raises(ValueError):
        ops.unpack_qkv_window_attn(wp[:-1], bp, heads)
