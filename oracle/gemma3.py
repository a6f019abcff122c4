"""ORACLE (test infrastructure, never on the product path): Gemma-3 vision encoder (SigLIP) on the CPU.

A plain-PyTorch restatement of eric/models/gemma3.py:18-136 and eric/models/layers/siglip.py:

* embeddings      Conv2d(k = s = patch, bias, padding valid) + learned positions (siglip.py:91-101,
                  the non-interpolating branch, which is the one gemma3.py takes);
* encoder layer   LayerNorm -> fused qkv -> full attention -> out_proj -> residual; LayerNorm -> fc1 ->
                  GELU(tanh) -> fc2 -> residual (siglip.py:104-189); xformers'
                  memory_efficient_attention_forward (third party, xformers 0.0.33.post1, not vendored)
                  is restated as softmax(q k^T * d^-0.5) v per image and head (attention.py:28-53);
* post layernorm  siglip.py:275-279,329-333;
* projector       transpose -> [B,H,side,side] -> AvgPool2d -> GemmaRMSNorm -> matmul (gemma3.py:33-49,
                  norm.py:90-113).

State-dict names are the checkpoint's (separate q_proj/k_proj/v_proj, which the reference fuses at load
time, eric/models/layers/linear.py:339-371).  Pinned by tests/test_oracle_models.py against
tests/golden/gemma3_small.npz, written by tests/golden/make_golden.py from the installed third-party
Hugging Face SiglipVisionModel + Gemma3MultiModalProjector.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F


@dataclass
class SiglipConfig:
    hidden_size: int = 1152
    intermediate_size: int = 4304
    num_hidden_layers: int = 27
    num_attention_heads: int = 16
    num_channels: int = 3
    image_size: int = 896
    patch_size: int = 14
    layer_norm_eps: float = 1e-6
    hidden_act: str = "gelu_pytorch_tanh"
    # projector
    mm_tokens_per_image: int = 256
    text_hidden_size: int = 2560


VT = "vision_tower.vision_model."
MM = "multi_modal_projector."


def gemma_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    orig = x.dtype
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    xf = xf * (1.0 + w.float())
    return xf.to(orig)


def full_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, nh: int, scale: float) -> torch.Tensor:
    """q,k,v: [B, S, H]; fp32 math on the stored-precision inputs, output in q.dtype."""
    B, S, H = q.shape
    d = H // nh
    qf, kf, vf = (t.float().view(B, S, nh, d).transpose(1, 2) for t in (q, k, v))
    out = torch.empty(B, nh, S, d)
    for b in range(B):  # per image to bound the size of the score matrix
        p = torch.softmax(torch.matmul(qf[b], kf[b].transpose(1, 2)) * scale, dim=-1)
        out[b] = torch.matmul(p, vf[b])
    return out.transpose(1, 2).reshape(B, S, H).to(q.dtype)


def vision_tower(sd: dict, cfg: SiglipConfig, pixel_values: torch.Tensor, dtype=torch.float32,
                 num_layers: int | None = None, post_norm: bool = True) -> torch.Tensor:
    """`num_layers` / `post_norm`: a tower built only up to a feature layer, without the final LayerNorm
    (siglip.py:301-335, as the LLaVA-family encoders build it, layers/vit.py:43-62)."""
    W = {k: v.to(dtype) for k, v in sd.items() if k.startswith(VT)}
    x = pixel_values.to(dtype)
    x = F.conv2d(x, W[VT + "embeddings.patch_embedding.weight"], W[VT + "embeddings.patch_embedding.bias"],
                 stride=cfg.patch_size)
    x = x.flatten(2).transpose(1, 2)
    x = x + W[VT + "embeddings.position_embedding.weight"][None, : x.shape[1]]
    H, nh = cfg.hidden_size, cfg.num_attention_heads
    for i in range(cfg.num_hidden_layers if num_layers is None else num_layers):
        p = f"{VT}encoder.layers.{i}."
        h = F.layer_norm(x, (H,), W[p + "layer_norm1.weight"], W[p + "layer_norm1.bias"], cfg.layer_norm_eps)
        q = F.linear(h, W[p + "self_attn.q_proj.weight"], W[p + "self_attn.q_proj.bias"])
        k = F.linear(h, W[p + "self_attn.k_proj.weight"], W[p + "self_attn.k_proj.bias"])
        v = F.linear(h, W[p + "self_attn.v_proj.weight"], W[p + "self_attn.v_proj.bias"])
        o = full_attention(q, k, v, nh, (H // nh) ** -0.5)
        x = x + F.linear(o, W[p + "self_attn.out_proj.weight"], W[p + "self_attn.out_proj.bias"])
        h = F.layer_norm(x, (H,), W[p + "layer_norm2.weight"], W[p + "layer_norm2.bias"], cfg.layer_norm_eps)
        h = F.gelu(F.linear(h, W[p + "mlp.fc1.weight"], W[p + "mlp.fc1.bias"]), approximate="tanh")
        x = x + F.linear(h, W[p + "mlp.fc2.weight"], W[p + "mlp.fc2.bias"])
    if not post_norm:
        return x
    return F.layer_norm(x, (H,), W[VT + "post_layernorm.weight"], W[VT + "post_layernorm.bias"], cfg.layer_norm_eps)


def projector(sd: dict, cfg: SiglipConfig, feats: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    B, S, H = feats.shape
    side = cfg.image_size // cfg.patch_size
    tokens_per_side = int(cfg.mm_tokens_per_image**0.5)
    k = side // tokens_per_side
    x = feats.transpose(1, 2).reshape(B, H, side, side).contiguous()
    x = F.avg_pool2d(x, kernel_size=k, stride=k).flatten(2).transpose(1, 2)
    x = gemma_rms_norm(x, sd[MM + "mm_soft_emb_norm.weight"].to(dtype), cfg.layer_norm_eps)
    return torch.matmul(x, sd[MM + "mm_input_projection_weight"].to(dtype)).type_as(feats)


def forward(sd: dict, cfg: SiglipConfig, pixel_values: list, num_crops: list, dtype=torch.float32) -> list:
    px = torch.cat(pixel_values, dim=0)
    n = (torch.cat([c.reshape(-1) for c in num_crops]) + 1).tolist()
    feats = vision_tower(sd, cfg, px, dtype)
    emb = projector(sd, cfg, feats, dtype)
    return [e.flatten(0, 1) for e in emb.split(n)]
