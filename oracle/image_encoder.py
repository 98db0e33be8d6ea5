"""Oracle: the SAM ViT image encoder that hosts the hot path (CPU, torch eager).

TEST INFRASTRUCTURE ONLY (see the package docstring).

A functional restatement over a flat state dict that uses the reference's
parameter names, so the same weights drive the oracle and the product
modules.  Reference functions followed:

encoder_forward   segment_anything_fast/modeling/image_encoder.py:107-117
block_forward     segment_anything_fast/modeling/image_encoder.py:167-183
patch embedding   segment_anything_fast/modeling/image_encoder.py:398-406
MLP               segment_anything_fast/modeling/common.py:25-26
LayerNorm2d       segment_anything_fast/modeling/common.py:38-43
hyper-parameters  segment_anything_fast/build_sam.py:14-44,102-120
preprocess        segment_anything_fast/modeling/sam.py:164-174,
                  build_sam.py:139-140 (pixel mean / std)

Pinned by (tests/test_oracle_encoder.py): LayerNorm2d against
F.layer_norm over the channel axis; the block against a composition of the
per-op oracles written with nn.Module library layers (nn.Linear,
nn.LayerNorm, nn.GELU, nn.Conv2d) carrying the same weights; shape and
parameter-name table against the one the reference constructors imply.
"""

from dataclasses import dataclass
from typing import Dict, Tuple

import torch
import torch.nn.functional as F

from . import relpos_attention as ra

PIXEL_MEAN = (123.675, 116.28, 103.53)   # build_sam.py:139
PIXEL_STD = (58.395, 57.12, 57.375)      # build_sam.py:140


@dataclass(frozen=True)
class EncoderConfig:
    embed_dim: int
    depth: int
    num_heads: int
    global_attn_indexes: Tuple[int, ...]
    window_size: int = 14
    img_size: int = 1024
    patch_size: int = 16
    out_chans: int = 256
    mlp_ratio: int = 4
    ln_eps: float = 1e-6


VIT_B = EncoderConfig(768, 12, 12, (2, 5, 8, 11))      # build_sam.py:37-44
VIT_L = EncoderConfig(1024, 24, 16, (5, 11, 17, 23))   # build_sam.py:27-34
VIT_H = EncoderConfig(1280, 32, 16, (7, 15, 23, 31))   # build_sam.py:14-21


def preprocess(images: torch.Tensor) -> torch.Tensor:
    """(x - mean) / std per channel on (B, 3, H, W); sam.py:167."""
    mean = torch.tensor(PIXEL_MEAN, dtype=images.dtype).view(1, 3, 1, 1)
    std = torch.tensor(PIXEL_STD, dtype=images.dtype).view(1, 3, 1, 1)
    return (images - mean) / std


def layer_norm_2d(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float = 1e-6):
    """Normalise (B, C, H, W) over C with biased variance; common.py:38-43."""
    mu = x.mean(dim=1, keepdim=True)
    var = (x - mu).pow(2).mean(dim=1, keepdim=True)
    xn = (x - mu) / torch.sqrt(var + eps)
    return xn * weight.view(1, -1, 1, 1) + bias.view(1, -1, 1, 1)


def block_forward(sd: Dict[str, torch.Tensor], prefix: str, x: torch.Tensor,
                  cfg: EncoderConfig, window_size: int, linear=F.linear,
                  use_sdpa: bool = False, mlp_linear=None) -> torch.Tensor:
    """One transformer block on (B, H, W, C); image_encoder.py:167-183."""
    mlp_linear = mlp_linear or linear
    C = cfg.embed_dim
    p = lambda name: sd[prefix + name]
    shortcut = x
    y = F.layer_norm(x, (C,), p("norm1.weight"), p("norm1.bias"), cfg.ln_eps)
    if window_size > 0:
        H, W = y.shape[1], y.shape[2]
        y, pad_hw = ra.window_partition(y, window_size)
    y = ra.attention_forward(
        y, p("attn.qkv.weight"), p("attn.qkv.bias"), p("attn.proj.weight"), p("attn.proj.bias"),
        p("attn.rel_pos_h"), p("attn.rel_pos_w"), cfg.num_heads, linear=linear,
        use_sdpa=use_sdpa,
    )
    if window_size > 0:
        y = ra.window_unpartition(y, window_size, pad_hw, (H, W))
    x = shortcut + y
    z = F.layer_norm(x, (C,), p("norm2.weight"), p("norm2.bias"), cfg.ln_eps)
    z = mlp_linear(z, p("mlp.lin1.weight"), p("mlp.lin1.bias"))
    z = F.gelu(z)  # exact erf GELU, the nn.GELU default (common.py:17)
    z = mlp_linear(z, p("mlp.lin2.weight"), p("mlp.lin2.bias"))
    return x + z


def encoder_forward(sd: Dict[str, torch.Tensor], images: torch.Tensor, cfg: EncoderConfig,
                    linear=F.linear, use_sdpa: bool = False, mlp_linear=None) -> torch.Tensor:
    """(B, 3, 1024, 1024) normalised images -> (B, 256, 64, 64) embeddings.

    `linear(x, w, b)` is used for the four Linears of every block (qkv, proj,
    lin1, lin2) - pass oracle.quant_linear.dynamic_int8_linear for the
    quantised path.  `mlp_linear`, if given, replaces it for lin1 / lin2 only (the
    2:4-sparse MLP configuration).  Patch embedding and neck are convolutions and stay float.
    use_sdpa=True routes attention through F.scaled_dot_product_attention with a
    materialised bias, which is what the reference executes on a CPU
    (flash_4.py:368-370); the default writes the softmax out.
    """
    x = F.conv2d(images, sd["patch_embed.proj.weight"], sd["patch_embed.proj.bias"],
                 stride=cfg.patch_size)
    x = x.permute(0, 2, 3, 1)
    if "pos_embed" in sd:
        x = x + sd["pos_embed"]
    for i in range(cfg.depth):
        ws = 0 if i in cfg.global_attn_indexes else cfg.window_size
        x = block_forward(sd, f"blocks.{i}.", x, cfg, ws, linear, use_sdpa, mlp_linear)
    x = x.permute(0, 3, 1, 2)
    x = F.conv2d(x, sd["neck.0.weight"])
    x = layer_norm_2d(x, sd["neck.1.weight"], sd["neck.1.bias"])
    x = F.conv2d(x, sd["neck.2.weight"], padding=1)
    x = layer_norm_2d(x, sd["neck.3.weight"], sd["neck.3.bias"])
    return x


def parameter_shapes(cfg: EncoderConfig) -> Dict[str, Tuple[int, ...]]:
    """Name -> shape of every encoder parameter, as the reference constructors
    create them (image_encoder.py:59-105,152-163,213-223,398-400; common.py:21-22,34-35)."""
    C, P, O = cfg.embed_dim, cfg.patch_size, cfg.out_chans
    G = cfg.img_size // P
    hd = C // cfg.num_heads
    shapes = {
        "pos_embed": (1, G, G, C),
        "patch_embed.proj.weight": (C, 3, P, P),
        "patch_embed.proj.bias": (C,),
        "neck.0.weight": (O, C, 1, 1),
        "neck.1.weight": (O,), "neck.1.bias": (O,),
        "neck.2.weight": (O, O, 3, 3),
        "neck.3.weight": (O,), "neck.3.bias": (O,),
    }
    for i in range(cfg.depth):
        S = G if i in cfg.global_attn_indexes else cfg.window_size
        b = f"blocks.{i}."
        shapes.update({
            b + "norm1.weight": (C,), b + "norm1.bias": (C,),
            b + "attn.qkv.weight": (3 * C, C), b + "attn.qkv.bias": (3 * C,),
            b + "attn.proj.weight": (C, C), b + "attn.proj.bias": (C,),
            b + "attn.rel_pos_h": (2 * S - 1, hd), b + "attn.rel_pos_w": (2 * S - 1, hd),
            b + "norm2.weight": (C,), b + "norm2.bias": (C,),
            b + "mlp.lin1.weight": (cfg.mlp_ratio * C, C), b + "mlp.lin1.bias": (cfg.mlp_ratio * C,),
            b + "mlp.lin2.weight": (C, cfg.mlp_ratio * C), b + "mlp.lin2.bias": (C,),
        })
    return shapes
