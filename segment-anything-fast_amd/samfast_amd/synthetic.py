"""Seeded synthetic weights and images for benchmarks and tests (no checkpoints
or datasets are available offline).

Weights: Linear / Conv weights ~ trunc_normal(std=0.02), their biases ~
N(0, 0.02), LayerNorm weight 1 / bias 0, pos_embed ~ trunc_normal(std=0.02),
rel_pos tables ~ N(0, 0.02).  (The reference initialises rel_pos to zeros,
modeling/image_encoder.py:222-223; non-zero tables are used so the bias path
carries signal.)  Images: uniform [0, 255] then (x - mean) / std with the SAM
pixel statistics (build_sam.py:139-140).
"""

from typing import Dict

import torch

PIXEL_MEAN = (123.675, 116.28, 103.53)
PIXEL_STD = (58.395, 57.12, 57.375)


def init_encoder_weights(encoder: torch.nn.Module, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Fill `encoder` in place (fp32, CPU generator => identical on every machine);
    returns its state dict."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    encoder = getattr(encoder, "_orig_mod", encoder)  # the fast registry's replay wrapper: same names as the bare encoder
    with torch.no_grad():
        for name, p in sorted(encoder.named_parameters(), key=lambda kv: kv[0]):
            t = torch.empty(p.shape, dtype=torch.float32)
            leaf = name.rsplit(".", 1)[-1]
            is_norm = ".norm" in name or name.startswith("neck.1.") or name.startswith("neck.3.")
            if is_norm:
                t.fill_(1.0 if leaf == "weight" else 0.0)
            elif "rel_pos" in name or leaf == "bias":
                t.normal_(0.0, 0.02, generator=gen)
            else:  # Linear / Conv weights, pos_embed
                torch.nn.init.trunc_normal_(t, std=0.02, a=-0.04, b=0.04, generator=gen)
            p.copy_(t.to(p.dtype))
    return encoder.state_dict()


def make_images(batch: int, size: int = 1024, seed: int = 1) -> torch.Tensor:
    """(B, 3, size, size) fp32 normalised images, CPU."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.rand((batch, 3, size, size), generator=gen, dtype=torch.float32) * 255.0
    mean = torch.tensor(PIXEL_MEAN).view(1, 3, 1, 1)
    std = torch.tensor(PIXEL_STD).view(1, 3, 1, 1)
    return (x - mean) / std
