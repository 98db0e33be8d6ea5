"""Container for the image-encoder side of SAM.

Only what the encoder hot path needs from segment_anything_fast/modeling/sam.py
is kept: the attribute layout (`image_encoder`, `pixel_mean`, `pixel_std`,
`image_format`, `device`) and `preprocess` (:164-174).  The prompt encoder and
mask decoder are outside this package; they can be attached as attributes by a
caller that owns them and are passed through untouched.
"""

from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .image_encoder import ImageEncoderViT


class Sam(nn.Module):
    mask_threshold: float = 0.0
    image_format: str = "RGB"

    def __init__(
        self,
        image_encoder: ImageEncoderViT,
        prompt_encoder: Optional[nn.Module] = None,
        mask_decoder: Optional[nn.Module] = None,
        pixel_mean: List[float] = [123.675, 116.28, 103.53],
        pixel_std: List[float] = [58.395, 57.12, 57.375],
    ) -> None:
        super().__init__()
        self.image_encoder = image_encoder
        self.prompt_encoder = prompt_encoder
        self.mask_decoder = mask_decoder
        self.register_buffer("pixel_mean", torch.tensor(pixel_mean).view(-1, 1, 1), False)
        self.register_buffer("pixel_std", torch.tensor(pixel_std).view(-1, 1, 1), False)

    @property
    def device(self):
        return self.pixel_mean.device

    def preprocess(self, x: torch.Tensor) -> torch.Tensor:
        """Normalise colours, then zero-pad bottom/right to the square encoder input."""
        x = (x - self.pixel_mean) / self.pixel_std
        h, w = x.shape[-2:]
        size = self.image_encoder.img_size
        return F.pad(x, (0, size - w, 0, size - h))

    def forward(self, *args, **kwargs):
        raise NotImplementedError(
            "samfast_amd covers the image encoder; prompt encoding and mask decoding "
            "are not part of this package")
