"""The encoder half of SamPredictor (segment_anything_fast/predictor.py:17-91).

`set_torch_image` keeps its contract - a (B, 3, H, W) image whose long side equals
the encoder input size is normalised, padded and encoded, and the embedding is
kept in `self.features` - so code that drives the image encoder through the
predictor runs unchanged.  Prompt decoding (`predict`, `predict_torch`) belongs
to the mask decoder, which this package does not contain.
"""

from typing import Tuple

import torch

from .modeling import Sam


class SamPredictor:
    def __init__(self, sam_model: Sam) -> None:
        self.model = sam_model
        self.reset_image()

    @property
    def device(self) -> torch.device:
        return self.model.device

    def reset_image(self) -> None:
        self.is_image_set = False
        self.features = None
        self.orig_h = self.orig_w = None
        self.input_h = self.input_w = None
        self.original_size = None
        self.input_size = None

    @torch.no_grad()
    def set_torch_image(self, transformed_image: torch.Tensor,
                        original_image_size: Tuple[int, ...]) -> None:
        size = self.model.image_encoder.img_size
        assert (transformed_image.dim() == 4 and transformed_image.shape[1] == 3
                and max(transformed_image.shape[2:]) == size), \
            f"set_torch_image input must be BCHW with long side {size}."
        self.reset_image()
        self.original_size = original_image_size
        self.input_size = tuple(transformed_image.shape[-2:])
        x = self.model.preprocess(transformed_image)
        dtype = next(self.model.image_encoder.parameters()).dtype
        self.features = self.model.image_encoder(x.to(dtype))
        self.is_image_set = True

    def get_image_embedding(self) -> torch.Tensor:
        if not self.is_image_set:
            raise RuntimeError("An image must be set with .set_image(...) to generate an embedding.")
        return self.features

    def predict(self, *args, **kwargs):
        raise NotImplementedError("mask decoding is not part of samfast_amd")

    predict_torch = predict
