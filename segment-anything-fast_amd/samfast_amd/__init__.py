"""samfast_amd - the SAM ViT image-encoder hot path on MI355X (gfx950).

Public names follow segment_anything_fast/__init__.py:7-20 for the part of the
API that touches the image encoder.
"""

from .build_sam import (
    build_sam,
    build_sam_fast,
    build_sam_fast_vit_b,
    build_sam_fast_vit_h,
    build_sam_fast_vit_l,
    build_sam_vit_b,
    build_sam_vit_h,
    build_sam_vit_l,
    sam_model_fast_registry,
    sam_model_registry,
)
from .predictor import SamPredictor
from .quant import Int8DynamicLinear, apply_dynamic_quant
from .sparse import Int8Sparse24Linear, apply_fake_sparsity, apply_sparse

__all__ = [
    "build_sam", "build_sam_vit_h", "build_sam_vit_l", "build_sam_vit_b", "sam_model_registry",
    "build_sam_fast", "build_sam_fast_vit_h", "build_sam_fast_vit_l", "build_sam_fast_vit_b",
    "sam_model_fast_registry", "SamPredictor", "Int8DynamicLinear", "apply_dynamic_quant",
    "Int8Sparse24Linear", "apply_fake_sparsity", "apply_sparse",
]
