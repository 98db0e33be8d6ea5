from .common import LayerNorm2d, MLPBlock
from .image_encoder import (
    Attention,
    Block,
    ImageEncoderViT,
    PatchEmbed,
    add_decomposed_rel_pos,
    get_rel_pos,
    window_partition,
    window_unpartition,
)
from .sam import Sam
