"""Model factories with the reference's registry keys and signatures
(segment_anything_fast/build_sam.py:14-92).

`sam_model_registry[name](checkpoint=None)` builds the float model;
`sam_model_fast_registry[name](checkpoint=None, compile_mode='max-autotune',
dtype=torch.bfloat16)` returns it in eval mode and `dtype`.  The fast path here
is the HIP kernels behind Attention / Int8DynamicLinear; nothing is traced or
autotuned.  What `compile_mode` keeps of the reference's
`torch.compile(sam.image_encoder, mode=compile_mode)` (:67-71) is the part that
matters at small batch: with any mode but None the image encoder is wrapped in
`graphs.ReplayedEncoder`, which records one forward per input shape into a HIP
graph and replays it while the batch is launch-bound (up to four images).
`compile_mode=None` leaves the encoder as it is.

Only the image encoder is constructed (hyper-parameters from :14-44,102-120);
checkpoint keys that belong to the prompt encoder / mask decoder are ignored on
load.
"""

from functools import partial

import torch

from .modeling import ImageEncoderViT, Sam

_ENCODER_SPECS = {
    "vit_h": dict(embed_dim=1280, depth=32, num_heads=16, global_attn_indexes=(7, 15, 23, 31)),
    "vit_l": dict(embed_dim=1024, depth=24, num_heads=16, global_attn_indexes=(5, 11, 17, 23)),
    "vit_b": dict(embed_dim=768, depth=12, num_heads=12, global_attn_indexes=(2, 5, 8, 11)),
}


def build_image_encoder(name: str) -> ImageEncoderViT:
    spec = _ENCODER_SPECS[name]
    return ImageEncoderViT(
        depth=spec["depth"], embed_dim=spec["embed_dim"], img_size=1024, mlp_ratio=4,
        norm_layer=partial(torch.nn.LayerNorm, eps=1e-6), num_heads=spec["num_heads"],
        patch_size=16, qkv_bias=True, use_rel_pos=True,
        global_attn_indexes=spec["global_attn_indexes"], window_size=14, out_chans=256)


def _build_sam(name: str, checkpoint=None) -> Sam:
    sam = Sam(image_encoder=build_image_encoder(name))
    sam.eval()
    if checkpoint is not None:
        with open(checkpoint, "rb") as f:
            state_dict = torch.load(f, weights_only=True)
        own = sam.state_dict()
        sam.load_state_dict({k: v for k, v in state_dict.items() if k in own}, strict=True)
    return sam


def build_sam_vit_h(checkpoint=None):
    return _build_sam("vit_h", checkpoint)


def build_sam_vit_l(checkpoint=None):
    return _build_sam("vit_l", checkpoint)


def build_sam_vit_b(checkpoint=None):
    return _build_sam("vit_b", checkpoint)


build_sam = build_sam_vit_h

sam_model_registry = {
    "default": build_sam_vit_h,
    "vit_h": build_sam_vit_h,
    "vit_l": build_sam_vit_l,
    "vit_b": build_sam_vit_b,
}


def _apply_eval_dtype_sam(model: Sam, dtype):
    for attr in ("image_encoder", "prompt_encoder", "mask_decoder"):
        sub = getattr(model, attr, None)
        if sub is None:
            continue
        sub = sub.eval()
        setattr(model, attr, sub.to(dtype) if dtype is not None else sub)
    return model


def _fast(builder, checkpoint, compile_mode, dtype):
    sam = _apply_eval_dtype_sam(builder(checkpoint), dtype)
    if compile_mode is not None:
        from .graphs import ReplayedEncoder
        sam.image_encoder = ReplayedEncoder(sam.image_encoder, compile_mode)
    return sam


def build_sam_fast_vit_h(checkpoint=None, compile_mode="max-autotune", dtype=torch.bfloat16):
    return _fast(build_sam_vit_h, checkpoint, compile_mode, dtype)


def build_sam_fast_vit_l(checkpoint=None, compile_mode="max-autotune", dtype=torch.bfloat16):
    return _fast(build_sam_vit_l, checkpoint, compile_mode, dtype)


def build_sam_fast_vit_b(checkpoint=None, compile_mode="max-autotune", dtype=torch.bfloat16):
    return _fast(build_sam_vit_b, checkpoint, compile_mode, dtype)


build_sam_fast = build_sam_fast_vit_h

sam_model_fast_registry = {
    "default": build_sam_fast_vit_h,
    "vit_h": build_sam_fast_vit_h,
    "vit_l": build_sam_fast_vit_l,
    "vit_b": build_sam_fast_vit_b,
}
