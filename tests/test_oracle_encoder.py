"""Pins the encoder oracle (oracle/image_encoder.py) against library layers carrying
the same weights, and checks the product modules agree with it on the CPU route
(where they execute exactly the reference's eager composition)."""

from functools import partial

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import image_encoder as oe
from oracle import relpos_attention as ora


def test_layer_norm_2d_is_channel_layer_norm():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 16, 5, 7, generator=g)
    w, b = torch.randn(16, generator=g), torch.randn(16, generator=g)
    got = oe.layer_norm_2d(x, w, b, 1e-6)
    ref = F.layer_norm(x.permute(0, 2, 3, 1), (16,), w, b, 1e-6).permute(0, 3, 1, 2)
    assert torch.allclose(got, ref, atol=1e-5)


def test_parameter_table_matches_modules():
    from samfast_amd.build_sam import build_image_encoder
    for name, cfg in (("vit_b", oe.VIT_B),):
        enc = build_image_encoder(name)
        shapes = {k: tuple(v.shape) for k, v in enc.state_dict().items()}
        assert shapes == oe.parameter_shapes(cfg)
    # hyper-parameters of the other two sizes (build_sam.py:14-34)
    assert (oe.VIT_H.embed_dim, oe.VIT_H.depth, oe.VIT_H.num_heads, oe.VIT_H.global_attn_indexes) == \
        (1280, 32, 16, (7, 15, 23, 31))
    assert (oe.VIT_L.embed_dim, oe.VIT_L.depth, oe.VIT_L.num_heads, oe.VIT_L.global_attn_indexes) == \
        (1024, 24, 16, (5, 11, 17, 23))
    n_h = sum(int(torch.tensor(s).prod()) for s in oe.parameter_shapes(oe.VIT_H).values())
    assert abs(n_h - 637e6) < 5e6  # the published ViT-H encoder size


def _tiny():
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.synthetic import init_encoder_weights
    enc = ImageEncoderViT(img_size=128, patch_size=16, embed_dim=64, depth=3, num_heads=2,
                          out_chans=16, use_rel_pos=True, window_size=3, global_attn_indexes=(2,),
                          norm_layer=partial(nn.LayerNorm, eps=1e-6))
    sd = {k: v.clone() for k, v in init_encoder_weights(enc, seed=3).items()}
    cfg = oe.EncoderConfig(64, 3, 2, (2,), window_size=3, img_size=128, out_chans=16)
    return enc.eval(), sd, cfg


def test_block_against_library_layers():
    """One windowed block rebuilt from nn.LayerNorm / nn.Linear / nn.GELU and the
    attention oracle, with 8x8 tokens padded to 9x9 for 3x3 windows."""
    enc, sd, cfg = _tiny()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 8, 8, 64, generator=g)
    got = oe.block_forward(sd, "blocks.0.", x, cfg, 3)
    p = lambda n: sd["blocks.0." + n]
    ln1, ln2 = nn.LayerNorm(64, eps=1e-6), nn.LayerNorm(64, eps=1e-6)
    qkv, proj = nn.Linear(64, 192), nn.Linear(64, 64)
    l1, l2 = nn.Linear(64, 256), nn.Linear(256, 64)
    with torch.no_grad():
        for mod, nm in ((ln1, "norm1"), (ln2, "norm2"), (qkv, "attn.qkv"), (proj, "attn.proj"),
                        (l1, "mlp.lin1"), (l2, "mlp.lin2")):
            mod.weight.copy_(p(nm + ".weight"))
            mod.bias.copy_(p(nm + ".bias"))
        y = ln1(x)
        yp = F.pad(y, (0, 0, 0, 1, 0, 1))
        wins = yp.view(2, 3, 3, 3, 3, 64).permute(0, 1, 3, 2, 4, 5).reshape(18, 9, 64)
        t = qkv(wins).view(18, 9, 3, 2, 32).permute(2, 0, 3, 1, 4)
        o = ora.attention_from_tables(t[0], t[1], t[2], p("attn.rel_pos_h"), p("attn.rel_pos_w"), (3, 3))
        o = proj(o.permute(0, 2, 1, 3).reshape(18, 9, 64))
        o = o.view(2, 3, 3, 3, 3, 64).permute(0, 1, 3, 2, 4, 5).reshape(2, 9, 9, 64)[:, :8, :8]
        x1 = x + o
        ref = x1 + l2(nn.GELU()(l1(ln2(x1))))
    assert torch.allclose(got, ref, atol=1e-5)


def test_modules_cpu_route_equals_oracle():
    enc, sd, cfg = _tiny()
    g = torch.Generator().manual_seed(2)
    img = torch.randn(2, 3, 128, 128, generator=g)
    with torch.no_grad():
        ref = oe.encoder_forward(sd, img, cfg)
        ref_sdpa = oe.encoder_forward(sd, img, cfg, use_sdpa=True)
        got = enc(img)
    assert ref.shape == (2, 16, 8, 8)
    assert torch.allclose(ref, ref_sdpa, atol=1e-4)
    assert torch.allclose(got, ref, atol=1e-4)


def test_preprocess_constants():
    x = torch.full((1, 3, 4, 4), 128.0)
    y = oe.preprocess(x)
    for c in range(3):
        assert torch.allclose(y[0, c], torch.tensor((128.0 - oe.PIXEL_MEAN[c]) / oe.PIXEL_STD[c]))
