"""GPU parity of the whole encoder: product modules on the HIP kernels against the
CPU oracle on the same seeded weights and images.  Floating-point end to end:
the bar is cosine similarity >= 0.999 per image (stated with each assert)."""

from functools import partial

import pytest
import torch

from oracle import image_encoder as oe
from oracle import quant_linear as oq

pytestmark = pytest.mark.gpu

COSINE_MIN = 0.999


def _cos(a, b):
    return torch.nn.functional.cosine_similarity(
        a.float().flatten(1).cpu(), b.float().flatten(1).cpu(), dim=1).min().item()


def _rounded(sd):
    return {k: v.to(torch.bfloat16).float() for k, v in sd.items()}


def _vit_b():
    from samfast_amd.build_sam import build_image_encoder
    from samfast_amd.synthetic import init_encoder_weights, make_images
    enc = build_image_encoder("vit_b")
    sd = {k: v.clone() for k, v in init_encoder_weights(enc, seed=0).items()}
    x = make_images(1, seed=1)
    return enc, sd, x


def test_vit_b_bf16_attention_kernels_vs_oracle():
    """Config: full ViT-B encoder, bs 1, bf16, attention on the HIP kernels, bf16 Linears."""
    enc, sd, x = _vit_b()
    with torch.no_grad():
        ref = oe.encoder_forward(_rounded(sd), x.to(torch.bfloat16).float(), oe.VIT_B, use_sdpa=True)
        out = enc.eval().to(torch.bfloat16).cuda()(x.to(torch.bfloat16).cuda())
    c = _cos(out, ref)
    print(f"vit_b bf16: cosine {c:.6f}", flush=True)
    assert torch.isfinite(out.float()).all() and c >= COSINE_MIN


def test_vit_b_int8_linears_vs_quantised_oracle():
    """Same encoder with every Linear on the int8 path, against the oracle that quantises
    the same way on the CPU (fp32 everywhere else)."""
    from samfast_amd import apply_dynamic_quant
    enc, sd, x = _vit_b()
    lin = lambda a, w, b: oq.dynamic_int8_linear(a, w, b).float()
    with torch.no_grad():
        ref_q = oe.encoder_forward(_rounded(sd), x.to(torch.bfloat16).float(), oe.VIT_B, linear=lin,
                                   use_sdpa=True)
        ref_f = oe.encoder_forward(_rounded(sd), x.to(torch.bfloat16).float(), oe.VIT_B, use_sdpa=True)
        enc = enc.eval().to(torch.bfloat16).cuda()
        apply_dynamic_quant(enc)
        out = enc(x.to(torch.bfloat16).cuda())
    cq, cf = _cos(out, ref_q), _cos(out, ref_f)
    print(f"vit_b int8: cosine vs quantised oracle {cq:.6f}, vs float oracle {cf:.6f}", flush=True)
    assert torch.isfinite(out.float()).all() and cq >= COSINE_MIN
    assert cf >= 0.995  # quantisation noise itself, against the unquantised model


def test_vit_h_slice_vs_pytorch_rocm_bf16():
    """ViT-H shapes (hd 80, 16 heads), 4 blocks with one global, bs 2: the HIP path
    (attention + int8 linears) against the same modules on PyTorch-ROCm bf16 eager
    (SDPA with materialised bias, nn.Linear) - the reference's bf16 route."""
    from samfast_amd import apply_dynamic_quant, flash_4
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.synthetic import init_encoder_weights, make_images
    make = lambda: ImageEncoderViT(depth=4, embed_dim=1280, num_heads=16, global_attn_indexes=(3,),
                                   window_size=14, use_rel_pos=True, mlp_ratio=4,
                                   norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
    a = make()
    sd = {k: v.clone() for k, v in init_encoder_weights(a, seed=2).items()}
    b = make()
    b.load_state_dict(sd)
    x = make_images(2, seed=3).to(torch.bfloat16).cuda()
    a = a.eval().to(torch.bfloat16).cuda()
    b = b.eval().to(torch.bfloat16).cuda()
    apply_dynamic_quant(a)
    with torch.no_grad():
        out = a(x)
        flash_4.USE_CUSTOM_KERNEL = False
        try:
            ref = b(x)
        finally:
            flash_4.USE_CUSTOM_KERNEL = True
    c = _cos(out, ref)
    print(f"vit_h slice: cosine vs torch bf16 eager {c:.6f}", flush=True)
    assert c >= COSINE_MIN


def test_vit_l_slice_vs_oracle():
    """ViT-L shapes (embed 1024, 16 heads of 64 channels, MLP 4096), 3 blocks with the last one
    global, bs 2: attention kernels + int8 linears (fused block) against the oracle that
    quantises the same way on the CPU.  Bar: cosine >= 0.999 per image."""
    from samfast_amd import apply_dynamic_quant
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.synthetic import init_encoder_weights, make_images
    enc = ImageEncoderViT(depth=3, embed_dim=1024, num_heads=16, global_attn_indexes=(2,),
                          window_size=14, use_rel_pos=True, mlp_ratio=4,
                          norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
    sd = {k: v.clone() for k, v in init_encoder_weights(enc, seed=5).items()}
    x = make_images(2, seed=6).to(torch.bfloat16)
    cfg = oe.EncoderConfig(1024, 3, 16, (2,))
    lin = lambda a, w, b: oq.dynamic_int8_linear(a, w, b).float()
    with torch.no_grad():
        ref = oe.encoder_forward(_rounded(sd), x.float(), cfg, linear=lin, use_sdpa=True)
        enc = enc.eval().to(torch.bfloat16).cuda()
        apply_dynamic_quant(enc)
        assert all(b._int8_fused_ok(torch.empty(2, 64, 64, 1024, dtype=torch.bfloat16, device="cuda"))
                   for b in enc.blocks)
        out = enc(x.cuda())
    c = _cos(out, ref)
    print(f"vit_l slice int8: cosine vs quantised oracle {c:.6f}", flush=True)
    assert torch.isfinite(out.float()).all() and c >= COSINE_MIN


def test_predictor_set_torch_image():
    import samfast_amd
    from samfast_amd.synthetic import init_encoder_weights
    sam = samfast_amd.sam_model_fast_registry["vit_b"]()
    init_encoder_weights(sam.image_encoder, seed=0)
    sam = sam.cuda()
    pred = samfast_amd.SamPredictor(sam)
    img = torch.rand(1, 3, 1024, 768, device="cuda") * 255
    pred.set_torch_image(img, (1024, 768))
    f = pred.get_image_embedding()
    assert f.shape == (1, 256, 64, 64) and f.dtype == torch.bfloat16 and torch.isfinite(f.float()).all()


class _ChainedTrunk(torch.nn.Module):
    """Patch embedding, position embedding and the transformer blocks of an encoder: everything
    but the neck, whose two convolutions run in MIOpen (its choice of algorithm is not ours to pin)."""

    def __init__(self, encoder):
        super().__init__()
        self.encoder = encoder

    def forward(self, x):
        e = self.encoder
        x = e.patch_embed(x)
        if e.pos_embed is not None:
            x = x + e.pos_embed
        return e.forward_blocks(x)


def test_fast_registry_replays_a_graph_bit_equal_to_eager():
    """The encoder the fast registry returns replays a HIP graph for small batches (what the
    reference's compile_mode='max-autotune' gives, build_sam.py:67-71).  On the trunk (everything
    this repository's kernels compute) a replay is bit-equal to the eager forward, replay after
    replay and on a second image; through the neck's library convolutions it agrees to a bf16 step.
    A module swap drops the recording; a batch beyond the launch-bound range runs eagerly."""
    import samfast_amd
    from samfast_amd.graphs import ReplayedEncoder
    from samfast_amd.sparse import mlp_only
    from samfast_amd.synthetic import init_encoder_weights, make_images
    sam = samfast_amd.sam_model_fast_registry["vit_b"]()
    init_encoder_weights(sam.image_encoder, seed=0)
    sam = sam.cuda()
    samfast_amd.apply_dynamic_quant(sam.image_encoder)
    enc = sam.image_encoder
    assert isinstance(enc, ReplayedEncoder)
    imgs = make_images(2, seed=3).to(torch.bfloat16).cuda()
    a, b = imgs[:1], imgs[1:]

    def close(x, y):
        return torch.allclose(x.float(), y.float(), rtol=2 ** -6, atol=2e-2)

    with torch.no_grad():
        # the trunk alone behind the same wrapper: bit for bit
        trunk = _ChainedTrunk(enc._orig_mod)
        trunk_replay = ReplayedEncoder(trunk.eval())
        want_a, want_b = trunk(a), trunk(b)
        assert trunk_replay.replays(a)
        got = [trunk_replay(a), trunk_replay(b), trunk_replay(a)]
        torch.cuda.synchronize()
        assert len(trunk_replay._graphs) == 1
        assert torch.equal(got[0], want_a) and torch.equal(got[2], want_a) and torch.equal(got[1], want_b)
        # the whole encoder as the registry hands it out
        eager_a, eager_b = enc._orig_mod(a), enc._orig_mod(b)
        assert enc.replays(a)
        first, other, again = enc(a), enc(b), enc(a)
        torch.cuda.synchronize()
        assert len(enc._graphs) == 1
        # (MIOpen's convolutions are not run-to-run deterministic, eagerly or replayed)
        assert close(first, eager_a) and close(again, eager_a) and close(other, eager_b)
        # the predictor goes through the same wrapper
        pred = samfast_amd.SamPredictor(sam)
        raw = torch.rand(1, 3, 1024, 1024, device="cuda") * 255
        pred.set_torch_image(raw, (1024, 1024))
        assert close(pred.get_image_embedding(), enc._orig_mod(sam.preprocess(raw).to(torch.bfloat16)))
        # swapping modules drops the recordings; the next forward records the new modules
        trunk_replay(a)
        samfast_amd.apply_sparse(enc, mlp_only)
        assert not enc._graphs
        trunk_replay.invalidate()  # (a wrapper outside the swapped model is told by hand)
        sparse_want = trunk(a)
        assert not torch.equal(sparse_want, want_a)
        assert torch.equal(trunk_replay(a), sparse_want) and torch.equal(trunk_replay(a), sparse_want)
        assert close(enc(a), enc._orig_mod(a))
        # eight images are not launch-bound: eager path, nothing recorded
        big = make_images(8, seed=4).to(torch.bfloat16).cuda()
        assert not enc.replays(big)
        n = len(enc._graphs)
        enc(big)
        assert len(enc._graphs) == n


def test_fused_block_equals_module_composition():
    """Block.forward as nine fused launches against the same block run module by module
    (LayerNorm, window partition, residual adds and GELU in PyTorch-ROCm), windowed and global."""
    from samfast_amd import apply_dynamic_quant
    from samfast_amd.modeling import Block
    from samfast_amd.modeling import image_encoder as ie
    for ws in (14, 0):
        torch.manual_seed(5)
        blk = Block(1280, 16, use_rel_pos=True, window_size=ws, input_size=(64, 64),
                    norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
        with torch.no_grad():
            blk.attn.rel_pos_h.normal_(0, 0.02)
            blk.attn.rel_pos_w.normal_(0, 0.02)
            blk.norm1.weight.normal_(1, 0.1)
            blk.norm1.bias.normal_(0, 0.1)
        blk = blk.eval().to(torch.bfloat16).cuda()
        apply_dynamic_quant(blk)
        x = torch.randn(2, 64, 64, 1280, device="cuda").to(torch.bfloat16)
        with torch.no_grad():
            assert blk._int8_fused_ok(x)
            fused = blk(x)
            ie.FUSED_BLOCK = False
            try:
                assert not blk._int8_fused_ok(x)
                plain = blk(x)
            finally:
                ie.FUSED_BLOCK = True
        d = (fused.float() - plain.float()).abs()
        c = _cos(fused, plain)
        print(f"fused block ws={ws}: cosine {c:.6f} max-abs {d.max().item():.4f} mean-abs {d.mean().item():.5f}",
              flush=True)
        assert c >= 0.9999 and d.mean().item() <= 2e-3


class _Trunk(torch.nn.Module):
    """Encoder without the neck: patch embedding, position embedding and the blocks."""

    def __init__(self, enc):
        super().__init__()
        self.enc = enc

    def forward(self, x):
        x = self.enc.patch_embed(x)
        if self.enc.pos_embed is not None:
            x = x + self.enc.pos_embed
        for blk in self.enc.blocks:
            x = blk(x)
        return x


def test_graphed_encoder_replays_equal_eager():
    """HIP-graph replay of the ViT-B encoder (int8 linears).  The trunk (everything on the HIP
    kernels) must equal the eager result bit for bit on every replay, with eager work and
    synchronisations between the replays; the whole encoder is compared by cosine because MIOpen's
    neck convolutions are not run-to-run deterministic and may use another solver under capture."""
    from samfast_amd import apply_dynamic_quant
    from samfast_amd.graphs import GraphedEncoder
    from samfast_amd.synthetic import make_images
    enc, _, _ = _vit_b()
    enc = enc.eval().to(torch.bfloat16).cuda()
    apply_dynamic_quant(enc)
    trunk = _Trunk(enc)
    xs = [make_images(1, seed=s).to(torch.bfloat16).cuda() for s in (1, 2, 3)]
    with torch.no_grad():
        eager = [trunk(x).clone() for x in xs]
        eager_full = [enc(x).clone() for x in xs]
    g = GraphedEncoder(trunk, xs[0])
    gf = GraphedEncoder(enc, xs[0])
    for rep in range(2):
        for x, ref, ref_full in zip(xs, eager, eager_full):
            out = g(x).clone()
            full = gf(x).clone()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), rep
            assert _cos(full, ref_full) >= 0.9995  # MIOpen may pick another solver while capturing
            with torch.no_grad():  # eager work between replays
                again = trunk(x)
            torch.cuda.synchronize()
            assert torch.equal(again.view(torch.int16), ref.view(torch.int16))
    with pytest.raises(RuntimeError, match="recorded for"):
        g(torch.zeros((2, 3, 1024, 1024), dtype=torch.bfloat16, device="cuda"))


def test_derived_weight_copies_follow_load_state_dict():
    """The K-block major weight copies and the padding-token rows are derived from module state;
    loading other weights after a forward must not leave stale copies behind."""
    from samfast_amd import apply_dynamic_quant
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.synthetic import init_encoder_weights, make_images
    make = lambda: ImageEncoderViT(depth=2, embed_dim=256, num_heads=4, global_attn_indexes=(1,),
                                   window_size=14, use_rel_pos=True, mlp_ratio=4,
                                   norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
    a, b = make(), make()
    init_encoder_weights(a, seed=1)
    init_encoder_weights(b, seed=2)
    a = a.eval().to(torch.bfloat16).cuda()
    b = b.eval().to(torch.bfloat16).cuda()
    apply_dynamic_quant(a)
    apply_dynamic_quant(b)
    x = make_images(1, seed=4).to(torch.bfloat16).cuda()
    with torch.no_grad():
        ref_b = b(x).clone()
        a(x)                                   # builds a's derived copies
        a.load_state_dict(b.state_dict())      # in place: same storage, new values
        out = a(x)
    # stale copies would give an unrelated output; the neck convolutions are not run-to-run exact
    assert _cos(out, ref_b) >= 0.9995


# ---- the ViT-H configurations at their full depth ------------------------------------------

def _vit_h_state(seed=0):
    from samfast_amd.build_sam import build_image_encoder
    from samfast_amd.synthetic import init_encoder_weights
    enc = build_image_encoder("vit_h")
    sd = {k: v.clone() for k, v in init_encoder_weights(enc, seed=seed).items()}
    return enc, sd


def _trunk_input(enc, images):
    """Patch embedding + position embedding (PyTorch-ROCm library GEMM), i.e. what block 0 receives."""
    x = enc.patch_embed(images)
    return x + enc.pos_embed if enc.pos_embed is not None else x


def _run_blocks(enc, x):
    return enc.forward_blocks(x)


def test_vit_h_all_32_blocks_vs_oracle():
    """The ViT-H encoder at its full depth (32 blocks, 4 global), batch 2, seeded weights and images:
    (a) attention kernels + int8 linears against the oracle that quantises the same way;
    (b) attention kernels + bf16 nn.Linear against the float oracle.
    Bar: cosine >= 0.999 per image, outputs finite."""
    from samfast_amd import apply_dynamic_quant
    enc, sd = _vit_h_state()
    from samfast_amd.synthetic import make_images
    x = make_images(2, seed=1).to(torch.bfloat16)
    sd_r, xf = _rounded(sd), x.float()
    lin = lambda a, w, b: oq.dynamic_int8_linear(a, w, b).float()
    with torch.no_grad():
        print("vit_h depth 32: float oracle ...", flush=True)
        ref_f = oe.encoder_forward(sd_r, xf, oe.VIT_H, use_sdpa=True)
        print("vit_h depth 32: quantised oracle ...", flush=True)
        ref_q = oe.encoder_forward(sd_r, xf, oe.VIT_H, linear=lin, use_sdpa=True)
        enc = enc.eval().to(torch.bfloat16).cuda()
        out_f = enc(x.cuda()).float().cpu()
        apply_dynamic_quant(enc)
        assert all(b._int8_fused_ok(torch.empty(2, 64, 64, 1280, dtype=torch.bfloat16, device="cuda"))
                   for b in enc.blocks)
        out_q = enc(x.cuda()).float().cpu()
    cf, cq, cqf = _cos(out_f, ref_f), _cos(out_q, ref_q), _cos(out_q, ref_f)
    print(f"vit_h depth 32 bs2: bf16 linears vs float oracle {cf:.6f}; int8 vs quantised oracle {cq:.6f}; "
          f"int8 vs float oracle {cqf:.6f}", flush=True)
    assert torch.isfinite(out_f).all() and torch.isfinite(out_q).all()
    assert cf >= COSINE_MIN and cq >= COSINE_MIN
    assert cqf >= 0.995  # quantisation noise itself, against the unquantised model


def test_vit_h_batch_16_blocks_bitwise_equal_batch_2_runs():
    """Images are independent and every kernel here is deterministic, so the 32 blocks applied to a
    batch of 16 must give, image by image, the very bits they give on batches of 2 - whatever tile,
    workgroup or wave count the larger launch picks.  (The patch embedding in front is a library
    GEMM whose algorithm may change with the batch: both runs start from the same embedded tokens.)"""
    from samfast_amd import apply_dynamic_quant
    from samfast_amd.synthetic import make_images
    enc, _ = _vit_h_state()
    enc = enc.eval().to(torch.bfloat16).cuda()
    apply_dynamic_quant(enc)
    with torch.no_grad():
        x0 = _trunk_input(enc, make_images(16, seed=1).to(torch.bfloat16).cuda())
        full = _run_blocks(enc, x0.clone())
        torch.cuda.synchronize()
        assert torch.isfinite(full.float()).all()
        for i in (0, 6, 14):
            part = _run_blocks(enc, x0[i:i + 2].clone())
            assert torch.equal(part.view(torch.int16), full[i:i + 2].view(torch.int16)), i
        out = enc.neck(full.permute(0, 3, 1, 2))
    assert out.shape == (16, 256, 64, 64) and torch.isfinite(out.float()).all()


def test_oversized_batch_goes_through_the_blocks_in_passes():
    """The int8 kernels address an activation with 32-bit offsets, which caps a pass through the
    blocks at 102 images for ViT-H; a larger batch is cut into passes.  Forced here with a cap of
    2 on 5 images of a two-block ViT-B-shaped encoder: same bits as one pass."""
    from samfast_amd import apply_dynamic_quant
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.synthetic import init_encoder_weights, make_images
    enc = ImageEncoderViT(depth=2, embed_dim=768, num_heads=12, global_attn_indexes=(1,),
                          window_size=14, use_rel_pos=True, mlp_ratio=4,
                          norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
    init_encoder_weights(enc, seed=7)
    enc = enc.eval().to(torch.bfloat16).cuda()
    apply_dynamic_quant(enc)
    with torch.no_grad():
        x0 = _trunk_input(enc, make_images(5, seed=8).to(torch.bfloat16).cuda())
        assert enc.images_per_pass(x0) == (2 ** 31 - 1) // (4096 * 3072)
        whole = enc.forward_blocks(x0.clone())
        enc.max_images_per_pass = 2
        parts = enc.forward_blocks(x0.clone())
    assert parts.shape == whole.shape
    assert torch.equal(parts.view(torch.int16), whole.view(torch.int16))


def test_vit_h_batch_32_sparse_mlp_bitwise_equals_dense_kernels_on_pruned_weights():
    """The int8 + 2:4 configuration at its real batch (32 images, all 32 blocks): the sparse matrix
    cores on the packed lin1 / lin2 weights must reproduce, bit for bit, the dense int8 kernels run on
    the same magnitude-pruned weights (integer accumulators are exact, the epilogues are shared)."""
    from samfast_amd import apply_dynamic_quant, apply_fake_sparsity, apply_sparse
    from samfast_amd.sparse import Int8Sparse24Linear, mlp_only
    from samfast_amd.synthetic import make_images
    a, sd = _vit_h_state()
    b, _ = _vit_h_state()
    a = a.eval().to(torch.bfloat16).cuda()
    b = b.eval().to(torch.bfloat16).cuda()
    apply_sparse(a, mlp_only)
    apply_dynamic_quant(a)
    apply_fake_sparsity(b, mlp_only)
    apply_dynamic_quant(b)
    assert isinstance(a.blocks[5].mlp.lin2, Int8Sparse24Linear) and not isinstance(b.blocks[5].mlp.lin2, Int8Sparse24Linear)
    with torch.no_grad():
        x0 = _trunk_input(a, make_images(32, seed=1).to(torch.bfloat16).cuda())
        ya = _run_blocks(a, x0.clone())
        yb = _run_blocks(b, x0.clone())
    torch.cuda.synchronize()
    assert torch.isfinite(ya.float()).all()
    assert torch.equal(ya.view(torch.int16), yb.view(torch.int16))


def test_chained_blocks_equal_separate_quantiser_launches(monkeypatch):
    """The encoder's blocks with every row quantiser inside the GEMM that produces its rows (five
    launches per block, blocks chained through lin2) against the same blocks with the quantisers as
    launches of their own, and against blocks called one by one: bit-equal."""
    from samfast_amd import apply_dynamic_quant, quant
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.synthetic import init_encoder_weights, make_images
    enc = ImageEncoderViT(depth=4, embed_dim=1280, num_heads=16, global_attn_indexes=(1, 3),
                          window_size=14, use_rel_pos=True, mlp_ratio=4,
                          norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
    init_encoder_weights(enc, seed=6)
    enc = enc.eval().to(torch.bfloat16).cuda()
    apply_dynamic_quant(enc)
    with torch.no_grad():
        x0 = _trunk_input(enc, make_images(3, seed=2).to(torch.bfloat16).cuda())
        monkeypatch.setattr(quant, "FUSED_QUANT", True)
        chained = enc.forward_blocks(x0.clone())
        one_by_one = x0.clone()
        for blk in enc.blocks:
            one_by_one = blk(one_by_one)
        monkeypatch.setattr(quant, "FUSED_QUANT", False)
        separate = enc.forward_blocks(x0.clone())
    torch.cuda.synchronize()
    assert torch.isfinite(chained.float()).all()
    assert torch.equal(chained.view(torch.int16), separate.view(torch.int16))
    assert torch.equal(chained.view(torch.int16), one_by_one.view(torch.int16))
