"""GPU parity: 2:4-sparse int8 linears (pack kernel + sparse-MFMA GEMM, through the C ABI)
against the CPU oracle.  Everything integer is bit-exact; the fused epilogues are compared
bit for bit with the dense int8 kernels run on the pruned dense weight."""

import numpy as np
import pytest
import torch

from helpers import linear_inputs
from oracle import quant_linear as orq

pytestmark = pytest.mark.gpu


def _pruned_int8(wq: torch.Tensor) -> np.ndarray:
    """Dense int8 matrix after the keep-2-largest-of-4 rule (ties: earlier position)."""
    return orq.prune_2_of_4(wq.to(torch.float32)).numpy().astype(np.int8)


@pytest.mark.parametrize("N,K,small", [(24, 128, False), (8, 64, True), (40, 320, True)])
def test_prune24_pack_matches_oracle(N, K, small):
    from samfast_amd import ops
    g = torch.Generator().manual_seed(N + K)
    hi = 4 if small else 128  # a small range forces magnitude ties and zeros
    wq = torch.randint(-hi + 1, hi, (N, K), generator=g, dtype=torch.int8)
    wc_ref, widx_ref = orq.pack_2_of_4(wq.numpy())
    wc, widx = ops.prune24_pack(wq.cuda())
    torch.cuda.synchronize()
    assert np.array_equal(wc.cpu().numpy(), wc_ref)
    assert np.array_equal(widx.cpu().numpy(), widx_ref)
    # the packed pair stands for exactly the pruned dense matrix
    assert np.array_equal(orq.unpack_2_of_4(wc_ref, widx_ref), _pruned_int8(wq))


@pytest.mark.parametrize("M,N,K", [
    (128, 256, 256), (1, 8, 256), (300, 264, 384), (513, 1280, 1280), (260, 5120, 1280),
    (129, 1280, 5120), (1000, 3072, 768), (31, 768, 3072),
])
def test_gemm_sparse24_i32_bit_exact(M, N, K):
    from samfast_amd import ops
    print(f"case sparse gemm M={M} N={N} K={K}", flush=True)
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    xq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    ref = orq.int8_gemm_i32(xq.numpy(), _pruned_int8(wq))
    wc, widx = ops.prune24_pack(wq.cuda())
    acc = ops.gemm_i8_sparse24_i32(xq.cuda(), wc, widx)
    torch.cuda.synchronize()
    assert np.array_equal(acc.cpu().numpy(), ref)


@pytest.mark.parametrize("M,N,K", [(300, 264, 256), (777, 5120, 1280), (130, 1280, 5120)])
def test_sparse24_linear_end_to_end_bit_exact(M, N, K):
    """prune (float) -> quantise -> pack -> sparse GEMM -> epilogue against the oracle."""
    from samfast_amd import _lib, ops
    from samfast_amd.quant import quantize_weight_per_channel
    from samfast_amd.sparse import prune_2_of_4
    print(f"case sparse linear M={M} N={N} K={K}", flush=True)
    x, w, b = linear_inputs(M, K, N, seed=M + N)
    ref = orq.sparse24_int8_linear(x, w, b)
    wp = prune_2_of_4(w.to(torch.float32))
    assert torch.equal(wp, orq.prune_2_of_4(w.to(torch.float32)))
    wq, sw = quantize_weight_per_channel(wp)
    wc, widx = ops.prune24_pack(wq.cuda())
    xq, sx = ops.quant_rowwise(x.cuda())
    y = ops.gemm_i8_sparse24_fused(xq, sx, wc, widx, sw.cuda(), b.to(torch.float32).cuda(),
                                   _lib.EPILOGUE_NONE)
    torch.cuda.synchronize()
    assert torch.equal(y.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(200, 512, 256), (1030, 5120, 1280), (515, 1280, 5120)])
def test_sparse24_fused_epilogues_equal_dense_kernels(M, N, K):
    """GELU and residual tails: same bits as the dense int8 kernel on the pruned weight."""
    from samfast_amd import _lib, ops
    print(f"case sparse fused M={M} N={N} K={K}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    xq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    sx = (torch.rand(M, generator=g) * 1e-2 + 1e-3).cuda()
    sw = (torch.rand(N, generator=g) * 1e-3 + 1e-4).cuda()
    bias = (torch.randn(N, generator=g) * 0.1).cuda()
    res = torch.randn((M, N), generator=g).to(torch.bfloat16).cuda()
    wd = torch.from_numpy(_pruned_int8(wq)).cuda()
    wc, widx = ops.prune24_pack(wq.cuda())
    for epi, kw in ((_lib.EPILOGUE_NONE, {}), (_lib.EPILOGUE_GELU, {}),
                    (_lib.EPILOGUE_RESIDUAL, {"residual": res})):
        dense = ops.gemm_i8_fused(xq, sx, wd, sw, bias, epi, **kw)
        sparse = ops.gemm_i8_sparse24_fused(xq, sx, wc, widx, sw, bias, epi, **kw)
        torch.cuda.synchronize()
        assert torch.equal(dense.view(torch.int16), sparse.view(torch.int16)), epi
    # in place on the residual stream, as the block uses it
    buf = res.clone()
    ops.gemm_i8_sparse24_fused(xq, sx, wc, widx, sw, bias, _lib.EPILOGUE_RESIDUAL, residual=buf, out=buf)
    torch.cuda.synchronize()
    assert torch.equal(buf.view(torch.int16), dense.view(torch.int16))


@pytest.mark.parametrize("M,N,K,layout", [
    (128, 256, 512, "rows"),        # one tile, the shortest K loop the resident form takes
    (384, 512, 640, "rows"),        # six tiles, fewer tiles than workgroup slots
    (1024, 768, 1280, "kb64"),      # K-block major codes as the encoder passes them
    (66560, 1280, 1280, "kb64"),    # 2600 tiles: five per resident workgroup, uneven lists
    (8192, 5120, 1280, "kb64"),     # lin1 shape: 1280 tiles
    (4096, 1280, 5120, "kb64"),     # lin2 shape: 160 tiles, 80 k-steps
])
def test_sparse24_resident_form_agrees(M, N, K, layout):
    """The resident-workgroup form of the 2:4 kernel (tile lists, the previous tile's output produced
    at the top of the next tile) against the one-workgroup-per-tile form, bit for bit over the whole
    output and for every epilogue (scale + bias, GELU, residual, residual in place), and against the
    dense kernel on the pruned weight."""
    from samfast_amd import _lib, ops
    print(f"case sparse resident M={M} N={N} K={K} {layout}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    xq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    sx = (torch.rand(M, generator=g) * 1e-2 + 1e-3).cuda()
    sw = (torch.rand(N, generator=g) * 1e-3 + 1e-4).cuda()
    bias = (torch.randn(N, generator=g) * 0.1).cuda()
    res = torch.randn((M, N), generator=g).to(torch.bfloat16).cuda()
    wd = torch.from_numpy(_pruned_int8(wq)).cuda()
    wc, widx = ops.prune24_pack(wq.cuda())
    L = _lib.LAYOUT_ROWMAJOR
    if layout == "kb64":
        L = _lib.LAYOUT_KB64
        xq, wd = ops.to_kb64(xq), ops.to_kb64(wd)

    def run(epi, in_place=False):
        if epi != _lib.EPILOGUE_RESIDUAL:
            return ops.gemm_i8_sparse24_fused(xq, sx, wc, widx, sw, bias, epi, layout=L)
        if in_place:
            buf = res.clone()
            return ops.gemm_i8_sparse24_fused(xq, sx, wc, widx, sw, bias, epi, residual=buf, out=buf, layout=L)
        return ops.gemm_i8_sparse24_fused(xq, sx, wc, widx, sw, bias, epi, residual=res, layout=L)

    for epi in (_lib.EPILOGUE_NONE, _lib.EPILOGUE_GELU, _lib.EPILOGUE_RESIDUAL):
        with _lib.knobs(SAMFAST_SPARSE_PERSIST=0):
            want = run(epi)
        with _lib.knobs(SAMFAST_SPARSE_PERSIST=2):
            got = run(epi)
            again = run(epi, in_place=True)
        kw = {"residual": res} if epi == _lib.EPILOGUE_RESIDUAL else {}
        dense = ops.gemm_i8_fused(xq, sx, wd, sw, bias, epi, layout=L, **kw)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), epi
        assert torch.equal(again.view(torch.int16), want.view(torch.int16)), epi
        assert torch.equal(dense.view(torch.int16), want.view(torch.int16)), epi


def test_sparse24_full_size_equals_dense_kernel():
    """lin1 of ViT-H at batch 16 (65536 x 5120 x 1280): accumulators of the sparse kernel
    equal those of the dense kernel on the pruned weight, compared on the GPU."""
    from samfast_amd import ops
    g = torch.Generator().manual_seed(77)
    M, N, K = 65536, 5120, 1280
    xq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    wd = torch.from_numpy(_pruned_int8(wq)).cuda()
    wc, widx = ops.prune24_pack(wq.cuda())
    a = ops.gemm_i8_sparse24_i32(xq, wc, widx)
    b = ops.gemm_i8_i32(xq, wd)
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_sparse24_rejects_bad_shapes():
    from samfast_amd import ops
    xq = torch.zeros((8, 192), dtype=torch.int8, device="cuda")
    wq = torch.zeros((8, 192), dtype=torch.int8, device="cuda")
    wc, widx = ops.prune24_pack(wq)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ops.gemm_i8_sparse24_i32(xq, wc, widx)
    with pytest.raises(RuntimeError):
        ops.prune24_pack(torch.zeros((8, 100), dtype=torch.int8, device="cuda"))


def test_apply_sparse_mlp_only_module_and_encoder():
    """apply_sparse(mlp_only) + apply_dynamic_quant on a ViT-H-shaped slice (2 blocks, one
    global): swapped modules, dense view of the packed weight, and the encoder output against
    the oracle that prunes and quantises the same way (cosine >= 0.999 per image)."""
    from functools import partial
    from samfast_amd import apply_dynamic_quant, apply_sparse
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.quant import Int8DynamicLinear, quantize_weight_per_channel
    from samfast_amd.sparse import Int8Sparse24Linear, mlp_only
    from samfast_amd.synthetic import init_encoder_weights, make_images
    from oracle import image_encoder as oe

    cfg = oe.EncoderConfig(embed_dim=1280, depth=2, num_heads=16, global_attn_indexes=(1,))
    enc = ImageEncoderViT(depth=2, embed_dim=1280, num_heads=16, global_attn_indexes=(1,),
                          window_size=14, use_rel_pos=True, mlp_ratio=4,
                          norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
    sd = {k: v.clone() for k, v in init_encoder_weights(enc, seed=3).items()}
    enc = enc.eval().to(torch.bfloat16).cuda()
    lin1_w = enc.blocks[0].mlp.lin1.weight.detach().float().cpu()
    apply_sparse(enc, mlp_only)          # float lin1 / lin2 -> 2:4 sparse int8
    apply_dynamic_quant(enc)             # the remaining Linears -> dense int8
    blk = enc.blocks[0]
    assert isinstance(blk.mlp.lin1, Int8Sparse24Linear) and isinstance(blk.mlp.lin2, Int8Sparse24Linear)
    assert isinstance(blk.attn.qkv, Int8DynamicLinear) and isinstance(blk.attn.proj, Int8DynamicLinear)
    wq_ref, _ = quantize_weight_per_channel(orq.prune_2_of_4(lin1_w))
    assert torch.equal(blk.mlp.lin1.wq.cpu(), wq_ref)

    x = make_images(1, seed=5).to(torch.bfloat16)
    dense = lambda a, w, b: orq.dynamic_int8_linear(a, w, b).float()
    sparse = lambda a, w, b: orq.sparse24_int8_linear(a, w, b).float()
    with torch.no_grad():
        out = enc(x.cuda()).float().cpu()
        sd_r = {k: v.to(torch.bfloat16).float() for k, v in sd.items()}
        ref = oe.encoder_forward(sd_r, x.float(), cfg, linear=dense, use_sdpa=True, mlp_linear=sparse)
    cos = torch.nn.functional.cosine_similarity(out.flatten(1), ref.flatten(1), dim=1).min().item()
    print(f"sparse mlp slice: cosine {cos:.6f}", flush=True)
    assert torch.isfinite(out).all() and cos >= 0.999, cos


def test_apply_sparse_every_linear_as_the_reference_does():
    """apply_sparse(model) with no filter - the reference's own scope (sparse.py:28-32 swaps every
    Linear): qkv, proj, lin1 and lin2 of a windowed and a global ViT-H block all become 2:4-sparse
    int8 Linears (proj without its row scatter, so windowed blocks take the module-by-module route
    or the in-place window kernel), and the encoder output follows the oracle that prunes and
    quantises all four the same way."""
    from functools import partial
    from samfast_amd import apply_sparse
    from samfast_amd.modeling import ImageEncoderViT
    from samfast_amd.sparse import Int8Sparse24Linear
    from samfast_amd.synthetic import init_encoder_weights, make_images
    from oracle import image_encoder as oe

    cfg = oe.EncoderConfig(embed_dim=1280, depth=2, num_heads=16, global_attn_indexes=(1,))
    enc = ImageEncoderViT(depth=2, embed_dim=1280, num_heads=16, global_attn_indexes=(1,),
                          window_size=14, use_rel_pos=True, mlp_ratio=4,
                          norm_layer=partial(torch.nn.LayerNorm, eps=1e-6))
    sd = {k: v.clone() for k, v in init_encoder_weights(enc, seed=7).items()}
    enc = enc.eval().to(torch.bfloat16).cuda()
    apply_sparse(enc)
    for blk in enc.blocks:
        for lin in (blk.attn.qkv, blk.attn.proj, blk.mlp.lin1, blk.mlp.lin2):
            assert isinstance(lin, Int8Sparse24Linear)
    x = make_images(1, seed=6).to(torch.bfloat16)
    sparse = lambda a, w, b: orq.sparse24_int8_linear(a, w, b).float()
    with torch.no_grad():
        out = enc(x.cuda()).float().cpu()
        sd_r = {k: v.to(torch.bfloat16).float() for k, v in sd.items()}
        ref = oe.encoder_forward(sd_r, x.float(), cfg, linear=sparse, use_sdpa=True)
    cos = torch.nn.functional.cosine_similarity(out.flatten(1), ref.flatten(1), dim=1).min().item()
    print(f"all-Linears sparse slice: cosine {cos:.6f}", flush=True)
    assert torch.isfinite(out).all() and cos >= 0.999, cos


def test_seeded_sweep_of_ragged_shapes_sparse_bit_exact():
    """Twenty random shapes: the 2:4 GEMM's accumulators equal the dense product with the pruned
    int8 matrix bit for bit (K in steps of 128 from 256, as the sparse kernel requires)."""
    from samfast_amd import ops
    rng = np.random.default_rng(77)
    for case in range(20):
        M = int(rng.integers(1, 600))
        N = 8 * int(rng.integers(1, 80))
        K = 128 * int(rng.integers(2, 12))
        print(f"case sparse sweep {case}: M={M} N={N} K={K}", flush=True)
        g = torch.Generator().manual_seed(500 + case)
        xq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
        wq = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
        wc, widx = ops.prune24_pack(wq.cuda())
        dense = orq.unpack_2_of_4(wc.cpu().numpy(), widx.cpu().numpy())
        ref = orq.int8_gemm_i64(xq.numpy(), dense)
        acc = ops.gemm_i8_sparse24_i32(xq.cuda(), wc, widx)
        assert np.array_equal(acc.cpu().numpy().astype(np.int64), ref)
