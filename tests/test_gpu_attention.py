"""GPU parity: HIP rel-pos attention (through the C ABI) against the CPU oracle.

Tolerance (attention is floating point): max-abs <= 2e-2 and mean-abs <= 1e-3
against the oracle evaluated in fp32 on the same bf16-rounded inputs.
"""

import math

import pytest
import torch

from helpers import attn_inputs, bias_inputs
from oracle import relpos_attention as ora

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
MEAN_ABS = 1e-3


def _check(out_gpu, ref, what):
    diff = (out_gpu.float().cpu() - ref.float()).abs()
    print(f"{what}: max-abs {diff.max().item():.3e} mean-abs {diff.mean().item():.3e}", flush=True)
    assert torch.isfinite(out_gpu.float()).all(), what
    assert diff.max().item() <= MAX_ABS, what
    assert diff.mean().item() <= MEAN_ABS, what


def _oracle_tables(q, k, v, rph, rpw, grid):
    outs = []
    for b in range(q.shape[0]):  # per image to bound memory
        outs.append(ora.attention_from_tables(q[b:b + 1], k[b:b + 1], v[b:b + 1], rph, rpw, grid,
                                              compute_dtype=torch.float32))
    return torch.cat(outs)


@pytest.mark.parametrize("B,nH,gh,gw,hd", [
    (1, 2, 64, 64, 64),     # ViT-B global shape, batch 1 (the case the reference cannot run)
    (2, 3, 64, 64, 80),     # ViT-H global shape
    (1, 2, 4, 64, 64),      # short grid: 256 tokens
    (3, 2, 14, 14, 64),     # ViT-B window
    (5, 3, 14, 14, 80),     # ViT-H window
    (2, 2, 7, 9, 80),       # ragged small window
    (1, 1, 13, 16, 64),     # largest window the kernel takes (208 keys)
])
def test_fused_tables_vs_oracle(B, nH, gh, gw, hd):
    from samfast_amd import ops
    print(f"case fused B={B} nH={nH} grid={gh}x{gw} hd={hd}", flush=True)
    q, k, v, rph, rpw = attn_inputs(B, nH, gh, gw, hd)
    ref = _oracle_tables(q, k, v, rph, rpw, (gh, gw))
    dev = "cuda"
    out = ops.attn_relpos(q.to(dev), k.to(dev), v.to(dev), rph.to(dev), rpw.to(dev), (gh, gw))
    torch.cuda.synchronize()
    _check(out, ref, f"fused {B}x{nH}x{gh}x{gw}x{hd}")


@pytest.mark.parametrize("B,nH,gh,gw,hd", [
    (1, 2, 64, 64, 64),
    (2, 2, 64, 64, 80),
    (4, 2, 14, 14, 80),
    (2, 2, 14, 14, 64),
])
def test_bias_form_vs_oracle(B, nH, gh, gw, hd):
    """Operand form of _attention_rel_h_rel_w with the reference test's input recipe."""
    from samfast_amd import ops
    print(f"case bias B={B} nH={nH} grid={gh}x{gw} hd={hd}", flush=True)
    q, k, v, rel_h, rel_w = bias_inputs(B, nH, gh, gw, hd)
    ref = ora.attention_rel_h_rel_w(q, k, v, rel_h, rel_w, compute_dtype=torch.float32)
    dev = "cuda"
    out = ops.attn_relpos_bias(q.to(dev), k.to(dev), v.to(dev),
                               rel_h.squeeze(-1).to(dev), rel_w.squeeze(-2).to(dev))
    torch.cuda.synchronize()
    _check(out, ref, f"bias {B}x{nH}x{gh}x{gw}x{hd}")


def test_token_major_strided_inputs():
    """q, k, v as strided views of a (B, N, 3, nH, hd) qkv buffer; output token-major."""
    from samfast_amd import ops
    B, nH, gh, gw, hd = 2, 4, 14, 14, 80
    q, k, v, rph, rpw = attn_inputs(B, nH, gh, gw, hd, seed=7)
    ref = _oracle_tables(q, k, v, rph, rpw, (gh, gw))
    qkv = torch.stack([q, k, v], dim=0).permute(1, 3, 0, 2, 4).contiguous().cuda()  # (B,N,3,nH,hd)
    qs, ks, vs = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    assert not qs.is_contiguous()
    out = ops.attn_relpos(qs, ks, vs, rph.cuda(), rpw.cuda(), (gh, gw))
    torch.cuda.synchronize()
    assert out.permute(0, 2, 1, 3).is_contiguous()  # token-major buffer
    _check(out, ref, "strided window")


def test_composite_and_operator_dispatch():
    """_attention_rel_h_rel_w and customflash::custom_flash_aligned reach the HIP kernel."""
    from samfast_amd.flash_4 import _attention_rel_h_rel_w
    B, nH, gh, gw, hd = 1, 2, 64, 64, 80
    q, k, v, rel_h, rel_w = bias_inputs(B, nH, gh, gw, hd, seed=3)
    ref = ora.attention_rel_h_rel_w(q, k, v, rel_h, rel_w, compute_dtype=torch.float32)
    dev = "cuda"
    out = _attention_rel_h_rel_w(q.to(dev), k.to(dev), v.to(dev), rel_h.to(dev), rel_w.to(dev))
    _check(out, ref, "composite global")
    rel_h_w = torch.cat([rel_h.squeeze(-1), rel_w.squeeze(-2)], dim=-1).to(dev)
    out2 = torch.ops.customflash.custom_flash_aligned(q.to(dev), k.to(dev), v.to(dev), rel_h_w,
                                                      1.0 / math.sqrt(hd))
    _check(out2, ref, "operator")
    # windows go through the composite too
    q, k, v, rel_h, rel_w = bias_inputs(3, 2, 14, 14, 64, seed=5)
    ref = ora.attention_rel_h_rel_w(q, k, v, rel_h, rel_w, compute_dtype=torch.float32)
    out3 = _attention_rel_h_rel_w(q.to(dev), k.to(dev), v.to(dev), rel_h.to(dev), rel_w.to(dev))
    _check(out3, ref, "composite window")


def test_invariants_full_size():
    """Config-sized global call (B=1, 12 heads, 4096 tokens, hd 64): properties that
    need no oracle - constant V gives constant output; zero tables equal plain SDPA."""
    from samfast_amd import ops
    B, nH, gh, gw, hd = 1, 12, 64, 64, 64
    q, k, v, rph, rpw = (t.cuda() for t in attn_inputs(B, nH, gh, gw, hd, seed=11))
    vc = torch.full_like(v, 0.75)
    out = ops.attn_relpos(q, k, vc, rph, rpw, (gh, gw))
    assert (out.float() - 0.75).abs().max().item() <= 4e-3
    zero_h, zero_w = torch.zeros_like(rph), torch.zeros_like(rpw)
    out0 = ops.attn_relpos(q, k, v, zero_h, zero_w, (gh, gw))
    sdpa = torch.nn.functional.scaled_dot_product_attention(q, k, v)
    d = (out0.float() - sdpa.float()).abs()
    assert d.max().item() <= MAX_ABS and d.mean().item() <= MEAN_ABS


def test_unsupported_shapes_raise():
    from samfast_amd import ops
    q = torch.zeros((1, 1, 100, 48), dtype=torch.bfloat16, device="cuda")
    t = torch.zeros((19, 48), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.attn_relpos(q, q, q, t, t, (10, 10))


@pytest.mark.parametrize("B,nH,H,W,ws,hd", [(2, 3, 20, 17, 14, 64), (1, 2, 64, 64, 14, 80), (2, 2, 9, 9, 3, 64),
                                           (1, 1, 14, 14, 14, 80), (1, 2, 15, 29, 7, 64), (3, 1, 27, 13, 13, 80),
                                           (1, 4, 1, 40, 14, 64), (2, 1, 33, 2, 11, 80)])
def test_windowed_on_image_tokens_equals_partitioned_windows(B, nH, H, W, ws, hd):
    """samfast_attn_relpos_windowed_fwd = window_partition + per-window attention +
    window_unpartition: same bits as running the window kernel on explicitly partitioned,
    padded windows whose padding tokens carry the pad rows; and within the attention
    tolerance of the fp32 oracle on those windows."""
    from samfast_amd import ops
    from oracle import relpos_attention as ora
    print(f"case windowed B={B} nH={nH} H={H} W={W} ws={ws} hd={hd}", flush=True)
    g = torch.Generator().manual_seed(B + H + W + hd)
    C = nH * hd
    qkv = torch.randn((B, H * W, 3, nH, hd), generator=g).to(torch.bfloat16)
    rph = (torch.randn((2 * ws - 1, hd), generator=g) * 0.02).to(torch.bfloat16)
    rpw = (torch.randn((2 * ws - 1, hd), generator=g) * 0.02).to(torch.bfloat16)
    pad_k = torch.randn((nH, hd), generator=g).to(torch.bfloat16)
    pad_v = torch.randn((nH, hd), generator=g).to(torch.bfloat16)
    scale = hd ** -0.5
    dq = qkv.cuda()
    q, k, v = (dq[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    out = ops.attn_relpos_windowed(q, k, v, rph.cuda(), rpw.cuda(), pad_k.cuda(), pad_v.cuda(), (H, W), ws, scale)
    torch.cuda.synchronize()
    assert out.shape == (B, H * W, nH, hd)

    # explicit partition on the CPU: padded positions get (anything, pad_k, pad_v)
    def part(t, fill):
        x = t.reshape(B, H, W, C).float()
        Hp, Wp = -(-H // ws) * ws, -(-W // ws) * ws
        full = fill.reshape(1, 1, 1, C).float().expand(B, Hp, Wp, C).clone()
        full[:, :H, :W] = x
        wins, _ = ora.window_partition(full, ws)
        return wins.reshape(-1, ws * ws, nH, hd).permute(0, 2, 1, 3).to(torch.bfloat16)
    zero = torch.zeros(C)
    qw, kw, vw = part(qkv[:, :, 0], zero), part(qkv[:, :, 1], pad_k), part(qkv[:, :, 2], pad_v)
    ow = ops.attn_relpos(qw.cuda().contiguous(), kw.cuda().contiguous(), vw.cuda().contiguous(),
                         rph.cuda(), rpw.cuda(), (ws, ws), scale)
    torch.cuda.synchronize()
    ow = ow.permute(0, 2, 1, 3).reshape(-1, ws, ws, C).float().cpu()
    Hp, Wp = -(-H // ws) * ws, -(-W // ws) * ws
    back = ora.window_unpartition(ow, ws, (Hp, Wp), (H, W)).reshape(B, H * W, nH, hd)
    assert torch.equal(out.float().cpu(), back)
    # oracle on the same windows (fp32): max-abs <= 2e-2, mean-abs <= 1e-3 on the real tokens
    ref = ora.attention_from_tables(qw, kw, vw, rph, rpw, (ws, ws))
    ref = ref.permute(0, 2, 1, 3).reshape(-1, ws, ws, C).float()
    ref = ora.window_unpartition(ref, ws, (Hp, Wp), (H, W)).reshape(B, H * W, nH, hd)
    err = (out.float().cpu() - ref).abs()
    assert err.max() <= 2e-2 and err.mean() <= 1e-3, (err.max(), err.mean())


@pytest.mark.parametrize("gh,gw,hd,ramp", [(64, 64, 80, 0.02), (64, 64, 64, 3.0), (14, 14, 80, 0.5), (14, 14, 64, 6.0)])
def test_rising_maximum_along_the_keys(gh, gw, hd, ramp):
    """The kernels rescale their accumulators only when the running maximum has grown by more than
    2^8 since the last rescale.  Keys whose logits rise steadily with the key index make the
    maximum move in every tile: slowly (never past the threshold after the first tile) or fast
    (past it every few tiles); both must agree with the oracle."""
    from samfast_amd import ops
    B, nH = 1, 2
    N = gh * gw
    q, k, v, rph, rpw = attn_inputs(B, nH, gh, gw, hd, seed=7)
    # one shared direction u: q gets a positive component along u, key n the component ramp*n/N*|u|
    g = torch.Generator().manual_seed(3)
    u = torch.randn(hd, generator=g)
    u = u / u.norm()
    steps = torch.arange(N, dtype=torch.float32) / N
    q = (q.float() + 4.0 * u).to(torch.bfloat16)
    k = (k.float() + (ramp * math.sqrt(hd) * 8.0) * steps[None, None, :, None] * u).to(torch.bfloat16)
    ref = _oracle_tables(q, k, v, rph, rpw, (gh, gw))
    dev = "cuda"
    out = ops.attn_relpos(q.to(dev), k.to(dev), v.to(dev), rph.to(dev), rpw.to(dev), (gh, gw))
    torch.cuda.synchronize()
    _check(out, ref, f"rising max {gh}x{gw}x{hd} ramp {ramp}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_window_kernel_with_large_bias_factors(dtype):
    """Relative-position tables 25 times the usual size: the bias factors <q, rel_pos row> reach
    +-20, the 16-bit operands that carry them (pre-divided by the softmax scale) about +-180 -
    inside the range include/samfast.h documents for fp16 - and the bias decides the softmax.
    fp16 keeps the bar of the other tests; bf16's eight-bit mantissa puts a factor of 20 on a grid
    of 0.06, so its bar is widened by that much."""
    from samfast_amd import ops
    B, nH, gh, gw, hd = 3, 2, 14, 14, 80
    q, k, v, rph, rpw = attn_inputs(B, nH, gh, gw, hd, seed=31, table_std=0.5, dtype=dtype)
    ref = _oracle_tables(q, k, v, rph, rpw, (gh, gw))
    out = ops.attn_relpos(q.cuda(), k.cuda(), v.cuda(), rph.cuda(), rpw.cuda(), (gh, gw))
    torch.cuda.synchronize()
    diff = (out.float().cpu() - ref.float()).abs()
    print(f"large bias {dtype}: max-abs {diff.max().item():.3e} mean-abs {diff.mean().item():.3e}", flush=True)
    assert torch.isfinite(out.float()).all()
    loose = 1 if dtype == torch.float16 else 8
    assert diff.max().item() <= loose * MAX_ABS and diff.mean().item() <= loose * MEAN_ABS


@pytest.mark.parametrize("B,nH,gh,gw,hd", [(5, 3, 14, 14, 80), (3, 2, 14, 14, 64), (2, 2, 7, 9, 80),
                                            (2, 2, 13, 16, 64), (2, 2, 5, 3, 80), (2, 2, 15, 13, 80)])
def test_both_window_key_layouts_vs_oracle(B, nH, gh, gw, hd):
    """The window kernel exists with the keys in token order (attn_window_kernel) and as grid rows
    padded to 16 (attn_window_rows_kernel, SAMFAST_ATTN_WINDOW_ROWS=1, built for gh <= 14).  Each is held to the
    oracle's bar on its own, with the tables and with caller-computed bias factors; a window of 15
    rows only fits the first."""
    from samfast_amd import _lib, ops
    print(f"case window layouts B={B} nH={nH} grid={gh}x{gw} hd={hd}", flush=True)
    q, k, v, rph, rpw = attn_inputs(B, nH, gh, gw, hd, seed=17)
    ref = _oracle_tables(q, k, v, rph, rpw, (gh, gw))
    qb, kb, vb, rel_h, rel_w = bias_inputs(B, nH, gh, gw, hd, seed=18)
    ref_b = ora.attention_rel_h_rel_w(qb, kb, vb, rel_h, rel_w, compute_dtype=torch.float32)
    for rows in (0, 1):
        with _lib.knobs(SAMFAST_ATTN_WINDOW_ROWS=rows):
            out = ops.attn_relpos(q.cuda(), k.cuda(), v.cuda(), rph.cuda(), rpw.cuda(), (gh, gw))
            out_b = ops.attn_relpos_bias(qb.cuda(), kb.cuda(), vb.cuda(), rel_h.cuda().squeeze(-1),
                                         rel_w.cuda().squeeze(-2))
            torch.cuda.synchronize()
        _check(out, ref, f"tables, rows layout {rows}")
        _check(out_b, ref_b, f"bias factors, rows layout {rows}")


@pytest.mark.parametrize("hd,gh", [(80, 64), (64, 64), (80, 8)])
def test_global_kernel_wave_count_variants_agree(hd, gh):
    """The global kernel runs with 128 or 256 queries per workgroup (4 or 8 wavefronts); the choice
    follows the grid size and can be forced.  A query's arithmetic does not depend on it."""
    from samfast_amd import _lib, ops
    B, nH, gw = 1, 2, 64
    q, k, v, rph, rpw = (t.cuda() for t in attn_inputs(B, nH, gh, gw, hd, seed=5))
    outs = {}
    for waves in ("4", "8"):
        with _lib.knobs(SAMFAST_ATTN_WAVES=int(waves)):
            outs[waves] = ops.attn_relpos(q, k, v, rph, rpw, (gh, gw)).clone()
    torch.cuda.synchronize()
    assert torch.equal(outs["4"], outs["8"])
    ref = _oracle_tables(q.cpu(), k.cpu(), v.cpu(), rph.cpu(), rpw.cpu(), (gh, gw))
    _check(outs["8"], ref, "8 wavefronts per workgroup")


@pytest.mark.parametrize("batch", [1, 8])
@pytest.mark.parametrize("head,hidden_dim", [(16, 80), (12, 64)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_test_recipe_against_sdpa(batch, head, hidden_dim, dtype):
    """The reference's own test of this operator (test/test_flash_4.py:5-43): its shapes (batch 1
    and 8, 16 heads x 80 / 12 heads x 64, 4096 tokens), its two dtypes (:41-43), its input recipe
    (seed 20, q / k / v and both bias factors ~ N(0, 0.5)) and its tolerance (rtol = atol = 1e-3)
    against scaled_dot_product_attention with the materialised bias; SDPA is evaluated in fp32 on
    the same half-precision inputs and rounded once."""
    from samfast_amd.flash_4 import _attention_rel_h_rel_w
    seq_len, device = 4096, "cuda"
    print(f"case reference recipe batch={batch} head={head} hd={hidden_dim} {dtype}", flush=True)
    torch.manual_seed(20)
    q, k, v = (torch.empty((batch, head, seq_len, hidden_dim), dtype=dtype, device=device).normal_(mean=0.0, std=0.5)
               for _ in range(3))
    w = int(seq_len ** 0.5)
    rel_h = torch.empty((batch, head, seq_len, w, 1), dtype=dtype, device=device).normal_(mean=0, std=0.5)
    rel_w = torch.empty((batch, head, seq_len, 1, w), dtype=dtype, device=device).normal_(mean=0, std=0.5)
    out = _attention_rel_h_rel_w(q, k, v, rel_h, rel_w)
    assert out.dtype == dtype and out.shape == q.shape
    for b in range(batch):  # one image at a time: the bias is 1 GB per image in fp32
        bias = (rel_h[b:b + 1].float() + rel_w[b:b + 1].float()).view(1, head, seq_len, seq_len)
        ref = torch.nn.functional.scaled_dot_product_attention(
            q[b:b + 1].float(), k[b:b + 1].float(), v[b:b + 1].float(), attn_mask=bias)
        torch.testing.assert_close(ref.to(dtype), out[b:b + 1], rtol=1e-3, atol=1e-3)


def test_seeded_sweep_of_window_and_grid_shapes():
    """Random window shapes up to the kernel's limits (gh <= 15, gw <= 16, <= 208 tokens) and 64-wide
    grids with an even number of rows, both head sizes, against the fp32 oracle at the stated bar."""
    import numpy as np
    from samfast_amd import ops
    rng = np.random.default_rng(31)
    shapes = []
    while len(shapes) < 14:
        gh, gw = int(rng.integers(1, 16)), int(rng.integers(1, 17))
        if gh * gw <= 208:
            shapes.append((int(rng.integers(1, 7)), int(rng.integers(1, 5)), gh, gw, (64, 80)[len(shapes) % 2]))
    for gh in (2, 6, 10, 30):
        shapes.append((int(rng.integers(1, 3)), int(rng.integers(1, 3)), gh, 64, (64, 80)[(gh // 2) % 2]))
    for case, (B, nH, gh, gw, hd) in enumerate(shapes):
        print(f"case attention sweep {case}: B={B} nH={nH} grid={gh}x{gw} hd={hd}", flush=True)
        q, k, v, rph, rpw = attn_inputs(B, nH, gh, gw, hd, seed=300 + case)
        ref = _oracle_tables(q, k, v, rph, rpw, (gh, gw))
        out = ops.attn_relpos(q.cuda(), k.cuda(), v.cuda(), rph.cuda(), rpw.cuda(), (gh, gw))
        torch.cuda.synchronize()
        _check(out, ref, f"sweep {B}x{nH}x{gh}x{gw}x{hd}")


@pytest.mark.parametrize("B,nH,gh,gw,hd", [(1, 2, 64, 64, 64), (2, 2, 64, 64, 80), (3, 2, 14, 14, 64),
                                           (4, 3, 14, 14, 80), (2, 2, 7, 9, 80), (1, 1, 13, 16, 64)])
def test_float16_operands_vs_oracle(B, nH, gh, gw, hd):
    """The float16 instantiation of both kernels (the reference's operator takes fp16 and bf16,
    flash_4.py:188,348): tables form and bias form against the fp32 oracle on the same
    fp16-rounded inputs, at the bar of the bf16 tests."""
    from samfast_amd import ops
    print(f"case fp16 B={B} nH={nH} grid={gh}x{gw} hd={hd}", flush=True)
    q, k, v, rph, rpw = attn_inputs(B, nH, gh, gw, hd, dtype=torch.float16)
    ref = _oracle_tables(q, k, v, rph, rpw, (gh, gw))
    out = ops.attn_relpos(q.cuda(), k.cuda(), v.cuda(), rph.cuda(), rpw.cuda(), (gh, gw))
    assert out.dtype == torch.float16
    _check(out, ref, f"fp16 fused {B}x{nH}x{gh}x{gw}x{hd}")
    q, k, v, rel_h, rel_w = bias_inputs(B, nH, gh, gw, hd, dtype=torch.float16)
    ref = ora.attention_rel_h_rel_w(q, k, v, rel_h, rel_w, compute_dtype=torch.float32)
    out = ops.attn_relpos_bias(q.cuda(), k.cuda(), v.cuda(), rel_h.squeeze(-1).cuda(), rel_w.squeeze(-2).cuda())
    _check(out, ref, f"fp16 bias {B}x{nH}x{gh}x{gw}x{hd}")


def test_float16_windowed_on_image_tokens_and_module():
    """fp16 through the image-ordered window entry point (padding rows included) against the oracle
    on explicitly partitioned windows, and through the Attention module (fp16 nn.Linear + the HIP
    kernel) against the module's eager route."""
    from samfast_amd import flash_4, ops
    from samfast_amd.modeling import Attention
    B, nH, H, W, ws, hd = 2, 3, 20, 17, 14, 80
    g = torch.Generator().manual_seed(5)
    C = nH * hd
    f16 = torch.float16
    qkv = torch.randn((B, H * W, 3, nH, hd), generator=g).to(f16)
    rph = (torch.randn((2 * ws - 1, hd), generator=g) * 0.02).to(f16)
    rpw = (torch.randn((2 * ws - 1, hd), generator=g) * 0.02).to(f16)
    pad_k, pad_v = torch.randn((nH, hd), generator=g).to(f16), torch.randn((nH, hd), generator=g).to(f16)
    dq = qkv.cuda()
    q, k, v = (dq[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    out = ops.attn_relpos_windowed(q, k, v, rph.cuda(), rpw.cuda(), pad_k.cuda(), pad_v.cuda(), (H, W), ws, hd ** -0.5)
    Hp, Wp = -(-H // ws) * ws, -(-W // ws) * ws

    def part(t, fill):
        full = fill.reshape(1, 1, 1, C).float().expand(B, Hp, Wp, C).clone()
        full[:, :H, :W] = t.reshape(B, H, W, C).float()
        wins, _ = ora.window_partition(full, ws)
        return wins.reshape(-1, ws * ws, nH, hd).permute(0, 2, 1, 3).to(f16)
    qw, kw, vw = part(qkv[:, :, 0], torch.zeros(C)), part(qkv[:, :, 1], pad_k), part(qkv[:, :, 2], pad_v)
    ref = ora.attention_from_tables(qw, kw, vw, rph, rpw, (ws, ws))
    ref = ref.permute(0, 2, 1, 3).reshape(-1, ws, ws, C).float()
    ref = ora.window_unpartition(ref, ws, (Hp, Wp), (H, W)).reshape(B, H * W, nH, hd)
    _check(out, ref, "fp16 windowed on image tokens")

    torch.manual_seed(1)
    att = Attention(256, 4, use_rel_pos=True, input_size=(14, 14))
    with torch.no_grad():
        att.rel_pos_h.normal_(0, 0.02)
        att.rel_pos_w.normal_(0, 0.02)
    att = att.eval().to(f16).cuda()
    x = torch.randn(3, 14, 14, 256, device="cuda").to(f16)
    with torch.no_grad():
        got = att(x)
        flash_4.USE_CUSTOM_KERNEL = False
        try:
            eager = att(x)
        finally:
            flash_4.USE_CUSTOM_KERNEL = True
    assert got.dtype == f16
    d = (got.float() - eager.float()).abs()
    assert d.max().item() <= 2e-2 and d.mean().item() <= 1e-3, (d.max().item(), d.mean().item())
