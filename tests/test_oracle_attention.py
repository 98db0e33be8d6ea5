"""Pins the attention oracle (oracle/relpos_attention.py) without running the
reference: closed forms, brute-force loops on tiny shapes, library routines and
invariants, each chosen so that a dropped term, a wrong sign / index or a
transposed operand fails."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import relpos_attention as ora


def _rand(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=dtype)


@pytest.mark.parametrize("S", [2, 3, 14, 64])
def test_get_rel_pos_closed_form(S):
    table = _rand(2 * S - 1, 5, seed=S)
    R = ora.get_rel_pos(S, S, table)
    assert R.shape == (S, S, 5)
    for i in range(S):
        for j in range(S):
            assert torch.equal(R[i, j], table[i - j + S - 1])


def test_get_rel_pos_resize_branch_is_halfpixel_linear():
    """L != 2S-1: the table is resized with half-pixel linear interpolation
    (F.interpolate mode='linear', align_corners False) before the gather."""
    S, L = 5, 13
    table = _rand(L, 3, seed=1)
    R = ora.get_rel_pos(S, S, table)
    span = 2 * S - 1
    resized = torch.empty(span, 3, dtype=table.dtype)
    for o in range(span):
        src = (o + 0.5) * L / span - 0.5
        src = min(max(src, 0.0), L - 1.0)
        lo = int(math.floor(src))
        hi = min(lo + 1, L - 1)
        w = src - lo
        resized[o] = (1 - w) * table[lo] + w * table[hi]
    for i in range(S):
        for j in range(S):
            assert torch.allclose(R[i, j], resized[i - j + S - 1], atol=1e-12)


def test_get_rel_pos_unequal_sizes():
    """q_size != k_size: coordinates scaled by the size ratio (image_encoder.py:331-333)."""
    q_size, k_size = 4, 8
    table = _rand(2 * 8 - 1, 2, seed=2)
    R = ora.get_rel_pos(q_size, k_size, table)
    for i in range(q_size):
        for j in range(k_size):
            idx = int(i * 2.0 - j * 1.0 + (k_size - 1) * 1.0)
            assert torch.equal(R[i, j], table[idx])


def test_add_decomposed_rel_pos_bruteforce():
    Bh, qh, qw, C = 2, 3, 4, 5
    q = _rand(Bh, qh * qw, C, seed=3)
    th, tw = _rand(2 * qh - 1, C, seed=4), _rand(2 * qw - 1, C, seed=5)
    rel_h, rel_w = ora.add_decomposed_rel_pos(q, th, tw, (qh, qw), (qh, qw))
    assert rel_h.shape == (Bh, qh * qw, qh, 1) and rel_w.shape == (Bh, qh * qw, 1, qw)
    for b in range(Bh):
        for y in range(qh):
            for x in range(qw):
                vec = q[b, y * qw + x]
                for j in range(qh):
                    assert abs(rel_h[b, y * qw + x, j, 0] - vec @ th[y - j + qh - 1]) < 1e-12
                for j in range(qw):
                    assert abs(rel_w[b, y * qw + x, 0, j] - vec @ tw[x - j + qw - 1]) < 1e-12


def test_add_decomposed_rel_pos_invariants():
    Bh, S, C = 1, 4, 6
    q = _rand(Bh, S * S, C, seed=6)
    zeros = torch.zeros(2 * S - 1, C, dtype=torch.float64)
    rel_h, rel_w = ora.add_decomposed_rel_pos(q, zeros, zeros, (S, S), (S, S))
    assert rel_h.abs().max() == 0 and rel_w.abs().max() == 0
    onehot = torch.zeros(Bh, S * S, C, dtype=torch.float64)
    onehot[..., 2] = 1.0
    th, tw = _rand(2 * S - 1, C, seed=7), _rand(2 * S - 1, C, seed=8)
    rel_h, rel_w = ora.add_decomposed_rel_pos(onehot, th, tw, (S, S), (S, S))
    for y in range(S):
        for x in range(S):
            for j in range(S):
                assert rel_h[0, y * S + x, j, 0] == th[y - j + S - 1, 2]
                assert rel_w[0, y * S + x, 0, j] == tw[x - j + S - 1, 2]


def _loop_attention(q, k, v, rel_h, rel_w):
    B, nH, N, hd = q.shape
    kh, kw = rel_h.shape[3], rel_w.shape[4]
    out = torch.zeros_like(q)
    for b in range(B):
        for h in range(nH):
            for i in range(N):
                logits = torch.empty(N, dtype=torch.float64)
                for n in range(N):
                    logits[n] = (q[b, h, i] @ k[b, h, n]) / math.sqrt(hd) \
                        + rel_h[b, h, i, n // kw, 0] + rel_w[b, h, i, 0, n % kw]
                w = torch.exp(logits - logits.max())
                w = w / w.sum()
                out[b, h, i] = w @ v[b, h]
    return out


def test_attention_against_loops():
    B, nH, kh, kw, hd = 1, 2, 3, 4, 5
    N = kh * kw
    q, k, v = (_rand(B, nH, N, hd, seed=s) for s in (10, 11, 12))
    rel_h, rel_w = _rand(B, nH, N, kh, 1, seed=13), _rand(B, nH, N, 1, kw, seed=14)
    got = ora.attention_rel_h_rel_w(q, k, v, rel_h, rel_w, compute_dtype=torch.float64)
    assert torch.allclose(got, _loop_attention(q, k, v, rel_h, rel_w), atol=1e-12)


@pytest.mark.parametrize("kh,kw,hd", [(14, 14, 80), (8, 64, 64)])
def test_attention_equals_sdpa_with_bias(kh, kw, hd):
    """The relation the reference's own test asserts (test/test_flash_4.py:32-39)."""
    B, nH, N = 2, 3, kh * kw
    q, k, v = (_rand(B, nH, N, hd, seed=s, dtype=torch.float32) * 0.5 for s in (20, 21, 22))
    rel_h = _rand(B, nH, N, kh, 1, seed=23, dtype=torch.float32) * 0.5
    rel_w = _rand(B, nH, N, 1, kw, seed=24, dtype=torch.float32) * 0.5
    got = ora.attention_rel_h_rel_w(q, k, v, rel_h, rel_w)
    bias = (rel_h + rel_w).view(B, nH, N, N)
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=bias)
    assert torch.allclose(got, ref, atol=2e-6, rtol=1e-5)
    assert torch.allclose(ora.attention_rel_h_rel_w_sdpa(q, k, v, rel_h, rel_w), ref)


def test_attention_invariants():
    B, nH, kh, kw, hd = 1, 2, 4, 5, 8
    N = kh * kw
    q, k, v = (_rand(B, nH, N, hd, seed=s) for s in (30, 31, 32))
    rel_h, rel_w = _rand(B, nH, N, kh, 1, seed=33), _rand(B, nH, N, 1, kw, seed=34)
    f = lambda *a: ora.attention_rel_h_rel_w(*a, compute_dtype=torch.float64)
    base = f(q, k, v, rel_h, rel_w)
    # zero bias = plain attention
    z_h, z_w = torch.zeros_like(rel_h), torch.zeros_like(rel_w)
    plain = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(hd), -1) @ v
    assert torch.allclose(f(q, k, v, z_h, z_w), plain, atol=1e-12)
    # a per-query constant in the bias cancels in the softmax
    shift = _rand(B, nH, N, 1, 1, seed=35)
    assert torch.allclose(f(q, k, v, rel_h + shift, rel_w), base, atol=1e-12)
    # constant V -> constant output
    assert torch.allclose(f(q, k, torch.full_like(v, 0.3), rel_h, rel_w),
                          torch.full_like(v, 0.3), atol=1e-12)
    # rel_h and rel_w are not interchangeable: swapping the roles changes the result
    assert not torch.allclose(
        f(q, k, v, rel_w.transpose(-1, -2)[..., :kh, :] if kh <= kw else rel_h, rel_w), base) or kh == kw
    # permuting key rows (kh axis) together with rel_h columns leaves the output unchanged
    perm = torch.tensor([2, 0, 3, 1])
    kp = k.view(B, nH, kh, kw, hd)[:, :, perm].reshape(B, nH, N, hd)
    vp = v.view(B, nH, kh, kw, hd)[:, :, perm].reshape(B, nH, N, hd)
    assert torch.allclose(f(q, kp, vp, rel_h[:, :, :, perm], rel_w), base, atol=1e-12)


def test_tables_composition_matches_manual_bias():
    B, nH, S, hd = 1, 2, 4, 8
    N = S * S
    q, k, v = (_rand(B, nH, N, hd, seed=s, dtype=torch.float32) for s in (40, 41, 42))
    th, tw = _rand(2 * S - 1, hd, seed=43, dtype=torch.float32), _rand(2 * S - 1, hd, seed=44, dtype=torch.float32)
    got = ora.attention_from_tables(q, k, v, th, tw, (S, S))
    bias = torch.zeros(B, nH, N, N)
    for y in range(S):
        for x in range(S):
            for jy in range(S):
                for jx in range(S):
                    bias[:, :, y * S + x, jy * S + jx] = (
                        q[:, :, y * S + x] @ th[y - jy + S - 1] + q[:, :, y * S + x] @ tw[x - jx + S - 1])
    ref = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(hd) + bias, -1) @ v
    assert torch.allclose(got, ref, atol=1e-5)
    assert torch.allclose(ora.attention_from_tables(q, k, v, th, tw, (S, S), use_sdpa=True), ref, atol=1e-5)


@pytest.mark.parametrize("H,W,ws", [(64, 64, 14), (14, 14, 14), (5, 9, 4)])
def test_window_partition_roundtrip_and_index_map(H, W, ws):
    B, C = 2, 3
    x = _rand(B, H, W, C, seed=50)
    win, (Hp, Wp) = ora.window_partition(x, ws)
    assert Hp % ws == 0 and Wp % ws == 0 and Hp - H < ws and Wp - W < ws
    nW = Wp // ws
    assert win.shape == (B * (Hp // ws) * nW, ws, ws, C)
    for b in range(B):
        for (y, xx) in [(0, 0), (H - 1, W - 1), (H // 2, W // 3)]:
            w_idx = b * (Hp // ws) * nW + (y // ws) * nW + xx // ws
            assert torch.equal(win[w_idx, y % ws, xx % ws], x[b, y, xx])
    # padded positions are zeros
    if Hp > H:
        last = win.view(B, Hp // ws, nW, ws, ws, C)[:, -1, :, (H % ws):, :, :]
        assert last.abs().max() == 0
    back = ora.window_unpartition(win, ws, (Hp, Wp), (H, W))
    assert torch.equal(back, x)
