"""Shared input recipes for the parity tests (CPU generators: the same tensors on
every machine)."""

import torch


def attn_inputs(B, nH, gh, gw, hd, seed=20, std=1.0, table_std=0.02, dtype=torch.bfloat16):
    """q, k, v ~ N(0, std) as (B, nH, N, hd); tables ~ N(0, table_std); all rounded to `dtype`
    (draw order q, k, v, rel_pos_h, rel_pos_w)."""
    g = torch.Generator().manual_seed(seed)
    N = gh * gw
    q, k, v = (torch.randn((B, nH, N, hd), generator=g) * std for _ in range(3))
    rph = torch.randn((2 * gh - 1, hd), generator=g) * table_std
    rpw = torch.randn((2 * gw - 1, hd), generator=g) * table_std
    return tuple(t.to(dtype) for t in (q, k, v, rph, rpw))


def bias_inputs(B, nH, gh, gw, hd, seed=20, std=0.5, dtype=torch.bfloat16):
    """The recipe of the reference's test/test_flash_4.py:10-28: everything ~ N(0, 0.5),
    rel_h (B, nH, N, gh, 1), rel_w (B, nH, N, 1, gw)."""
    g = torch.Generator().manual_seed(seed)
    N = gh * gw
    q, k, v = (torch.randn((B, nH, N, hd), generator=g) * std for _ in range(3))
    rel_h = torch.randn((B, nH, N, gh, 1), generator=g) * std
    rel_w = torch.randn((B, nH, N, 1, gw), generator=g) * std
    return tuple(t.to(dtype) for t in (q, k, v, rel_h, rel_w))


def linear_inputs(M, K, N, seed=4, outlier_frac=0.001, dtype=torch.bfloat16):
    """Activations ~ N(0, 1) with a fraction of rows scaled 20x; weights ~ N(0, 0.02);
    bias ~ N(0, 0.02)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=g)
    n_out = max(1, int(round(M * outlier_frac)))
    rows = torch.randperm(M, generator=g)[:n_out]
    x[rows] *= 20.0
    w = torch.randn((N, K), generator=g) * 0.02
    b = torch.randn((N,), generator=g) * 0.02
    return x.to(dtype), w.to(dtype), b.to(dtype)
