"""Oracle: attention with decomposed relative-position bias (CPU, torch eager).

TEST INFRASTRUCTURE ONLY (see the package docstring).

Reference functions restated here
---------------------------------
get_rel_pos             segment_anything_fast/modeling/image_encoder.py:305-335
add_decomposed_rel_pos  segment_anything_fast/modeling/image_encoder.py:338-372
attention_rel_h_rel_w   segment_anything_fast/flash_4.py:335-370 (the eager
                        branch :368-370, which is the definition every other
                        branch of that function is tested against in
                        test/test_flash_4.py:32-39)
window_partition        segment_anything_fast/modeling/image_encoder.py:256-277
window_unpartition      segment_anything_fast/modeling/image_encoder.py:280-302
attention_forward       segment_anything_fast/modeling/image_encoder.py:225-253

How each is pinned (tests/test_oracle_attention.py)
---------------------------------------------------
get_rel_pos (same-size branch): closed form R[i, j] = table[i - j + S - 1],
    brute-force double loop.
get_rel_pos (resize branch): restated with the same library routine the
    reference calls (F.interpolate, mode="linear"); additionally checked
    against the closed-form half-pixel linear interpolation.  Never reached
    at SAM sizes (tables are exactly 2S-1 rows).
add_decomposed_rel_pos: triple loop on tiny shapes; zero tables give zero
    bias; a one-hot q returns a table column.
attention_rel_h_rel_w: float64 loop softmax on tiny shapes; equality with
    F.scaled_dot_product_attention(attn_mask=bias) (the relation the
    reference's own test asserts); bias==0 reduces to plain attention; a
    per-row constant added to the bias changes nothing; constant V gives
    constant output; permuting keys with their bias columns changes nothing.
window_partition / window_unpartition: round trip, zero padding, brute-force
    index map.
"""

import math
from typing import Tuple

import torch
import torch.nn.functional as F


def get_rel_pos(q_size: int, k_size: int, rel_pos: torch.Tensor) -> torch.Tensor:
    """Gather the (q_size, k_size, C) table of relative-position embeddings.

    Follows image_encoder.py:305-335.  `rel_pos` is (L, C).  When L differs
    from 2*max(q_size, k_size)-1 the table is first resized along L with
    linear interpolation (:319-328).  The row picked for query i and key j is
    i*max(k/q,1) - j*max(q/k,1) + (k_size-1)*max(q/k,1), truncated to an
    integer (:331-335).
    """
    span = 2 * max(q_size, k_size) - 1
    table = rel_pos
    if table.shape[0] != span:
        # (L, C) -> (1, C, L) -> resize L -> (span, C)
        table = F.interpolate(
            table.t().unsqueeze(0), size=span, mode="linear"
        ).squeeze(0).t()
    q_step = max(k_size / q_size, 1.0)
    k_step = max(q_size / k_size, 1.0)
    qi = torch.arange(q_size, device=rel_pos.device, dtype=torch.float32).unsqueeze(1) * q_step
    kj = torch.arange(k_size, device=rel_pos.device, dtype=torch.float32).unsqueeze(0) * k_step
    idx = (qi - kj + (k_size - 1) * k_step).long()
    return table[idx]


def add_decomposed_rel_pos(
    q: torch.Tensor,
    rel_pos_h: torch.Tensor,
    rel_pos_w: torch.Tensor,
    q_size: Tuple[int, int],
    k_size: Tuple[int, int],
) -> Tuple[torch.Tensor, torch.Tensor]:
    """The two bias factors of image_encoder.py:338-372.

    q is (Bh, q_h*q_w, C) and is NOT pre-scaled.  Returns
    rel_h (Bh, q_h*q_w, k_h, 1) with rel_h[b, (y, x), j] = <q[b, y, x], Rh[y, j]>
    rel_w (Bh, q_h*q_w, 1, k_w) with rel_w[b, (y, x), j] = <q[b, y, x], Rw[x, j]>.
    """
    q_h, q_w = q_size
    k_h, k_w = k_size
    Rh = get_rel_pos(q_h, k_h, rel_pos_h)
    Rw = get_rel_pos(q_w, k_w, rel_pos_w)
    Bh, _, C = q.shape
    grid = q.reshape(Bh, q_h, q_w, C)
    # (Bh, y, x, C) x (y, j, C) -> (Bh, y, x, j): batch over y
    rel_h = torch.matmul(grid.permute(1, 0, 2, 3).reshape(q_h, Bh * q_w, C), Rh.transpose(1, 2))
    rel_h = rel_h.reshape(q_h, Bh, q_w, k_h).permute(1, 0, 2, 3)
    # (Bh, y, x, C) x (x, j, C) -> (Bh, y, x, j): batch over x
    rel_w = torch.matmul(grid.permute(2, 0, 1, 3).reshape(q_w, Bh * q_h, C), Rw.transpose(1, 2))
    rel_w = rel_w.reshape(q_w, Bh, q_h, k_w).permute(1, 2, 0, 3)
    return (
        rel_h.reshape(Bh, q_h * q_w, k_h, 1),
        rel_w.reshape(Bh, q_h * q_w, 1, k_w),
    )


def attention_rel_h_rel_w(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    rel_h: torch.Tensor,
    rel_w: torch.Tensor,
    compute_dtype: torch.dtype = torch.float32,
) -> torch.Tensor:
    """softmax(q k^T / sqrt(hd) + rel_h + rel_w) v, written out.

    Follows flash_4.py:335-370: scale 1/sqrt(hd) (:343) applies to q.k only;
    key n = j_h*k_w + j_w gets bias rel_h[..., j_h, 0] + rel_w[..., 0, j_w]
    (:368-369).  q, k, v are (B, nH, N, hd); rel_h (B, nH, N, k_h, 1);
    rel_w (B, nH, N, 1, k_w).  All arithmetic in `compute_dtype`; the result
    is returned in that dtype.
    """
    B, nH, N, hd = q.shape
    k_h, k_w = rel_h.shape[3], rel_w.shape[4]
    assert k.shape[2] == k_h * k_w
    qc, kc, vc = q.to(compute_dtype), k.to(compute_dtype), v.to(compute_dtype)
    logits = torch.matmul(qc, kc.transpose(-1, -2)) * (1.0 / math.sqrt(hd))
    bias = rel_h.to(compute_dtype) + rel_w.to(compute_dtype)  # (B, nH, N, k_h, k_w)
    logits = logits + bias.reshape(B, nH, N, k_h * k_w)
    probs = torch.softmax(logits, dim=-1)
    return torch.matmul(probs, vc)


def attention_rel_h_rel_w_sdpa(q, k, v, rel_h, rel_w) -> torch.Tensor:
    """The same function through the library call the reference itself makes on
    a CPU (flash_4.py:368-370): materialise rel_h + rel_w as an additive mask and
    hand it to F.scaled_dot_product_attention.  Used as the timed CPU baseline and
    as the cross-check of attention_rel_h_rel_w."""
    B, nH, N, _ = q.shape
    bias = (rel_h + rel_w).reshape(B, nH, N, rel_h.shape[3] * rel_w.shape[4])
    return F.scaled_dot_product_attention(q, k, v, attn_mask=bias)


def attention_from_tables(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    rel_pos_h: torch.Tensor,
    rel_pos_w: torch.Tensor,
    grid_hw: Tuple[int, int],
    compute_dtype: torch.dtype = torch.float32,
    use_sdpa: bool = False,
) -> torch.Tensor:
    """Bias from the (2S-1, hd) tables, then attention_rel_h_rel_w.

    The composition image_encoder.py:234-245 performs.  q, k, v (B, nH, N, hd).
    """
    B, nH, N, hd = q.shape
    qc = q.to(compute_dtype).reshape(B * nH, N, hd)
    rel_h, rel_w = add_decomposed_rel_pos(
        qc, rel_pos_h.to(compute_dtype), rel_pos_w.to(compute_dtype), grid_hw, grid_hw
    )
    rel_h = rel_h.reshape(B, nH, N, grid_hw[0], 1)
    rel_w = rel_w.reshape(B, nH, N, 1, grid_hw[1])
    if use_sdpa:
        return attention_rel_h_rel_w_sdpa(
            q.to(compute_dtype), k.to(compute_dtype), v.to(compute_dtype), rel_h, rel_w)
    return attention_rel_h_rel_w(q, k, v, rel_h, rel_w, compute_dtype)


def window_partition(x: torch.Tensor, window_size: int):
    """(B, H, W, C) -> (B*nWin, ws, ws, C), zero padded on the bottom/right.

    Follows image_encoder.py:256-277.  Window order is (b, win_row, win_col).
    """
    B, H, W, C = x.shape
    pad_h = (-H) % window_size
    pad_w = (-W) % window_size
    if pad_h or pad_w:
        x = F.pad(x, (0, 0, 0, pad_w, 0, pad_h))
    Hp, Wp = H + pad_h, W + pad_w
    nh, nw = Hp // window_size, Wp // window_size
    tiles = x.reshape(B, nh, window_size, nw, window_size, C).transpose(2, 3)
    return tiles.reshape(B * nh * nw, window_size, window_size, C), (Hp, Wp)


def window_unpartition(windows: torch.Tensor, window_size: int, pad_hw, hw) -> torch.Tensor:
    """Inverse of window_partition, cropping the padding.

    Follows image_encoder.py:280-302.
    """
    Hp, Wp = pad_hw
    H, W = hw
    nh, nw = Hp // window_size, Wp // window_size
    B = windows.shape[0] // (nh * nw)
    x = windows.reshape(B, nh, nw, window_size, window_size, -1).transpose(2, 3)
    x = x.reshape(B, Hp, Wp, -1)
    return x[:, :H, :W, :].contiguous()


def attention_forward(
    x: torch.Tensor,
    qkv_weight: torch.Tensor,
    qkv_bias: torch.Tensor,
    proj_weight: torch.Tensor,
    proj_bias: torch.Tensor,
    rel_pos_h: torch.Tensor,
    rel_pos_w: torch.Tensor,
    num_heads: int,
    linear=F.linear,
    use_sdpa: bool = False,
) -> torch.Tensor:
    """Attention.forward of image_encoder.py:225-253 on (B, H, W, C) tokens.

    `linear(x, w, b)` is the Linear used for qkv and proj, so the same
    function serves the float path and the int8 dynamic-quant path.
    """
    B, H, W, C = x.shape
    N = H * W
    hd = C // num_heads
    qkv = linear(x.reshape(B, N, C), qkv_weight, qkv_bias)
    qkv = qkv.reshape(B, N, 3, num_heads, hd).permute(2, 0, 3, 1, 4)  # (3, B, nH, N, hd)
    q, k, v = qkv[0], qkv[1], qkv[2]
    out = attention_from_tables(q, k, v, rel_pos_h, rel_pos_w, (H, W), compute_dtype=q.dtype,
                                use_sdpa=use_sdpa)
    out = out.permute(0, 2, 1, 3).reshape(B, N, C)  # heads back into channels
    out = linear(out, proj_weight, proj_bias)
    return out.reshape(B, H, W, C)
