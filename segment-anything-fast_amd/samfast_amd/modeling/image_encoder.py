"""SAM ViT image encoder with the hot path on the HIP kernels.

Class names, constructor signatures, parameter names (hence state-dict keys) and
tensor contracts follow segment_anything_fast/modeling/image_encoder.py:
ImageEncoderViT :18-117, Block :120-183, Attention :186-253, window_partition
:256-277, window_unpartition :280-302, get_rel_pos :305-335,
add_decomposed_rel_pos :338-372, PatchEmbed :375-406.

What differs is Attention.forward on a GPU in bf16: q, k and v are read by the
attention kernel straight out of the qkv Linear's (B, N, 3, nH, hd) output
through strides, the two bias factors are computed inside the kernel from
rel_pos_h / rel_pos_w, and the result is written token-major, so the head
split/merge copies (:228-230, :249) and the bias tensors (:234-242) never exist.
Any other input (CPU, fp32, shapes the kernels do not cover) follows the
reference's own composition through flash_4._attention_rel_h_rel_w.

When, in addition, the four Linears of a Block have been swapped for
quant.Int8DynamicLinear, Block.forward (:167-183) runs with no eager glue as nine kernel
launches: LayerNorm + quantise, qkv GEMM, attention, quantise, proj GEMM + residual, LayerNorm
+ quantise, lin1 GEMM + GELU, quantise, lin2 GEMM + residual.  With SAMFAST_FUSED_QUANT=1 the
three quantisers that follow a GEMM run inside that GEMM (proj + norm2 + quantise, lin1 +
quantise, lin2 + the NEXT block's norm1 + quantise: five launches per block, same bits; slower
at the measured shapes, hence not the default).  SAMFAST_FUSED_BLOCK=0 keeps the
module-by-module composition.
"""

import os
from typing import Optional, Tuple, Type

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import _lib, flash_4, ops
from ..flash_4 import _attention_rel_h_rel_w
from .common import LayerNorm2d, MLPBlock

KB64_OPERANDS = os.environ.get("SAMFAST_KB64", "1") != "0"
WINDOWS_IN_PLACE = os.environ.get("SAMFAST_WINDOWS_IN_PLACE", "1") != "0"
FUSED_BLOCK = bool(int(os.environ.get("SAMFAST_FUSED_BLOCK", 1)))


class ImageEncoderViT(nn.Module):
    def __init__(
        self,
        img_size: int = 1024,
        patch_size: int = 16,
        in_chans: int = 3,
        embed_dim: int = 768,
        depth: int = 12,
        num_heads: int = 12,
        mlp_ratio: float = 4.0,
        out_chans: int = 256,
        qkv_bias: bool = True,
        norm_layer: Type[nn.Module] = nn.LayerNorm,
        act_layer: Type[nn.Module] = nn.GELU,
        use_abs_pos: bool = True,
        use_rel_pos: bool = False,
        rel_pos_zero_init: bool = True,
        window_size: int = 0,
        global_attn_indexes: Tuple[int, ...] = (),
    ) -> None:
        super().__init__()
        self.img_size = img_size
        grid = img_size // patch_size
        self.patch_embed = PatchEmbed(
            kernel_size=(patch_size, patch_size), stride=(patch_size, patch_size),
            in_chans=in_chans, embed_dim=embed_dim)
        self.pos_embed: Optional[nn.Parameter] = None
        if use_abs_pos:
            self.pos_embed = nn.Parameter(torch.zeros(1, grid, grid, embed_dim))
        self.blocks = nn.ModuleList([
            Block(
                dim=embed_dim, num_heads=num_heads, mlp_ratio=mlp_ratio, qkv_bias=qkv_bias,
                norm_layer=norm_layer, act_layer=act_layer, use_rel_pos=use_rel_pos,
                rel_pos_zero_init=rel_pos_zero_init,
                window_size=0 if i in global_attn_indexes else window_size,
                input_size=(grid, grid))
            for i in range(depth)
        ])
        self.neck = nn.Sequential(
            nn.Conv2d(embed_dim, out_chans, kernel_size=1, bias=False),
            LayerNorm2d(out_chans),
            nn.Conv2d(out_chans, out_chans, kernel_size=3, padding=1, bias=False),
            LayerNorm2d(out_chans),
        )

    # images per pass through the blocks; None = as many as the int8 kernels can address
    max_images_per_pass: Optional[int] = None

    def images_per_pass(self, x: torch.Tensor) -> int:
        """The int8 GEMMs and the row quantiser address an activation of M rows and K columns with
        32-bit offsets (M * K < 2^31).  The widest one is lin2's input, 4C per token: 102 images of
        64 x 64 tokens at ViT-H.  Images are independent, so a larger batch goes through the blocks
        in passes of at most that many."""
        if self.max_images_per_pass is not None:
            return max(1, int(self.max_images_per_pass))
        from ..quant import Int8LinearBase
        widest = max((m.in_features for m in self.modules() if isinstance(m, Int8LinearBase)), default=0)
        if widest == 0:
            return x.shape[0]
        return max(1, (2 ** 31 - 1) // (x.shape[1] * x.shape[2] * widest))

    def forward_blocks(self, x: torch.Tensor) -> torch.Tensor:
        """The transformer blocks on (B, H, W, C) tokens.  Consecutive blocks on the fused int8
        path are chained: a block's lin2 launch also runs the next block's norm1 and the qkv
        Linear's quantiser on the rows it has just written."""
        per_pass = self.images_per_pass(x)
        if x.shape[0] > per_pass:
            return torch.cat([self.forward_blocks(x[i:i + per_pass]) for i in range(0, x.shape[0], per_pass)])
        carry = None
        for i, blk in enumerate(self.blocks):
            if not blk._int8_fused_ok(x):
                x, carry = blk(x), None
                continue
            nxt = self.blocks[i + 1] if i + 1 < len(self.blocks) else None
            next_norm = None
            if nxt is not None and nxt._int8_fused_ok(x) and nxt._chains_from_previous():
                next_norm = (nxt.norm1.weight, nxt.norm1.bias, nxt.norm1.eps)
            x, carry = blk._forward_int8_fused(x, carry, next_norm)
        return x

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = self.patch_embed(x)
        if self.pos_embed is not None:
            x = x + self.pos_embed
        x = self.forward_blocks(x)
        return self.neck(x.permute(0, 3, 1, 2))


class Block(nn.Module):
    """Pre-norm transformer block; window_size > 0 runs attention inside
    non-overlapping windows, 0 runs it over the whole grid."""

    def __init__(
        self,
        dim: int,
        num_heads: int,
        mlp_ratio: float = 4.0,
        qkv_bias: bool = True,
        norm_layer: Type[nn.Module] = nn.LayerNorm,
        act_layer: Type[nn.Module] = nn.GELU,
        use_rel_pos: bool = False,
        rel_pos_zero_init: bool = True,
        window_size: int = 0,
        input_size: Optional[Tuple[int, int]] = None,
    ) -> None:
        super().__init__()
        self.norm1 = norm_layer(dim)
        self.attn = Attention(
            dim, num_heads=num_heads, qkv_bias=qkv_bias, use_rel_pos=use_rel_pos,
            rel_pos_zero_init=rel_pos_zero_init,
            input_size=input_size if window_size == 0 else (window_size, window_size))
        self.norm2 = norm_layer(dim)
        self.mlp = MLPBlock(embedding_dim=dim, mlp_dim=int(dim * mlp_ratio), act=act_layer)
        self.window_size = window_size

    def _int8_fused_ok(self, x: torch.Tensor) -> bool:
        from ..quant import Int8LinearBase
        attn, mlp = self.attn, self.mlp
        if not (FUSED_BLOCK and flash_4.USE_CUSTOM_KERNEL and x.is_cuda
                and x.dtype == torch.bfloat16 and x.dim() == 4 and attn.use_rel_pos):
            return False
        if not all(isinstance(m, Int8LinearBase) for m in (attn.qkv, attn.proj, mlp.lin1, mlp.lin2)):
            return False
        if self.window_size > 0 and not attn.proj.supports_row_scatter:
            return False
        if not (isinstance(self.norm1, nn.LayerNorm) and isinstance(self.norm2, nn.LayerNorm)
                and self.norm1.elementwise_affine and self.norm2.elementwise_affine
                and self.norm1.bias is not None and self.norm2.bias is not None
                and self.norm1.weight.dtype == torch.bfloat16
                and attn.rel_pos_h.dtype == torch.bfloat16 and attn.rel_pos_w.dtype == torch.bfloat16
                and isinstance(mlp.act, nn.GELU) and getattr(mlp.act, "approximate", "none") == "none"):
            return False
        B, H, W, C = x.shape
        g = self.window_size if self.window_size > 0 else None
        gh, gw = (g, g) if g else (H, W)
        return (attn.rel_pos_h.shape[0] == 2 * gh - 1 and attn.rel_pos_w.shape[0] == 2 * gw - 1
                and ops.attn_supported(gh * gw, (gh, gw), C // attn.num_heads, x.dtype))

    def _pad_rows(self, nH: int, hd: int, device):
        """(nH, hd) bf16 k and v rows of a zero-padded token: the qkv bias, rounded as the
        Linear's epilogue rounds it."""
        bias = self.attn.qkv.bias_f32
        key = None if bias is None else (bias.data_ptr(), self.attn.qkv.bias_bits._version, str(device))
        if getattr(self, "_pad_key", "unset") != key:
            C = nH * hd
            if bias is None:
                pk = pv = torch.zeros((nH, hd), dtype=torch.bfloat16, device=device)
            else:
                pk = bias[C:2 * C].to(torch.bfloat16).view(nH, hd).contiguous()
                pv = bias[2 * C:3 * C].to(torch.bfloat16).view(nH, hd).contiguous()
            self._pad_key, self._pad_kv = key, (pk, pv)
        return self._pad_kv

    def _chains_from_previous(self) -> bool:
        """Whether this block's norm1 + quantiser can run in the previous block's lin2 launch:
        its rows must be the image-ordered tokens (no window gather in front of qkv)."""
        return self.window_size == 0 or WINDOWS_IN_PLACE

    def _forward_int8_fused(self, x: torch.Tensor, carry=None, next_norm=None):
        """image_encoder.py:167-183 with every step on the HIP kernels.

        `carry` = (xq, sx): this block's norm1 output, already quantised by the previous block's
        lin2 launch.  `next_norm` = (gamma, beta, eps) of the next block's norm1: lin2 then
        also returns that block's carry.  Returns (tokens (B, H, W, C), carry for the next block)."""
        B, H, W, C = x.shape
        attn, mlp = self.attn, self.mlp
        nH = attn.num_heads
        hd = C // nH
        tokens = x.contiguous().view(B * H * W, C)
        # int8 activations travel K-block major between the quantisers and the GEMMs
        L = _lib.LAYOUT_KB64 if (C % 64 == 0 and KB64_OPERANDS) else _lib.LAYOUT_ROWMAJOR
        ws = self.window_size
        norm2 = (self.norm2.weight, self.norm2.bias, self.norm2.eps)
        if ws > 0 and not WINDOWS_IN_PLACE:
            # windows materialised: the partition is a row gather in the LayerNorm+quant kernel,
            # the unpartition a row scatter in the proj epilogue
            row_map, _ = ops.window_row_maps(B, H, W, ws, x.device)
            N = ws * ws
            xq, sx = ops.layernorm_quant(tokens, self.norm1.weight, self.norm1.bias, self.norm1.eps, row_map, layout=L)
            Bw = sx.shape[0] // N
            qkv = attn.qkv.linear_fused(xq, sx, _lib.EPILOGUE_NONE, layout=L).view(Bw, N, 3, nH, hd)
            q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
            o = ops.attn_relpos(q, k, v, attn.rel_pos_h, attn.rel_pos_w, (ws, ws), attn.scale)
            oq, so = ops.quant_rowwise(o.permute(0, 2, 1, 3).reshape(Bw * N, C), layout=L)
            tokens = attn.proj.linear_fused(oq, so, _lib.EPILOGUE_RESIDUAL, residual=tokens, dst_row=row_map, layout=L)
            hq, sh = ops.layernorm_quant(tokens, *norm2, layout=L)
        else:
            # norm1 + qkv's activation quantiser (unless the previous block's lin2 launch has done
            # it), qkv GEMM on the image-ordered tokens
            if carry is not None:
                xq, sx = carry
            else:
                xq, sx = ops.layernorm_quant(tokens, self.norm1.weight, self.norm1.bias, self.norm1.eps, layout=L)
            qkv = attn.qkv.linear_fused(xq, sx, _lib.EPILOGUE_NONE, layout=L).view(B, H * W, 3, nH, hd)
            q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
            if ws > 0:
                # the attention kernel cuts the windows itself; the reference's zero-padded tokens
                # enter as keys / values with the rows a zero input gives the qkv Linear: its bias
                pad_k, pad_v = self._pad_rows(nH, hd, x.device)
                o = ops.attn_relpos_windowed(q, k, v, attn.rel_pos_h, attn.rel_pos_w, pad_k, pad_v,
                                             (H, W), ws, attn.scale).view(B * H * W, C)
            else:
                o = ops.attn_relpos(q, k, v, attn.rel_pos_h, attn.rel_pos_w, (H, W), attn.scale)
                o = o.permute(0, 2, 1, 3).reshape(B * H * W, C)
            oq, so = ops.quant_rowwise(o, layout=L)
            # proj + `shortcut + x`, then norm2 + lin1's quantiser on the rows just written
            tokens, hq, sh = attn.proj.linear_fused_quant(oq, so, _lib.EPILOGUE_RESIDUAL, residual=tokens,
                                                          layout=L, ln=norm2, out_layout=L)
        # lin1 + GELU + lin2's quantiser, lin2 + `x + mlp(...)` (+ the next block's norm1 and quantiser)
        _, gq, sg = mlp.lin1.linear_fused_quant(hq, sh, _lib.EPILOGUE_GELU, layout=L, out_layout=L)
        if next_norm is not None:
            tokens, nq, sn = mlp.lin2.linear_fused_quant(gq, sg, _lib.EPILOGUE_RESIDUAL, residual=tokens,
                                                         out=tokens, layout=L, ln=next_norm, out_layout=L)
            return tokens.view(B, H, W, C), (nq, sn)
        tokens = mlp.lin2.linear_fused(gq, sg, _lib.EPILOGUE_RESIDUAL, residual=tokens, out=tokens, layout=L)
        return tokens.view(B, H, W, C), None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self._int8_fused_ok(x):
            return self._forward_int8_fused(x)[0]
        shortcut = x
        x = self.norm1(x)
        if self.window_size > 0:
            H, W = x.shape[1], x.shape[2]
            x, pad_hw = window_partition(x, self.window_size)
        x = self.attn(x)
        if self.window_size > 0:
            x = window_unpartition(x, self.window_size, pad_hw, (H, W))
        x = shortcut + x
        return x + self.mlp(self.norm2(x))


class Attention(nn.Module):
    """Multi-head attention over a (B, H, W, C) token grid with decomposed
    relative-position bias."""

    def __init__(
        self,
        dim: int,
        num_heads: int = 8,
        qkv_bias: bool = True,
        use_rel_pos: bool = False,
        rel_pos_zero_init: bool = True,
        input_size: Optional[Tuple[int, int]] = None,
    ) -> None:
        super().__init__()
        self.num_heads = num_heads
        head_dim = dim // num_heads
        self.scale = head_dim ** -0.5
        self.qkv = nn.Linear(dim, dim * 3, bias=qkv_bias)
        self.proj = nn.Linear(dim, dim)
        self.use_rel_pos = use_rel_pos
        if self.use_rel_pos:
            assert input_size is not None, \
                "Input size must be provided if using relative positional encoding."
            self.rel_pos_h = nn.Parameter(torch.zeros(2 * input_size[0] - 1, head_dim))
            self.rel_pos_w = nn.Parameter(torch.zeros(2 * input_size[1] - 1, head_dim))

    def _fused_ok(self, qkv: torch.Tensor, H: int, W: int, hd: int) -> bool:
        return (self.use_rel_pos and flash_4.USE_CUSTOM_KERNEL and qkv.is_cuda
                and self.rel_pos_h.shape[0] == 2 * H - 1 and self.rel_pos_w.shape[0] == 2 * W - 1
                and ops.attn_supported(H * W, (H, W), hd, qkv.dtype))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        B, H, W, C = x.shape
        nH = self.num_heads
        hd = C // nH
        qkv = self.qkv(x).reshape(B, H * W, 3, nH, hd)
        if self._fused_ok(qkv, H, W, hd):
            # strided (B, nH, N, hd) views of the token-major qkv buffer: no copies
            q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
            out = ops.attn_relpos(q, k, v, self.rel_pos_h, self.rel_pos_w, (H, W), self.scale)
            x = out.permute(0, 2, 1, 3).reshape(B, H, W, C)  # already token-major: a view
            return self.proj(x)

        q, k, v = qkv.permute(2, 0, 3, 1, 4).reshape(3, B * nH, H * W, hd).unbind(0)
        if self.use_rel_pos:
            rel_h, rel_w = add_decomposed_rel_pos(q, self.rel_pos_h, self.rel_pos_w, (H, W), (H, W))
            rel_h = rel_h.view(B, nH, H * W, H, 1)
            rel_w = rel_w.view(B, nH, H * W, 1, W)
        q, k, v = (t.view(B, nH, H * W, hd) for t in (q, k, v))
        if self.use_rel_pos:
            x = _attention_rel_h_rel_w(q, k, v, rel_h, rel_w)
        else:
            x = F.scaled_dot_product_attention(q, k, v)
        x = x.view(B, nH, H, W, hd).permute(0, 2, 3, 1, 4).reshape(B, H, W, C)
        return self.proj(x)


def window_partition(x: torch.Tensor, window_size: int) -> Tuple[torch.Tensor, Tuple[int, int]]:
    """(B, H, W, C) -> ((B * nWindows, ws, ws, C), (Hp, Wp)), zero padding the
    bottom and right edges up to a multiple of the window."""
    B, H, W, C = x.shape
    pad_h = (-H) % window_size
    pad_w = (-W) % window_size
    if pad_h or pad_w:
        x = F.pad(x, (0, 0, 0, pad_w, 0, pad_h))
    Hp, Wp = H + pad_h, W + pad_w
    x = x.reshape(B, Hp // window_size, window_size, Wp // window_size, window_size, C)
    windows = x.transpose(2, 3).reshape(-1, window_size, window_size, C)
    return windows, (Hp, Wp)


def window_unpartition(windows: torch.Tensor, window_size: int, pad_hw: Tuple[int, int],
                       hw: Tuple[int, int]) -> torch.Tensor:
    """Inverse of window_partition: back to (B, H, W, C) without the padding."""
    Hp, Wp = pad_hw
    H, W = hw
    per_image = (Hp // window_size) * (Wp // window_size)
    B = windows.shape[0] // per_image
    x = windows.view(B, Hp // window_size, Wp // window_size, window_size, window_size, -1)
    x = x.transpose(2, 3).reshape(B, Hp, Wp, -1)
    if Hp > H or Wp > W:
        x = x[:, :H, :W, :].contiguous()
    return x


def get_rel_pos(q_size: int, k_size: int, rel_pos: torch.Tensor) -> torch.Tensor:
    """(q_size, k_size, C) relative-position embeddings gathered from an (L, C)
    table, resizing the table linearly when L != 2*max(q_size, k_size) - 1."""
    span = int(2 * max(q_size, k_size) - 1)
    table = rel_pos
    if table.shape[0] != span:
        table = F.interpolate(table.t()[None], size=span, mode="linear")[0].t()
    q_pos = torch.arange(q_size, device=rel_pos.device)[:, None] * max(k_size / q_size, 1.0)
    k_pos = torch.arange(k_size, device=rel_pos.device)[None, :] * max(q_size / k_size, 1.0)
    rel = (q_pos - k_pos) + (k_size - 1) * max(q_size / k_size, 1.0)
    return table[rel.long()]


def add_decomposed_rel_pos(
    q: torch.Tensor,
    rel_pos_h: torch.Tensor,
    rel_pos_w: torch.Tensor,
    q_size: Tuple[int, int],
    k_size: Tuple[int, int],
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Bias factors for q (Bh, q_h*q_w, C): rel_h (Bh, q_h*q_w, k_h, 1) and
    rel_w (Bh, q_h*q_w, 1, k_w)."""
    q_h, q_w = q_size
    k_h, k_w = k_size
    Rh = get_rel_pos(q_h, k_h, rel_pos_h)
    Rw = get_rel_pos(q_w, k_w, rel_pos_w)
    Bh, _, dim = q.shape
    grid = q.reshape(Bh, q_h, q_w, dim)
    rel_h = torch.einsum("byxc,ykc->byxk", grid, Rh)
    rel_w = torch.einsum("byxc,xkc->byxk", grid, Rw)
    return (rel_h.reshape(Bh, q_h * q_w, k_h, 1), rel_w.reshape(Bh, q_h * q_w, 1, k_w))


class PatchEmbed(nn.Module):
    """Image to patch embedding: strided convolution, output (B, H, W, C)."""

    def __init__(
        self,
        kernel_size: Tuple[int, int] = (16, 16),
        stride: Tuple[int, int] = (16, 16),
        padding: Tuple[int, int] = (0, 0),
        in_chans: int = 3,
        embed_dim: int = 768,
    ) -> None:
        super().__init__()
        self.proj = nn.Conv2d(in_chans, embed_dim, kernel_size=kernel_size, stride=stride,
                              padding=padding)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        p = self.proj
        kh, kw = p.kernel_size
        if (x.is_cuda and p.stride == p.kernel_size and p.padding == (0, 0) and p.dilation == (1, 1)
                and p.groups == 1 and x.shape[2] % kh == 0 and x.shape[3] % kw == 0):
            # non-overlapping patches: the convolution is one GEMM over (channel, dy, dx) whose
            # output is already (B, H, W, C)
            B, C, H, W = x.shape
            gh, gw = H // kh, W // kw
            cols = x.reshape(B, C, gh, kh, gw, kw).permute(0, 2, 4, 1, 3, 5).reshape(B * gh * gw, C * kh * kw)
            y = F.linear(cols, p.weight.reshape(p.out_channels, C * kh * kw), p.bias)
            return y.view(B, gh, gw, p.out_channels)
        return self.proj(x).permute(0, 2, 3, 1)
