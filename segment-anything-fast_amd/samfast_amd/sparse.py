"""2:4 magnitude sparsity for the quantised Linears, on the sparse int8 matrix cores.

Mirrors segment_anything_fast/sparse.py: `apply_fake_sparsity(model)` zeroes the two
smallest-magnitude weights of every 4 consecutive input features (the rule of
torch.ao.pruning.WeightNormSparsifier with sparse_block_shape (1, 4), zeros_per_block 2,
sparsity_level 1.0, sparse.py:6-25) and `apply_sparse(model)` then swaps the Linears for
modules that keep only the surviving half of the weight (sparse.py:28-32).  Here the
compressed weight is int8 and feeds v_smfmac_i32_32x32x64_i8; the activation side is the
same dynamic per-token int8 quantiser as Int8DynamicLinear.

Both functions take an optional `filter_fn(module, fqn)`; the reference applies them to every
Linear, the int8 + 2:4 benchmark configuration only to the MLP (`mlp_only`).
"""

from typing import Callable, Optional

import torch
import torch.nn as nn

from . import _lib, ops
from .quant import Int8DynamicLinear, Int8LinearBase, quantize_weight_per_channel
from .tools import replace_with_custom_fn_if_matches_filter


def mlp_only(mod: nn.Module, fqn: str) -> bool:
    """filter_fn selecting lin1 / lin2 of every MLPBlock (modeling/common.py:21-22)."""
    return fqn.endswith(".mlp.lin1") or fqn.endswith(".mlp.lin2")


def prune_2_of_4(weight: torch.Tensor) -> torch.Tensor:
    """Keep the 2 largest |w| of every 4 consecutive along the last axis (ties: the earlier
    position), zero the rest."""
    N, K = weight.shape
    if K % 4 != 0:
        raise ValueError("prune_2_of_4 needs in_features % 4 == 0")
    blocks = weight.detach().reshape(N, K // 4, 4)
    order = torch.sort(blocks.abs().to(torch.float32), dim=-1, descending=True, stable=True).indices
    keep = torch.zeros_like(blocks, dtype=torch.bool)
    keep.scatter_(-1, order[..., :2], True)
    return (blocks * keep).reshape(N, K)


class Int8Sparse24Linear(Int8LinearBase):
    """Dynamic int8 Linear whose weight is stored 2:4-compressed (`wc`, `widx`; layout in
    include/samfast.h).  Built on the GPU: packing runs as a HIP kernel."""

    supports_row_scatter = False

    def __init__(self, in_features: int, out_features: int, wc: torch.Tensor, widx: torch.Tensor,
                 sw: torch.Tensor, bias: Optional[torch.Tensor]) -> None:
        super().__init__(in_features, out_features, sw, bias)
        self.register_buffer("wc", wc)
        self.register_buffer("widx", widx)

    @classmethod
    def from_int8(cls, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor]):
        """wq (N, K) int8 on the GPU (pruned here by int8 magnitude if it is not 2:4 yet)."""
        wc, widx = ops.prune24_pack(wq.contiguous())
        return cls(wq.shape[1], wq.shape[0], wc, widx, sw, bias)

    @classmethod
    def from_float(cls, linear: nn.Module) -> "Int8Sparse24Linear":
        """From an nn.Linear (or Int8DynamicLinear): prune the float weight, quantise per
        output channel (pruning never removes a row's absmax, so scales are unchanged)."""
        if isinstance(linear, Int8DynamicLinear):
            # already quantised: the int8 codes order like the float weights up to rounding ties
            return cls.from_int8(linear.wq, linear.sw, linear.bias)
        w = prune_2_of_4(linear.weight.detach().to(torch.float32))
        wq, sw = quantize_weight_per_channel(w)
        if not wq.is_cuda:
            raise RuntimeError("samfast: move the model to the GPU before apply_sparse "
                               "(the 2:4 packer is a HIP kernel; there is no CPU route)")
        return cls.from_int8(wq, sw, linear.bias)

    @property
    def wq(self) -> torch.Tensor:
        """Dense int8 (N, K) view of the packed weight (inspection only)."""
        KB, N, _ = self.wc.shape
        dev = self.wc.device
        g = torch.arange(8, device=dev)
        h = torch.arange(2, device=dev)
        base = (32 * (g // 4))[None, :] + 16 * h[:, None] + (4 * (g % 4))[None, :]  # (2, 8)
        shifts = (4 * g).to(torch.int64)
        nib = (self.widx.to(torch.int64)[..., None] >> shifts) & 15            # (KB, N, 2, 8)
        vals = self.wc.view(KB, N, 2, 8, 2)
        out = torch.zeros((N, KB, 64), dtype=torch.int8, device=dev)
        for e, pos in ((0, nib & 3), (1, nib >> 2)):
            col = (base[None, None] + pos).permute(1, 0, 2, 3).reshape(N, KB, 16)
            out.scatter_(2, col, vals[..., e].permute(1, 0, 2, 3).reshape(N, KB, 16))
        return out.reshape(N, KB * 64)

    def linear_fused(self, xq, sx, epilogue, residual=None, dst_row=None, out=None,
                     layout=_lib.LAYOUT_ROWMAJOR):
        if dst_row is not None:
            raise RuntimeError("samfast: the sparse GEMM has no row scatter")
        return ops.gemm_i8_sparse24_fused(xq, sx, self.wc, self.widx, self.sw, self.bias_f32,
                                          epilogue, residual=residual, out=out, layout=layout)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                "int8 dynamic, 2:4 sparse weight")


def _is_linear(mod: nn.Module) -> bool:
    return isinstance(mod, (nn.Linear, Int8DynamicLinear))


def _wrap(filter_fn: Optional[Callable[[nn.Module, str], bool]]):
    if filter_fn is None:
        return lambda mod, fqn: _is_linear(mod)
    return lambda mod, fqn: _is_linear(mod) and filter_fn(mod, fqn)


def apply_fake_sparsity(model: nn.Module,
                        filter_fn: Optional[Callable[[nn.Module, str], bool]] = None) -> None:
    """Zero, in place, the 2 smallest-magnitude weights of every 4 of each selected
    nn.Linear (sparse.py:6-25).  Dense storage, dense kernels: accuracy simulation only."""
    from .graphs import invalidate_recordings
    invalidate_recordings(model)
    sel = _wrap(filter_fn)
    for name, mod in model.named_modules():
        if isinstance(mod, nn.Linear) and sel(mod, name):
            with torch.no_grad():
                mod.weight.copy_(prune_2_of_4(mod.weight))


def apply_sparse(model: nn.Module,
                 filter_fn: Optional[Callable[[nn.Module, str], bool]] = None) -> None:
    """Swap each selected Linear (float or already int8) for Int8Sparse24Linear, in place
    (sparse.py:28-32)."""
    replace_with_custom_fn_if_matches_filter(model, Int8Sparse24Linear.from_float, _wrap(filter_fn))
