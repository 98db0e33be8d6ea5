"""Dynamic symmetric int8 Linear on the HIP kernels.

`apply_dynamic_quant(model)` has the call shape of
torchao.quantization.apply_dynamic_quant as the reference uses it
(experiments/eval_combo.py:357-359): every nn.Linear under `model` (optionally
filtered) is replaced, in place, by a module that

  * holds the weight quantised once per output channel to int8 with
    scale absmax/127 (row-major (N, K), so both GEMM operands are K-contiguous),
  * quantises its input per token at run time (fused absmax/round/pack kernel),
  * multiplies on the int8 matrix cores with int32 accumulation and applies
    (acc * s_x[m]) * s_w[n] + bias[n] -> bf16 in the GEMM epilogue.

The swapped module keeps `in_features`, `out_features`, a float `bias`
parameter and a `weight` property (the dequantised weight), so code that only
inspects shapes keeps working.  Forward needs GPU bf16 activations; there is no
CPU route.
"""

import os
from typing import Callable, Optional

import torch
import torch.nn as nn

from . import ops
from ._lib import EPILOGUE_NONE, LAYOUT_KB64, LAYOUT_ROWMAJOR
from .tools import replace_with_custom_fn_if_matches_filter

# The next Linear's row quantiser inside the producing GEMM (one launch, five per block) or after
# it (two launches, nine per block).  Both give the same bits.  Measured on the ViT-H batch-16
# encoder the single launch is the slower one (the workgroup that quantises a row tile holds
# one of its CU's two GEMM slots for the duration, and the device-scope release of every tile
# writes the L2 back), so the separate launches are the default; SAMFAST_FUSED_QUANT=1 selects
# the fused form.
FUSED_QUANT = os.environ.get("SAMFAST_FUSED_QUANT", "0") != "0"


WEIGHT_CONVENTIONS = ("absmax127", "torchao")


def quantize_weight_per_channel(weight: torch.Tensor, convention: str = "absmax127"):
    """(N, K) float -> (int8 (N, K), fp32 scale (N,)), done once at swap time.

    "absmax127" (default): fp32 arithmetic, scale = max(absmax, 1e-5) / 127,
        q = clamp(rint(w / scale), -127, 127) - the symmetric convention of the activation
        quantiser; codes never reach -128.
    "torchao": torchao's `dynamically_quantize_per_channel(w, -128, 127, torch.int8)` as its
        apply_dynamic_quant runs it on the weight (call site experiments/eval_combo.py:357-359),
        restated from the published routine: scale = max(absmax / 127.5, eps) with eps = float32
        machine epsilon (the symmetric range is split as (quant_max - quant_min) / 2), the scale
        is stored in the WEIGHT's dtype and the division runs in that dtype too (the reference
        casts the encoder to bfloat16 before it quantises, eval_combo.py:351-352), then
        q = clamp(rint(w / scale), -128, 127): the extreme weight of a channel lands on +-127.5,
        i.e. on 127 (clamped from 128) or -128.  Not checked against torchao itself, which is
        not installable here.
    Either way the kernels only see int8 codes and an fp32 scale per channel."""
    w = weight.detach()
    if convention == "absmax127":
        w = w.to(torch.float32)
        scale = w.abs().amax(dim=1).clamp_min(1e-5) / 127.0
        q = torch.round(w / scale[:, None]).clamp_(-127, 127).to(torch.int8)
    elif convention == "torchao":
        if not w.is_floating_point():
            raise ValueError("the weight must be a floating-point tensor")
        absmax = torch.maximum(w.amax(dim=1).clamp_min(0), (-w.amin(dim=1)).clamp_min(0))
        scale = (absmax / 127.5).clamp(min=torch.finfo(torch.float32).eps).to(w.dtype)
        q = torch.round(w / scale[:, None]).clamp_(-128, 127).to(torch.int8)
    else:
        raise ValueError(f"weight convention must be one of {WEIGHT_CONVENTIONS}, got {convention!r}")
    return q.contiguous(), scale.to(torch.float32).contiguous()


class Int8LinearBase(nn.Module):
    """What every int8 Linear here shares: shapes, per-channel weight scales and bias.

    Scales and the fp32 bias are registered as int32 bit patterns so that a
    later `model.to(torch.bfloat16)` (which casts every floating-point buffer)
    cannot round them; they are viewed back as fp32 at call time.  The bias has
    this one home: `bias` is a read-only fp32 view of it, and a state dict that
    carries a float `bias` entry (an nn.Linear's) is folded into it on load."""

    supports_row_scatter = True  # linear_fused accepts dst_row

    def __init__(self, in_features: int, out_features: int, sw: torch.Tensor,
                 bias: Optional[torch.Tensor]) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("sw_bits", sw.to(torch.float32).contiguous().view(torch.int32))
        if bias is not None:
            self.register_buffer(
                "bias_bits", bias.detach().to(torch.float32).contiguous().view(torch.int32))
        else:
            self.bias_bits = None

    @property
    def sw(self) -> torch.Tensor:
        return self.sw_bits.view(torch.float32)

    @property
    def bias_f32(self) -> Optional[torch.Tensor]:
        return None if self.bias_bits is None else self.bias_bits.view(torch.float32)

    @property
    def bias(self) -> Optional[torch.Tensor]:
        return self.bias_f32

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        key = prefix + "bias"
        if key in state_dict:
            value = state_dict.pop(key)
            if self.bias_bits is not None and prefix + "bias_bits" not in state_dict:
                state_dict[prefix + "bias_bits"] = (
                    value.detach().to(torch.float32).contiguous().view(torch.int32))
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    @property
    def weight(self) -> torch.Tensor:
        return self.wq.to(torch.float32) * self.sw[:, None]

    def linear_fused(self, xq, sx, epilogue, residual=None, dst_row=None, out=None,
                     layout=LAYOUT_ROWMAJOR):
        raise NotImplementedError

    def linear_fused_quant(self, xq, sx, epilogue, residual=None, out=None, layout=LAYOUT_ROWMAJOR,
                           ln=None, out_layout=LAYOUT_ROWMAJOR):
        """linear_fused followed by the next Linear's row quantiser (behind a LayerNorm when
        ln = (gamma, beta, eps) is given): returns (y, yq, sy).  Here as separate launches;
        Int8DynamicLinear runs all of it inside its GEMM."""
        y = self.linear_fused(xq, sx, epilogue, residual=residual, out=out, layout=layout)
        if ln is not None:
            yq, sy = ops.layernorm_quant(y, ln[0], ln[1], ln[2], layout=out_layout)
        else:
            yq, sy = ops.quant_rowwise(y, layout=out_layout)
        return y, yq, sy

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """The kernels compute on bf16 rows; any other floating input is cast on the way in and
        the result cast back, so the module keeps its input's dtype as nn.Linear does."""
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.in_features)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        xq, sx = ops.quant_rowwise(x2)
        y = self.linear_fused(xq, sx, EPILOGUE_NONE)
        return y.reshape(*lead, self.out_features).to(x.dtype)


class Int8DynamicLinear(Int8LinearBase):
    """Dense int8 weight `wq` (N, K)."""

    def __init__(self, in_features: int, out_features: int, wq: torch.Tensor, sw: torch.Tensor,
                 bias: Optional[torch.Tensor]) -> None:
        super().__init__(in_features, out_features, sw, bias)
        self.register_buffer("wq", wq)
        self._wq_kb64 = None  # derived K-block major copy, not part of the state dict
        self._wq_kb64_key = None

    @classmethod
    def from_float(cls, linear: nn.Linear, weight_convention: str = "absmax127") -> "Int8DynamicLinear":
        wq, sw = quantize_weight_per_channel(linear.weight, weight_convention)
        return cls(linear.in_features, linear.out_features, wq, sw, linear.bias)

    def linear_fused(self, xq: torch.Tensor, sx: torch.Tensor, epilogue: int,
                     residual: Optional[torch.Tensor] = None, dst_row: Optional[torch.Tensor] = None,
                     out: Optional[torch.Tensor] = None, layout: int = LAYOUT_ROWMAJOR) -> torch.Tensor:
        """The GEMM + epilogue on already quantised rows (see ops.gemm_i8_fused); `layout` is
        the layout xq comes in.  The K-block major copy of the weight is made on first use."""
        return ops.gemm_i8_fused(xq, sx, self._weight_for(layout), self.sw, self.bias_f32, epilogue,
                                 residual=residual, dst_row=dst_row, out=out, layout=layout)

    def _weight_for(self, layout: int) -> torch.Tensor:
        if layout != LAYOUT_KB64:
            return self.wq
        key = (self.wq.data_ptr(), self.wq._version, str(self.wq.device))
        if self._wq_kb64 is None or self._wq_kb64_key != key:  # rebuilt after load_state_dict / .to()
            self._wq_kb64, self._wq_kb64_key = ops.to_kb64(self.wq), key
        return self._wq_kb64

    def linear_fused_quant(self, xq, sx, epilogue, residual=None, out=None, layout=LAYOUT_ROWMAJOR,
                           ln=None, out_layout=LAYOUT_ROWMAJOR):
        """GEMM + epilogue + the next Linear's quantiser as one launch (ops.gemm_i8_fused_quant);
        FUSED_QUANT = False keeps the quantiser a launch of its own (same results)."""
        if not FUSED_QUANT:
            return super().linear_fused_quant(xq, sx, epilogue, residual=residual, out=out, layout=layout,
                                              ln=ln, out_layout=out_layout)
        return ops.gemm_i8_fused_quant(xq, sx, self._weight_for(layout), self.sw, self.bias_f32, epilogue,
                                       residual=residual, out=out, layout=layout, ln=ln,
                                       out_layout=out_layout)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, int8 dynamic"


def apply_dynamic_quant(model: nn.Module,
                        filter_fn: Optional[Callable[[nn.Module, str], bool]] = None,
                        weight_convention: str = "absmax127") -> None:
    """Swap every nn.Linear under `model` for Int8DynamicLinear, in place.
    `weight_convention` picks the per-channel weight quantiser (quantize_weight_per_channel):
    "torchao" reproduces the codes and scales torchao's own swap would hold."""
    if weight_convention not in WEIGHT_CONVENTIONS:
        raise ValueError(f"weight convention must be one of {WEIGHT_CONVENTIONS}, got {weight_convention!r}")
    if filter_fn is None:
        filter_fn = lambda mod, fqn: isinstance(mod, nn.Linear)
    else:
        user = filter_fn
        filter_fn = lambda mod, fqn: isinstance(mod, nn.Linear) and user(mod, fqn)
    make = lambda linear: Int8DynamicLinear.from_float(linear, weight_convention)
    replace_with_custom_fn_if_matches_filter(model, make, filter_fn)
