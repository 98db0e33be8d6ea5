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

from typing import Callable, Optional

import torch
import torch.nn as nn

from . import ops
from ._lib import EPILOGUE_NONE, LAYOUT_KB64, LAYOUT_ROWMAJOR
from .tools import replace_with_custom_fn_if_matches_filter


def quantize_weight_per_channel(weight: torch.Tensor):
    """(N, K) float -> (int8 (N, K), fp32 scale (N,)), scale = max(absmax, 1e-5)/127,
    q = clamp(rint(w / scale), -127, 127).  fp32 arithmetic, done once at swap time."""
    w = weight.detach().to(torch.float32)
    absmax = w.abs().amax(dim=1).clamp_min(1e-5)
    scale = absmax / 127.0
    q = torch.round(w / scale[:, None]).clamp_(-127, 127).to(torch.int8)
    return q.contiguous(), scale.contiguous()


class Int8LinearBase(nn.Module):
    """What every int8 Linear here shares: shapes, per-channel weight scales and bias.

    Scales and the fp32 bias are registered as int32 bit patterns so that a
    later `model.to(torch.bfloat16)` (which casts every floating-point buffer)
    cannot round them; they are viewed back as fp32 at call time."""

    supports_row_scatter = True  # linear_fused accepts dst_row

    def __init__(self, in_features: int, out_features: int, sw: torch.Tensor,
                 bias: Optional[torch.Tensor]) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("sw_bits", sw.to(torch.float32).contiguous().view(torch.int32))
        if bias is not None:
            self.bias = nn.Parameter(bias.detach().clone(), requires_grad=False)
            self.register_buffer(
                "bias_bits", bias.detach().to(torch.float32).contiguous().view(torch.int32))
        else:
            self.bias = None
            self.bias_bits = None

    @property
    def sw(self) -> torch.Tensor:
        return self.sw_bits.view(torch.float32)

    @property
    def bias_f32(self) -> Optional[torch.Tensor]:
        return None if self.bias_bits is None else self.bias_bits.view(torch.float32)

    @property
    def weight(self) -> torch.Tensor:
        return self.wq.to(torch.float32) * self.sw[:, None]

    def linear_fused(self, xq, sx, epilogue, residual=None, dst_row=None, out=None,
                     layout=LAYOUT_ROWMAJOR):
        raise NotImplementedError

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.in_features)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        xq, sx = ops.quant_rowwise(x2)
        y = self.linear_fused(xq, sx, EPILOGUE_NONE)
        return y.reshape(*lead, self.out_features)


class Int8DynamicLinear(Int8LinearBase):
    """Dense int8 weight `wq` (N, K)."""

    def __init__(self, in_features: int, out_features: int, wq: torch.Tensor, sw: torch.Tensor,
                 bias: Optional[torch.Tensor]) -> None:
        super().__init__(in_features, out_features, sw, bias)
        self.register_buffer("wq", wq)
        self._wq_kb64 = None  # derived K-block major copy, not part of the state dict
        self._wq_kb64_key = None

    @classmethod
    def from_float(cls, linear: nn.Linear) -> "Int8DynamicLinear":
        wq, sw = quantize_weight_per_channel(linear.weight)
        return cls(linear.in_features, linear.out_features, wq, sw, linear.bias)

    def linear_fused(self, xq: torch.Tensor, sx: torch.Tensor, epilogue: int,
                     residual: Optional[torch.Tensor] = None, dst_row: Optional[torch.Tensor] = None,
                     out: Optional[torch.Tensor] = None, layout: int = LAYOUT_ROWMAJOR) -> torch.Tensor:
        """The GEMM + epilogue on already quantised rows (see ops.gemm_i8_fused); `layout` is
        the layout xq comes in.  The K-block major copy of the weight is made on first use."""
        if layout == LAYOUT_KB64:
            key = (self.wq.data_ptr(), self.wq._version, str(self.wq.device))
            if self._wq_kb64 is None or self._wq_kb64_key != key:  # rebuilt after load_state_dict / .to()
                self._wq_kb64, self._wq_kb64_key = ops.to_kb64(self.wq), key
            w = self._wq_kb64
        else:
            w = self.wq
        return ops.gemm_i8_fused(xq, sx, w, self.sw, self.bias_f32, epilogue,
                                 residual=residual, dst_row=dst_row, out=out, layout=layout)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, int8 dynamic"


def apply_dynamic_quant(model: nn.Module,
                        filter_fn: Optional[Callable[[nn.Module, str], bool]] = None) -> None:
    """Swap every nn.Linear under `model` for Int8DynamicLinear, in place."""
    if filter_fn is None:
        filter_fn = lambda mod, fqn: isinstance(mod, nn.Linear)
    else:
        user = filter_fn
        filter_fn = lambda mod, fqn: isinstance(mod, nn.Linear) and user(mod, fqn)
    replace_with_custom_fn_if_matches_filter(model, Int8DynamicLinear.from_float, filter_fn)
