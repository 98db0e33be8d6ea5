"""Host-side mirror of the reference's attention operator layer.

Keeps the names, argument meaning and dispatch behaviour of
segment_anything_fast/flash_4.py so that callers written against it work
unchanged:

  _attention_rel_h_rel_w(q_, k_, v_, rel_h_, rel_w_)      flash_4.py:335-370
  torch.ops.customflash.custom_flash_aligned(q, k, v, rel_h_w, sm_scale)
                                                          flash_4.py:268-329
  SEGMENT_ANYTHING_FAST_USE_FLASH_4 (default 1)           flash_4.py:332

Differences, all on the side of doing more in the kernel: head_dim 80 is run
natively (no pad to 128, :358-367), batch size 1 with head_dim 64 is correct
(:350-351 disables it there), and 14x14 windows go to the HIP kernel as well
(the reference sends them to SDPA with a materialised bias, :368-370).

Both half types run on the kernels (fp16 and bf16, :188,:348).  As in the reference, inputs the
kernels do not cover (fp32, CPU tensors, the switch set to 0, odd shapes) take the eager
F.scaled_dot_product_attention(attn_mask=rel_h + rel_w) route (:368-370); a GPU
half-precision call that the kernels DO cover never falls back - a missing or
failing library raises.
"""

import math
import os

import torch
import torch.nn.functional as F

from . import ops

USE_CUSTOM_KERNEL = bool(int(os.environ.get("SEGMENT_ANYTHING_FAST_USE_FLASH_4", 1)))

# Operator schema of flash_4.py:268-269.  The namespace may already hold the
# definition when the reference package is imported in the same process.
_lib_def = torch.library.Library("customflash", "FRAGMENT")
try:
    _lib_def.define(
        "custom_flash_aligned(Tensor q, Tensor k, Tensor v, Tensor rel_h_w, float sm_scale) -> Tensor")
    _OWNS_SCHEMA = True
except RuntimeError:
    _OWNS_SCHEMA = False


def _custom_flash_aligned_meta(q, k, v, rel_h_w, sm_scale):
    return q.contiguous()


def _custom_flash_aligned_gpu(q, k, v, rel_h_w, sm_scale):
    """rel_h_w is (B, nH, N, 128): columns [0, 64) are rel_h over key rows,
    [64, 128) rel_w over key columns (flash_4.py:98-101,115-117,352)."""
    assert q.shape == k.shape == v.shape
    assert rel_h_w.shape[-1] == 128 and rel_h_w.shape[-2] == q.shape[-2]
    assert rel_h_w.dtype == q.dtype
    # key n sits at grid row n // 64, column n % 64 (flash_4.py:115-116): N / 64 key rows, of
    # which the first N / 64 columns of the rel_h half are the ones the kernel reads
    N = q.shape[-2]
    if N % 128 != 0 or N // 64 > 64:
        raise RuntimeError(
            f"customflash::custom_flash_aligned: {N} tokens are not a 64-wide key grid of at most 64 "
            "rows (an even number of them)")
    gh = N // 64
    if rel_h_w.stride(-1) != 1:
        rel_h_w = rel_h_w.contiguous()
    if q.stride(-1) != 1:
        q = q.contiguous()
    if k.stride(-1) != 1:
        k = k.contiguous()
    if v.stride(-1) != 1:
        v = v.contiguous()
    return ops.attn_relpos_bias(q, k, v, rel_h_w[..., :gh], rel_h_w[..., 64:], sm_scale)


if _OWNS_SCHEMA:
    _lib_def.impl("custom_flash_aligned", _custom_flash_aligned_meta, "Meta")
    _lib_def.impl("custom_flash_aligned", _custom_flash_aligned_gpu, "CUDA")  # HIP key on ROCm


def _kernel_guards(q_, k_, v_) -> bool:
    # half types only, as flash_4.py:345-348
    return (q_.is_cuda and q_.dtype in (torch.bfloat16, torch.float16) and q_.dtype == k_.dtype
            and k_.dtype == v_.dtype and USE_CUSTOM_KERNEL)


def _attention_rel_h_rel_w(q_, k_, v_, rel_h_, rel_w_):
    """q_, k_, v_: (B, nH, N, hd); rel_h_: (B, nH, N, k_h, 1); rel_w_: (B, nH, N, 1, k_w).
    Returns (B, nH, N, hd) = softmax(q k^T / sqrt(hd) + rel_h + rel_w) v."""
    hd = q_.size(-1)
    k_h, k_w = rel_h_.size(3), rel_w_.size(4)
    if _kernel_guards(q_, k_, v_) and ops.attn_supported(q_.size(-2), (k_h, k_w), hd, q_.dtype):
        sm_scale = 1.0 / math.sqrt(hd)
        if k_w == 64 and k_h == 64:
            # same operand packing as the reference (flash_4.py:352), through the operator
            rel_h_w = torch.cat([rel_h_.squeeze(-1), rel_w_.squeeze(-2)], dim=-1)
            return torch.ops.customflash.custom_flash_aligned(q_, k_, v_, rel_h_w, sm_scale)
        rel_h = rel_h_.squeeze(-1)
        rel_w = rel_w_.squeeze(-2)
        if rel_h.stride(-1) != 1:
            rel_h = rel_h.contiguous()
        if rel_w.stride(-1) != 1:
            rel_w = rel_w.contiguous()
        qq = q_ if q_.stride(-1) == 1 else q_.contiguous()
        kk = k_ if k_.stride(-1) == 1 else k_.contiguous()
        vv = v_ if v_.stride(-1) == 1 else v_.contiguous()
        return ops.attn_relpos_bias(qq, kk, vv, rel_h, rel_w, sm_scale)
    attn_bias = (rel_h_ + rel_w_).view(q_.size(0), q_.size(1), rel_h_.size(2), k_h * k_w)
    return F.scaled_dot_product_attention(q_, k_, v_, attn_mask=attn_bias)
