"""Tensor-level wrappers over the C ABI: device pointers, strides and the current
HIP stream are taken from torch tensors; all compute happens in libsamfast.so.

Every function requires tensors on a GPU device and raises otherwise - there is
no CPU or eager path behind these names.
"""

import math
from typing import Optional, Tuple

import torch

from . import _lib


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


# Optional per-launch timing: while a list is installed with record_launches(), every
# kernel launch is bracketed by two events on the stream it is enqueued on and
# (kernel, algorithmic work, unit, start, end) is appended.  Used by the benchmark to
# get per-kernel durations of a real encoder step; off (None) otherwise.
_launch_log = None


class record_launches:
    def __init__(self):
        self.entries = []

    def __enter__(self):
        global _launch_log
        self._prev, _launch_log = _launch_log, self.entries
        return self

    def __exit__(self, *exc):
        global _launch_log
        _launch_log = self._prev
        return False

    def summary(self):
        """{kernel: dict(launches, work, unit, ms)} after synchronising."""
        torch.cuda.synchronize()
        out = {}
        for name, work, unit, e0, e1, nbytes in self.entries:
            d = out.setdefault(name, dict(launches=0, work=0.0, unit=unit, ms=0.0, bytes=0.0))
            d["launches"] += 1
            d["work"] += work
            d["bytes"] += nbytes
            d["ms"] += e0.elapsed_time(e1)
        return out


def _timed(name: str, work: float, unit: str, launch, nbytes: float = 0.0):
    log = _launch_log
    if log is None:
        return launch()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    code = launch()
    e1.record()
    log.append((name, work, unit, e0, e1, nbytes))
    return code


def _require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("samfast ops need GPU tensors (no CPU path exists)")


def _bnhd_strides(t: torch.Tensor) -> Tuple[int, int, int]:
    """(batch, head, token) element strides of a logical (B, nH, N, hd) tensor."""
    if t.stride(3) != 1:
        raise RuntimeError("samfast: the head_dim axis must be contiguous")
    return t.stride(0), t.stride(1), t.stride(2)


def _dtype_code(t: torch.Tensor) -> int:
    """Element type code of the C ABI.  The attention kernels exist for both half types; the
    int8 linears take bfloat16 only and refuse the float16 code themselves."""
    if t.dtype == torch.bfloat16:
        return _lib.SAMFAST_BF16
    if t.dtype == torch.float16:
        return _lib.SAMFAST_F16
    raise RuntimeError(f"samfast: unsupported dtype {t.dtype} (the kernels take bfloat16 or float16)")


def _check_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: Optional[torch.Tensor],
               tokens: int) -> None:
    """The library only receives the grid: it walks `tokens` rows of every (batch, head)
    slice whatever the tensors hold, so their shapes are pinned here, before any launch."""
    if q.dim() != 4 or q.shape[2] != tokens:
        raise RuntimeError(f"samfast: q must be (B, nH, {tokens}, hd) for this grid, got {tuple(q.shape)}")
    if k.shape != q.shape or v.shape != q.shape:
        raise RuntimeError("samfast: k and v must have the shape of q")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("samfast: k and v must have the dtype of q")
    if out is not None and (out.shape != q.shape or out.dtype != q.dtype or out.device != q.device):
        raise RuntimeError("samfast: out must have the shape, dtype and device of q")


def attn_supported(N: int, grid_hw: Tuple[int, int], hd: int, dtype: torch.dtype) -> bool:
    """Shapes the HIP attention kernels cover (mirrors the checks in the library)."""
    gh, gw = grid_hw
    if dtype not in (torch.bfloat16, torch.float16) or hd not in (64, 80) or gh * gw != N:
        return False
    global_ok = gw == 64 and N % 128 == 0 and gh <= 64
    window_ok = gh <= 15 and gw <= 16 and N <= 208
    return global_ok or window_ok


def attn_relpos(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                rel_pos_h: torch.Tensor, rel_pos_w: torch.Tensor,
                grid_hw: Tuple[int, int], sm_scale: Optional[float] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(q k^T * scale + rel_h + rel_w) v with the bias computed in-kernel
    from the (2S-1, hd) tables.  q, k, v: logical (B, nH, N, hd), any batch / head /
    token strides (head_dim contiguous).  Returns (B, nH, N, hd) laid out
    token-major, i.e. as a (B, N, nH*hd) buffer viewed head-major, unless `out`
    is given."""
    gh, gw = grid_hw
    _check_qkv(q, k, v, out, gh * gw)
    _require_gpu(q, k, v, rel_pos_h, rel_pos_w)
    B, nH, N, hd = q.shape
    if out is None:
        out = torch.empty((B, N, nH, hd), dtype=q.dtype, device=q.device).permute(0, 2, 1, 3)
    rel_pos_h = rel_pos_h.contiguous()
    rel_pos_w = rel_pos_w.contiguous()
    if rel_pos_h.shape != (2 * gh - 1, hd) or rel_pos_w.shape != (2 * gw - 1, hd):
        raise RuntimeError("samfast: relative-position tables must be (2*S-1, head_dim)")
    if rel_pos_h.dtype != q.dtype or rel_pos_w.dtype != q.dtype:
        rel_pos_h, rel_pos_w = rel_pos_h.to(q.dtype), rel_pos_w.to(q.dtype)
    scale = float(sm_scale) if sm_scale is not None else 1.0 / math.sqrt(hd)
    lib = _lib.load()
    code = _timed(
        "attn_global" if gw == 64 else "attn_window", 4.0 * B * nH * N * N * hd, "flop",
        lambda: lib.samfast_attn_relpos_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), rel_pos_h.data_ptr(), rel_pos_w.data_ptr(),
            out.data_ptr(), B, nH, gh, gw, hd,
            *_bnhd_strides(q), *_bnhd_strides(k), *_bnhd_strides(v), *_bnhd_strides(out),
            _dtype_code(q), scale, _stream()),
        nbytes=0.0 if gw == 64 else 4.0 * B * nH * N * hd * q.element_size())
    _lib.check(code, "attn_relpos_fwd")
    return out


def attn_relpos_windowed(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                         rel_pos_h: torch.Tensor, rel_pos_w: torch.Tensor,
                         pad_k: torch.Tensor, pad_v: torch.Tensor,
                         grid_hw: Tuple[int, int], window: int, scale: float) -> torch.Tensor:
    """Windowed attention on image-ordered tokens (partition + attention + unpartition).
    q, k, v: (B, nH, H*W, hd) views with contiguous hd; pad_k / pad_v: (nH, hd) rows standing
    for the zero-padded tokens.  Returns (B, H*W, nH, hd) contiguous."""
    H, W = grid_hw
    _check_qkv(q, k, v, None, H * W)
    _require_gpu(q, k, v, rel_pos_h, rel_pos_w, pad_k, pad_v)
    B, nH, N, hd = q.shape
    if tuple(rel_pos_h.shape) != (2 * window - 1, hd) or tuple(rel_pos_w.shape) != (2 * window - 1, hd):
        raise RuntimeError("samfast: rel_pos tables must be (2*window-1, head_dim)")
    # the kernel reads the tables as q's element type
    rel_pos_h = rel_pos_h.to(q.dtype).contiguous()
    rel_pos_w = rel_pos_w.to(q.dtype).contiguous()
    for t in (pad_k, pad_v):
        if tuple(t.shape) != (nH, hd) or not t.is_contiguous() or t.dtype != q.dtype:
            raise RuntimeError("samfast: pad_k / pad_v must be contiguous (nH, hd) tensors of q's dtype")
    out = torch.empty((B, N, nH, hd), dtype=q.dtype, device=q.device)
    o = out.permute(0, 2, 1, 3)
    lib = _lib.load()
    nwin = B * (-(-H // window)) * (-(-W // window))
    nt = window * window
    code = _timed(
        "attn_window", 4.0 * nwin * nH * nt * nt * hd, "flop",
        lambda: lib.samfast_attn_relpos_windowed_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), rel_pos_h.data_ptr(),
            rel_pos_w.data_ptr(), pad_k.data_ptr(), pad_v.data_ptr(), out.data_ptr(),
            B, nH, H, W, window, hd,
            *_bnhd_strides(q), *_bnhd_strides(k), *_bnhd_strides(v), *_bnhd_strides(o),
            _dtype_code(q), float(scale), _stream()),
        nbytes=4.0 * nwin * nH * nt * hd * q.element_size())
    _lib.check(code, "attn_relpos_windowed_fwd")
    return out


def attn_relpos_bias(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                     rel_h: torch.Tensor, rel_w: torch.Tensor,
                     sm_scale: Optional[float] = None,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Same attention with caller-computed bias factors rel_h (B, nH, N, gh) and
    rel_w (B, nH, N, gw) (last axis contiguous).  Returns a contiguous
    (B, nH, N, hd) tensor unless `out` is given."""
    gh, gw = rel_h.shape[-1], rel_w.shape[-1]
    _check_qkv(q, k, v, out, gh * gw)
    B, nH, N, hd = q.shape
    if tuple(rel_h.shape) != (B, nH, N, gh) or tuple(rel_w.shape) != (B, nH, N, gw):
        raise RuntimeError("samfast: bias factors must be (B, nH, N, gh) and (B, nH, N, gw) with gh*gw == N")
    if rel_h.dtype != q.dtype or rel_w.dtype != q.dtype:
        raise RuntimeError("samfast: bias factors must have the dtype of q")
    _require_gpu(q, k, v, rel_h, rel_w)
    if out is None:
        out = torch.empty((B, nH, N, hd), dtype=q.dtype, device=q.device)
    scale = float(sm_scale) if sm_scale is not None else 1.0 / math.sqrt(hd)
    lib = _lib.load()
    code = _timed(
        "attn_global_bias" if gw == 64 else "attn_window_bias", 4.0 * B * nH * N * N * hd, "flop",
        lambda: lib.samfast_attn_relpos_bias_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), rel_h.data_ptr(), rel_w.data_ptr(),
            out.data_ptr(), B, nH, gh, gw, hd,
            *_bnhd_strides(q), *_bnhd_strides(k), *_bnhd_strides(v), *_bnhd_strides(out),
            *_bnhd_strides(rel_h), *_bnhd_strides(rel_w),
            _dtype_code(q), scale, _stream()))
    _lib.check(code, "attn_relpos_bias_fwd")
    return out


def _xq_empty(M: int, K: int, layout: int, device) -> torch.Tensor:
    """int8 activation buffer: (M, K) row-major, or (K/64, M, 64) K-block major."""
    if layout == _lib.LAYOUT_KB64:
        if K % 64 != 0:
            raise RuntimeError("samfast: the K-block major layout needs K % 64 == 0")
        return torch.empty((K // 64, M, 64), dtype=torch.int8, device=device)
    return torch.empty((M, K), dtype=torch.int8, device=device)


def to_kb64(q: torch.Tensor) -> torch.Tensor:
    """(R, K) int8 row-major -> (K/64, R, 64) K-block major copy (weights, once)."""
    R, K = q.shape
    return q.view(R, K // 64, 64).permute(1, 0, 2).contiguous()


def from_kb64(q: torch.Tensor) -> torch.Tensor:
    """(K/64, R, 64) K-block major -> (R, K) row-major copy."""
    KB, R, _ = q.shape
    return q.permute(1, 0, 2).reshape(R, KB * 64)


def _operand_shape(q: torch.Tensor, layout: int) -> Tuple[int, int]:
    """(rows, K) of an int8 GEMM operand in either layout."""
    if q.dtype != torch.int8 or not q.is_contiguous():
        raise RuntimeError("samfast: int8 GEMM operands must be contiguous int8 tensors")
    if layout == _lib.LAYOUT_KB64:
        if q.dim() != 3 or q.shape[2] != 64:
            raise RuntimeError("samfast: a K-block major operand has shape (K/64, rows, 64)")
        return q.shape[1], q.shape[0] * 64
    if q.dim() != 2:
        raise RuntimeError("samfast: a row-major operand has shape (rows, K)")
    return q.shape[0], q.shape[1]


def quant_rowwise(x: torch.Tensor, layout: int = _lib.LAYOUT_ROWMAJOR) -> Tuple[torch.Tensor, torch.Tensor]:
    """(M, K) bf16 (row stride free, K contiguous) -> (int8 codes in `layout`, fp32 scales (M,))."""
    _require_gpu(x)
    if x.dim() != 2 or x.stride(1) != 1:
        raise RuntimeError("samfast: quant_rowwise needs a 2-D tensor with contiguous rows")
    M, K = x.shape
    xq = _xq_empty(M, K, layout, x.device)
    sx = torch.empty((M,), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    code = _timed(
        "quant_rowwise", 3.0 * M * K + 4.0 * M, "byte",
        lambda: lib.samfast_quant_rowwise_i8(
            x.data_ptr(), x.stride(0), xq.data_ptr(), sx.data_ptr(), M, K, _dtype_code(x),
            int(layout), _stream()))
    _lib.check(code, "quant_rowwise_i8")
    return xq, sx


def gemm_i8_i32(xq: torch.Tensor, wq: torch.Tensor) -> torch.Tensor:
    """int8 (M, K) x int8 (N, K)^T -> int32 (M, N), exact."""
    _require_gpu(xq, wq)
    if xq.dtype != torch.int8 or wq.dtype != torch.int8:
        raise RuntimeError("samfast: gemm_i8_i32 needs int8 operands")
    if not (xq.is_contiguous() and wq.is_contiguous()) or xq.shape[1] != wq.shape[1]:
        raise RuntimeError("samfast: gemm_i8_i32 needs contiguous (M, K) and (N, K)")
    M, K = xq.shape
    N = wq.shape[0]
    acc = torch.empty((M, N), dtype=torch.int32, device=xq.device)
    lib = _lib.load()
    code = _timed(
        "gemm_i8_i32", 2.0 * M * N * K, "op",
        lambda: lib.samfast_gemm_i8_i32(xq.data_ptr(), wq.data_ptr(), acc.data_ptr(), M, N, K,
                                        _stream()))
    _lib.check(code, "gemm_i8_i32")
    return acc


def gemm_i8_scale_bias(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                       bias: Optional[torch.Tensor], out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16 (M, N) = (float(xq wq^T) * sx[:, None]) * sw[None, :] + bias."""
    _require_gpu(xq, sx, wq, sw, bias)
    if not (xq.is_contiguous() and wq.is_contiguous()) or xq.shape[1] != wq.shape[1]:
        raise RuntimeError("samfast: gemm_i8_scale_bias needs contiguous (M, K) and (N, K)")
    M, K = xq.shape
    N = wq.shape[0]
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != M or sw.numel() != N:
        raise RuntimeError("samfast: scales must be fp32 of length M and N")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N):
        raise RuntimeError("samfast: bias must be fp32 of length N")
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=xq.device)
    lib = _lib.load()
    code = _timed(
        "gemm_i8_scale_bias", 2.0 * M * N * K, "op",
        lambda: lib.samfast_gemm_i8_scale_bias(
            xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(),
            bias.data_ptr() if bias is not None else None, out.data_ptr(), out.stride(0),
            M, N, K, _lib.SAMFAST_BF16, _stream()))
    _lib.check(code, "gemm_i8_scale_bias")
    return out


def layernorm_quant(x: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor, eps: float,
                    src_row: Optional[torch.Tensor] = None,
                    layout: int = _lib.LAYOUT_ROWMAJOR) -> Tuple[torch.Tensor, torch.Tensor]:
    """LayerNorm over the last axis of x (R, K) bf16, optional row gather (src_row int32 (M,),
    -1 = zero row), then the per-row int8 quantiser.  Returns (int8 (M, K), fp32 (M,))."""
    _require_gpu(x, gamma, beta, src_row)
    if x.dim() != 2 or x.stride(1) != 1:
        raise RuntimeError("samfast: layernorm_quant needs a 2-D tensor with contiguous rows")
    K = x.shape[1]
    M = x.shape[0] if src_row is None else src_row.numel()
    if gamma.dtype != x.dtype or beta.dtype != x.dtype or gamma.numel() != K or beta.numel() != K:
        raise RuntimeError("samfast: gamma / beta must match x in dtype and length K")
    if src_row is not None and (src_row.dtype != torch.int32 or not src_row.is_contiguous()):
        raise RuntimeError("samfast: src_row must be a contiguous int32 tensor")
    xq = _xq_empty(M, K, layout, x.device)
    sx = torch.empty((M,), dtype=torch.float32, device=x.device)
    lib = _lib.load()
    code = _timed(
        "layernorm_quant", 2.0 * min(M, x.shape[0]) * K + 1.0 * M * K + 4.0 * M, "byte",
        lambda: lib.samfast_layernorm_quant_i8(
            x.data_ptr(), x.stride(0), gamma.contiguous().data_ptr(), beta.contiguous().data_ptr(),
            float(eps), src_row.data_ptr() if src_row is not None else None,
            xq.data_ptr(), sx.data_ptr(), M, K, _dtype_code(x), int(layout), _stream()))
    _lib.check(code, "layernorm_quant_i8")
    return xq, sx


def gemm_i8_fused(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                  bias: Optional[torch.Tensor], epilogue: int,
                  residual: Optional[torch.Tensor] = None, dst_row: Optional[torch.Tensor] = None,
                  out: Optional[torch.Tensor] = None, layout: int = _lib.LAYOUT_ROWMAJOR) -> torch.Tensor:
    """gemm_i8_scale_bias with a fused tail (see include/samfast.h); `layout` is the layout of
    both xq and wq:
    _lib.EPILOGUE_GELU, or _lib.EPILOGUE_RESIDUAL with `residual` (rows_out, N) bf16 and an
    optional int32 row scatter `dst_row` (M,), -1 = dropped.  For RESIDUAL the output has the
    shape of `residual` (and may alias it via `out=residual`)."""
    _require_gpu(xq, sx, wq, sw, bias, residual, dst_row)
    M, K = _operand_shape(xq, layout)
    N, Kw = _operand_shape(wq, layout)
    if K != Kw:
        raise RuntimeError("samfast: gemm_i8_fused operands disagree on K")
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != M or sw.numel() != N:
        raise RuntimeError("samfast: scales must be fp32 of length M and N")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N):
        raise RuntimeError("samfast: bias must be fp32 of length N")
    if epilogue == _lib.EPILOGUE_RESIDUAL:
        if residual is None or residual.dim() != 2 or residual.shape[1] != N or residual.stride(1) != 1 \
                or residual.dtype != torch.bfloat16:
            raise RuntimeError("samfast: residual must be a bf16 (rows, N) tensor")
        if dst_row is None and residual.shape[0] != M:
            raise RuntimeError("samfast: residual rows must equal M without a row map")
        if dst_row is not None and (dst_row.dtype != torch.int32 or dst_row.numel() != M
                                    or not dst_row.is_contiguous()):
            raise RuntimeError("samfast: dst_row must be a contiguous int32 tensor of length M")
        if out is None:
            out = torch.empty_like(residual)
    elif out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=xq.device)
    lib = _lib.load()
    name = {_lib.EPILOGUE_NONE: "gemm_i8_scale_bias", _lib.EPILOGUE_GELU: "gemm_i8_gelu",
            _lib.EPILOGUE_RESIDUAL: "gemm_i8_residual"}.get(epilogue, "gemm_i8_fused")
    code = _timed(
        name, 2.0 * M * N * K, "op",
        lambda: lib.samfast_gemm_i8_fused(
            xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(),
            bias.data_ptr() if bias is not None else None, out.data_ptr(), out.stride(0),
            M, N, K, _lib.SAMFAST_BF16, int(epilogue),
            residual.data_ptr() if residual is not None else None,
            residual.stride(0) if residual is not None else 0,
            dst_row.data_ptr() if dst_row is not None else None, int(layout), _stream()))
    _lib.check(code, "gemm_i8_fused")
    return out


_tile_counters = {}


def tile_counters(rows: int, device) -> torch.Tensor:
    """The zeroed int32 workspace samfast_gemm_i8_fused_quant wants (one entry per 128 rows).
    Outside graph capture: one buffer per (device, stream) - launches on one stream cannot overlap -
    whose entries are cleared on the stream before every use (a fill kernel): a launch leaves them
    zero again, but one that ended early (an error, a killed kernel) would not, and nothing else
    would ever notice.  Under capture: a buffer of the recording's own (from the graph's memory
    pool), so that two recorded graphs replayed on different streams never share counters."""
    need = -(-rows // 128)
    if torch.cuda.is_current_stream_capturing():
        return torch.zeros(max(need, 1), dtype=torch.int32, device=device)
    key = (str(device), torch.cuda.current_stream().cuda_stream)
    buf = _tile_counters.get(key)
    if buf is None or buf.numel() < need:
        buf = torch.empty(max(need, 1024), dtype=torch.int32, device=device)
        _tile_counters[key] = buf
    buf[:need].zero_()
    return buf


def gemm_i8_fused_quant(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                        bias: Optional[torch.Tensor], epilogue: int,
                        residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                        layout: int = _lib.LAYOUT_ROWMAJOR,
                        ln: Optional[Tuple[torch.Tensor, torch.Tensor, float]] = None,
                        out_layout: int = _lib.LAYOUT_ROWMAJOR,
                        counters: Optional[torch.Tensor] = None):
    """gemm_i8_fused (no row scatter) that also returns its output rows quantised for the next
    Linear: (y, yq, sy), with yq / sy what quant_rowwise(y) - or, with ln = (gamma, beta, eps),
    layernorm_quant(y, gamma, beta, eps) - returns, bit for bit, in `out_layout`."""
    _require_gpu(xq, sx, wq, sw, bias, residual)
    M, K = _operand_shape(xq, layout)
    N, Kw = _operand_shape(wq, layout)
    if K != Kw:
        raise RuntimeError("samfast: gemm_i8_fused_quant operands disagree on K")
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != M or sw.numel() != N:
        raise RuntimeError("samfast: scales must be fp32 of length M and N")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N):
        raise RuntimeError("samfast: bias must be fp32 of length N")
    if epilogue == _lib.EPILOGUE_RESIDUAL:
        if residual is None or tuple(residual.shape) != (M, N) or residual.stride(1) != 1 \
                or residual.dtype != torch.bfloat16:
            raise RuntimeError("samfast: residual must be a bf16 (M, N) tensor")
        if out is None:
            out = torch.empty_like(residual)
    elif out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=xq.device)
    if tuple(out.shape) != (M, N) or out.dtype != torch.bfloat16 or out.stride(1) != 1:
        raise RuntimeError("samfast: out must be a bf16 (M, N) tensor with contiguous rows")
    gamma = beta = None
    eps = 0.0
    if ln is not None:
        gamma, beta, eps = ln
        _require_gpu(gamma, beta)
        if gamma.dtype != torch.bfloat16 or beta.dtype != torch.bfloat16 or gamma.numel() != N or beta.numel() != N:
            raise RuntimeError("samfast: LayerNorm weight / bias must be bf16 of length N")
        gamma, beta = gamma.contiguous(), beta.contiguous()
    yq = _xq_empty(M, N, out_layout, xq.device)
    sy = torch.empty((M,), dtype=torch.float32, device=xq.device)
    if counters is None:
        counters = tile_counters(M, xq.device)
    if counters.dtype != torch.int32 or counters.numel() * 128 < M or not counters.is_contiguous():
        raise RuntimeError("samfast: the counter workspace must hold ceil(M / 128) int32")
    lib = _lib.load()
    name = {_lib.EPILOGUE_NONE: "gemm_i8_scale_bias", _lib.EPILOGUE_GELU: "gemm_i8_gelu",
            _lib.EPILOGUE_RESIDUAL: "gemm_i8_residual"}.get(epilogue, "gemm_i8_fused") \
        + ("_lnquant" if ln is not None else "_quant")
    code = _timed(
        name, 2.0 * M * N * K, "op",
        lambda: lib.samfast_gemm_i8_fused_quant(
            xq.data_ptr(), sx.data_ptr(), wq.data_ptr(), sw.data_ptr(),
            bias.data_ptr() if bias is not None else None, out.data_ptr(), out.stride(0),
            M, N, K, _lib.SAMFAST_BF16, int(epilogue),
            residual.data_ptr() if residual is not None else None,
            residual.stride(0) if residual is not None else 0, int(layout),
            gamma.data_ptr() if gamma is not None else None,
            beta.data_ptr() if beta is not None else None, float(eps),
            yq.data_ptr(), sy.data_ptr(), int(out_layout), counters.data_ptr(), _stream()))
    _lib.check(code, "gemm_i8_fused_quant")
    return out, yq, sy


def prune24_pack(wq: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """int8 (N, K) -> packed 2:4 form (wc int8 (K/64, N, 32), widx int32 (K/64, N, 2)): per
    aligned group of 4 along K the two largest magnitudes are kept (ties: lowest position).
    Lossless for a matrix that already is 2:4.  Layout: include/samfast.h."""
    _require_gpu(wq)
    if wq.dtype != torch.int8 or wq.dim() != 2 or not wq.is_contiguous():
        raise RuntimeError("samfast: prune24_pack needs a contiguous int8 (N, K) tensor")
    N, K = wq.shape
    if K % 64 != 0:
        raise RuntimeError("samfast: prune24_pack needs K % 64 == 0")
    wc = torch.empty((K // 64, N, 32), dtype=torch.int8, device=wq.device)
    widx = torch.empty((K // 64, N, 2), dtype=torch.int32, device=wq.device)
    code = _lib.load().samfast_prune24_pack_i8(wq.data_ptr(), wc.data_ptr(), widx.data_ptr(), N, K,
                                               _stream())
    _lib.check(code, "prune24_pack_i8")
    return wc, widx


def _check_sparse24(xq: torch.Tensor, wc: torch.Tensor, widx: torch.Tensor,
                    layout: int = _lib.LAYOUT_ROWMAJOR) -> Tuple[int, int, int]:
    M, K = _operand_shape(xq, layout)
    if (wc.dtype != torch.int8 or widx.dtype != torch.int32 or wc.dim() != 3 or widx.dim() != 3
            or not (wc.is_contiguous() and widx.is_contiguous())
            or wc.shape[0] * 64 != K or wc.shape[2] != 32
            or tuple(widx.shape) != (wc.shape[0], wc.shape[1], 2)):
        raise RuntimeError("samfast: packed weight must be int8 (K/64, N, 32) + int32 (K/64, N, 2)")
    return M, wc.shape[1], K


def gemm_i8_sparse24_i32(xq: torch.Tensor, wc: torch.Tensor, widx: torch.Tensor) -> torch.Tensor:
    """int8 (M, K) x packed 2:4 int8 weight -> int32 (M, N), exact."""
    _require_gpu(xq, wc, widx)
    M, N, K = _check_sparse24(xq, wc, widx)
    acc = torch.empty((M, N), dtype=torch.int32, device=xq.device)
    lib = _lib.load()
    code = _timed(
        "gemm_i8_sp24_i32", 1.0 * M * N * K, "op",
        lambda: lib.samfast_gemm_i8_sparse24_i32(xq.data_ptr(), wc.data_ptr(), widx.data_ptr(),
                                                 acc.data_ptr(), M, N, K, _stream()))
    _lib.check(code, "gemm_i8_sparse24_i32")
    return acc


def gemm_i8_sparse24_fused(xq: torch.Tensor, sx: torch.Tensor, wc: torch.Tensor, widx: torch.Tensor,
                           sw: torch.Tensor, bias: Optional[torch.Tensor], epilogue: int,
                           residual: Optional[torch.Tensor] = None,
                           out: Optional[torch.Tensor] = None,
                           layout: int = _lib.LAYOUT_ROWMAJOR) -> torch.Tensor:
    """gemm_i8_fused (no row scatter) with the weight in the packed 2:4 form; `layout` is the
    layout of xq.  The work
    reported to record_launches is the multiply-adds the sparse matrix cores execute
    (half the dense count)."""
    _require_gpu(xq, sx, wc, widx, sw, bias, residual)
    M, N, K = _check_sparse24(xq, wc, widx, layout)
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != M or sw.numel() != N:
        raise RuntimeError("samfast: scales must be fp32 of length M and N")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N):
        raise RuntimeError("samfast: bias must be fp32 of length N")
    if epilogue == _lib.EPILOGUE_RESIDUAL:
        if residual is None or tuple(residual.shape) != (M, N) or residual.stride(1) != 1 \
                or residual.dtype != torch.bfloat16:
            raise RuntimeError("samfast: residual must be a bf16 (M, N) tensor")
        if out is None:
            out = torch.empty_like(residual)
    elif out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=xq.device)
    lib = _lib.load()
    name = {_lib.EPILOGUE_NONE: "gemm_i8_sp24_scale_bias", _lib.EPILOGUE_GELU: "gemm_i8_sp24_gelu",
            _lib.EPILOGUE_RESIDUAL: "gemm_i8_sp24_residual"}.get(epilogue, "gemm_i8_sp24_fused")
    code = _timed(
        name, 1.0 * M * N * K, "op",
        lambda: lib.samfast_gemm_i8_sparse24_fused(
            xq.data_ptr(), sx.data_ptr(), wc.data_ptr(), widx.data_ptr(), sw.data_ptr(),
            bias.data_ptr() if bias is not None else None, out.data_ptr(), out.stride(0),
            M, N, K, _lib.SAMFAST_BF16, int(epilogue),
            residual.data_ptr() if residual is not None else None,
            residual.stride(0) if residual is not None else 0, int(layout), _stream()))
    _lib.check(code, "gemm_i8_sparse24_fused")
    return out


_window_maps = {}


def window_row_maps(B: int, H: int, W: int, window: int, device) -> Tuple[torch.Tensor, Tuple[int, int]]:
    """int32 map for window_partition on (B, H, W) tokens: entry r of the window-ordered,
    zero-padded token list holds the flat index of its source token, or -1 for a padding
    position.  The same tensor is the scatter map of window_unpartition.  Cached."""
    key = (B, H, W, window, str(device))
    hit = _window_maps.get(key)
    if hit is not None:
        return hit
    Hp = H + (-H) % window
    Wp = W + (-W) % window
    idx = torch.arange(B * H * W, dtype=torch.int32).view(B, H, W)
    padded = torch.full((B, Hp, Wp), -1, dtype=torch.int32)
    padded[:, :H, :W] = idx
    wins = padded.view(B, Hp // window, window, Wp // window, window).permute(0, 1, 3, 2, 4)
    res = (wins.reshape(-1).contiguous().to(device), (Hp, Wp))
    _window_maps[key] = res
    return res
