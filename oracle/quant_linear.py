"""Oracle: dynamic symmetric int8 linear (CPU, numpy integers + fp32).

TEST INFRASTRUCTURE ONLY (see the package docstring).

What the reference does on this path
------------------------------------
experiments/eval_combo.py:357-360 calls `torchao.quantization.apply_dynamic_quant`
on the image encoder.  torchao is a third-party dependency that setup.py:16
names without a version, that is not vendored under the reference tree and is
not installed here.  Its published algorithm (torchao 0.1, quant_primitives:
`quantize_activation_per_token_absmax`, `dynamically_quantize_per_channel`,
`quant_int8_per_token_matmul`) is restated below in the form the benchmark
configuration of this build fixes it:

  activations, per token (row):  s_x[m] = absmax(x[m, :]) / 127
  weights, per output channel:   s_w[n] = absmax(w[n, :]) / 127
  q = clamp(round_half_even(value / s), -127, 127) as int8
  acc[m, n] = sum_k xq[m, k] * wq[n, k]            (int32, exact)
  y[m, n]   = (float(acc) * s_x[m]) * s_w[n] + bias[n]   -> bf16

All floating-point steps are single fp32 operations in the order written
(no fused multiply-add), so a GPU kernel can reproduce them bit for bit.
An all-zero row or channel gets absmax floored at 1e-5 (torchao's eps), which
only changes rows that quantise to all zeros anyway.

PARITY UNPINNED against torchao itself: the reference holds no test, golden
vector or fixture for the quantised path, and torchao cannot be imported in
this environment, so its exact scale/rounding conventions (127 vs 127.5
divisors, bf16 vs fp32 division) are not checked.  What IS pinned
(tests/test_oracle_quant.py): the integer GEMM against int64 matmul and
torch._int_mm (the library routine torchao calls); the quantisers against
their closed form and invariants (|q| <= 127, the absmax element maps to
+-127, positive rescaling of a row leaves q unchanged, rows are independent,
dequantisation error <= s/2); the epilogue against float64.
"""

import numpy as np
import torch

EPS = np.float32(1e-5)
QMAX = np.float32(127.0)


def _to_f32_numpy(t) -> np.ndarray:
    if isinstance(t, torch.Tensor):
        return t.detach().to(torch.float32).cpu().numpy()
    return np.asarray(t, dtype=np.float32)


def quantize_rows_absmax(x):
    """Per-row symmetric int8: returns (q int8 (M, K), scale fp32 (M,)).

    Stands for torchao's per-token activation quantiser (called from
    experiments/eval_combo.py:357-359) and, applied to a (N, K) weight, for
    its per-output-channel weight quantiser.
    """
    xf = x.detach().to(torch.float32) if isinstance(x, torch.Tensor) else torch.from_numpy(_to_f32_numpy(x))
    assert xf.dim() == 2
    # torch's CPU element-wise kernels: one IEEE fp32 operation per call (several threads);
    # amax propagates a NaN, round() is round-half-to-even
    absmax = xf.abs().amax(dim=1).clamp_min(float(EPS))
    scale = absmax / float(QMAX)
    ratio = xf / scale[:, None]
    q = ratio.round().clamp_(-127.0, 127.0).to(torch.int8)
    return q.numpy(), scale.numpy()


def int8_gemm_i32(xq: np.ndarray, wq: np.ndarray) -> np.ndarray:
    """acc[m, n] = sum_k xq[m, k] * wq[n, k] as int32 (torch._int_mm semantics).

    |acc| <= K * 128^2 < 2^31 for K <= 131 000, so int32 never wraps here.  Large
    products run as a float64 matrix product on the BLAS threads: every product and
    every partial sum is an integer far below 2^53, so the result is exact whatever
    the summation order (torch._int_mm on a CPU gives the same numbers 50x slower;
    tests/test_oracle_quant.py checks the two and the int64 product against each other).
    """
    assert xq.dtype == np.int8 and wq.dtype == np.int8
    M, K = xq.shape
    if M * wq.shape[0] * K >= 1 << 22:
        a = torch.from_numpy(np.ascontiguousarray(xq)).to(torch.float64)
        b = torch.from_numpy(np.ascontiguousarray(wq)).to(torch.float64)
        return (a @ b.t()).to(torch.int32).numpy()
    return (xq.astype(np.int32) @ wq.astype(np.int32).T).astype(np.int32)


def int8_gemm_i64(xq: np.ndarray, wq: np.ndarray) -> np.ndarray:
    """Same product through int64 numpy matmul: the independent check of int8_gemm_i32."""
    return xq.astype(np.int64) @ wq.astype(np.int64).T


def scale_bias_epilogue(acc: np.ndarray, sx: np.ndarray, sw: np.ndarray, bias) -> torch.Tensor:
    """y = (float(acc) * sx[m]) * sw[n] + bias[n], each step one fp32 op, -> bf16.
    (torch's CPU element-wise kernels: one IEEE operation per call, several threads.)"""
    t = torch.from_numpy(np.ascontiguousarray(acc)).to(torch.float32)  # int32 -> fp32, round to nearest even
    t = t * torch.from_numpy(np.ascontiguousarray(sx, dtype=np.float32))[:, None]
    t = t * torch.from_numpy(np.ascontiguousarray(sw, dtype=np.float32))[None, :]
    if bias is not None:
        t = t + torch.from_numpy(_to_f32_numpy(bias))[None, :]
    return t.to(torch.bfloat16)


def dynamic_int8_linear(x: torch.Tensor, weight: torch.Tensor, bias) -> torch.Tensor:
    """Whole dynamic-quant Linear on (..., K) activations; returns bf16 (..., N)."""
    lead = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    xq, sx = quantize_rows_absmax(x2)
    wq, sw = quantize_rows_absmax(weight)
    acc = int8_gemm_i32(xq, wq)
    y = scale_bias_epilogue(acc, sx, sw, bias)
    return y.reshape(*lead, weight.shape[0])


def prune_2_of_4(weight: torch.Tensor) -> torch.Tensor:
    """Zero the 2 smallest-magnitude entries of every 4 consecutive along K.

    Follows segment_anything_fast/sparse.py:6-25 (WeightNormSparsifier with
    sparse_block_shape=(1, 4), zeros_per_block=2, sparsity_level=1.0).  Ties
    keep the earlier index (the sparsifier leaves tie order unspecified).
    """
    w = _to_f32_numpy(weight)
    N, K = w.shape
    assert K % 4 == 0
    blocks = np.abs(w).reshape(N, K // 4, 4)
    # stable sort descending by magnitude: keep the first two positions
    order = np.argsort(-blocks, axis=-1, kind="stable")
    keep = np.zeros_like(blocks, dtype=bool)
    np.put_along_axis(keep, order[..., :2], True, axis=-1)
    out = (w.reshape(N, K // 4, 4) * keep).reshape(N, K)
    return torch.from_numpy(out).to(weight.dtype if isinstance(weight, torch.Tensor) else torch.float32)


def _group_dense_offset(g: int, h: int) -> int:
    """First dense k (inside a 64-wide block) of group g of lane half h, as the gfx950
    sparse matrix instruction v_smfmac_i32_32x32x64_i8 pairs stored A bytes with B."""
    return 32 * (g // 4) + 16 * h + 4 * (g % 4)


def pack_2_of_4(wq: np.ndarray):
    """Packed form of an int8 (N, K) matrix for the sparse int8 GEMM (layout documented at
    samfast_prune24_pack_i8 in include/samfast.h): per aligned group of 4 along K the two
    largest magnitudes (ties: lowest position) are kept.  The compress step of
    segment_anything_fast/sparse.py:32 (to_sparse_semi_structured), restated for int8 and
    the gfx950 operand order.  Pure-Python loops: small matrices only.

    Returns (wc int8 (K/64, N, 32), widx int32 (K/64, N, 2)).
    """
    assert wq.dtype == np.int8 and wq.ndim == 2 and wq.shape[1] % 64 == 0
    N, K = wq.shape
    wc = np.zeros((K // 64, N, 32), dtype=np.int8)
    widx = np.zeros((K // 64, N, 2), dtype=np.uint32)
    for kb in range(K // 64):
        for n in range(N):
            for h in range(2):
                word = 0
                for g in range(8):
                    base = 64 * kb + _group_dense_offset(g, h)
                    grp = wq[n, base:base + 4].astype(np.int32)
                    order = sorted(range(4), key=lambda p: (-abs(int(grp[p])), p))
                    p0, p1 = sorted(order[:2])
                    wc[kb, n, 16 * h + 2 * g] = grp[p0]
                    wc[kb, n, 16 * h + 2 * g + 1] = grp[p1]
                    word |= (p0 | (p1 << 2)) << (4 * g)
                widx[kb, n, h] = word
    return wc, widx.view(np.int32)


def unpack_2_of_4(wc: np.ndarray, widx: np.ndarray) -> np.ndarray:
    """Inverse of pack_2_of_4: the dense int8 (N, K) matrix a packed weight stands for."""
    KB, N, _ = wc.shape
    out = np.zeros((N, KB * 64), dtype=np.int8)
    words = widx.view(np.uint32)
    for kb in range(KB):
        for n in range(N):
            for h in range(2):
                word = int(words[kb, n, h])
                for g in range(8):
                    base = 64 * kb + _group_dense_offset(g, h)
                    nib = (word >> (4 * g)) & 15
                    out[n, base + (nib & 3)] = wc[kb, n, 16 * h + 2 * g]
                    out[n, base + (nib >> 2)] = wc[kb, n, 16 * h + 2 * g + 1]
    return out


def sparse24_int8_linear(x: torch.Tensor, weight: torch.Tensor, bias) -> torch.Tensor:
    """Dynamic int8 Linear whose float weight is first magnitude-pruned to 2:4
    (sparse.py:6-25), then quantised per output channel: the combination the
    benchmark's int8 + 2:4 MLP configuration uses."""
    return dynamic_int8_linear(x, prune_2_of_4(weight), bias)
