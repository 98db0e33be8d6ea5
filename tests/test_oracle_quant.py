"""Pins the quantised-linear oracle (oracle/quant_linear.py): integer GEMM against
int64 matmul and torch._int_mm; quantisers against closed form and invariants;
epilogue against float64; 2:4 pruning against brute force and the library
sparsifier."""

import numpy as np
import pytest
import torch

from helpers import linear_inputs
from oracle import quant_linear as orq


def test_quantiser_closed_form_small():
    x = torch.tensor([[1.0, -2.0, 0.5, 127.0], [0.0, 0.0, 0.0, 0.0], [-3.0, 1.5, 0.75, 0.1]])
    q, s = orq.quantize_rows_absmax(x)
    assert np.array_equal(s, np.array([1.0, np.float32(1e-5) / np.float32(127), np.float32(3.0) / np.float32(127)], dtype=np.float32))
    assert q[0].tolist() == [1, -2, 0, 127]          # 0.5 -> 0 (half to even)
    assert q[1].tolist() == [0, 0, 0, 0]
    assert q[2].tolist() == [-127, 64, 32, 4]        # 63.5 -> 64, 31.75 -> 32, 4.23 -> 4


def test_quantiser_half_to_even():
    x = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]])
    q, s = orq.quantize_rows_absmax(x)
    assert s[0] == 1.0
    assert q[0].tolist() == [127, 0, 2, 2, 0, -2, -2, 4]


def test_quantiser_invariants():
    x, _, _ = linear_inputs(200, 256, 8, seed=1)
    xf = x.float()
    q, s = orq.quantize_rows_absmax(x)
    assert q.dtype == np.int8 and np.abs(q.astype(np.int32)).max() <= 127
    amax_idx = xf.abs().argmax(dim=1).numpy()
    assert np.all(np.abs(q[np.arange(200), amax_idx].astype(np.int32)) == 127)
    # dequantisation error at most half a step
    err = np.abs(q.astype(np.float32) * s[:, None] - xf.numpy())
    assert np.all(err <= 0.5 * s[:, None] * (1 + 1e-3))
    # positive power-of-two rescaling of a row leaves the codes unchanged
    q2, s2 = orq.quantize_rows_absmax(xf * 4.0)
    assert np.array_equal(q2, q) and np.allclose(s2, 4 * s)
    # rows are independent: changing one row changes only that row
    y = xf.clone()
    y[7] *= 20.0
    q3, _ = orq.quantize_rows_absmax(y)
    keep = np.arange(200) != 7
    assert np.array_equal(q3[keep], q[keep])


@pytest.mark.parametrize("M,N,K", [(3, 8, 8), (17, 24, 64), (130, 264, 1280), (256, 1280, 1280)])
def test_int8_gemm_three_ways(M, N, K):
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).numpy()
    b = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).numpy()
    ref64 = orq.int8_gemm_i64(a, b)
    got = orq.int8_gemm_i32(a, b)
    assert got.dtype == np.int32 and np.array_equal(got.astype(np.int64), ref64)
    if M > 16 and K % 8 == 0 and N % 8 == 0:  # the library routine the reference's quantised Linear calls
        lib = torch._int_mm(torch.from_numpy(a), torch.from_numpy(b).t())
        assert np.array_equal(lib.numpy(), got)
    # brute force on a corner
    for (i, j) in [(0, 0), (M - 1, N - 1)]:
        assert ref64[i, j] == sum(int(a[i, t]) * int(b[j, t]) for t in range(K))
    # worst case does not wrap
    ones = np.full((32, 5120), 127, dtype=np.int8)
    assert orq.int8_gemm_i32(ones, -ones)[0, 0] == -5120 * 127 * 127


def test_epilogue_against_float64():
    g = torch.Generator().manual_seed(0)
    acc = torch.randint(-2_000_000, 2_000_000, (50, 40), generator=g, dtype=torch.int32).numpy()
    sx = (torch.rand(50, generator=g) * 0.05 + 1e-3).numpy()
    sw = (torch.rand(40, generator=g) * 1e-3 + 1e-5).numpy()
    bias = torch.randn(40, generator=g) * 0.02
    y = orq.scale_bias_epilogue(acc, sx, sw, bias).float().numpy()
    exact = acc.astype(np.float64) * sx[:, None].astype(np.float64) * sw[None, :].astype(np.float64) \
        + bias.double().numpy()[None, :]
    assert np.all(np.abs(y - exact) <= np.abs(exact) * 2 ** -8 + 1e-30)  # one bf16 rounding
    y0 = orq.scale_bias_epilogue(acc, sx, sw, None).float().numpy()
    assert np.all(np.abs(y0 - (exact - bias.double().numpy())) <= np.abs(exact - bias.double().numpy()) * 2 ** -8 + 1e-30)


def test_dynamic_linear_close_to_float_linear():
    x, w, b = linear_inputs(64, 1280, 96, seed=3)
    y = orq.dynamic_int8_linear(x, w, b).float()
    ref = torch.nn.functional.linear(x.float(), w.float(), b.float())
    rel = (y - ref).norm() / ref.norm()
    assert rel < 0.02, rel
    y3 = orq.dynamic_int8_linear(x.reshape(4, 16, 1280), w, b)
    assert y3.shape == (4, 16, 96) and torch.equal(y3.reshape(64, 96), orq.dynamic_int8_linear(x, w, b))


def test_prune_2_of_4_bruteforce_and_library():
    g = torch.Generator().manual_seed(5)
    w = torch.randn(12, 32, generator=g)
    p = orq.prune_2_of_4(w)
    for n in range(12):
        for blk in range(8):
            seg = w[n, 4 * blk:4 * blk + 4]
            kept = p[n, 4 * blk:4 * blk + 4]
            assert (kept != 0).sum() == 2
            top2 = seg.abs().topk(2).indices.tolist()
            for t in range(4):
                assert kept[t] == (seg[t] if t in top2 else 0)
    # the routine the reference calls (sparse.py:12-25)
    from torch.ao.pruning import WeightNormSparsifier
    lin = torch.nn.Linear(32, 12, bias=False)
    with torch.no_grad():
        lin.weight.copy_(w)
    sp = WeightNormSparsifier(sparsity_level=1.0, sparse_block_shape=(1, 4), zeros_per_block=2)
    sp.prepare(torch.nn.Sequential(lin), [{"tensor_fqn": "0.weight"}])
    sp.step()
    sp.squash_mask()
    assert torch.equal(lin.weight.detach(), p)


def test_pack_2_of_4_round_trip_and_invariants():
    """The packed 2:4 form stands for exactly the magnitude-pruned matrix; positions are
    ordered and every group keeps two entries.  (Which stored byte the hardware pairs with
    which dense k is fixed by the GPU bit-exact tests, not here.)"""
    rng = np.random.default_rng(11)
    for hi in (128, 3):  # full range, and a range that forces ties and zeros
        wq = rng.integers(-hi + 1, hi, size=(6, 192), dtype=np.int8)
        wc, widx = orq.pack_2_of_4(wq)
        assert wc.shape == (3, 6, 32) and widx.shape == (3, 6, 2) and widx.dtype == np.int32
        dense = orq.unpack_2_of_4(wc, widx)
        pruned = orq.prune_2_of_4(torch.from_numpy(wq.astype(np.float32))).numpy().astype(np.int8)
        assert np.array_equal(dense, pruned)
        words = widx.view(np.uint32)
        for g in range(8):
            nib = (words >> (4 * g)) & 15
            assert np.all((nib & 3) < (nib >> 2))
        # a matrix that already is 2:4 is packed without loss
        wc2, widx2 = orq.pack_2_of_4(pruned)
        assert np.array_equal(orq.unpack_2_of_4(wc2, widx2), pruned)
