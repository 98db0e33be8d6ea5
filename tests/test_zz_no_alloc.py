"""The entry point that allocates nothing (samfast_gemm_i8_fused_quant_noalloc: its counter
workspace is a device array inside the library) against the entry point that takes the workspace
from the caller, raw through the C ABI: y, codes and scales bit-equal, on two calls in a row of
which the second is the smaller one, for both kinds of fused quantiser."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(lib, fn_name, t, M, N, K, epilogue, counters):
    from samfast_amd import _lib
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    yq = torch.empty((N // 64, M, 64), dtype=torch.int8, device="cuda")
    sy = torch.empty((M,), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    res = t["res"]
    args = [t["xq"].data_ptr(), t["sx"].data_ptr(), t["wq"].data_ptr(), t["sw"].data_ptr(), t["bias"].data_ptr(),
            y.data_ptr(), N, M, N, K, _lib.SAMFAST_BF16, epilogue,
            res.data_ptr() if res is not None else None, N if res is not None else 0, _lib.LAYOUT_KB64,
            t["gamma"].data_ptr() if t["gamma"] is not None else None,
            t["beta"].data_ptr() if t["beta"] is not None else None, 1e-6,
            yq.data_ptr(), sy.data_ptr(), _lib.LAYOUT_KB64]
    if counters is not None:
        args.append(counters.data_ptr())
    args.append(stream)
    _lib.check(getattr(lib, fn_name)(*args), fn_name)
    torch.cuda.synchronize()
    return y, yq, sy


def _inputs(M, N, K, ln, seed):
    from samfast_amd import _lib, ops
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).cuda()
    xq, sx = ops.quant_rowwise(x, _lib.LAYOUT_KB64)
    wq, sw = ops.quant_rowwise(w, _lib.LAYOUT_KB64)
    t = {"xq": xq, "sx": sx, "wq": wq, "sw": sw, "bias": (torch.randn(N, generator=g) * 0.02).cuda(),
         "res": None, "gamma": None, "beta": None}
    if ln:
        t["res"] = torch.randn((M, N), generator=g).to(torch.bfloat16).cuda()
        t["gamma"] = (1 + 0.1 * torch.randn(N, generator=g)).to(torch.bfloat16).cuda()
        t["beta"] = (0.1 * torch.randn(N, generator=g)).to(torch.bfloat16).cuda()
    return t


@pytest.mark.parametrize("N,K,ln", [(5120, 1280, False), (1280, 5120, True)])
def test_no_alloc_entry_point_equals_workspace_entry_point(N, K, ln):
    from samfast_amd import _lib
    lib = _lib.load()
    epilogue = _lib.EPILOGUE_RESIDUAL if ln else _lib.EPILOGUE_GELU
    for M, seed in ((4096 + 77, 1), (300, 2)):     # the second call is the smaller one
        print(f"case no-alloc N={N} K={K} ln={ln} M={M}", flush=True)
        t = _inputs(M, N, K, ln, seed)
        counters = torch.zeros(-(-M // 128), dtype=torch.int32, device="cuda")
        y0, q0, s0 = _call(lib, "samfast_gemm_i8_fused_quant", t, M, N, K, epilogue, counters)
        y1, q1, s1 = _call(lib, "samfast_gemm_i8_fused_quant_noalloc", t, M, N, K, epilogue, None)
        assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
        assert torch.equal(q0, q1)
        assert torch.equal(s0.view(torch.int32), s1.view(torch.int32))


def test_no_alloc_entry_point_rejects_sizes_beyond_its_workspace():
    from samfast_amd import _lib
    lib = _lib.load()
    M = 32768 * 128 + 1
    rc = lib.samfast_gemm_i8_fused_quant_noalloc(None, None, None, None, None, None, 1280, M, 1280, 1280, 0, 2,
                                                 None, 1280, 1, None, None, 1e-6, None, None, 1, None)
    assert rc == -1 and b"row-tile counters" in lib.samfast_last_error()


def test_no_alloc_entry_point_under_graph_capture():
    """What the entry point is for: recorded into a HIP graph (no allocation may happen while
    capturing; the counters are cleared by a kernel, not a memset node) and replayed several times
    with eager work and synchronisations in between, every replay must reproduce the eager result."""
    from samfast_amd import _lib
    lib = _lib.load()
    M, N, K = 1000, 1280, 1280
    t = _inputs(M, N, K, True, 3)
    counters = torch.zeros(-(-M // 128), dtype=torch.int32, device="cuda")
    y0, q0, s0 = _call(lib, "samfast_gemm_i8_fused_quant", t, M, N, K, _lib.EPILOGUE_RESIDUAL, counters)
    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    yq = torch.empty((N // 64, M, 64), dtype=torch.int8, device="cuda")
    sy = torch.empty((M,), dtype=torch.float32, device="cuda")

    def launch():
        args = [t["xq"].data_ptr(), t["sx"].data_ptr(), t["wq"].data_ptr(), t["sw"].data_ptr(), t["bias"].data_ptr(),
                y.data_ptr(), N, M, N, K, _lib.SAMFAST_BF16, _lib.EPILOGUE_RESIDUAL, t["res"].data_ptr(), N,
                _lib.LAYOUT_KB64, t["gamma"].data_ptr(), t["beta"].data_ptr(), 1e-6, yq.data_ptr(), sy.data_ptr(),
                _lib.LAYOUT_KB64, torch.cuda.current_stream().cuda_stream]
        _lib.check(lib.samfast_gemm_i8_fused_quant_noalloc(*args), "fused_quant_noalloc")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()  # the first call on a device looks the array's address up: keep that out of the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    for rep in range(3):
        y.zero_(); yq.zero_(); sy.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), y0.view(torch.int16)), rep
        assert torch.equal(yq, q0) and torch.equal(sy.view(torch.int32), s0.view(torch.int32)), rep
        _call(lib, "samfast_gemm_i8_fused_quant_noalloc", _inputs(300, N, K, True, 9), 300, N, K,
              _lib.EPILOGUE_RESIDUAL, None)  # eager work on the same array between replays
