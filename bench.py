#!/usr/bin/env python3
"""Benchmark of the SAM ViT image-encoder hot path on one MI355X.

One step = one forward of the ViT-H image encoder over a batch of 16 synthetic
1024x1024 images (bf16 activations, rel-pos attention on the HIP flash kernels,
all four Linears of every block on the dynamic-int8 HIP kernels), inputs and
weights resident in HBM before the timed region.

Prints ONE JSON line: images/s plus
  roofline       the dominant kernel (by time inside a step) against its bound,
                 from per-launch event timings of an instrumented step;
  kernels        the same figures for every hand-written kernel in the step (window attention also
                 against the HBM roof, which is its bound);
  attention_combined  all rel-pos attention of a step against the bf16 MFMA peak;
  config_1       the single global attention operator (B=1, 12 heads, 4096 tokens, head_dim 64) on the
                 kernel and through the reference's CPU route;
  gpu_baseline   the same encoder through PyTorch-ROCm bf16 SDPA + bf16 Linear;
  other_configs  the two other encoder configurations of the benchmark, measured the same way in the
                 same process: ViT-H batch 32 with 2:4-sparse MLP linears, and ViT-B batch 1 (eager
                 launches and replayed as one HIP graph); --main-only leaves them out;
  mfma_ceiling   what a loop of nothing but matrix instructions sustains on this GPU, on constant and
                 on random operands (--no-mfma-ceiling leaves it out);
  cpu_baseline   the CPU oracle (the reference's eager route) on one image.
"""

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "segment-anything-fast_amd"))
sys.path.insert(0, str(ROOT))

PEAK = {"op": ("mfma", 5.0e15, "TOP/s"),       # int8 dense MFMA
        "flop": ("mfma", 2.5e15, "TFLOP/s"),   # bf16 dense MFMA
        "byte": ("hbm", 8.0e12, "GB/s")}       # HBM3E

# Bytes per launch that cross the L2 <-> fabric boundary (average over the launches of one
# encoder step), from the two `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of this
# script summarised in TRAFFIC_SOURCE, each counter scaled by what it reads for the 1 GiB
# --calibration-copy dispatch (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  Counters cannot be read
# from inside a timed run, so the figure is a recorded one: it is reported only for the default
# workload (vit_h, batch 16, dense int8 linears) and only while the kernel family's source files
# still have the hash they had when the counters were taken (otherwise `traffic` is null).
TRAFFIC_SOURCE = "profiles/bench_vit_h_bs16_pmc_traffic.txt"
TRAFFIC = {"gemm_i8_kernel": (1.0042e9, "gemm_i8.hip+gemm_i8_persist.hip+gemm_i8_shared.hpp", "bfc90be515ad881e")}


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=10)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--model", default="vit_h", choices=["vit_h", "vit_l", "vit_b"])
    p.add_argument("--batch", type=int, default=16)
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--no-gpu-baseline", action="store_true")
    p.add_argument("--no-compiled-baseline", action="store_true",
                   help="skip the torch.compile variant of the PyTorch-ROCm baseline (about 30 s)")
    p.add_argument("--main-only", action="store_true",
                   help="measure only the workload named by --model / --batch (no other_configs object)")
    p.add_argument("--no-mfma-ceiling", action="store_true", help="skip the matrix-instruction-only loops")
    p.add_argument("--mfma-ceiling", action="store_true",
                   help="run ONLY the matrix-instruction-only loops and print their JSON object")
    p.add_argument("--gemm-variants", action="store_true",
                   help="run ONLY the int8 GEMM variant table: the four ViT-H linears at 65536 rows under every "
                        "kernel-variant knob, on all-zero and on model-like codes, and print its JSON object")
    p.add_argument("--bf16-linears", action="store_true", help="keep nn.Linear (attention kernels only)")
    p.add_argument("--sparse-mlp", action="store_true",
                   help="lin1 / lin2 magnitude-pruned 2:4 on the sparse int8 matrix cores (the int8 + 2:4 "
                        "configuration); every other Linear dense int8")
    p.add_argument("--graph", action="store_true",
                   help="replay the forward as one HIP graph (launch-bound shapes, e.g. vit_b batch 1)")
    p.add_argument("--also-graph", action="store_true",
                   help="besides the eager launches, time the forward replayed as a HIP graph and through "
                        "sam_model_fast_registry (hip_graph_replay / fast_registry_replay objects)")
    p.add_argument("--calibration-copy", action="store_true",
                   help="also run one 1 GiB device-to-device copy (a known-size reference for "
                        "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    p.add_argument("--library-yardsticks", action="store_true",
                   help="also time the ROCm libraries on the encoder's operator shapes (torch._int_mm = "
                        "hipBLASLt int8, bf16 F.linear, F.scaled_dot_product_attention) next to the "
                        "hand-written kernels; adds a 'library_yardsticks' object to the JSON line")
    return p.parse_args()


def time_steps(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def kernel_table(summary):
    rows = {}
    for name, d in summary.items():
        bound, peak, unit = PEAK[d["unit"]]
        sec = d["ms"] * 1e-3
        rate = d["work"] / sec if sec > 0 else 0.0
        scale = 1e-9 if unit == "GB/s" else 1e-12
        rows[name] = {
            "launches": d["launches"], "ms_total": round(d["ms"], 3),
            "avg_us": round(1e3 * d["ms"] / d["launches"], 2),
            "bound": bound, "achieved": round(rate * scale, 2), "peak": peak * scale,
            "unit": unit, "frac": round(rate / peak, 4),
        }
        if d.get("bytes") and sec > 0:
            # a kernel whose arithmetic intensity puts it under the HBM roof (window attention: ~100
            # flop per byte against 312 at the ridge): its algorithmic bytes against the HBM peak as well
            rows[name]["bound"] = "hbm"
            rows[name]["hbm"] = {"achieved": round(d["bytes"] / sec * 1e-9, 1), "peak": 8000.0, "unit": "GB/s",
                                 "frac": round(d["bytes"] / sec / 8.0e12, 4),
                                 "flop_per_byte": round(d["work"] / d["bytes"], 1)}
    return rows


def attention_combined(summary):
    """Rel-pos attention as a whole (global + windowed launches of one step) against the bf16 MFMA peak:
    the second half of the benchmark's metric."""
    ms = sum(d["ms"] for n, d in summary.items() if n.startswith("attn_"))
    flop = sum(d["work"] for n, d in summary.items() if n.startswith("attn_"))
    if ms <= 0:
        return None
    rate = flop / (ms * 1e-3)
    return {"what": "all rel-pos attention launches of one step (4 B nH N^2 hd flop each)", "ms_per_step": round(ms, 3),
            "TFLOP_per_step": round(flop * 1e-12, 3), "achieved": round(rate * 1e-12, 1), "peak": 2500.0,
            "unit": "TFLOP/s", "frac": round(rate / 2.5e15, 4)}


def library_yardsticks(batch, heads, hd, width):
    """The encoder's operator shapes on the ROCm libraries that PyTorch calls, next to the kernels of
    this repository on the same operands (events around 10 calls each, after 2 warm-up calls)."""
    import torch
    import torch.nn.functional as F
    from samfast_amd import _lib, ops

    def rate(fn, work, n=10):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return round(work / (e0.elapsed_time(e1) / n * 1e-3) / 1e12, 1)

    res = {"unit": "TOP/s (linears), TFLOP/s (attention)", "linears": {}, "attention": {}}
    M = batch * 4096
    g = torch.Generator(device="cuda").manual_seed(4)
    epi = {"qkv": _lib.EPILOGUE_NONE, "proj": _lib.EPILOGUE_RESIDUAL, "lin1": _lib.EPILOGUE_GELU,
           "lin2": _lib.EPILOGUE_RESIDUAL}
    for name, N, K in (("qkv", 3 * width, width), ("proj", width, width), ("lin1", 4 * width, width),
                       ("lin2", width, 4 * width)):
        x = torch.randn((M, K), device="cuda", generator=g)
        x[torch.randperm(M, device="cuda", generator=g)[:max(1, M // 1000)]] *= 20.0
        x = x.to(torch.bfloat16)
        w = (torch.randn((N, K), device="cuda", generator=g) * 0.02).to(torch.bfloat16)
        xq, sx = ops.quant_rowwise(x)
        wq, sw = ops.quant_rowwise(w)
        xk, wk = ops.to_kb64(xq), ops.to_kb64(wq)
        bias = torch.zeros(N, device="cuda")
        resid = torch.randn((M, N), device="cuda").to(torch.bfloat16) if epi[name] == _lib.EPILOGUE_RESIDUAL else None
        out = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        work = 2.0 * M * N * K
        row = {"this_repo_fused_epilogue_bf16_out": rate(
            lambda: ops.gemm_i8_fused(xk, sx, wk, sw, bias, epi[name], residual=resid, out=out,
                                      layout=_lib.LAYOUT_KB64), work)}
        try:
            wt = wq.t()
            row["torch_int_mm_int32_out"] = rate(lambda: torch._int_mm(xq, wt), work)
        except Exception as e:  # not every build exposes it
            row["torch_int_mm_int32_out"] = f"unavailable: {str(e)[:60]}"
        row["torch_bf16_linear"] = rate(lambda: F.linear(x, w), work)
        res["linears"][name] = row
        del x, w, xq, wq, xk, wk, out, resid
    for what, B, N, grid in (("global", batch, 4096, (64, 64)), ("window", batch * 25, 196, (14, 14))):
        q, k, v = (torch.randn((B, heads, N, hd), device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
        rph = (torch.randn((2 * grid[0] - 1, hd), device="cuda", generator=g) * 0.02).to(torch.bfloat16)
        rpw = (torch.randn((2 * grid[1] - 1, hd), device="cuda", generator=g) * 0.02).to(torch.bfloat16)
        work = 4.0 * B * heads * N * N * hd
        row = {"this_repo_with_relpos_bias": rate(lambda: ops.attn_relpos(q, k, v, rph, rpw, grid, hd ** -0.5), work),
               "torch_sdpa_no_bias": rate(lambda: F.scaled_dot_product_attention(q, k, v), work)}
        bias = torch.randn((B, heads, N, N), device="cuda", generator=g).to(torch.bfloat16)
        row["torch_sdpa_materialised_bias"] = rate(
            lambda: F.scaled_dot_product_attention(q, k, v, attn_mask=bias), work, n=3)
        res["attention"][what] = row
        del q, k, v, bias
    torch.cuda.empty_cache()
    return res


def source_sha16(names):
    """sha256 (first 16 hex digits) over the named kernel sources, in order ('a.hip+b.hip')"""
    import hashlib
    h = hashlib.sha256()
    for name in names.split("+"):
        path = ROOT / "segment-anything-fast_amd" / "csrc" / name
        if not path.exists():
            return None
        h.update(path.read_bytes())
    return h.hexdigest()[:16]


def mfma_ceiling():
    """Loops of nothing but matrix instructions (operands in registers, no memory traffic), on
    operands that are all zero, small constants, and random like a GEMM's / attention's: the
    rate this GPU's matrix pipe sustains under its power limit, in POP/s (int8) and PFLOP/s (bf16)."""
    import ctypes
    import torch
    from samfast_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    out = torch.zeros(1024, dtype=torch.int32, device=dev)
    g = torch.Generator(device="cuda").manual_seed(7)
    n8 = 8 * 256 * 16   # bytes of one operand buffer
    operands = {
        0: {"zeros": torch.zeros(n8, dtype=torch.int8, device=dev),
            "small_ints": torch.randint(0, 3, (n8,), generator=g, dtype=torch.int8, device=dev),
            "gaussian_codes": (torch.randn(n8, generator=g, device=dev) * 28).round().clamp(-127, 127).to(torch.int8),
            "random_int8": torch.randint(-127, 128, (n8,), generator=g, dtype=torch.int8, device=dev)},
        1: {"zeros": torch.zeros(n8 // 2, dtype=torch.bfloat16, device=dev),
            "ones": torch.ones(n8 // 2, dtype=torch.bfloat16, device=dev),
            "random_normal": torch.randn(n8 // 2, generator=g, device=dev).to(torch.bfloat16)},
    }
    # the same codes without their signs, and one (A, B) pair repeated for every instruction
    operands[0]["gaussian_codes_non_negative"] = operands[0]["gaussian_codes"].abs()
    operands[0]["random_int8_same_pair_every_instruction"] = \
        operands[0]["random_int8"].view(4, -1)[:1].repeat(4, 1).reshape(-1).contiguous()
    res = {"what": "8 independent MFMAs per round and wavefront, operands in registers, 512 workgroups of "
                   "4 wavefronts (2 wavefronts per SIMD on 256 CUs), ~40 ms per launch, events on the launch stream",
           "int8_v_mfma_i32_32x32x32_i8": {"unit": "POP/s", "published_peak": 5.0},
           "bf16_v_mfma_f32_32x32x16_bf16": {"unit": "PFLOP/s", "published_peak": 2.5}}
    stream = torch.cuda.current_stream().cuda_stream
    for instr, key, iters in ((0, "int8_v_mfma_i32_32x32x32_i8", 120000), (1, "bf16_v_mfma_f32_32x32x16_bf16", 100000)):
        for name, buf in operands[instr].items():
            ops = ctypes.c_int64(0)
            launch = lambda: _lib.check(lib.samfast_bench_mfma_ceiling(
                instr, buf.data_ptr(), 512, iters, ctypes.byref(ops), out.data_ptr(), stream), "bench_mfma_ceiling")
            launch()
            torch.cuda.synchronize()
            best = 0.0
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                launch()
                e1.record()
                torch.cuda.synchronize()
                best = max(best, ops.value / (e0.elapsed_time(e1) * 1e-3) / 1e15)
            res[key][name] = round(best, 3)
    # the same question asked of the real GEMM kernel: one encoder shape (qkv, 65536 x 3840 x 1280,
    # scale + bias epilogue) on all-zero codes and on codes like the encoder's, ten launches back to back
    from samfast_amd import ops
    M, N, K = 65536, 3840, 1280
    sx = torch.full((M,), 0.01, device=dev)
    sw = torch.full((N,), 0.001, device=dev)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    gemm = {"what": f"gemm_i8 {M}x{N}x{K}, scale + bias -> bf16, 10 launches back to back", "unit": "POP/s"}
    for name in ("zeros", "gaussian_codes"):
        if name == "zeros":
            xq = torch.zeros((K // 64, M, 64), dtype=torch.int8, device=dev)
            wq = torch.zeros((K // 64, N, 64), dtype=torch.int8, device=dev)
        else:
            xq = (torch.randn((K // 64, M, 64), device=dev, generator=g) * 28).round().clamp(-127, 127).to(torch.int8)
            wq = (torch.randn((K // 64, N, 64), device=dev, generator=g) * 28).round().clamp(-127, 127).to(torch.int8)
        run = lambda: ops.gemm_i8_fused(xq, sx, wq, sw, None, _lib.EPILOGUE_NONE, out=y, layout=_lib.LAYOUT_KB64)
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            run()
        e1.record()
        torch.cuda.synchronize()
        gemm[name] = round(2.0 * M * N * K * 10 / (e0.elapsed_time(e1) * 1e-3) / 1e15, 3)
        del xq, wq
    res["gemm_i8_kernel_same_shape_different_data"] = gemm

    # how much vector work fits under another wavefront's MFMAs on the same SIMD: one 8-wavefront
    # workgroup per CU, wavefronts 0-3 only MFMAs, wavefronts 4-7 only vector instructions, sized so
    # that either side alone takes the same time; overlap = (alone_a + alone_b - both) / min(alone)
    def timed(kind, mfma_rounds, vector_rounds):
        launch = lambda: _lib.check(lib.samfast_bench_mfma_valu_overlap(
            kind, buf.data_ptr(), 256, mfma_rounds, vector_rounds, out.data_ptr(), stream), "bench_mfma_valu_overlap")
        launch()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            launch()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1))
        return best

    overlap = {"what": "256 workgroups of 8 wavefronts: wavefronts 0-3 v_mfma_f32_32x32x16_bf16 only, wavefronts 4-7 "
                       "(their SIMD partners) vector instructions only; ms alone, ms together, share of the shorter "
                       "side that ran under the other"}
    rounds = 20000
    # on all-zero MFMA operands the matrix pipe draws little power, so the clock does not fall when
    # the vector side joins: that pair isolates the issue limit from the power limit
    for data in ("zeros", "random_normal"):
        buf = operands[1][data]
        t_mfma = timed(0, rounds, 0)
        for kind, name in ((0, "v_fma_f32"), (1, "v_exp_f32_then_v_mul_f32")):
            probe = timed(kind, 0, 2000)
            vr = max(1, int(2000 * t_mfma / probe))
            t_vec = timed(kind, 0, vr)
            t_both = timed(kind, rounds, vr)
            overlap[f"{name}_mfma_operands_{data}"] = {
                "mfma_alone_ms": round(t_mfma, 3), "vector_alone_ms": round(t_vec, 3), "together_ms": round(t_both, 3),
                "overlap": round((t_mfma + t_vec - t_both) / min(t_mfma, t_vec), 3)}
    res["mfma_and_vector_wavefronts_on_one_simd"] = overlap
    return res


def gemm_variants(batch=16, width=1280):
    """The four Linears of a ViT-H block at batch * 4096 rows (K-block major operands, the epilogue the
    encoder uses) under each variant of the int8 GEMM kernel, ten launches back to back after three
    warm-up launches, events on the launch stream; on all-zero codes (no operand toggling: the clock
    stays up, what is left is the kernel's structure) and on Gaussian codes like the encoder's."""
    import torch
    from samfast_amd import _lib, ops
    dev = torch.device("cuda:0")
    M = batch * 4096
    g = torch.Generator(device="cuda").manual_seed(11)
    variants = [("three_workgroups_per_cu", {"SAMFAST_GEMM_PERSIST": 0}),
                ("two_workgroups_per_cu", {"SAMFAST_GEMM_PERSIST": 0, "SAMFAST_GEMM_WG3": 0}),
                ("persistent, all workgroups start together", {"SAMFAST_GEMM_PERSIST": 2, "SAMFAST_GEMM_PERSIST_SKEW": 0}),
                ("persistent, every second workgroup starts a tile late", {"SAMFAST_GEMM_PERSIST": 2}),
                ("persistent, skewed, no wave priorities", {"SAMFAST_GEMM_PERSIST": 2, "SAMFAST_GEMM_PERSIST_PRIO": 0})]
    shapes = [("qkv", 3 * width, width, _lib.EPILOGUE_NONE), ("proj", width, width, _lib.EPILOGUE_RESIDUAL),
              ("lin1", 4 * width, width, _lib.EPILOGUE_GELU), ("lin2", width, 4 * width, _lib.EPILOGUE_RESIDUAL)]
    res = {"what": f"gemm_i8 at M={M}, us per launch (10 back to back) and TOP/s, per variant knob, on "
                   "all-zero / Gaussian int8 codes", "rows": {}}
    for name, N, K, epi in shapes:
        sx = torch.full((M,), 0.01, device=dev)
        sw = torch.full((N,), 0.001, device=dev)
        bias = torch.zeros((N,), device=dev)
        y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        resid = torch.randn((M, N), device=dev, generator=g).to(torch.bfloat16) if epi == _lib.EPILOGUE_RESIDUAL else None
        row = {}
        for data in ("zeros", "gaussian"):
            if data == "zeros":
                xq = torch.zeros((K // 64, M, 64), dtype=torch.int8, device=dev)
                wq = torch.zeros((K // 64, N, 64), dtype=torch.int8, device=dev)
            else:
                xq = (torch.randn((K // 64, M, 64), device=dev, generator=g) * 28).round().clamp(-127, 127).to(torch.int8)
                wq = (torch.randn((K // 64, N, 64), device=dev, generator=g) * 28).round().clamp(-127, 127).to(torch.int8)
            run = lambda: ops.gemm_i8_fused(xq, sx, wq, sw, bias, epi, residual=resid, out=y, layout=_lib.LAYOUT_KB64)
            for label, knobs in variants:
                with _lib.knobs(**knobs):
                    for _ in range(3):
                        run()
                    torch.cuda.synchronize()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(10):
                        run()
                    e1.record()
                    torch.cuda.synchronize()
                us = e0.elapsed_time(e1) * 100.0
                row.setdefault(label, {})[data] = {"us": round(us, 1), "TOP/s": round(2.0 * M * N * K / us / 1e6, 1)}
            del xq, wq
        res["rows"][f"{name} {M}x{N}x{K}"] = row
        del y, resid
    # the 2:4-sparse kernel's two forms on the MLP shapes (weights pruned to 2:4, Gaussian codes)
    sparse_variants = [("one workgroup per tile", {"SAMFAST_SPARSE_PERSIST": 0}),
                       ("resident workgroups", {"SAMFAST_SPARSE_PERSIST": 2})]
    for name, N, K, epi in shapes[2:]:
        w = (torch.randn((N, K), device=dev, generator=g) * 28).round().clamp(-127, 127)
        w4 = w.view(N, K // 4, 4)
        keep = torch.zeros_like(w4, dtype=torch.bool).scatter_(-1, w4.abs().topk(2, dim=-1).indices, True)
        wc, widx = ops.prune24_pack((w4 * keep).view(N, K).to(torch.int8))
        sx = torch.full((M,), 0.01, device=dev)
        sw = torch.full((N,), 0.001, device=dev)
        bias = torch.zeros((N,), device=dev)
        y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        resid = torch.randn((M, N), device=dev, generator=g).to(torch.bfloat16) if epi == _lib.EPILOGUE_RESIDUAL else None
        xq = (torch.randn((K // 64, M, 64), device=dev, generator=g) * 28).round().clamp(-127, 127).to(torch.int8)
        run = lambda: ops.gemm_i8_sparse24_fused(xq, sx, wc, widx, sw, bias, epi, residual=resid, out=y,
                                                 layout=_lib.LAYOUT_KB64)
        row = {}
        for label, knobs in sparse_variants:
            with _lib.knobs(**knobs):
                for _ in range(3):
                    run()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(10):
                    run()
                e1.record()
                torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 100.0
            row[label] = {"gaussian": {"us": round(us, 1), "TOP/s executed": round(1.0 * M * N * K / us / 1e6, 1)}}
        res["rows"][f"2:4 {name} {M}x{N}x{K}"] = row
        del y, resid, xq, wc, widx
    torch.cuda.empty_cache()
    return res


def config_1(cores):
    """The benchmark's operator configuration: ONE global rel-pos attention call at the ViT-B shape
    (B = 1, 12 heads, 64 x 64 = 4096 tokens, head_dim 64; q, k, v ~ N(0, 1), tables ~ N(0, 0.02), CPU
    generator seed 20).  bf16 on the HIP kernel (events around 20 calls) and the reference's CPU route -
    fp32 add_decomposed_rel_pos + F.scaled_dot_product_attention with the materialised bias
    (flash_4.py:368-370), restated in oracle/ - timed on the host cores; both on the same inputs, the
    kernel's output checked against the CPU result."""
    import torch
    from samfast_amd import ops
    from oracle import relpos_attention as ora
    B, nH, g, hd = 1, 12, 64, 64
    gen = torch.Generator().manual_seed(20)
    q, k, v = (torch.randn((B, nH, g * g, hd), generator=gen) for _ in range(3))
    rph = torch.randn((2 * g - 1, hd), generator=gen) * 0.02
    rpw = torch.randn((2 * g - 1, hd), generator=gen) * 0.02
    flop = 4.0 * B * nH * (g * g) ** 2 * hd
    dq, dk, dv, dh, dw = (t.to(torch.bfloat16).cuda() for t in (q, k, v, rph, rpw))
    run = lambda: ops.attn_relpos(dq, dk, dv, dh, dw, (g, g))
    for _ in range(3):
        out = run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        run()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / 20
    torch.set_num_threads(cores)
    b16 = lambda t: t.to(torch.bfloat16).float()  # the CPU route on the kernel's bf16-rounded inputs, in fp32
    cpu_in = (b16(q), b16(k), b16(v), b16(rph), b16(rpw))
    with torch.no_grad():
        ref = ora.attention_from_tables(*cpu_in, (g, g), use_sdpa=True)
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            ora.attention_from_tables(*cpu_in, (g, g), use_sdpa=True)
            times.append(time.perf_counter() - t0)
    cpu_s = sorted(times)[1]
    diff = (out.float().cpu() - ref).abs()
    return {"workload": "single global rel-pos attention op, B=1, 12 heads, 64x64 = 4096 tokens, head_dim 64",
            "flop": flop,
            "gpu_bf16": {"us_per_call": round(us, 1), "achieved": round(flop / us * 1e-6, 1), "peak": 2500.0,
                         "unit": "TFLOP/s", "frac": round(flop / (us * 1e-6) / 2.5e15, 4)},
            "cpu_fp32": {"ms_per_call": round(cpu_s * 1e3, 1), "achieved": round(flop / cpu_s * 1e-12, 3),
                         "unit": "TFLOP/s", "cores": cores, "kind": "port",
                         "sample": "the whole operator, median of 3 calls after 1 warm-up, fp32 SDPA with the "
                                   "materialised 4096 x 4096 bias per head"},
            "max_abs_diff_gpu_vs_cpu": round(diff.max().item(), 5), "mean_abs_diff_gpu_vs_cpu": round(diff.mean().item(), 6)}


def run_config(model, batch, steps, warmup, sparse_mlp=False, bf16_linears=False, graph=False,
               gpu_baseline=True, calibration_copy=False, yardsticks=False, also_graph=False,
               compiled_baseline=False):
    """Build the encoder, time `steps` forwards after `warmup`, run one instrumented forward for the
    per-kernel figures and (optionally) the PyTorch-ROCm eager baseline on the same weights."""
    import torch
    from samfast_amd import apply_dynamic_quant, apply_sparse, flash_4, ops
    from samfast_amd.sparse import mlp_only
    from samfast_amd.build_sam import build_image_encoder
    from samfast_amd.synthetic import init_encoder_weights, make_images
    dev = torch.device("cuda:0")

    enc = build_image_encoder(model)
    sd_fp32 = {k: v.clone() for k, v in init_encoder_weights(enc, seed=0).items()}
    enc = enc.eval().to(torch.bfloat16).to(dev)
    if sparse_mlp:
        apply_sparse(enc, mlp_only)
    if not bf16_linears:
        apply_dynamic_quant(enc)
    images = make_images(batch, seed=1).to(torch.bfloat16).to(dev)

    if calibration_copy:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    extra = {}
    with torch.no_grad():
        step = lambda: enc(images)
        if graph or also_graph:
            from samfast_amd.graphs import GraphedEncoder
            graphed = GraphedEncoder(enc, images)
        timed = (lambda: graphed(images)) if graph else step
        sec = time_steps(timed, steps, warmup)
        if also_graph and not graph:
            gsec = time_steps(lambda: graphed(images), steps, warmup)
            extra["hip_graph_replay"] = {"value": round(batch / gsec, 3), "unit": "images/s",
                                         "ms_per_step": round(gsec * 1e3, 3)}
            # the same model as a user of the drop-in API gets it: sam_model_fast_registry (compile_mode
            # 'max-autotune' = graph replay for launch-bound batches), Linears swapped on the returned model
            from samfast_amd import sam_model_fast_registry
            sam = sam_model_fast_registry[model]()
            sam.image_encoder._orig_mod.load_state_dict(sd_fp32)
            sam = sam.to(dev)
            if sparse_mlp:
                apply_sparse(sam.image_encoder, mlp_only)
            if not bf16_linears:
                apply_dynamic_quant(sam.image_encoder)
            rsec = time_steps(lambda: sam.image_encoder(images), steps, warmup)
            cos_r = torch.nn.functional.cosine_similarity(
                sam.image_encoder(images).float().flatten(1), step().float().flatten(1), dim=1).min().item()
            extra["fast_registry_replay"] = {
                "what": "sam_model_fast_registry[...]().image_encoder(images): HIP-graph replay behind the registry, "
                        "input copy and output clone included",
                "value": round(batch / rsec, 3), "unit": "images/s", "ms_per_step": round(rsec * 1e3, 3),
                "min_cosine_vs_eager": round(cos_r, 6)}  # (bit-equal up to the neck's MIOpen convolutions)
            del sam
        out = step()
        finite = bool(torch.isfinite(out.float()).all())

        # instrumented step: events around every hand-written kernel launch
        with ops.record_launches() as rec:
            step()
        summary = rec.summary()
        kernels = kernel_table(summary)
        extra["attention_combined"] = attention_combined(summary)

    # the dominant kernel: every epilogue variant of gemm_i8_kernel counts as one kernel
    fam = {}
    for name, d in summary.items():
        key = ("gemm_i8_sp24_kernel" if name.startswith("gemm_i8_sp24") else
               "gemm_i8_kernel" if name.startswith("gemm_i8") else name)
        f = fam.setdefault(key, dict(launches=0, work=0.0, unit=d["unit"], ms=0.0))
        f["launches"] += d["launches"]
        f["work"] += d["work"]
        f["ms"] += d["ms"]
    families = kernel_table(fam)
    dominant = max(families, key=lambda n: families[n]["ms_total"])
    dk = families[dominant]
    traffic, traffic_note = None, "not measured for this workload"
    if (model, batch, sparse_mlp, bf16_linears) == ("vit_h", 16, False, False) and dominant in TRAFFIC:
        value, src_name, sha = TRAFFIC[dominant]
        if source_sha16(src_name) == sha:
            traffic, traffic_note = value, f"rocprofv3 FETCH_SIZE / WRITE_SIZE runs summarised in {TRAFFIC_SOURCE}"
        else:
            traffic_note = (f"{src_name} changed since the counters in {TRAFFIC_SOURCE} were taken "
                            f"(then {value / 1e6:.0f} MB per launch)")
    roofline = {"kernel": dominant, "bound": dk["bound"], "achieved": dk["achieved"],
                "peak": dk["peak"], "unit": dk["unit"], "frac": dk["frac"],
                "traffic": traffic, "traffic_source": traffic_note,
                "avg_us": dk["avg_us"], "launches_per_step": dk["launches"],
                "ms_per_step": dk["ms_total"]}

    result = {
        "value": round(batch / sec, 3), "unit": "images/s", "ms_per_step": round(sec * 1e3, 3),
        "steps": steps, "warmup": warmup,
        "dtype": ("bf16" if bf16_linears and not sparse_mlp else
                  "bf16 attention + int8 linears (int32 accumulate)"
                  + (", lin1/lin2 2:4 sparse" if sparse_mlp else "")),
        "config": {"workload": f"SAM {model} image encoder forward, batch {batch}, "
                               "1024x1024, rel-pos attention + "
                               + ("bf16 linears" if bf16_linears and not sparse_mlp else "dynamic int8 linears")
                               + (" (lin1 / lin2 pruned 2:4, sparse int8 MFMA)" if sparse_mlp else ""),
                   "batch": batch, "image": 1024},
        "hip_graph": bool(graph),
        "output_finite": finite,
        "roofline": roofline,
        "kernels": kernels,
    }
    result.update(extra)

    if gpu_baseline:
        # same weights, PyTorch-ROCm eager: bf16 nn.Linear + SDPA with a materialised bias
        base = build_image_encoder(model)
        base.load_state_dict(sd_fp32)
        base = base.eval().to(torch.bfloat16).to(dev)
        if sparse_mlp:  # same pruned weights, dense bf16 kernels
            from samfast_amd import apply_fake_sparsity
            apply_fake_sparsity(base, mlp_only)
        flash_4.USE_CUSTOM_KERNEL = False
        try:
            with torch.no_grad():
                bsec = time_steps(lambda: base(images), 3, 1)
                ref = base(images)
            cos = torch.nn.functional.cosine_similarity(
                out.float().flatten(1), ref.float().flatten(1), dim=1).min().item()
            compiled = None
            if compiled_baseline:
                # the reference's "SDPA" configuration is this eager model under torch.compile
                # (build_sam.py:67-71); default mode: no autotuning, ~20 s of compilation
                try:
                    cbase = torch.compile(base)
                    with torch.no_grad():
                        csec = time_steps(lambda: cbase(images), 3, 2)
                    compiled = {"what": "the same model under torch.compile, mode='default' (no autotuning; the "
                                        "reference builds with mode='max-autotune', build_sam.py:70, which adds "
                                        "autotuned GEMM configurations and graph replay)",
                                "mode": "default",
                                "value": round(batch / csec, 3), "unit": "images/s",
                                "ms_per_step": round(csec * 1e3, 3), "speedup": round(csec / sec, 3)}
                    del cbase
                    try:  # the compiler's pool of worker processes must not outlive this script
                        from torch._inductor.async_compile import shutdown_compile_workers
                        shutdown_compile_workers()
                    except Exception:
                        pass
                except Exception as e:  # the baseline is optional: a compiler problem must not lose the line
                    compiled = {"what": "torch.compile failed", "error": f"{type(e).__name__}: {str(e)[:200]}"}
        finally:
            flash_4.USE_CUSTOM_KERNEL = True
        result["gpu_baseline"] = {"what": "same encoder, PyTorch-ROCm eager bf16 SDPA(attn_mask) + bf16 nn.Linear",
                                  "value": round(batch / bsec, 3), "unit": "images/s",
                                  "ms_per_step": round(bsec * 1e3, 3),
                                  "speedup": round(bsec / sec, 3),
                                  "min_cosine_vs_this_path": round(cos, 6)}
        if compiled is not None:
            result["gpu_baseline"]["torch_compile"] = compiled
        del base, ref

    if yardsticks:
        blk = enc.blocks[0].attn
        with torch.no_grad():
            result["library_yardsticks"] = library_yardsticks(
                batch, blk.num_heads, blk.qkv.in_features // blk.num_heads, blk.qkv.in_features)
    del enc, images, out
    torch.cuda.empty_cache()
    return result, sd_fp32


def brief(r):
    """What an other_configs entry keeps of a run_config result."""
    keep = {k: r[k] for k in ("value", "unit", "ms_per_step", "steps", "warmup", "dtype", "output_finite")}
    keep["workload"] = r["config"]["workload"]
    rf = r["roofline"]
    keep["dominant_kernel"] = {k: rf[k] for k in ("kernel", "bound", "achieved", "peak", "unit", "frac",
                                                   "avg_us", "launches_per_step", "ms_per_step")}
    keep["kernels"] = {n: {k: d[k] for k in ("launches", "ms_total", "achieved", "unit", "frac")}
                       for n, d in r["kernels"].items()}
    for k in ("gpu_baseline", "hip_graph_replay", "fast_registry_replay"):
        if k in r:
            keep[k] = r[k]
    return keep


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives exist on this path); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from samfast_amd.synthetic import make_images

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(torch.device("cuda:0"))

    if args.mfma_ceiling:
        print(json.dumps({"mfma_ceiling": mfma_ceiling()}))
        return
    if args.gemm_variants:
        print(json.dumps({"gemm_variants": gemm_variants()}))
        return

    main_run, sd_fp32 = run_config(
        args.model, args.batch, args.steps, args.warmup, sparse_mlp=args.sparse_mlp,
        bf16_linears=args.bf16_linears, graph=args.graph, gpu_baseline=not args.no_gpu_baseline,
        calibration_copy=args.calibration_copy, yardsticks=args.library_yardsticks,
        compiled_baseline=not args.no_gpu_baseline and not args.no_compiled_baseline, also_graph=args.also_graph)

    result = {
        "metric": ("images/s ViT-H encoder bs16 1024^2" if (args.model, args.batch) == ("vit_h", 16)
                   else f"images/s {args.model} encoder bs{args.batch} 1024^2")
        + (" (2:4 sparse MLP)" if args.sparse_mlp else ""),
        "value": main_run["value"], "unit": "images/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_run["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": main_run["dtype"],
        "data": "synthetic (seeded uniform images, random-init weights)",
        "config": main_run["config"],
    }
    for k in ("hip_graph", "output_finite", "roofline", "kernels", "attention_combined", "gpu_baseline",
              "library_yardsticks", "hip_graph_replay", "fast_registry_replay"):
        if k in main_run:
            result[k] = main_run[k]

    default_workload = (args.model, args.batch, args.sparse_mlp, args.bf16_linears, args.graph) == \
        ("vit_h", 16, False, False, False)
    if default_workload and not args.main_only:
        # the benchmark's two other encoder configurations, same protocol, fewer steps
        others = {}
        r, _ = run_config("vit_h", 32, max(3, args.steps // 2), 2, sparse_mlp=True,
                          gpu_baseline=not args.no_gpu_baseline)
        others["vit_h_bs32_int8_sparse24_mlp"] = brief(r)
        r, _ = run_config("vit_b", 1, max(20, args.steps), 5, gpu_baseline=not args.no_gpu_baseline,
                          also_graph=True)
        others["vit_b_bs1_int8"] = brief(r)
        result["other_configs"] = others

    if not args.no_mfma_ceiling:
        result["mfma_ceiling"] = mfma_ceiling()

    if not args.no_cpu_baseline:
        from oracle import image_encoder as oe
        cfg = {"vit_h": oe.VIT_H, "vit_l": oe.VIT_L, "vit_b": oe.VIT_B}[args.model]
        # the host share of a one-GPU box is 16 cores whatever os.cpu_count() shows there
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
        torch.set_num_threads(cores)
        if default_workload and not args.main_only:
            result["config_1"] = config_1(cores)
        n_cpu = 3 if args.model == "vit_h" else 6  # about 10-15 s of host work
        xs = make_images(n_cpu, seed=1)
        with torch.no_grad():
            t0 = time.perf_counter()
            for i in range(n_cpu):
                oe.encoder_forward(sd_fp32, xs[i:i + 1], cfg, use_sdpa=True)
            csec = (time.perf_counter() - t0) / n_cpu
        result["cpu_baseline"] = {"value": round(1.0 / csec, 4), "unit": "images/s", "cores": cores,
                                  "kind": "port",
                                  "sample": f"{n_cpu} images, one at a time, through the whole {args.model} encoder, "
                                            "fp32 eager (SDPA with materialised bias, fp32 Linear)"}

    print(json.dumps(result))


if __name__ == "__main__":
    main()
