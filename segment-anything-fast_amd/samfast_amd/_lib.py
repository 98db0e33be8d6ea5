"""ctypes binding of libsamfast.so (the C ABI declared in include/samfast.h, plus the
measurement aids of include/samfast_bench.h).

The library is looked up next to this package (lib/libsamfast.so, built in-tree
by segment-anything-fast_amd/build.py).  There is no fallback: if it is missing
or a call fails, a RuntimeError carrying samfast_last_error() is raised.
"""

import ctypes
import os
from pathlib import Path

_LIB_PATH = Path(__file__).resolve().parent / "lib" / "libsamfast.so"
_lib = None

SAMFAST_BF16 = 0
SAMFAST_F16 = 1  # attention entry points only

_i32, _i64, _f32, _ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

_SIGNATURES = {
    "samfast_version": (_i32, []),
    "samfast_arch": (ctypes.c_char_p, []),
    "samfast_last_error": (ctypes.c_char_p, []),
    "samfast_attn_relpos_fwd": (
        _i32, [_ptr] * 6 + [_i32] * 5 + [_i64] * 12 + [_i32, _f32, _ptr]),
    "samfast_attn_relpos_windowed_fwd": (
        _i32, [_ptr] * 8 + [_i32] * 6 + [_i64] * 12 + [_i32, _f32, _ptr]),
    "samfast_attn_relpos_bias_fwd": (
        _i32, [_ptr] * 6 + [_i32] * 5 + [_i64] * 18 + [_i32, _f32, _ptr]),
    "samfast_quant_rowwise_i8": (_i32, [_ptr, _i64, _ptr, _ptr, _i64, _i32, _i32, _i32, _ptr]),
    "samfast_gemm_i8_i32": (_i32, [_ptr, _ptr, _ptr, _i64, _i32, _i32, _ptr]),
    "samfast_gemm_i8_scale_bias": (
        _i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _i32, _i32, _ptr]),
    "samfast_layernorm_quant_i8": (
        _i32, [_ptr, _i64, _ptr, _ptr, _f32, _ptr, _ptr, _ptr, _i64, _i32, _i32, _i32, _ptr]),
    "samfast_gemm_i8_fused": (
        _i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _i32, _i32, _i32,
               _ptr, _i64, _ptr, _i32, _ptr]),
    "samfast_gemm_i8_fused_quant": (
        _i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _i32, _i32, _i32,
               _ptr, _i64, _i32, _ptr, _ptr, _f32, _ptr, _ptr, _i32, _ptr, _ptr]),
    "samfast_gemm_i8_fused_quant_noalloc": (
        _i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _i32, _i32, _i32,
               _ptr, _i64, _i32, _ptr, _ptr, _f32, _ptr, _ptr, _i32, _ptr]),
    "samfast_prune24_pack_i8": (_i32, [_ptr, _ptr, _ptr, _i32, _i32, _ptr]),
    "samfast_gemm_i8_sparse24_i32": (_i32, [_ptr, _ptr, _ptr, _ptr, _i64, _i32, _i32, _ptr]),
    "samfast_gemm_i8_sparse24_fused": (
        _i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _i32, _i32, _i32,
               _ptr, _i64, _i32, _ptr]),
}

# include/samfast_bench.h: measurement and tuning aids, not part of the path's ABI
_BENCH_SIGNATURES = {
    "samfast_bench_set_knob": (_i32, [ctypes.c_char_p, _i32, _i32]),
    "samfast_bench_mfma_ceiling": (_i32, [_i32, _ptr, _i32, _i32, ctypes.POINTER(_i64), _ptr, _ptr]),
    "samfast_bench_mfma_valu_overlap": (_i32, [_i32, _ptr, _i32, _i32, _i32, _ptr, _ptr]),
}

EPILOGUE_NONE, EPILOGUE_GELU, EPILOGUE_RESIDUAL = 0, 1, 2
LAYOUT_ROWMAJOR, LAYOUT_KB64 = 0, 1

EXPORTED_SYMBOLS = tuple(_SIGNATURES)
BENCH_SYMBOLS = tuple(_BENCH_SIGNATURES)


def lib_path() -> Path:
    return Path(os.environ.get("SAMFAST_LIB", str(_LIB_PATH)))


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not path.exists():
            raise RuntimeError(
                f"samfast: {path} not found - build it with "
                "`python segment-anything-fast_amd/build.py` (there is no fallback path)")
        lib = ctypes.CDLL(str(path))
        for name, (restype, argtypes) in {**_SIGNATURES, **_BENCH_SIGNATURES}.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().samfast_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"samfast: {what} failed ({code}): {msg}")


class knobs:
    """Context manager that sets kernel-variant knobs (include/samfast_bench.h) for the calls inside
    it and puts them back to "not given" afterwards: `with knobs(SAMFAST_GEMM_WG3=0): ...`.  The
    library reads the environment variables of the same names once, at its first launch, so
    changing os.environ later has no effect; this is the way to switch variants inside a process."""

    def __init__(self, **values: int) -> None:
        self.values = values

    def __enter__(self):
        lib = load()
        for name, value in self.values.items():
            check(lib.samfast_bench_set_knob(name.encode(), int(value), 0), "bench_set_knob")
        return self

    def __exit__(self, *exc):
        lib = load()
        for name in self.values:
            check(lib.samfast_bench_set_knob(name.encode(), 0, 1), "bench_set_knob")
        return False
