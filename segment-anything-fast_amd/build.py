"""Build libsamfast.so (HIP kernels + C ABI) in-tree for gfx950.

Usage: python segment-anything-fast_amd/build.py [--force]
hipcc cross-compiles without a GPU; the shared object lands next to the Python
package (samfast_amd/lib/libsamfast.so) so that it travels with the tree.
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
INCLUDE = HERE.parent / "include"
LIB_DIR = HERE / "samfast_amd" / "lib"
LIB_PATH = LIB_DIR / "libsamfast.so"
OBJ_DIR = HERE / "build"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    f"-I{INCLUDE}", f"-I{CSRC}",
]


def sources():
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = True, jobs: int = 4) -> Path:
    """Compile every .hip under csrc/ and link libsamfast.so.  Returns its path."""
    srcs = sources()
    deps = srcs + list(CSRC.glob("*.hpp")) + list(INCLUDE.glob("*.h"))
    if not force and LIB_PATH.exists():
        newest = max(p.stat().st_mtime for p in deps)
        if LIB_PATH.stat().st_mtime >= newest:
            return LIB_PATH
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(LIB_PATH)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv or True)
    print(path)
