"""Ahead-of-time build of libsqhip.so for gfx950 (hipcc; no JIT, no torch extension machinery)."""

from __future__ import annotations

import os
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libsqhip.so"
SOURCES = ["sq_api.hip", "sq_dequant.hip", "sq_small_generic.hip", "sq_gemv.hip", "sq_gemv_b16d8.hip",
           "sq_gemv_b12d4.hip", "sq_gemv_b10d4.hip", "sq_gemv_b8d4.hip", "sq_gemm.hip", "sq_gemm256.hip", "sq_stream.hip",
           "sq_q8.hip", "sq_neighbours.hip", "sq_segs.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False, extra_flags: tuple = ()) -> Path:
    """Compile every kernel translation unit and link libsqhip.so next to this file."""
    hipcc = _hipcc()
    objdir = CSRC / "build"
    objdir.mkdir(exist_ok=True)

    def one(src: str) -> Path:
        obj = objdir / (Path(src).stem + ".o")
        cmd = [hipcc, *FLAGS, *extra_flags, "-c", str(CSRC / src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip():
            print(err)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 4)) as ex:
        objs = list(ex.map(one, SOURCES))
    r = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
