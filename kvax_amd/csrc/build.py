"""Compile the HIP sources in this directory into ``kvax_amd/libkvax_amd.so`` for gfx950.

Usage: ``python -m kvax_amd.csrc.build`` (or ``build()`` from Python).  hipcc cross-compiles, so
no GPU is needed.  The library is built in-tree next to the Python package.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent
PKG = CSRC.parent
ROOT = PKG.parent
LIB = PKG / "libkvax_amd.so"
OBJ = CSRC / "build"

SOURCES = ["abi.cpp", "mask_builder.hip", "fa_tiles.hip", "fa_fwd.hip", "fa_bwd.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results go to ordinary vector registers (where the element-wise code reads them) also in
    # kernels that run one wavefront per SIMD and may use the accumulation registers as well
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]


def _compile(src: str, extra: list[str]) -> Path:
    OBJ.mkdir(exist_ok=True)
    out = OBJ / (src + ".o")
    cmd = [HIPCC, *FLAGS, *extra, "-x", "hip", "-c", str(CSRC / src), "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 target feature: harmless
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return out


def build(extra_flags: list[str] | None = None, jobs: int = 4, lib: Path | None = None) -> Path:
    """Compile and link; ``lib`` overrides the output path (used for experimental variants,
    loaded by pointing the KVAX_AMD_LIB environment variable at them)."""
    global LIB, OBJ
    if lib is not None:
        LIB = Path(lib).resolve()
        OBJ = LIB.parent / (LIB.stem + "_obj")
    extra = list(extra_flags or [])
    sources = [s for s in SOURCES if (CSRC / s).exists()]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra), sources))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    args = sys.argv[1:]
    out = None
    if args and args[0] == "-o":
        out, args = Path(args[1]), args[2:]
    print(build(args, lib=out))
