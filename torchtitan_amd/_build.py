"""Build the gfx950 HIP library in-tree with hipcc (cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB = PKG / "libmxfp8_gfx950.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}",
    f"-I{CSRC}",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def build(verbose: bool = False, jobs: int = 8, defines: tuple[str, ...] = (), out: Path | None = None) -> Path:
    """Compile every csrc/*.hip and link libmxfp8_gfx950.so next to the package.

    `defines` / `out` build a variant for measurements instead (the timing ablations the kernel
    sources name, e.g. MX_ABL_NO_EPILOGUE): objects go to a directory of their own, the library
    to `out`, and the product library is left alone.  bench.py loads such a variant when the
    environment variable MXFP8_LIBRARY names it."""
    if bool(defines) != (out is not None):
        raise ValueError("a variant build needs both defines and an output path")
    objdir = PKG / "build" if out is None else Path(out).with_suffix(".objs")
    objdir.mkdir(parents=True, exist_ok=True)
    lib = LIB if out is None else Path(out)
    dflags = [f"-D{d}" for d in defines]

    def compile_one(src: Path) -> Path:
        obj = objdir / (src.stem + ".o")
        cmd = [HIPCC, *FLAGS, *dflags, "-c", str(src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stderr}")
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(lib), *map(str, objs)]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return lib


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--define", action="append", default=[], help="extra -D for a measurement variant (needs --out)")
    ap.add_argument("--out", default=None, help="path of the variant library")
    a = ap.parse_args()
    print(build(verbose=True, defines=tuple(a.define), out=Path(a.out) if a.out else None))
