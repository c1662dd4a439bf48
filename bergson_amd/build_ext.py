"""Builds libbergson_amd.so (the C-ABI library of HIP kernels) in-tree for gfx950.

    python -m bergson_amd.build_ext [--force]

hipcc cross-compiles without a GPU; the built library sits next to the sources
so that it travels with the tree.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
LIB = PKG / "libbergson_amd.so"
SOURCES = ["capi.hip", "collect.hip", "scan.hip", "adam.hip", "fullgrad.hip", "precond.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed fp32 VALU ops are kept off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unknown-warning-option",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


# sources whose compiled code is inspected before linking (see isa_checks.py)
INSPECTED = ("scan.hip", "adam.hip")


def _compile(src: str, verbose: bool, temps: Path | None = None) -> Path:
    """Compiles one source.  With `temps`, the compiler's intermediate files -- among them the device
    assembly the object was assembled from -- are kept in that directory next to a copy of the object."""
    obj = CSRC / (Path(src).stem + ".o")
    cmd = [HIPCC, *FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    if temps is not None:
        cmd = [HIPCC, *FLAGS, "-save-temps=obj", "-c", str(CSRC / src), "-o", str(temps / obj.name)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError(f"hipcc failed on {src}")
    if verbose and res.stderr.strip():
        # the host pass reports that it does not know the packed-fp32 feature: harmless
        lines = [l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l]
        if lines:
            sys.stderr.write("\n".join(lines) + "\n")
    if temps is not None:
        shutil.copyfile(temps / obj.name, obj)
    return obj


def device_assembly(temps: Path, src: str) -> str:
    found = sorted(temps.glob(f"{Path(src).stem}-hip-amdgcn-amd-amdhsa-gfx950*.s"))
    if not found:
        raise RuntimeError(f"no device assembly for {src} in {temps}")
    return found[0].read_text()


def build(verbose: bool = True) -> Path:
    """Compile every HIP source, check the compiled code of the hand-scheduled kernels, and link the shared
    library.  Always rebuilds; raises without linking when a kernel breaks one of the rules of isa_checks."""
    from . import isa_checks

    temps = Path(tempfile.mkdtemp(prefix="bgx_build_"))
    try:
        with ThreadPoolExecutor(max_workers=min(6, len(SOURCES))) as ex:
            objs = list(ex.map(lambda s: _compile(s, verbose, temps if s in INSPECTED else None), SOURCES))
        bad = isa_checks.all_violations({src: device_assembly(temps, src) for src in INSPECTED})
    finally:
        shutil.rmtree(temps, ignore_errors=True)
    if bad:
        LIB.unlink(missing_ok=True)
        raise RuntimeError("compiled kernels break the scheduling rules they rely on:\n  " + "\n  ".join(bad))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *map(str, objs), "-o", str(LIB)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc link failed")
    return LIB


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("-q", "--quiet", action="store_true")
    args = ap.parse_args()
    lib = build(verbose=not args.quiet)
    print(f"built {lib} ({lib.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
