"""Builds libaxhip.so (the C-ABI gfx950 backend) with hipcc, in-tree.

    python -m axiom_amd.build            # compile every source, link
    python -m axiom_amd.build --host     # also build the C++ host layer and its test programs

Each .hip file is compiled to an object in parallel, then linked into
axiom_amd/lib/libaxhip.so.  hipcc cross-compiles for gfx950 without a GPU.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
import time
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
OBJ_DIR = PKG / "build"
LIB = LIB_DIR / "libaxhip.so"

ARCH = "gfx950"
# packed-fp32 VALU forms are disabled for every device translation unit
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{ROOT / 'include'}", f"-I{CSRC}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found: the gfx950 backend cannot be built")
    return exe


def _run(cmd: list[str], what: str) -> float:
    t0 = time.time()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"{what} failed:\n{' '.join(cmd)}\n{out}")
    if out.strip():
        print(out)
    return time.time() - t0


def build_library(verbose: bool = True, jobs: int | None = None) -> Path:
    hipcc = _hipcc()
    LIB_DIR.mkdir(exist_ok=True)
    OBJ_DIR.mkdir(exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    jobs = jobs or min(len(sources), os.cpu_count() or 4, 8)

    def compile_one(src: Path) -> tuple[str, float]:
        obj = OBJ_DIR / (src.stem + ".o")
        dt = _run([hipcc, *HIP_FLAGS, "-c", str(src), "-o", str(obj)], f"compile {src.name}")
        return src.name, dt

    with cf.ThreadPoolExecutor(max_workers=jobs) as pool:
        for name, dt in pool.map(compile_one, sources):
            if verbose:
                print(f"[axiom_amd.build] {name}: {dt:.1f}s", flush=True)
    objs = [str(OBJ_DIR / (s.stem + ".o")) for s in sources]
    dt = _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objs, "-o", str(LIB)], "link libaxhip.so")
    if verbose:
        print(f"[axiom_amd.build] linked {LIB} ({dt:.1f}s)", flush=True)
    return LIB


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--host", action="store_true", help="also build the C++ host layer")
    args = ap.parse_args(argv)
    build_library()
    if args.host:
        from . import build_host  # noqa: WPS433 (optional second stage)

        build_host.build_all()
    return 0


if __name__ == "__main__":
    sys.exit(main())
