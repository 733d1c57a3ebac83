"""Builds the C++ host layer (axiom_amd/host) and its test programs with g++.

    libaxiom_hip.so     Axiom's Tensor / ops / lazy graph / nn interface for the hot path,
                        over the C ABI of libaxhip.so (no CPU compute, no fallback)
    host_bench          times BASELINE's configurations along the whole host-layer path
    host_tests          test program; links the host layer and, as the checker only, the
                        CPU oracle (oracle/libaxiom_oracle.so)
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import shutil
import subprocess
import time
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
HOST = PKG / "host"
LIB_DIR = PKG / "lib"
OBJ_DIR = PKG / "build" / "host"
HOST_LIB = LIB_DIR / "libaxiom_hip.so"
TEST_BIN = LIB_DIR / "host_tests"
BENCH_BIN = LIB_DIR / "host_bench"

CXXFLAGS = ["-O2", "-g", "-std=c++20", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter",
            f"-I{HOST / 'include'}", f"-I{HOST / 'src'}", f"-I{ROOT / 'include'}"]


def _run(cmd, what):
    t0 = time.time()
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if p.returncode != 0:
        raise RuntimeError(f"{what} failed:\n{' '.join(map(str, cmd))}\n{p.stdout}")
    if p.stdout.strip():
        print(p.stdout)
    return time.time() - t0


def _compile_all(sources, tag, extra=()):
    cxx = shutil.which("g++") or "g++"
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    objs = []

    def one(src: Path):
        obj = OBJ_DIR / f"{tag}_{src.stem}.o"
        _run([cxx, *CXXFLAGS, *extra, "-c", str(src), "-o", str(obj)], f"compile {src.name}")
        return obj

    with cf.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 4)) as pool:
        objs = list(pool.map(one, sources))
    return objs


def build_all(verbose: bool = True) -> None:
    cxx = shutil.which("g++") or "g++"
    LIB_DIR.mkdir(exist_ok=True)
    t0 = time.time()
    objs = _compile_all(sorted((HOST / "src").glob("*.cpp")), "lib")
    _run([cxx, "-shared", "-o", str(HOST_LIB), *map(str, objs), f"-L{LIB_DIR}", "-laxhip", "-Wl,-rpath,$ORIGIN"], "link libaxiom_hip.so")
    tests = sorted((HOST / "tests").glob("*.cpp"))
    if tests:
        tobjs = _compile_all(tests, "test", extra=(f"-I{ROOT / 'oracle'}",))
        oracle_dir = ROOT / "oracle"
        _run([cxx, "-o", str(TEST_BIN), *map(str, tobjs), f"-L{LIB_DIR}", "-laxiom_hip", "-laxhip", f"-L{oracle_dir}", "-laxiom_oracle",
              "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,$ORIGIN/../../oracle", "-lpthread"], "link host_tests")
    bench = HOST / "bench" / "host_bench.cpp"
    if bench.exists():
        _run([cxx, *CXXFLAGS, str(bench), "-o", str(BENCH_BIN), f"-L{LIB_DIR}", "-laxiom_hip", "-laxhip", "-Wl,-rpath,$ORIGIN"], "build host_bench")
    for example in sorted((HOST / "examples").glob("*.cpp")):
        _run([cxx, *CXXFLAGS, str(example), "-o", str(LIB_DIR / example.stem), f"-L{LIB_DIR}", "-laxiom_hip", "-laxhip", "-Wl,-rpath,$ORIGIN"],
             f"build {example.stem}")
    if verbose:
        print(f"[axiom_amd.build_host] built {HOST_LIB.name}" + (f" and {TEST_BIN.name}" if tests else "") + f" ({time.time() - t0:.1f}s)", flush=True)


if __name__ == "__main__":
    build_all()
