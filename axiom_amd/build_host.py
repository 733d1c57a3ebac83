"""Builds the C++ host layer (axiom_amd/host) and its test programs with g++.

    libaxiom_hip.so     Axiom's Tensor / ops / lazy graph / nn interface for the hot path,
                        over the C ABI of libaxhip.so (no CPU compute, no fallback)
    host_bench          times BASELINE's configurations along the whole host-layer path
    host_tests          test program; links the host layer and, as the checker only, the
                        CPU oracle (oracle/libaxiom_oracle.so)

    python -m axiom_amd.build_host              the above, into axiom_amd/lib/
    python -m axiom_amd.build_host --sanitize   the host layer and host_tests once more with AddressSanitizer and
                                                UndefinedBehaviorSanitizer (host code only: the HIP library underneath
                                                is the ordinary one), into axiom_amd/lib/sanitize/; run its CPU cases
                                                with run_sanitized_cpu_tests()
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


def _compile_all(sources, tag, extra=(), flags=None):
    cxx = shutil.which("g++") or "g++"
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    objs = []

    def one(src: Path):
        obj = OBJ_DIR / f"{tag}_{src.stem}.o"
        _run([cxx, *(CXXFLAGS if flags is None else flags), *extra, "-c", str(src), "-o", str(obj)], f"compile {src.name}")
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


SANITIZE_DIR = LIB_DIR / "sanitize"
SANITIZE_FLAGS = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"]


def build_sanitized(verbose: bool = True) -> Path:
    """The host layer and its test program with -fsanitize=address,undefined (g++, host code), beside the ordinary
    build.  Returns the test program's path."""
    cxx = shutil.which("g++") or "g++"
    SANITIZE_DIR.mkdir(parents=True, exist_ok=True)
    t0 = time.time()
    flags = ["-O1" if f == "-O2" else f for f in CXXFLAGS] + SANITIZE_FLAGS
    objs = _compile_all(sorted((HOST / "src").glob("*.cpp")), "san_lib", flags=flags)
    lib = SANITIZE_DIR / "libaxiom_hip.so"
    _run([cxx, "-shared", *SANITIZE_FLAGS, "-o", str(lib), *map(str, objs), f"-L{LIB_DIR}", "-laxhip", "-Wl,-rpath,$ORIGIN/.."], "link sanitized libaxiom_hip.so")
    tobjs = _compile_all(sorted((HOST / "tests").glob("*.cpp")), "san_test", extra=(f"-I{ROOT / 'oracle'}",), flags=flags)
    exe = SANITIZE_DIR / "host_tests"
    _run([cxx, *SANITIZE_FLAGS, "-o", str(exe), *map(str, tobjs), f"-L{SANITIZE_DIR}", "-laxiom_hip", f"-L{LIB_DIR}", "-laxhip", f"-L{ROOT / 'oracle'}",
          "-laxiom_oracle", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath,$ORIGIN/../../../oracle", "-lpthread"], "link sanitized host_tests")
    if verbose:
        print(f"[axiom_amd.build_host] built {exe.relative_to(ROOT)} ({time.time() - t0:.1f}s)", flush=True)
    return exe


def run_sanitized_cpu_tests(timeout: float = 600.0) -> subprocess.CompletedProcess:
    """Runs the sanitized test program's CPU cases (`host_tests --cpu`), building it first when it is missing.
    Leak detection is off: the HIP runtime the library links keeps its own allocations until exit."""
    exe = SANITIZE_DIR / "host_tests"
    if not exe.exists():
        build_sanitized(verbose=False)
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:abort_on_error=0"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    return subprocess.run([str(exe), "--cpu"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout, env=env)


if __name__ == "__main__":
    import sys

    if "--sanitize" in sys.argv[1:]:
        build_sanitized()
    else:
        build_all()
