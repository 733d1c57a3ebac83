"""Writes tests/golden/ref_pcg64.json and tests/golden/ref_sgemm.npz.

The values come from oracle/_ref/libaxiom_ref.so, i.e. from the reference's own
PCG64 generator (include/axiom/random.hpp) and native BLAS tier
(src/backends/cpu/blas/blas_native.cpp) compiled from its sources.  That
library exists only where the reference tree is present; the fixtures it
produces are plain data and are what tests/test_oracle.py checks the C
restatement against everywhere else.

    python tests/golden/make_ref_fixtures.py
"""
import ctypes as C
import json
import pathlib
import sys

import numpy as np

HERE = pathlib.Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))
from oracle import axo  # noqa: E402

PCG_CASES = [(42, 1), (0, 1), (123456789, 7), (2**63 + 5, 3)]
# (M, N, K, transA, transB, alpha, beta): sizes on both sides of the 64x64x256 tile edges
SGEMM_CASES = [(7, 5, 9, 0, 0, 1.0, 0.0), (64, 64, 64, 0, 1, 0.125, 0.0), (37, 64, 37, 0, 0, 1.0, 1.0), (70, 130, 300, 1, 0, 0.5, 0.75),
               (3, 129, 513, 1, 1, 2.0, 0.0), (5, 4, 3, 0, 0, 0.0, 0.5), (65, 65, 257, 0, 1, 1.0, 0.0)]


def sgemm_inputs(case):
    M, N, K, tA, tB, _, _ = case
    r = np.random.default_rng(1000 * M + 10 * N + K)
    A = r.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
    B = r.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
    C0 = r.standard_normal((M, N)).astype(np.float32)
    return A, B, C0


def main():
    ref = axo.ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libaxiom_ref.so is missing: build it with `make -C oracle ref` where the reference tree exists")
    pcg = []
    for seed, stream in PCG_CASES:
        out = np.empty(32, np.uint64)
        ref.axref_pcg64(C.c_uint64(seed), C.c_uint64(stream), out.ctypes.data_as(C.c_void_p), out.size)
        pcg.append({"seed": seed, "stream": stream, "values": [int(v) for v in out]})
    out = np.empty(8, np.uint64)
    ref.axref_pcg64_default(out.ctypes.data_as(C.c_void_p), out.size)
    (HERE / "ref_pcg64.json").write_text(json.dumps({"cases": pcg, "default_constructed": [int(v) for v in out]}, indent=1) + "\n")

    arrays = {"cases": np.array(SGEMM_CASES, np.float64)}
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    for i, case in enumerate(SGEMM_CASES):
        M, N, K, tA, tB, alpha, beta = case
        A, B, C0 = sgemm_inputs(case)
        got = C0.copy()
        ref.axref_sgemm(tA, tB, M, N, K, alpha, p(A), A.shape[1], p(B), B.shape[1], beta, p(got), N)
        arrays[f"out{i}"] = got
    np.savez_compressed(HERE / "ref_sgemm.npz", **arrays)
    print("wrote", HERE / "ref_pcg64.json", HERE / "ref_sgemm.npz")


if __name__ == "__main__":
    main()
