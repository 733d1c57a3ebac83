"""Runs the C++ test program of the host layer (axiom_amd/host/tests): the cases that
mirror the reference's GoogleTest files.  Device-free cases run everywhere; GPU cases
go through libaxiom_hip.so -> libaxhip.so on the card and take their expected values
from the oracle linked into the test program only."""
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
LIB = ROOT / "axiom_amd" / "lib"
BIN = LIB / "host_tests"


def _ensure_built():
    if not BIN.exists():  # normally built beforehand by __graft_entry__.build()
        from axiom_amd import build_host
        from oracle import axo

        axo.build()
        build_host.build_all()


def _run(*args, timeout=600, env=None):
    _ensure_built()
    p = subprocess.run([str(BIN), *args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout, env=env)
    print(p.stdout[-6000:])
    return p


def test_host_cases_without_device():
    p = _run("--cpu")
    assert p.returncode == 0, p.stdout[-3000:]
    assert " 0 failed" in p.stdout


def test_safetensors_reader_on_a_file_from_the_python_package(tmp_path):
    """The C++ reader against the format's own implementation: every dtype the weights of a
    model can have, a 0-d tensor, and the package's metadata block."""
    import os

    import numpy as np
    import torch
    from safetensors.torch import save_file

    ramp = torch.arange(15, dtype=torch.float32).reshape(3, 5)
    tensors = {"ramp_f32": ramp, "ramp_f16": ramp.half(), "ramp_bf16": ramp.bfloat16(), "ramp_i64": ramp.long(), "ramp_i32": ramp.int(),
               "ramp_u8": ramp.to(torch.uint8), "mask": torch.tensor([False, True, False]), "scalar": torch.tensor(2.5)}
    path = tmp_path / "from_python.safetensors"
    save_file(tensors, str(path), metadata={"format": "pt", "note": "written by safetensors"})
    assert np.frombuffer(path.read_bytes()[:8], np.uint64)[0] > 0
    p = _run("--cpu", "SafeTensors", env={**os.environ, "AXIOM_TEST_SAFETENSORS": str(path)})
    assert p.returncode == 0, p.stdout[-3000:]
    assert " 0 failed" in p.stdout and " 0 skipped" in p.stdout


def test_host_cases_without_device_under_address_and_undefined_behaviour_sanitizers():
    """The host layer built once more with -fsanitize=address,undefined (python -m axiom_amd.build_host --sanitize;
    built here when it is missing) passes its device-free cases with no report from either sanitizer."""
    from axiom_amd import build_host
    from oracle import axo

    _ensure_built()
    axo.build()
    p = build_host.run_sanitized_cpu_tests()
    print(p.stdout[-6000:])
    assert p.returncode == 0, p.stdout[-3000:]
    assert " 0 failed" in p.stdout
    assert "AddressSanitizer" not in p.stdout and "runtime error:" not in p.stdout


def test_product_libraries_do_not_link_the_oracle():
    _ensure_built()
    for lib in ("libaxhip.so", "libaxiom_hip.so"):
        out = subprocess.run(["readelf", "-d", str(LIB / lib)], stdout=subprocess.PIPE, text=True, check=True).stdout
        needed = [l for l in out.splitlines() if "NEEDED" in l]
        assert not any("oracle" in l for l in needed), needed
    out = subprocess.run(["readelf", "-d", str(LIB / "libaxiom_hip.so")], stdout=subprocess.PIPE, text=True, check=True).stdout
    assert "libaxhip.so" in out  # the host layer sits on the C ABI


@pytest.mark.gpu
def test_host_cases_on_gpu():
    p = _run("--gpu")
    assert p.returncode == 0, p.stdout[-6000:]
    assert " 0 failed" in p.stdout and " 0 skipped" in p.stdout
