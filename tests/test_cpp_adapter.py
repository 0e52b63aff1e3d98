"""The C++ host adapter (tritium_amd/csrc/tritium_backend.hpp) driven through its TernaryBackend
interface by tests/cpp/conformance_runner (built beforehand by tests/cpp/Makefile / build())."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
RUNNER = os.path.join(HERE, "cpp", "conformance_runner")


def _run(*args):
    if not os.path.exists(RUNNER):
        pytest.fail("tests/cpp/conformance_runner is not built; run `make -C tests/cpp` (or __graft_entry__.build())")
    return subprocess.run([RUNNER, *args], capture_output=True, text=True, timeout=170)


def test_registry_skips_missing_device_host_side():
    r = _run("--nogpu")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "OK" in r.stdout


@pytest.mark.gpu
def test_cpp_adapter_conformance():
    r = _run()
    print(r.stdout[-2000:], flush=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "89/89 vectors passed" in r.stdout and r.stdout.strip().endswith("OK")
