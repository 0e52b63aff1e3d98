"""CPU-side checks of the product's host code: the C-ABI library loads and exports every symbol
the header declares; the host packers equal the oracle's; the registry and TernaryLinear host
logic behave like the reference's. No compute call is made (no GPU here)."""
import os
import re

import numpy as np
import pytest

import tritium_amd as T
from oracle_lib import FMT_TQ1_0, FMT_TQ2_0

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "tritium_mi355x.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    declared = set(re.findall(r"\b(tk_[a-z0-9_]+)\s*\(", hdr))
    assert len(declared) >= 40
    lib = T._lib.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(T._lib.SIGNATURES), declared ^ set(T._lib.SIGNATURES)


def test_packed_len():
    assert T.packed_len(6912, 2560, T.TernaryFormat.Tq2_0) == 4_561_920
    assert T.packed_len(8192, 2048, T.TernaryFormat.Tq2_0) == 4_325_376
    assert T.packed_len(1, 257, T.TernaryFormat.Tq1_0) == 108
    assert T.packed_len(3, 256, T.TernaryFormat.I2sInt8) == 0


@pytest.mark.parametrize("fmt,ofmt", [(T.TernaryFormat.Tq2_0, FMT_TQ2_0), (T.TernaryFormat.Tq1_0, FMT_TQ1_0)])
@pytest.mark.parametrize("n,k", [(1, 1), (3, 255), (2, 256), (5, 257), (2, 4096), (7, 300)])
def test_host_packers_equal_oracle(oracle, fmt, ofmt, n, k):
    rng = np.random.default_rng(n * 1000 + k)
    w = rng.integers(-1, 2, (n, k)).astype(np.int8)
    mine = T.pack_rows(w, n, k, fmt)
    assert (mine == oracle.pack_matrix(w, n, k, ofmt)).all()
    assert (T.unpack_rows(mine, n, k, fmt) == w).all()


def test_host_packer_goldens():
    for v, byte in ((0, 0x55), (1, 0xAA), (-1, 0x00)):
        p = T.pack_rows(np.full(256, v, np.int8), 1, 256, T.TernaryFormat.Tq2_0)
        assert (p[:64] == byte).all() and bytes(p[64:]) == b"\x00\x3c"
    for v, qs, qh in ((0, 0x80, 0x7F), (1, 0xFF, 0xFD), (-1, 0, 0)):
        p = T.pack_rows(np.full(256, v, np.int8), 1, 256, T.TernaryFormat.Tq1_0)
        assert (p[:48] == qs).all() and (p[48:52] == qh).all() and bytes(p[52:]) == b"\x00\x3c"


def test_host_packer_errors():
    with pytest.raises(T.ShapeMismatch) as e:
        T.pack_rows(np.zeros(255, np.int8), 1, 256)
    assert (e.value.expected, e.value.got) == (256, 255)
    with pytest.raises(T.InvalidInput):
        T.pack_rows(np.full(256, 2, np.int8), 1, 256)
    with pytest.raises(T.UnsupportedFormat):
        T.pack_rows(np.zeros(256, np.int8), 1, 256, T.TernaryFormat.I2sInt8)
    bad = np.full(66, 0x55, np.uint8)
    bad[3] = 0xFF
    with pytest.raises(T.Backend):
        T.unpack_rows(bad, 1, 256)
    with pytest.raises(T.ShapeMismatch):
        T.unpack_rows(np.zeros(65, np.uint8), 1, 256)


def test_registry_skips_failing_backend(capsys):
    """crates/tritium-runtime/src/lib.rs:148-166,250-299: a failing init is logged and skipped."""
    def boom():
        raise T.Backend("no device")

    class Dummy:
        def capabilities(self):
            return T.DeviceCaps("dummy", "dummy device")

    reg = T.Registry([T.BackendEntry("broken", boom), T.BackendEntry("dummy", Dummy)])
    assert len(reg) == 1 and reg.get("broken") is None and reg.get("dummy") is not None
    assert reg.enumerate()[0].backend == "dummy"
    assert "backend `broken` failed to initialise, skipping" in capsys.readouterr().err
    assert T.BACKENDS[0].name == "mi355x"


def test_weights_format_env(monkeypatch):
    from tritium_amd.linear import weights_format
    monkeypatch.delenv("TRITIUM_WEIGHTS", raising=False)
    assert weights_format() == T.TernaryFormat.Tq2_0
    monkeypatch.setenv("TRITIUM_WEIGHTS", "tq1")
    assert weights_format() == T.TernaryFormat.Tq1_0
    monkeypatch.setenv("TRITIUM_WEIGHTS", "tq3")
    with pytest.raises(T.InvalidInput):
        weights_format()


def test_gemm_shape():
    s = T.GemmShape(2, 3, 4)
    assert s.macs() == 24 and s.buffers_fit(8, 12, 6) and not s.buffers_fit(8, 12, 7)
