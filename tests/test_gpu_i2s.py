"""I2_S ingest on the device path: a tensor uploaded from its I2_S payload gives the bits of the same
trits uploaded as TQ2_0, with the per-tensor scale broadcast over the output channels
(crates/tritium-format/src/i2s_int8.rs:36-68)."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import same_bits, ternary
from oracle_lib import FMT_TQ2_0
from test_oracle_i2s import i2s_payload

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,k", [(48, 2560), (33, 640), (2, 192)])
def test_i2s_upload_equals_tq2_upload(backend, oracle, n, k):
    print("case i2s-upload", n, k, flush=True)
    rng = np.random.default_rng(n + k)
    w = ternary(rng, n, k)
    payload = i2s_payload(w, 1.2188548, pad=28)
    buf, scale = backend.upload_weights_i2s(payload, T.GemmShape(0, n, k))
    assert scale == np.float32(1.2188548)
    m = 3
    act = rng.standard_normal((m, k)).astype(np.float32)
    scales = np.full(n, scale, np.float32)
    out = np.zeros((m, n), np.float32)
    backend.mpgemm_with_act_quant(T.MpGemm(act, buf, scales, T.GemmShape(m, n, k), T.TernaryFormat.Tq2_0, out))
    rc, want = oracle.cpu_mpgemm_with_act_quant(oracle.pack_matrix(w, n, k, FMT_TQ2_0), FMT_TQ2_0, act, scales, m, n, k)
    assert rc == 0 and same_bits(out, want)
    assert (buf.download_trits() == w).all()
    buf.free()


def test_i2s_upload_errors(backend):
    with pytest.raises(T.InvalidInput):  # reserved code
        bad = i2s_payload(np.zeros(128, np.int8), 1.0)
        bad[0] = 0xFF
        backend.upload_weights_i2s(bad, T.GemmShape(0, 1, 128))
    with pytest.raises(T.ShapeMismatch):  # payload without its scale
        backend.upload_weights_i2s(np.zeros(32, np.uint8), T.GemmShape(0, 1, 128))
