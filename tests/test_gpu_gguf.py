"""A GGUF checkpoint's ternary tensors onto the device: each tensor uploaded from the file gives the
bits of the same trits and row scales through the oracle's CPU backend, for the three tensor types
the model loader accepts (crates/tritium-nn/src/model/weights.rs:177-333)."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import same_bits, ternary
from oracle_lib import FMT_TQ1_0, FMT_TQ2_0
from test_oracle_gguf import I2S, TQ1, TQ2, Builder, f16_bits, oracle_load
from test_oracle_i2s import i2s_payload

pytestmark = pytest.mark.gpu


def checkpoint(oracle, rng):
    """Three weight tensors in one file: I2_S, TQ2_0 with one scale per row, TQ1_0 with one scale and
    its exact f32 value in metadata."""
    tensors, data = {}, b""

    def add(name, dims, ty, payload):
        nonlocal data
        data += bytes(-len(data) % 32)
        tensors[name] = (dims, ty, len(data))
        data += payload

    w = ternary(rng, 48, 2560)
    add("blk.0.attn_q.weight", [2560, 48], I2S, i2s_payload(w, 1.2188548, pad=28).tobytes())
    rows = b""
    for r in range(33):
        rc, packed = oracle.pack_row(ternary(rng, 1, 512).reshape(-1), FMT_TQ2_0,
                                     np.full(2, f16_bits(0.25 * (r % 5 + 1)), np.uint16))
        rows += packed.tobytes()
    add("output.weight", [512, 33], TQ2, rows)
    rows = b""
    for r in range(20):
        rc, packed = oracle.pack_row(ternary(rng, 1, 768).reshape(-1), FMT_TQ1_0, np.full(3, f16_bits(0.0371), np.uint16))
        rows += packed.tobytes()
    add("blk.0.ffn_down.weight", [768, 20], TQ1, rows)
    b = Builder(3).meta_string("general.architecture", "bitnet")
    b.meta_f32("tritium.i2s_scale.blk.0.ffn_down.weight", np.float32(np.float16(0.0371)) + np.float32(2e-6))
    for name, (dims, ty, off) in tensors.items():
        b.tensor(name, dims, ty, off)
    return b.build(32, data), list(tensors)


def test_upload_from_gguf_matches_the_cpu_backend(backend, oracle):
    rng = np.random.default_rng(11)
    blob, names = checkpoint(oracle, rng)
    g = T.read_gguf(blob)
    raw = np.frombuffer(blob, np.uint8)
    for name in names:
        print("case gguf-upload", name, flush=True)
        want_trits, want_scales = oracle_load(oracle, blob, name)
        n, k = want_trits.shape
        buf, scales = backend.upload_weights_gguf(g, raw, name)
        assert scales.tobytes() == want_scales.tobytes() and (buf.download_trits() == want_trits).all()
        fmt = T.TernaryFormat(buf.format)
        m = 5
        act = rng.standard_normal((m, k)).astype(np.float32)
        out = np.zeros((m, n), np.float32)
        backend.mpgemm_with_act_quant(T.MpGemm(act, buf, scales, T.GemmShape(m, n, k), fmt, out))
        rc, want = oracle.cpu_mpgemm_with_act_quant(oracle.pack_matrix(want_trits, n, k, FMT_TQ2_0), FMT_TQ2_0, act,
                                                    want_scales, m, n, k)
        assert rc == 0 and same_bits(out, want)
        buf.free()
    assert len({s for s in backend.upload_weights_gguf(g, raw, "output.weight")[1]}) == 5  # rows kept their own scales


def test_upload_from_gguf_errors(backend, oracle):
    blob, _ = checkpoint(oracle, np.random.default_rng(12))
    g = T.read_gguf(blob)
    raw = np.frombuffer(blob, np.uint8)
    with pytest.raises(T.InvalidInput):
        backend.upload_weights_gguf(g, raw, "absent")
    with pytest.raises(T.InvalidInput):   # the file cut inside the tensor's payload
        backend.upload_weights_gguf(g, raw[:g.tensor_data_offset + 100], "blk.0.attn_q.weight")
