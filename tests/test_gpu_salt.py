"""Block-scale additive planes (SALT) through the device-resident C ABI.

The host definition (dequantize the row, planes in order; then one f32 accumulator over k:
crates/tritium-format/src/salt.rs:720-738, crates/tritium-nn/src/layers/packed_salt.rs:585-628) is the
oracle. The reference-order kernel must reproduce it bit for bit; the matrix-core form is held to the
bound the reference sets for its own GPU kernel, 1e-4 (crates/tritium-cuda/kernels/tq2_0_add.cu:651-655)."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, bf16_bits_to_f32, f32_to_bf16_bits, rel_err, same_bits, ternary
from test_oracle_salt import f16_bits

pytestmark = pytest.mark.gpu

SALT_REL = 1e-4  # tq2_0_add.cu:651-655


def make_planes(backend, oracle, rng, n, k, t_planes):
    nb = (k + 255) // 256
    packed, bufs = [], []
    for p in range(t_planes):
        trits = ternary(rng, n, k, (0.4, 0.7, 0.85, 0.85)[p])
        sc = f16_bits(rng.uniform(0.02, 1.0, (n, nb)) * (0.5 ** p))
        packed.append(oracle.pack_matrix_scaled(trits, sc, n, k))
        bufs.append(backend.upload_weights_scaled(packed[-1], T.GemmShape(0, n, k)))
    return packed, bufs


@pytest.mark.parametrize("m,n,k,t_planes", [(1, 48, 256, 1), (3, 33, 700, 2), (5, 130, 1000, 3), (17, 20, 300, 4)])
def test_reference_order_kernel_is_bit_exact(backend, oracle, m, n, k, t_planes):
    print("case salt-seq", m, n, k, t_planes, flush=True)
    rng = np.random.default_rng(m * 13 + n + k)
    packed, bufs = make_planes(backend, oracle, rng, n, k, t_planes)
    act = rng.standard_normal((m, k)).astype(np.float32)
    rc, want = oracle.salt_mpgemm(packed, n, k, act, m)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_salt(bufs, dact, m, dout, seq=True)
    assert rc == 0 and same_bits(dout.to_host(), want)
    for a in [dact, dout] + bufs:
        a.free()


@pytest.mark.parametrize("t_planes", [1, 2, 3, 4])
@pytest.mark.parametrize("m,n,k", [(1, 48, 256), (2, 130, 700), (4, 64, 2048), (5, 33, 1000), (8, 257, 2560), (16, 96, 2048)])
def test_matrix_core_form_within_the_reference_bound(backend, oracle, m, n, k, t_planes):
    print("case salt-flow", m, n, k, t_planes, flush=True)
    rng = np.random.default_rng(m * 17 + n + k + t_planes)
    packed, bufs = make_planes(backend, oracle, rng, n, k, t_planes)
    bits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32) * 2)
    act = bf16_bits_to_f32(bits).reshape(m, k)
    rc, want = oracle.salt_mpgemm(packed, n, k, act, m)
    for dtype, dev in (("bf16", bits), ("f32", act)):
        dact, dout = backend.to_device(dev, dtype), backend.empty(m * n, "f32")
        backend.linear_salt(bufs, dact, m, dout)
        got = dout.to_host().reshape(m, n)
        assert rc == 0 and accepts(got, want, rel=SALT_REL, floor=1.0).all()
        assert rel_err(got, want) < 2e-5  # what it actually achieves: the f32 fold's own rounding
        dact.free()
        dout.free()
    for b in bufs:
        b.free()


def test_tokens_with_nan_or_inf_take_the_host_order(backend, oracle):
    rng = np.random.default_rng(40)
    m, n, k = 4, 40, 600
    packed, bufs = make_planes(backend, oracle, rng, n, k, 2)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[1, 7] = np.nan
    act[2, 300] = np.inf
    rc, want = oracle.salt_mpgemm(packed, n, k, act, m)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_salt(bufs, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    assert same_bits(got[1], want[1]) and same_bits(got[2], want[2])
    assert accepts(got[[0, 3]], want[[0, 3]], rel=SALT_REL, floor=1.0).all()
    for a in [dact, dout] + bufs:
        a.free()


def test_more_than_16_tokens_run_in_slices(backend, oracle):
    """40 tokens are three slices (16, 16, 8) of the matrix-core form, the ragged last one included."""
    rng = np.random.default_rng(41)
    m, n, k = 40, 72, 768
    packed, bufs = make_planes(backend, oracle, rng, n, k, 2)
    act = rng.standard_normal((m, k)).astype(np.float32)
    rc, want = oracle.salt_mpgemm(packed, n, k, act, m)
    for dtype in ("f32", "bf16"):
        dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, dtype)
        backend.linear_salt(bufs, dact, m, dout)
        got = dout.to_host().reshape(m, n)
        if dtype == "bf16":
            got = bf16_bits_to_f32(got).reshape(m, n)
            assert accepts(got, want, rel=4e-3, floor=1.0).all()  # bf16 output: 8 bits
        else:
            assert accepts(got, want, rel=SALT_REL, floor=1.0).all() and rel_err(got, want) < 2e-5
        dact.free()
        dout.free()
    for b in bufs:
        b.free()


def test_rows_too_long_for_lds_fall_back(backend, oracle):
    """K = 10240 needs 164 KiB for the rows of 16 tokens: the launch takes the reference-order kernel."""
    rng = np.random.default_rng(43)
    m, n, k = 2, 20, 10240
    packed, bufs = make_planes(backend, oracle, rng, n, k, 1)
    act = rng.standard_normal((m, k)).astype(np.float32)
    rc, want = oracle.salt_mpgemm(packed, n, k, act, m)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_salt(bufs, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    assert accepts(got, want, rel=SALT_REL, floor=1.0).all()
    for a in [dact, dout] + bufs:
        a.free()


def test_scaled_upload_still_serves_the_plain_contract(backend, oracle):
    """mpgemm ignores block scales (crates/tritium-cpu/src/lib.rs:302-345), also on a buffer that kept them;
    and a buffer without them is refused by the block-scale entry point."""
    rng = np.random.default_rng(42)
    m, n, k = 2, 20, 512
    packed, bufs = make_planes(backend, oracle, rng, n, k, 1)
    act = rng.standard_normal((m, k)).astype(np.float32)
    sc = rng.uniform(0.01, 0.1, n).astype(np.float32)
    out = np.zeros((m, n), np.float32)
    backend.mpgemm(T.MpGemm(act, bufs[0], sc, T.GemmShape(m, n, k), T.TernaryFormat.Tq2_0, out))
    from oracle_lib import FMT_TQ2_0
    rc, want = oracle.cpu_mpgemm(packed[0], FMT_TQ2_0, act, sc, m, n, k)
    assert rc == 0 and same_bits(out, want)
    plain = backend.upload_weights(packed[0], T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    with pytest.raises(T.InvalidInput):
        backend.linear_salt([plain], dact, m, dout)
    for a in [dact, dout, plain] + bufs:
        a.free()


def test_every_f16_block_scale_reaches_the_kernels_exactly(backend, oracle):
    """One row per f16 bit pattern, one non-zero trit against an activation of 1: the output is the
    block scale itself, so the device's f16 -> f32 conversion is checked over all 65,536 patterns
    (subnormals, zeros, infinities, NaNs) through both kernels."""
    n, k = 65536, 256
    trits = np.zeros((n, k), np.int8)
    trits[:, 0] = 1
    bits = np.arange(n, dtype=np.uint16).reshape(n, 1)
    packed = oracle.pack_matrix_scaled(trits, bits, n, k)
    buf = backend.upload_weights_scaled(packed, T.GemmShape(0, n, k))
    act = np.zeros((1, k), np.float32)
    act[0, 0] = 1.0
    rc, want = oracle.salt_mpgemm([packed], n, k, act, 1)
    want = want.reshape(-1)
    scale = bits.reshape(-1).view(np.float16).astype(np.float32)
    finite = np.isfinite(scale)
    scale[0x8000] = 0.0  # 0.0 + (-0.0) * 1 is +0.0: the one pattern whose row is not the scale's own bits
    assert rc == 0 and (want[finite].view(np.uint32) == scale[finite].view(np.uint32)).all()
    assert np.isnan(want[~finite]).all()  # an infinite scale times a zero trit is NaN, on the host too
    dact, dout = backend.to_device(act, "f32"), backend.empty(n, "f32")
    backend.linear_salt([buf], dact, 1, dout, seq=True)
    got = dout.to_host()
    assert np.isnan(got[~finite]).all() and (got[finite].view(np.uint32) == want[finite].view(np.uint32)).all()
    # the matrix-core form multiplies the block's integer sum by the scale once: the same values for
    # every finite scale (an infinite or NaN scale gives Inf or NaN there, the host NaN)
    backend.linear_salt([buf], dact, 1, dout)
    got = dout.to_host()
    assert (got[finite].view(np.uint32) == want[finite].view(np.uint32)).all()
    assert (~np.isfinite(got[~finite])).all()
    for a in (dact, dout, buf):
        a.free()
