"""SALT containers and SALT V2 on the GPU. Row sidecars (dense and sparse residuals, rows of different plane
counts) must give the bits of the dense planes they stand for through the block-scale kernels, and the oracle's
dequantize-then-fold within the reference's 1e-4 (crates/tritium-cuda/kernels/tq2_0_add.cu:651-656). The SALT V2
exact forward and the row gather must carry the bits of the CPU reference's pinned order
(crates/tritium-cpu/src/salt_v2.rs:10-23,316-423), for all three codecs, ragged tiles and both scale groups;
non-finite inputs or results are refused and leave the output untouched (crates/tritium-cuda/src/cuda/tests.rs:246-280)."""
import numpy as np
import pytest

import salt_oracle_lib as S
import tritium_amd as T
from helpers import same_bits
from test_oracle_salt_formats import lcg_trits, sparse_residual, tq2_row

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def so():
    return S.load()


def test_salt_rows_dense_and_sparse_through_the_block_scale_kernels(backend, oracle, so):
    print("case salt-rows", flush=True)
    rng = np.random.default_rng(1)
    n, k, m = 70, 700, 5
    row_planes, encoded = [], []
    for r in range(n):
        t = int(rng.integers(1, 4))
        planes = [tq2_row(oracle, lcg_trits(k, r), np.float16(rng.uniform(0.1, 1.0)).view(np.uint16))]
        for j in range(1, t):
            planes.append(sparse_residual(oracle, k, int(rng.choice([3, 40, 64]))))
        row_planes.append(planes)
        rc, data = (so.pack_salt_row(k, planes) if r % 3 == 0 else so.pack_progressive_salt_row(k, planes, 0.10))
        assert rc == 0
        encoded.append(data)
    blob = np.concatenate(encoded)
    bufs = backend.upload_salt_rows(blob, n, k)
    assert len(bufs) == max(len(p) for p in row_planes)
    # what the tensor is: per plane a row-major TQ2_0 tensor; rows without that plane are zero trits, scale 0
    zero_row = np.tile(np.concatenate([np.full(64, 0x55, np.uint8), np.zeros(2, np.uint8)]), (k + 255) // 256)
    dense = [np.concatenate([(row_planes[r][p] if p < len(row_planes[r]) else zero_row) for r in range(n)]) for p in range(len(bufs))]
    direct = [backend.upload_weights_scaled(d, T.GemmShape(0, n, k)) for d in dense]
    act = rng.standard_normal((m, k)).astype(np.float32)
    dact, o1, o2 = backend.to_device(act, "f32"), backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
    for seq in (False, True):
        backend.linear_salt(bufs, dact, m, o1, seq=seq)
        backend.linear_salt(direct, dact, m, o2, seq=seq)
        assert same_bits(o1.to_host(), o2.to_host())
        rc, want = oracle.salt_mpgemm(dense, n, k, act, m)
        got = o1.to_host().reshape(m, n)
        if seq:
            assert same_bits(got, want)
        else:
            assert np.abs(got - want).max() <= 1e-4 * max(1.0, np.abs(want).max())
    # a prefix of every row: the lower tiers of the progressive format
    one = backend.upload_salt_rows(blob, n, k, 1)
    assert len(one) == 1
    backend.linear_salt(one, dact, m, o1, seq=True)
    assert same_bits(o1.to_host().reshape(m, n), oracle.salt_mpgemm(dense[:1], n, k, act, m)[1])
    with pytest.raises(T.ShapeMismatch):
        backend.upload_salt_rows(blob, n, k + 1)
    with pytest.raises(T.InvalidInput):
        backend.upload_salt_rows(blob[:-1], n, k)
    with pytest.raises(T.InvalidInput):
        backend.upload_salt_rows(blob, n - 1, k)
    for b in bufs + direct + one:
        b.free()
    for a in (dact, o1, o2):
        a.free()


@pytest.mark.parametrize("codec", [S.D2, S.B3, S.S34])
@pytest.mark.parametrize("n,k,counts,group,m", [(3, 173, [1, 3, 2], 128, 2), (5, 173, [1, 3, 2, 3], 128, 1), (64, 256, None, 128, 9),
                                                 (7, 100, None, 64, 3), (33, 1024, None, 128, 17), (1, 4, [1], 128, 1),
                                                 (130, 2048, None, 64, 8), (10, 384, None, 128, 5), (9, 192, None, 64, 2),
                                                 (70, 640, None, 128, 13)])
def test_v2_forward_and_gather_carry_the_reference_bits(backend, so, codec, n, k, counts, group, m):
    print("case salt-v2", codec, n, k, group, m, flush=True)
    if codec == S.S34 and (n * k) % 4:
        n += 4 - (n * k) % 4
        counts = None
    if counts is not None and len(counts) != (n * k + 255) // 256:
        counts = None
    rng = np.random.default_rng(codec * 1000 + n * 10 + k + m)
    t = S.random_v2_tensor(so, rng, codec, n, k, counts, group)
    # the product's own packer gives the same payload
    mine = np.concatenate([T.salt_v2_pack(codec, tr[j]) for tr, _ in t.tiles for j in range(tr.shape[0])])
    assert (mine == t.payload).all()
    dev = backend.salt_v2_upload(codec, group, t.payload, t.scales, t.plane_counts, n, k)
    act = (rng.uniform(-0.75, 0.75, (m, k)) * 10.0 ** rng.integers(-2, 3, (m, k))).astype(np.float32)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    dev.forward(dact, m, dout)
    rc, want = so.v2_forward(t, act, m)
    assert rc == 0 and same_bits(dout.to_host().reshape(m, n), want)
    rows = np.array([n - 1, 0, n - 1, n // 2], np.uint32)
    gout = backend.empty(rows.size * k, "f32")
    dev.gather_rows(rows, gout)
    got = gout.to_host().reshape(rows.size, k)
    for i, r in enumerate(rows):
        for c in sorted({0, k - 1, k // 2, min(127, k - 1), min(128, k - 1)}):
            rc, v = so.v2_coefficient(t, int(r) * k + c)
            assert rc == 0 and got[i, c].view(np.uint32) == v.view(np.uint32)
    assert np.abs(got - t.dense()[rows]).max() <= 1e-5 * max(1.0, np.abs(t.dense()).max())
    with pytest.raises(T.InvalidInput):
        dev.gather_rows(np.array([n], np.uint32), gout)
    for a in (dact, dout, gout):
        a.free()
    dev.free()


def test_v2_refuses_non_finite_and_leaves_the_output_alone(backend, so):
    fmax16 = np.float16(65504).view(np.uint16)
    fmax = np.float32(np.finfo(np.float32).max)
    sentinel = np.full(1, np.float32(19.0))
    # opposite trits cancel before the maximum scale is applied (crates/tritium-cpu/src/salt_v2.rs:1014-1026)
    t = S.V2Tensor(so, S.D2, 128, 1, 2, [(np.array([[1, -1]], np.int8), np.array([[fmax16]], np.uint16))])
    dev = backend.salt_v2_upload(S.D2, 128, t.payload, t.scales, t.plane_counts, 1, 2)
    dact, dout = backend.to_device(np.array([fmax, fmax], np.float32), "f32"), backend.to_device(sentinel, "f32")
    dev.forward(dact, 1, dout)
    assert dout.to_host()[0] == 0.0
    dev.free()
    # the same trits adding up overflow: refused, nothing stored (crates/tritium-cuda/src/cuda/tests.rs:246-280)
    t = S.V2Tensor(so, S.D2, 128, 1, 2, [(np.array([[1, 1]], np.int8), np.array([[0x3C00]], np.uint16))])
    dev = backend.salt_v2_upload(S.D2, 128, t.payload, t.scales, t.plane_counts, 1, 2)
    dout.copy_from(sentinel)
    with pytest.raises(T.InvalidInput):
        dev.forward(dact, 1, dout)
    assert dout.to_host()[0] == np.float32(19.0)
    dact.copy_from(np.array([np.nan, 1.0], np.float32))
    with pytest.raises(T.InvalidInput):
        dev.forward(dact, 1, dout)
    assert dout.to_host()[0] == np.float32(19.0)
    dev.free()
    dact.free()
    dout.free()


def test_v2_refusals_in_the_lane_per_row_form(backend, so):
    """Rows of whole scale groups take the form that keeps its terms in a workspace: the same refusals there,
    and the first row block's finiteness check covers every token."""
    one16 = 0x3C00
    fmax = np.float32(np.finfo(np.float32).max)
    trits = np.zeros((1, 256), np.int8)
    trits[0, :2] = 1          # row 0: columns 0 and 1
    trits[0, 128 + 5] = -1    # row 1: column 5
    t = S.V2Tensor(so, S.D2, 128, 2, 128, [(trits, np.array([[one16, one16]], np.uint16))])
    dev = backend.salt_v2_upload(S.D2, 128, t.payload, t.scales, t.plane_counts, 2, 128)
    m = 11
    act = np.zeros((m, 128), np.float32)
    act[:, 0], act[:, 1], act[:, 5] = 1.5, 2.25, 4.0
    dact, dout = backend.to_device(act, "f32"), backend.to_device(np.full(m * 2, 19.0, np.float32), "f32")
    dev.forward(dact, m, dout)
    assert (dout.to_host().reshape(m, 2) == np.array([3.75, -4.0], np.float32)).all()
    for bad_tok, a0, a1 in ((m - 1, fmax, fmax), (3, np.nan, 0.0), (8, 0.0, np.inf)):
        dout.copy_from(np.full(m * 2, 19.0, np.float32))
        bad = act.copy()
        bad[bad_tok, 0], bad[bad_tok, 1] = a0, a1
        if bad_tok == 8:
            bad[bad_tok, 100] = a1  # a column under zero trits only: still an input that is not finite
            bad[bad_tok, 1] = 0.0
        dact.copy_from(bad)
        with pytest.raises(T.InvalidInput):
            dev.forward(dact, m, dout)
        assert (dout.to_host() == np.float32(19.0)).all()
    dev.free()
    dact.free()
    dout.free()


def test_v2_upload_rejections(backend, so):
    rng = np.random.default_rng(3)
    t = S.random_v2_tensor(so, rng, S.B3, 3, 173, [1, 3, 2], 128)
    up = lambda **kw: backend.salt_v2_upload(kw.get("codec", S.B3), kw.get("group", 128), kw.get("payload", t.payload),
                                             kw.get("scales", t.scales), kw.get("counts", t.plane_counts), kw.get("n", 3), 173)
    bad = t.payload.copy(); bad[5] = 250
    with pytest.raises(T.InvalidInput, match="InvalidB3Code"):
        up(payload=bad)
    with pytest.raises(T.ShapeMismatch):
        up(payload=t.payload[:-1])
    with pytest.raises(T.ShapeMismatch):
        up(scales=t.scales[:-1])
    with pytest.raises(T.ShapeMismatch):
        up(counts=t.plane_counts[:-1])
    with pytest.raises(T.InvalidInput):
        up(counts=np.array([1, 4, 2], np.uint8))
    with pytest.raises(T.UnsupportedFormat):
        up(group=100)
    with pytest.raises(T.UnsupportedFormat):
        up(codec=7)
    up().free()
