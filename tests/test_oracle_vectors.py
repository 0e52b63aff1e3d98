"""Pins the regenerated conformance set (crates/tritium-testkit/src/generate.rs, frozen.rs:36-45).

The reference's frozen file vectors/v070.jsonl is absent from its checkout; by its own gate it
equals generate_vectors(0xC0FFEE, 64) (frozen.rs:89-98), which is integer xorshift plus single
IEEE f32 operations, so it is regenerated here and checked structurally.
"""
import numpy as np

from oracle_lib import FMT_TQ1_0, FMT_TQ2_0

FROZEN_SEED, FROZEN_COUNT = 0xC0FFEE, 64


def test_xorshift_known_answer(oracle):
    import ctypes as C
    s = C.c_uint64(1)
    # Marsaglia xorshift64 (13,7,17) from state 1: 0x40822041
    assert oracle.lib.to_xorshift64_next(C.byref(s)) == 0x40822041 == 1082269761
    assert s.value == 0x40822041


def test_frozen_set_structure(oracle):
    vs = oracle.generate_vectors(FROZEN_SEED, FROZEN_COUNT)
    assert len(vs) == 64 + 25
    for i, v in enumerate(vs[:64]):
        assert v["id"] == f"rand-{i}"
        assert 1 <= v["m"] <= 64 and 1 <= v["n"] <= 32 and v["k"] in (256, 512)
        assert v["format"] == (FMT_TQ2_0 if i % 2 == 0 else FMT_TQ1_0)
    shapes = [(1, 1, 256), (1, 32, 256), (64, 1, 256), (64, 32, 512), (1, 1, 512)]
    kinds = ["allzero", "allpos", "allneg", "mixed-tq2", "mixed-tq1"]
    fm = [FMT_TQ2_0, FMT_TQ2_0, FMT_TQ1_0, FMT_TQ2_0, FMT_TQ1_0]
    for si, shp in enumerate(shapes):
        for j, kind in enumerate(kinds):
            v = vs[64 + si * 5 + j]
            assert v["id"] == f"boundary-{si}-{kind}"
            assert (v["m"], v["n"], v["k"]) == shp and v["format"] == fm[j]
        g = vs[64 + si * 5: 64 + si * 5 + 5]
        assert (g[0]["weights"] == 0).all() and (g[1]["weights"] == 1).all() and (g[2]["weights"] == -1).all()
        assert (g[3]["weights"] == g[4]["weights"]).all()
        for v in g[1:]:
            assert (v["activation"] == g[0]["activation"]).all() and (v["scales"] == g[0]["scales"]).all()
        assert (g[0]["expected"] == 0).all()
        assert (g[1]["expected"] == -g[2]["expected"]).all()


def test_value_ranges_and_expected(oracle):
    vs = oracle.generate_vectors(FROZEN_SEED, FROZEN_COUNT)
    for v in vs:
        a100 = np.rint(v["activation"].astype(np.float64) * 100)
        assert (np.abs(v["activation"] * 100 - a100) < 1e-3).all()
        assert a100.min() >= -1000 and a100.max() <= 999       # generate.rs:45-47
        # and the value is the single f32 division the generator performs
        assert (v["activation"] == (a100.astype(np.float32) / np.float32(100))).all()
        s100 = np.rint(v["scales"].astype(np.float64) * 100)
        assert s100.min() >= 1 and s100.max() <= 200            # generate.rs:50-52
        assert set(np.unique(v["weights"])) <= {-1, 0, 1}
        m, n, k = v["m"], v["n"], v["k"]
        want = (v["activation"].reshape(m, k).astype(np.float64)
                @ v["weights"].reshape(n, k).T.astype(np.float64)) * v["scales"].astype(np.float64)
        got = v["expected"].reshape(m, n)
        assert (np.abs(got - want) <= 1e-4 * np.maximum(1, np.abs(want))).all()


def test_determinism_and_prefix_property(oracle):
    a = oracle.generate_vectors(42, 8)
    b = oracle.generate_vectors(42, 8)
    assert len(a) == 8 + 25
    for x, y in zip(a, b):
        assert x["id"] == y["id"] and (x["expected"] == y["expected"]).all()
    # frozen.rs:126-140 : a smaller count is a prefix of the frozen set, boundary set identical
    big = oracle.generate_vectors(FROZEN_SEED, 64)
    small = oracle.generate_vectors(FROZEN_SEED, 16)
    for i in range(16):
        assert (big[i]["activation"] == small[i]["activation"]).all()
        assert (big[i]["weights"] == small[i]["weights"]).all()
    for x, y in zip(big[64:], small[16:]):
        assert x["id"] == y["id"] and (x["weights"] == y["weights"]).all()


def test_oracle_cpu_backend_passes_conformance(oracle):
    """crates/tritium-cpu/src/lib.rs:710-735,741-765 — the CPU backend's own gates, run on the
    restatement: plain mpgemm is bit-equal to `expected`; the fused path equals quant+fold."""
    for seed, count in ((FROZEN_SEED, 64), (1, 24), (7, 24)):
        for v in oracle.generate_vectors(seed, count):
            m, n, k, fmt = v["m"], v["n"], v["k"], v["format"]
            packed = oracle.pack_matrix(v["weights"], n, k, fmt)
            rc, got = oracle.cpu_mpgemm(packed, fmt, v["activation"], v["scales"], m, n, k)
            assert rc == 0 and (got.reshape(-1).view(np.uint32) == v["expected"].view(np.uint32)).all()
