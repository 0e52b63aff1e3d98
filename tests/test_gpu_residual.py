"""Fused residual-add epilogue: out = residual + ((float)acc * s_w[n]) * s_a[m], one f32 add, as the
reference's tq2_0_add_mpgemm_tiled_i8_scaled_residual computes it
(crates/tritium-cuda/kernels/tq2_0_add.cu:577-637: `__fadd_rn(residual[idx], (float)acc * scales[ni] *
act_scale[mi])`). Expected = the CPU oracle's W1.58A8 composition plus the residual, added in f32."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import bf16_bits_to_f32, f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["auto", "ksplit", "stream", "flow", "flow32"], autouse=True)
def decode_kernel(request, backend):
    backend.set_decode_kernel({"auto": 0, "ksplit": 1, "stream": 2, "flow": 3, "flow32": 3}[request.param])
    backend.set_flow_mfma(32 if request.param == "flow32" else (16 if request.param == "flow" else 0))
    yield request.param
    backend.set_decode_kernel(0)
    backend.set_flow_mfma(0)


@pytest.mark.parametrize("m,n,k,planes", [(1, 7, 300, 1), (5, 130, 257, 2), (33, 40, 512, 1), (64, 48, 1024, 3),
                                            (100, 136, 700, 2), (130, 131, 512, 1), (70, 2100, 768, 1)])
def test_residual_add_bit_exact(backend, oracle, m, n, k, planes, decode_kernel):
    if m > 64 and decode_kernel != "auto":
        pytest.skip("the prefill kernel does not depend on the decode kernel choice")
    print("case residual", m, n, k, planes, decode_kernel, flush=True)
    rng = np.random.default_rng(m * 3 + n + k + planes)
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    layer = backend.linear(packed, scs, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    if m > 3:
        act[2, 1] = np.nan  # a token on the exact path gets the residual too
    res = (rng.standard_normal((m, n)) * 3).astype(np.float32)
    value = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k).reshape(m, n)
    want = res + value  # one f32 add per element
    dact, dres, dout = backend.to_device(act, "f32"), backend.to_device(res, "f32"), backend.empty(m * n, "f32")
    backend.linear_a8_residual(layer, dact, m, dres, dout)
    got = dout.to_host().reshape(m, n)
    fin = ~np.isnan(want)
    assert (np.isnan(got) == ~fin).all() and same_bits(got[fin], want[fin])
    # in place: the residual stream is updated where it lies
    backend.linear_a8_residual(layer, dact, m, dres, dres)
    assert same_bits(dres.to_host().reshape(m, n)[fin], want[fin])
    # bf16 residual and output: widened, added in f32, rounded once
    rb = f32_to_bf16_bits(res)
    want_b = f32_to_bf16_bits(bf16_bits_to_f32(rb).reshape(m, n) + value).reshape(m, n)
    drb, dob = backend.to_device(rb, "bf16"), backend.empty(m * n, "bf16")
    backend.linear_a8_residual(layer, dact, m, drb, dob)
    assert (dob.to_host().reshape(m, n)[fin] == want_b[fin]).all()
    # already-quantized activations (gemm_prequantized with the residual epilogue)
    q, s_a = oracle.quantize_act_int8(np.nan_to_num(act), m, k)
    dq, dsa = backend.to_device(q.astype(np.int8), "i8"), backend.to_device(s_a, "f32")
    backend.linear_i8_residual(layer, dq, dsa, m, backend.to_device(res, "f32"), dout)
    value2 = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, np.nan_to_num(act), m, n, k).reshape(m, n)
    assert same_bits(dout.to_host().reshape(m, n), res + value2)
    for a in (dact, dres, dout, drb, dob, dq, dsa):
        a.free()
    layer.free()


def test_residual_needs_a_pointer(backend, oracle):
    rng = np.random.default_rng(1)
    n, k = 16, 256
    layer = backend.linear([T.pack_rows(ternary(rng, n, k), n, k)], [scales(rng, n)], n, k)
    dact, dout = backend.to_device(rng.standard_normal((1, k)).astype(np.float32), "f32"), backend.empty(n, "f32")

    class Null:
        ptr = None
    with pytest.raises(T.InvalidInput):
        backend.linear_a8_residual(layer, dact, 1, Null, dout)
    dact.free()
    dout.free()
    layer.free()
