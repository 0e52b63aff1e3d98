#!/usr/bin/env python3
"""Benchmark of the packed ternary linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Headline workload (BASELINE.json configs[1]): two-plane additive ternary GEMV, K=2048, N=8192,
bf16 N(0,1) activations, per-channel f32 scales, batch sweep 1,2,4,8,16 — the HBM-bound decode
regime. One "step" is one pass of the sweep: five launches of the decode kernel, each over
COPIES distinct resident copies of the layer (1.07 GB of 2-bit codes per launch, far above the
256 MB last-level cache, so the figure is an HBM figure and not a cache one).

Prints ONE JSON line. `value` is algorithmic GB/s of the whole timed region (activation prep
launches included); `roofline` is the decode kernel alone, timed with events on the stream it runs
on; `cpu_baseline` is the CPU oracle's restatement of tritium-cpu timed on this host on one pass
of the same sweep. `extra` carries the other configs measured in the same run: the batch-1 f32
layer (configs[0]), the prefill GEMM (configs[2]), the projection-stack tokens/s (configs[3]) and
the three-plane decode and prefill (configs[4]), and decode launches at layer widths that none of the
configurations names (`decode_other_widths`). Every timed region follows an untimed pre-warm of
PREWARM_S seconds of the same work: from idle the clocks take tens of milliseconds to settle, and a
cold first few milliseconds under-report a kernel by 10-25%.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0     # MI355X HBM3E, published
# HBM bytes per launch of the decode kernel (sweep average), from two rocprofv3 --pmc runs
# (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0 after calibration against a 1 GiB copy kernel):
# profiles/decode_flow_c2_sweep_traffic.txt
DECODE_TRAFFIC_BYTES_PER_LAUNCH = 1_166_242_550
INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA, published
FP32_PEAK_TFLOPS = 157.3  # MI355X fp32, published

K2, N2, PLANES2 = 2048, 8192, 2
SWEEP = (1, 2, 4, 8, 16)
COPIES = 128


def ternary(rng, n, k, p_zero):
    u = rng.random((n, k), dtype=np.float32)
    half = (1.0 - p_zero) / 2
    return np.where(u < p_zero, 0, np.where(u < p_zero + half, 1, -1)).astype(np.int8)


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def algorithmic_bytes(m, n, k, planes, act_bytes, out_bytes, a8=False):
    """Minimum traffic of one linear: 2-bit codes (64 B per 256 trits, block scales excluded),
    activations, per-channel scales, output (+ per-token scales on the int8 path)."""
    nb = (k + 255) // 256
    return planes * n * nb * 64 + m * k * act_bytes + planes * n * 4 + m * n * out_bytes + (4 * m if a8 else 0)


PREWARM_S = 0.25  # untimed: the clock governor needs some tens of milliseconds of load to settle


def bf16_to_f32(bits):
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def check_a8(name, got_bits_or_f32, ws, scs, act, out_dtype):
    """Every leg that reports a W1.58A8 number checks sampled tokens of one member against the exact
    composition, computed here with numpy alone: per-token absmax int8 quantization (one f32 divide
    127/gamma, one multiply, ties to even), integer contraction (f32 BLAS on integers below 2^24 is
    exact), ((float)acc * s_w[n]) summed over planes in order, times the per-token scale. The contract
    is bit-exact, so any difference stops the benchmark."""
    act = np.ascontiguousarray(act, np.float32)
    gamma = np.abs(act).max(axis=1, keepdims=True)
    with np.errstate(divide="ignore", invalid="ignore"):
        s = np.where(gamma > 0, np.float32(127.0) / gamma, np.float32(0.0)).astype(np.float32)
    q = np.clip(np.rint(act * s), -128, 127).astype(np.float32)
    scale = (gamma / np.float32(127.0)).astype(np.float32)
    out = None
    for w, sc in zip(ws, scs):
        t = (q @ np.ascontiguousarray(w.T, np.float32)) * np.asarray(sc, np.float32)[None, :]
        out = t if out is None else out + t
    want = (out * scale).astype(np.float32)
    if out_dtype == "bf16":
        ok = (np.asarray(got_bits_or_f32, np.uint16).reshape(want.shape) == f32_to_bf16_bits(want).reshape(want.shape)).all()
    else:
        ok = (np.asarray(got_bits_or_f32, np.float32).reshape(want.shape).view(np.uint32) == want.view(np.uint32)).all()
    if not ok:
        sys.exit(f"bench.py: leg `{name}` produced outputs that differ from the exact W1.58A8 composition")
    return f"{want.shape[0]} token(s) x {want.shape[1]} outputs bit-exact"


def check_float(name, got, ws, scs, act):
    """Float-contract legs: sampled tokens of one member against a float64 evaluation, at the bound the
    contract states (1e-3 of the largest output; the kernels are normally ~1e-6)."""
    exact = sum((act.astype(np.float64) @ w.T.astype(np.float64)) * np.asarray(sc, np.float64)[None, :] for w, sc in zip(ws, scs))
    err = np.abs(np.asarray(got, np.float64).reshape(exact.shape) - exact).max() / max(np.abs(exact).max(), 1e-30)
    if not err <= 1e-3:
        sys.exit(f"bench.py: leg `{name}` is off by {err:.3e} of the largest output (bound 1e-3)")
    return f"{exact.shape[0]} token(s) x {exact.shape[1]} outputs within {err:.1e} of float64"


def prewarm(be, fn, seconds=PREWARM_S):
    """Run fn() untimed until `seconds` of wall clock have passed (at least once)."""
    t0 = time.perf_counter()
    while True:
        fn()
        be.sync()
        if time.perf_counter() - t0 >= seconds:
            return


def time_steps(be, steps, warmup, step_fn):
    """Untimed: a fixed pre-warm, then W steps. Timed: exactly K steps between two events on the
    library's stream (`value`). Then the same K steps once more with an event pair around every launch of
    the decode kernel (`roofline`): event markers between dependent launches cost a few microseconds
    each, so they stay out of the region `value` is taken from."""
    start, stop = be.event(), be.event()
    prewarm(be, lambda: step_fn(None))
    for _ in range(warmup):
        step_fn(None)
    be.sync()
    start.record()
    for _ in range(steps):
        step_fn(None)
    stop.record()
    be.sync()
    total_ms = start.elapsed_ms(stop)
    marks = []
    for _ in range(steps):
        step_fn(marks)
    be.sync()
    kernel_ms = sum(a.elapsed_ms(b) for a, b in marks)
    for a, b in marks:
        a.destroy()
        b.destroy()
    return total_ms, kernel_ms, len(marks)


def bench_decode(T, be, steps, warmup, rng):
    host = []
    for _ in range(2):  # two distinct host layers, replicated to COPIES distinct device copies
        trits = [ternary(rng, N2, K2, p0) for p0 in (0.4, 0.7)]
        planes = [T.pack_rows(w, N2, K2) for w in trits]
        scs = [rng.uniform(0.01, 0.1, N2).astype(np.float32) for _ in range(PLANES2)]
        host.append((planes, scs, trits))
    layers = [be.linear(host[i % 2][0], host[i % 2][1], N2, K2) for i in range(COPIES)]
    mmax = max(SWEEP)
    act_bits = [f32_to_bf16_bits(rng.standard_normal((mmax, K2)).astype(np.float32)) for _ in range(COPIES)]
    acts = [be.to_device(b, "bf16") for b in act_bits]
    outs = [be.empty(mmax * N2, "f32") for _ in range(COPIES)]
    groups = {m: be.group([(layers[i], acts[i], m, outs[i]) for i in range(COPIES)], 0, "bf16", "f32") for m in SWEEP}
    verified = {}
    for m in SWEEP:  # the last copy of every batch size against float64
        groups[m].launch()
        be.sync()
        c = COPIES - 1
        verified[str(m)] = check_float(f"decode sweep batch {m}", outs[c].to_host()[: m * N2], host[c % 2][2], host[c % 2][1],
                                       bf16_to_f32(act_bits[c]).reshape(mmax, K2)[:m])

    def step(marks):
        for m in SWEEP:
            g = groups[m]
            g.launch_parts(True, False)
            if marks is None:
                g.launch_parts(False, True)
            else:
                a = be.event().record()
                g.launch_parts(False, True)
                marks.append((a, be.event().record()))

    total_ms, kernel_ms, launches = time_steps(be, steps, warmup, step)
    per_launch = {m: COPIES * algorithmic_bytes(m, N2, K2, PLANES2, 2, 4) for m in SWEEP}
    step_bytes = sum(per_launch.values())

    # per-batch figures: the decode kernel alone, each batch size timed separately
    per_m = {}
    for m in SWEEP:
        g = groups[m]
        g.launch_parts(True, False)
        for _ in range(20):
            g.launch_parts(False, True)
        be.sync()
        a = be.event().record()
        for _ in range(50):
            g.launch_parts(False, True)
        b = be.event().record()
        be.sync()
        ms = a.elapsed_ms(b) / 50
        per_m[str(m)] = {"kernel_GB/s": round(per_launch[m] / ms / 1e6, 1), "frac_of_hbm_peak": round(per_launch[m] / ms / 1e6 / HBM_PEAK_GBS, 4),
                         "kernel_us_per_layer": round(ms * 1e3 / COPIES, 3)}
    res = {
        "ms_per_step": total_ms / steps,
        "value": step_bytes * steps / total_ms / 1e6,
        "kernel_gbs": step_bytes * steps / kernel_ms / 1e6,
        "kernel_avg_ms": kernel_ms / launches,
        "bytes_per_launch_avg": step_bytes / len(SWEEP),
        "per_batch": per_m,
        "verified": verified,
    }
    for g in groups.values():
        g.destroy()
    for x in acts + outs:
        x.free()
    for l in layers:
        l.free()
    return res


def time_calls(be, fn, iters):
    """Pre-warm, then `iters` calls of fn(i) between two events; returns ms per call."""
    prewarm(be, lambda: fn(0))
    a = be.event().record()
    for i in range(iters):
        fn(i)
    b = be.event().record()
    be.sync()
    return a.elapsed_ms(b) / iters


def bench_prefill(T, be, rng, m, k, n, planes=1, iters=100):
    """Prefill GEMM: bf16 activations quantized per token to int8 (fused prep launch), int8 MFMA with
    int32 accumulation over `planes` additive planes, bf16 output after per-channel x per-token scale."""
    p0s = (0.4, 0.7, 0.85)[:planes]
    hostw = []
    for _ in range(2):
        hostw.append(([ternary(rng, n, k, p0) for p0 in p0s], [rng.uniform(0.01, 0.1, n).astype(np.float32) for _ in p0s]))
    layers = [be.linear([T.pack_rows(w, n, k) for w in ws], scs, n, k) for ws, scs in hostw]
    abits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    act = be.to_device(abits, "bf16")
    out = be.empty(m * n, "bf16")
    be.linear_a8(layers[1], act, m, out)
    tok = [0, m // 2 + 1, m - 1]
    verified = check_a8(f"prefill M={m} K={k} N={n}", out.to_host().reshape(m, n)[tok], hostw[1][0], hostw[1][1],
                        bf16_to_f32(abits).reshape(m, k)[tok], "bf16")
    ms = time_calls(be, lambda i: be.linear_a8(layers[i % 2], act, m, out), iters)
    kernel = be.last_kernel()
    # the contraction alone: the same call on already-quantized int8 rows (their re-ordering launch stays in)
    q = be.to_device(rng.integers(-127, 128, (m, k)).astype(np.int8), "i8")
    qs = be.to_device(rng.uniform(0.01, 0.05, m).astype(np.float32), "f32")
    ms_i8 = time_calls(be, lambda i: be.linear_i8(layers[i % 2], q, qs, m, out), iters)
    ops = 2.0 * m * n * k * planes
    for l in layers:
        l.free()
    for x in (act, out, q, qs):
        x.free()
    return {"workload": f"prefill GEMM M={m} K={k} N={n} {planes} plane(s), bf16 act -> int8 per token -> int32 acc -> bf16",
            "ms_per_call_incl_quant": round(ms, 4), "TOPS": round(ops / ms / 1e9, 1),
            "frac_of_int8_peak": round(ops / ms / 1e9 / INT8_PEAK_TOPS, 4), "kernel": kernel,
            "int8_input_call": {"ms_per_call": round(ms_i8, 4), "TOPS": round(ops / ms_i8 / 1e9, 1),
                                "frac_of_int8_peak": round(ops / ms_i8 / 1e9 / INT8_PEAK_TOPS, 4),
                                "note": "activations already int8 (no absmax pass; the operand re-ordering launch included)"},
            "verified": verified}


def bench_config1(T, be, rng, iters=200):
    """configs[0]: one ternary linear, K=2560 N=6912, one plane, f32 N(0,1) activation, batch 1.
    (a) the HBM figure: COPIES distinct resident copies of the layer (0.57 GB of codes, above the 256 MB
        last-level cache) in one grouped launch; kernel alone and the whole step with its digit-split launch;
    (b) one device-resident call on a single 4.4 MB layer (one launch: the decode kernel splits the token's digits
        itself; beside it the same call as two launches -- cache resident and launch-bound, so latency figures,
        not bandwidth ones);
    (c) the adapter call on host slices (through the context's pinned block: host memcpy, copy kernel, decode
        launch, sync, host memcpy per call)."""
    n, k = 6912, 2560
    trits = [ternary(rng, n, k, 0.4) for _ in range(2)]
    packed = [T.pack_rows(w, n, k) for w in trits]
    scs = [rng.uniform(0.01, 0.1, n).astype(np.float32) for _ in range(2)]
    layers = [be.linear([packed[i % 2]], [scs[i % 2]], n, k) for i in range(COPIES)]
    act_h = [rng.standard_normal((1, k)).astype(np.float32) for _ in range(COPIES)]
    acts = [be.to_device(a, "f32") for a in act_h]
    outs = [be.empty(n, "f32") for _ in range(COPIES)]
    g = be.group([(layers[i], acts[i], 1, outs[i]) for i in range(COPIES)], 0, "f32", "f32")
    g.launch()
    be.sync()
    c = COPIES - 1
    verified = check_float("config1 grouped", outs[c].to_host(), [trits[c % 2]], [scs[c % 2]], act_h[c])
    ms_step = time_calls(be, lambda i: g.launch(), iters)
    g.launch_parts(True, False)
    ms_kernel = time_calls(be, lambda i: g.launch_parts(False, True), iters)
    by = COPIES * algorithmic_bytes(1, n, k, 1, 4, 4)
    g.destroy()
    ms_single = time_calls(be, lambda i: be.linear_float(layers[0], acts[0], 1, outs[0]), iters)
    be.set_fuse_tokens(0)  # the same call as two launches (digit split, then the decode kernel)
    ms_single_two = time_calls(be, lambda i: be.linear_float(layers[0], acts[0], 1, outs[0]), iters)
    be.set_fuse_tokens(-1)
    buf = be.upload_weights(packed[0], T.GemmShape(1, n, k), T.TernaryFormat.Tq2_0)
    out = np.zeros(n, np.float32)
    call = T.MpGemm(act_h[0].reshape(-1), buf, scs[0], T.GemmShape(1, n, k), T.TernaryFormat.Tq2_0, out)
    for _ in range(20):
        be.mpgemm(call)
    t0 = time.perf_counter()
    for _ in range(iters):
        be.mpgemm(call)
    host_us = (time.perf_counter() - t0) / iters * 1e6
    buf.free()
    for x in acts + outs:
        x.free()
    for l in layers:
        l.free()
    by1 = algorithmic_bytes(1, n, k, 1, 4, 4)
    return {"workload": f"K=2560 N=6912 1 plane, f32 activation, batch 1; {COPIES} resident layer copies per grouped launch",
            "kernel_GB/s": round(by / ms_kernel / 1e6, 1), "kernel_frac_of_hbm_peak": round(by / ms_kernel / 1e6 / HBM_PEAK_GBS, 4),
            "kernel_us_per_layer": round(ms_kernel * 1e3 / COPIES, 3),
            "step_GB/s_incl_digit_split": round(by / ms_step / 1e6, 1),
            "step_frac_of_hbm_peak": round(by / ms_step / 1e6 / HBM_PEAK_GBS, 4),
            "single_layer_device_resident_call_us": round(ms_single * 1e3, 2),
            "single_layer_call_as_two_launches_us": round(ms_single_two * 1e3, 2),
            "single_layer_GB/s": round(by1 / ms_single / 1e6, 1),
            "adapter_call_on_host_slices_us": round(host_us, 1),
            "verified": verified}


def bench_sweep_a8(T, be, rng, iters=100):
    """The headline sweep again under the other contract: activations quantized per token to int8
    (what TernaryLinear::forward asks of a backend, mpgemm_with_act_quant), bit-exact to the CPU. One
    operand row per token instead of the four digit rows of the float contract, so every batch size
    of the sweep stays in the bandwidth regime. Kernel only, like `per_batch`."""
    host = []
    for _ in range(2):
        trits = [ternary(rng, N2, K2, p0) for p0 in (0.4, 0.7)]
        host.append(([T.pack_rows(w, N2, K2) for w in trits], [rng.uniform(0.01, 0.1, N2).astype(np.float32) for _ in range(PLANES2)], trits))
    layers = [be.linear(host[i % 2][0], host[i % 2][1], N2, K2) for i in range(COPIES)]
    mmax = max(SWEEP)
    act_bits = [f32_to_bf16_bits(rng.standard_normal((mmax, K2)).astype(np.float32)) for _ in range(COPIES)]
    acts = [be.to_device(b, "bf16") for b in act_bits]
    outs = [be.empty(mmax * N2, "f32") for _ in range(COPIES)]
    res, tot_b, tot_ms, tot_step = {}, 0, 0.0, 0.0
    c = COPIES - 1
    for m in SWEEP:
        g = be.group([(layers[i], acts[i], m, outs[i]) for i in range(COPIES)], 1, "bf16", "f32")
        g.launch()
        be.sync()
        ver = check_a8(f"int8 sweep batch {m}", outs[c].to_host()[: m * N2], host[c % 2][2], host[c % 2][1],
                       bf16_to_f32(act_bits[c]).reshape(mmax, K2)[:m], "f32")
        ms_step = time_calls(be, lambda i: g.launch(), iters)
        g.launch_parts(True, False)
        ms = time_calls(be, lambda i: g.launch_parts(False, True), iters)
        by = COPIES * algorithmic_bytes(m, N2, K2, PLANES2, 2, 4, a8=True)
        res[str(m)] = {"kernel_GB/s": round(by / ms / 1e6, 1), "kernel_us_per_layer": round(ms * 1e3 / COPIES, 3),
                       "step_GB/s_incl_quant": round(by / ms_step / 1e6, 1), "verified": ver}
        tot_b += by
        tot_ms += ms
        tot_step += ms_step
        g.destroy()
    for x in acts + outs:
        x.free()
    for l in layers:
        l.free()
    return {"workload": "the headline sweep with per-token int8 activations (W1.58A8): decode kernel alone, and the step with its quantization launch",
            "per_batch": res, "kernel_sweep_GB/s": round(tot_b / tot_ms / 1e6, 1),
            "kernel_frac_of_hbm_peak": round(tot_b / tot_ms / 1e6 / HBM_PEAK_GBS, 4),
            "step_sweep_GB/s_incl_quant": round(tot_b / tot_step / 1e6, 1),
            "step_frac_of_hbm_peak": round(tot_b / tot_step / 1e6 / HBM_PEAK_GBS, 4)}


def bench_config5(T, be, rng):
    """configs[4]: 27B-class dense ternary projections, three additive planes (P(0)=0.4/0.7/0.85), hidden
    5120, FFN 17408, 64 layers. The config does not give the attention shapes; assumed here: 40 query heads
    and 8 KV heads of 128, i.e. q and o 5120 x 5120, k and v 1024 x 5120 (with gate/up 17408 x 5120 and down
    5120 x 17408 that is 330 M weights per layer and plane, 15.9 GB of 2-bit codes for the stack).
    Decode: all 64 layers x 7 projections at batch 64 (W1.58A8, bf16 in and out) on given inputs in ONE
    grouped launch, quantization included. The layers are 64 distinct device copies of one host set per
    shape. Prefill: the 4096-token GEMM of the up and of the down projection."""
    h, f, kvd, layers_n, m = 5120, 17408, 1024, 64, 64
    shapes = {"q": (h, h), "k": (kvd, h), "v": (kvd, h), "o": (h, h), "gate": (f, h), "up": (f, h), "down": (h, f)}
    hostw = {}
    for n, k in sorted(set(shapes.values())):
        ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)]
        hostw[(n, k)] = (ws, [rng.uniform(0.01, 0.1, n).astype(np.float32) for _ in range(3)], [T.pack_rows(w, n, k) for w in ws])
    lins = [{name: be.linear(hostw[sh][2], hostw[sh][1], *sh) for name, sh in shapes.items()} for _ in range(layers_n)]
    srcs_h = {key: f32_to_bf16_bits(rng.standard_normal((m, kk)).astype(np.float32)) for key, kk in (("hid", h), ("att", h), ("mid", f))}
    srcs = {key: be.to_device(v, "bf16") for key, v in srcs_h.items()}
    wiring = (("q", "hid"), ("k", "hid"), ("v", "hid"), ("o", "att"), ("gate", "hid"), ("up", "hid"), ("down", "mid"))
    members, outs = [], []
    for L in lins:
        for name, key in wiring:
            o = be.empty(m * shapes[name][0], "bf16")
            outs.append(o)
            members.append((L[name], srcs[key], m, o))
    g = be.group(members, 1, "bf16", "bf16")
    g.launch()
    be.sync()
    verified = {}
    tok = [0, 33, m - 1]
    for j, (name, key) in enumerate(wiring):  # the last layer's seven projections
        idx = (layers_n - 1) * len(wiring) + j
        n, k = shapes[name]
        ws, scs, _ = hostw[shapes[name]]
        verified[name] = check_a8(f"config5 decode {name}", outs[idx].to_host().reshape(m, n)[tok], ws, scs,
                                  bf16_to_f32(srcs_h[key]).reshape(m, k)[tok], "bf16")
    ms = time_calls(be, lambda i: g.launch(), 10)
    g.launch_parts(True, False)
    ms_k = time_calls(be, lambda i: g.launch_parts(False, True), 10)
    by = layers_n * sum(algorithmic_bytes(m, n, k, 3, 2, 2, a8=True) for n, k in shapes.values())
    ops = layers_n * sum(2.0 * m * n * k * 3 for n, k in shapes.values())
    res = {"assumed_attention_shapes": "40 query heads, 8 KV heads of 128: q,o 5120x5120; k,v 1024x5120 (not given by the config)",
           "decode_batch64": {"workload": f"{layers_n} layers x (q,k,v,o,gate,up,down), 3 planes, batch 64, one grouped launch on given inputs",
                              "ms_per_step_incl_quant": round(ms, 4), "GB/s": round(by / ms / 1e6, 1),
                              "frac_of_hbm_peak": round(by / ms / 1e6 / HBM_PEAK_GBS, 4),
                              "tokens_per_s": round(m / ms * 1e3, 1),
                              "kernels_only": {"ms": round(ms_k, 4), "GB/s": round(by / ms_k / 1e6, 1),
                                               "frac_of_hbm_peak": round(by / ms_k / 1e6 / HBM_PEAK_GBS, 4),
                                               "TOPS": round(ops / ms_k / 1e9, 1)},
                              "code_bytes": int(layers_n * sum(3 * n * ((k + 255) // 256) * 64 for n, k in shapes.values())),
                              "verified": verified}}
    g.destroy()
    # the same projections as single calls (one linear per launch, quantization included), rotating over
    # the 64 layers: rows beyond LDS -> the prefill kernel
    single = {}
    for name, key in (("q", "hid"), ("k", "hid"), ("up", "hid"), ("down", "mid")):
        n, k = shapes[name]
        o = outs[[w[0] for w in wiring].index(name)]
        ms1 = time_calls(be, lambda i: be.linear_a8(lins[i % layers_n][name], srcs[key], m, o), 64)
        by1 = algorithmic_bytes(m, n, k, 3, 2, 2, a8=True)
        single[name] = {"us_per_call_incl_quant": round(ms1 * 1e3, 1), "GB/s": round(by1 / ms1 / 1e6, 1),
                        "frac_of_hbm_peak": round(by1 / ms1 / 1e6 / HBM_PEAK_GBS, 4)}
    res["decode_batch64_single_calls"] = dict(single, workload="one projection per call, 3 planes, batch 64, incl. quantization")
    for x in outs + list(srcs.values()):
        x.free()
    for L in lins:
        for l in L.values():
            l.free()
    res["prefill_4096_up"] = bench_prefill(T, be, rng, 4096, h, f, planes=3, iters=20)
    res["prefill_4096_down"] = bench_prefill(T, be, rng, 4096, f, h, planes=3, iters=20)
    return res


def bench_zero_skip(T, be, rng, iters=60):
    """Zero-chunk skip on the headline shape (two planes, K=2048, N=8192, W1.58A8, batch 1, 4, 16, 32 and 64, 128
    layer copies per launch). Plane 2 has P(0)=0.85 in two forms: block-structured (75% of its 16-row x
    256-trit chunks all zero, the rest i.i.d. with P(0)=0.4) and i.i.d. Each is timed with the map the upload
    keeps by the 0.5% rule and with maps disabled; for the i.i.d. plane also with a map forced on (it has no
    zero chunk: the rule keeps none, so the default costs nothing). Batch 32 takes the 32x32x32 form of the
    kernel, the others the 16x16x64 form. GB/s are the dense algorithmic bytes over time, so a skip shows as a
    figure above what the memory could deliver for the full planes."""
    nt, nb = N2 // 16, K2 // 256
    p1 = ternary(rng, N2, K2, 0.4)
    structured = ternary(rng, N2, K2, 0.4)
    z = rng.random((nt, nb)) < 0.75
    structured.reshape(nt, 16, nb, 256)[z[:, None, :, None].repeat(16, 1).repeat(256, 3)] = 0
    iid = ternary(rng, N2, K2, 0.85)
    scs = [rng.uniform(0.01, 0.1, N2).astype(np.float32) for _ in range(2)]
    res = {"workload": f"two planes K={K2} N={N2}, plane 2 with P(0)=0.85 block-structured ({z.mean():.2f} of its chunks zero) or i.i.d.; "
                       f"W1.58A8, {COPIES} layer copies per launch, decode kernel alone",
           "zero_fraction_of_plane2": {"structured": round(float((structured == 0).mean()), 3), "iid": round(float((iid == 0).mean()), 3)}}
    packed1 = T.pack_rows(p1, N2, K2)
    batches = (1, 4, 16, 32, 64)
    acts = [be.to_device(f32_to_bf16_bits(rng.standard_normal((max(batches), K2)).astype(np.float32)), "bf16") for _ in range(COPIES)]
    outs = [be.empty(max(batches) * N2, "f32") for _ in range(COPIES)]
    ref_out = {}
    for name, plane2, modes in (("structured", structured, (0, 1)), ("iid", iid, (0, 1, 2))):
        packed2 = T.pack_rows(plane2, N2, K2)
        for mode in modes:
            be.set_zero_skip(mode)
            layers = [be.linear([packed1, packed2], scs, N2, K2) for _ in range(COPIES)]
            kept = layers[0].planes[1].zero_chunks()
            tag = f"{name}_{('by_rule', 'maps_off', 'map_forced')[mode]}"
            res[tag] = {"plane2_zero_chunks": kept[0], "chunks": kept[1], "map_kept": kept[2]}
            for m in batches:
                g = be.group([(layers[i], acts[i], m, outs[i]) for i in range(COPIES)], 1, "bf16", "f32")
                g.launch()
                be.sync()
                got = outs[COPIES - 1].to_host()[: m * N2].copy()
                if (name, m) in ref_out and not (got.view(np.uint32) == ref_out[(name, m)].view(np.uint32)).all():
                    sys.exit(f"bench.py: zero-skip leg: bits differ between map settings ({tag}, batch {m})")
                ref_out[(name, m)] = got
                ms = time_calls(be, lambda i: g.launch_parts(False, True), iters)
                by = COPIES * algorithmic_bytes(m, N2, K2, PLANES2, 2, 4, a8=True)
                res[tag][f"batch{m}"] = {"kernel_us_per_launch": round(ms * 1e3, 1), "dense_GB/s": round(by / ms / 1e6, 1)}
                g.destroy()
            for l in layers:
                l.free()
    be.set_zero_skip(0)
    res["bits"] = "identical across map settings (checked on the last layer copy of every launch)"
    for x in acts + outs:
        x.free()
    return res


def bench_base3(T, be, rng, iters=60):
    """A/B of the two weight streams of the decode kernel: 2-bit codes (64 bytes per 256 trits of a row) against
    the base-3 stream (52 bytes, TQ1_0-coded bytes decoded in the kernel), same layers, same activations,
    128 layer copies per launch, decode kernel alone. configs[0]'s layer uploaded in TQ1_0 (one plane,
    K=2560, N=6912) and the headline layer (two planes, K=2048, N=8192). GB/s are the 2-bit algorithmic
    bytes over time for both, so the ratio is the speed-up of the base-3 stream; outputs must carry the
    same bits."""
    res = {"workload": f"{COPIES} layer copies per launch, decode kernel alone; GB/s on the 2-bit algorithmic bytes for both streams"}
    shapes = (("config1_layer_tq1_0", 6912, 2560, 1, T.TernaryFormat.Tq1_0, ((1, "f32", 0), (1, "bf16", 1), (4, "bf16", 1), (16, "bf16", 1))),
              ("headline_layer", N2, K2, 2, T.TernaryFormat.Tq2_0, ((1, "bf16", 0), (2, "bf16", 0), (4, "bf16", 0), (8, "bf16", 0), (16, "bf16", 1))))
    for name, n, k, planes, fmt, cases in shapes:
        host = []
        for _ in range(2):
            trits = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7)[:planes]]
            host.append(([T.pack_rows(w, n, k, fmt) for w in trits], [rng.uniform(0.01, 0.1, n).astype(np.float32) for _ in range(planes)]))
        layers = {}
        for mode in (0, 2):
            be.set_base3_stream(mode)
            layers[mode] = [be.linear(host[i % 2][0], host[i % 2][1], n, k, fmt) for i in range(COPIES)]
        be.set_base3_stream(0)
        res[name] = {"base3_bytes_per_plane": layers[2][0].planes[0].base3_bytes(), "two_bit_bytes_per_plane": ((n + 15) // 16) * ((k + 255) // 256) * 1024}
        for m, dt, gmode in cases:
            mk = lambda: rng.standard_normal((m, k)).astype(np.float32)
            acts = [be.to_device(mk() if dt == "f32" else f32_to_bf16_bits(mk()), dt) for _ in range(COPIES)]
            outs = [be.empty(m * n, "f32") for _ in range(COPIES)]
            by = COPIES * algorithmic_bytes(m, n, k, planes, 4 if dt == "f32" else 2, 4, a8=(gmode == 1))
            row, ref = {}, None
            for mode, tag in ((0, "two_bit"), (2, "base3")):
                g = be.group([(layers[mode][i], acts[i], m, outs[i]) for i in range(COPIES)], gmode, dt, "f32")
                g.launch()
                be.sync()
                got = outs[COPIES - 1].to_host().copy()
                if ref is not None and not (got.view(np.uint32) == ref.view(np.uint32)).all():
                    sys.exit(f"bench.py: base-3 leg: bits differ between the two streams ({name}, batch {m})")
                ref = got
                ms = time_calls(be, lambda i: g.launch_parts(False, True), iters)
                row[tag] = {"kernel_us_per_launch": round(ms * 1e3, 1), "GB/s": round(by / ms / 1e6, 1)}
                g.destroy()
            row["base3_over_two_bit"] = round(row["two_bit"]["kernel_us_per_launch"] / row["base3"]["kernel_us_per_launch"], 3)
            res[name][f"batch{m}_{dt}_{'a8' if gmode else 'float'}"] = row
            for x in acts + outs:
                x.free()
        for mode in (0, 2):
            for l in layers[mode]:
                l.free()
    res["bits"] = "identical between the two streams (checked on the last layer copy of every launch)"
    return res


def bench_salt(T, be, rng, iters=30):
    """Block-scale additive planes (SALT): the headline shape K=2048 x 2 planes with per-256-block f16
    scales, one tall layer of N = 262,144 output channels per launch (2 x 134 MB of codes; two
    layers alternate, so the 0.54 GB working set exceeds the last-level cache), bf16 activations, f32
    out. Algorithmic bytes count the block scales at their f16 size."""
    k, n_unit, reps, planes = K2, N2, 32, 2
    n = n_unit * reps
    nb = (k + 255) // 256
    layers = []
    for _ in range(2):
        bufs = []
        for p0 in (0.4, 0.7):
            trits = ternary(rng, n_unit, k, p0)
            packed = T.pack_rows(trits, n_unit, k).reshape(n_unit, nb, 66).copy()
            sc = rng.uniform(0.02, 1.0, (n_unit, nb)).astype(np.float16).view(np.uint16)
            packed[:, :, 64] = (sc & 0xFF).astype(np.uint8)
            packed[:, :, 65] = (sc >> 8).astype(np.uint8)
            bufs.append(be.upload_weights_scaled(np.tile(packed.reshape(-1), reps), T.GemmShape(0, n, k)))
        layers.append(bufs)
    res = {"workload": f"2 block-scale planes, K={k}, N={n} per launch (two layers alternate), bf16 activations, f32 out, "
                       "digit split + contraction"}
    for m in (1, 4, 16):
        act = be.to_device(f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32)), "bf16")
        out = be.empty(m * n, "f32")
        ms = time_calls(be, lambda i: be.linear_salt(layers[i % 2], act, m, out), iters)
        by = planes * n * nb * (64 + 2) + m * k * 2 + m * n * 4
        res[f"batch{m}"] = {"ms_per_call": round(ms, 4), "GB/s": round(by / ms / 1e6, 1),
                            "frac_of_hbm_peak": round(by / ms / 1e6 / HBM_PEAK_GBS, 4)}
        act.free()
        out.free()
    for bufs in layers:
        for b in bufs:
            b.free()
    return res


def bench_salt_v2(T, be, rng, iters=10):
    """SALT V2 exact matvec (the reference's pinned scalar order per output: correctness first, no matrix
    cores): 4096 x 4096 coefficients in 65,536 allocation tiles of two planes each, D2 codec, scale groups
    of 128; f32 activations and outputs. Sampled outputs are checked against a float64 product of the
    dequantized matrix."""
    n = k = 4096
    tiles = n * k // 256
    planes = []
    for p0 in (0.4, 0.7):
        trits = ternary(rng, n, k, p0).reshape(-1)
        planes.append((trits, T.salt_v2_pack(T.SALT_V2_D2, trits).reshape(tiles, 64),
                       rng.uniform(0.02, 1.0, (tiles, 2)).astype(np.float16)))
    payload = np.stack([planes[0][1], planes[1][1]], axis=1).reshape(-1)   # tile after tile, planes in order
    scales = np.stack([planes[0][2], planes[1][2]], axis=1).reshape(-1)    # one per (plane, group of 128)
    dev = be.salt_v2_upload(T.SALT_V2_D2, 128, payload, scales.view(np.uint16), np.full(tiles, 2, np.uint8), n, k)
    res = {"workload": f"SALT V2 {n} x {k}, two planes per tile, D2 codec, scale group 128, exact order, f32 in/out"}
    rows = np.array([0, 1, n // 2, n - 1])
    dense = np.zeros((rows.size, k))
    for trits, _, sc in planes:
        for i, r in enumerate(rows):
            seg = slice(int(r) * k, int(r) * k + k)
            dense[i] += trits[seg].astype(np.float64) * np.repeat(sc.reshape(-1)[int(r) * k // 128:(int(r) * k + k) // 128].astype(np.float64), 128)
    for m in (1, 8):
        a = rng.standard_normal((m, k)).astype(np.float32)
        act, out = be.to_device(a, "f32"), be.empty(m * n, "f32")
        dev.forward(act, m, out)
        got = out.to_host().reshape(m, n)[:, rows].astype(np.float64)
        want = a.astype(np.float64) @ dense.T
        err = float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))
        if err > 1e-4:
            raise SystemExit(f"salt_v2 leg: output off by {err:.2e} of the largest value")
        ms = time_calls(be, lambda i: dev.forward(act, m, out), iters)
        by = payload.size + scales.size * 2 + m * k * 4 + m * n * 4
        res[f"batch{m}"] = {"ms_per_call": round(ms, 4), "GB/s": round(by / ms / 1e6, 1),
                            "frac_of_hbm_peak": round(by / ms / 1e6 / HBM_PEAK_GBS, 4),
                            "verified": f"{m} token(s) x {rows.size} outputs within {err:.1e} of float64"}
        act.free()
        out.free()
    dev.free()
    return res


def bench_other_widths(T, be, rng, iters=30):
    """Decode launches at layer widths that none of the reference's configurations names (hidden 4096 / 5120, FFN
    11008 / 17408): W1.58A8, bf16 in and out, 32 resident layer copies per grouped launch, decode kernel alone.
    These are the launches whose run lengths, workgroup sizes and kernel choice come from the library's rules rather
    than from a fit to the headline's shape."""
    copies = 32
    res = {"workload": f"{copies} layer copies per launch, W1.58A8, bf16 in/out, decode kernel alone (prep launch excluded)"}
    for n, k, planes in ((11008, 4096, 1), (5120, 5120, 3), (17408, 5120, 3)):
        hostw = []
        for _ in range(2):
            ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
            hostw.append((ws, [rng.uniform(0.01, 0.1, n).astype(np.float32) for _ in range(planes)]))
        layers = [be.linear([T.pack_rows(w, n, k) for w in hostw[i % 2][0]], hostw[i % 2][1], n, k) for i in range(copies)]
        leg = {}
        for m in (1, 8, 24, 32):
            abits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
            act = be.to_device(abits, "bf16")
            outs = [be.empty(m * n, "bf16") for _ in range(copies)]
            g = be.group([(layers[i], act, m, outs[i]) for i in range(copies)], 1, "bf16", "bf16")
            g.launch()
            be.sync()
            tok = sorted({0, m // 2, m - 1})
            c = copies - 1
            ver = check_a8(f"other widths {n}x{k}x{planes} batch {m}", outs[c].to_host().reshape(m, n)[tok], hostw[c % 2][0],
                           hostw[c % 2][1], bf16_to_f32(abits).reshape(m, k)[tok], "bf16")
            g.launch_parts(True, False)
            ms = time_calls(be, lambda i: g.launch_parts(False, True), iters)
            nbytes = copies * algorithmic_bytes(m, n, k, planes, 1, 2, a8=True)
            leg[f"batch{m}"] = {"kernel_us_per_launch": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1),
                                "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "verified": ver}
            g.destroy()
            for x in outs + [act]:
                x.free()
        res[f"N{n}_K{k}_{planes}plane{'s' if planes > 1 else ''}"] = leg
        for l in layers:
            l.free()
    return res


def bench_vjp(T, be, rng, iters=5):
    """mpgemm_projected_vjp on the configs[2] projection (M=2048 tokens, K=2560, N=6912, one plane),
    device-resident f32 operands. Each gradient is timed on its own; flops = one multiply and one add
    per term (kept unfused for the CPU backend's rounding), priced against the published fp32 vector
    rate, which counts a fused multiply-add per lane and clock."""
    m, k, n = 2048, 2560, 6912
    buf = be.upload_weights(T.pack_rows(ternary(rng, n, k, 0.4), n, k), T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
    sc = be.to_device(rng.uniform(0.01, 0.1, n).astype(np.float32), "f32")
    act = be.to_device(rng.standard_normal((m, k)).astype(np.float32), "f32")
    gy = be.to_device(rng.standard_normal((m, n)).astype(np.float32), "f32")
    ga, gw, gb = be.empty(m * k, "f32"), be.empty(n * k, "f32"), be.empty(n, "f32")
    res = {"workload": f"projected VJP M={m} K={k} N={n}, 1 plane, f32 operands resident on the device"}
    flops = 2.0 * m * n * k
    for name, outs in (("grad_act", (ga, None, None)), ("grad_projected_weight", (None, gw, None)),
                       ("grad_bias", (None, None, gb)), ("all_three", (ga, gw, gb))):
        ms = time_calls(be, lambda i: be.projected_vjp(buf, sc, act, gy, m, *outs), iters)
        res[name] = {"ms_per_call": round(ms, 4)}
        if name != "grad_bias":
            f = flops * (2 if name == "all_three" else 1)
            res[name].update({"TFLOP/s": round(f / ms / 1e9, 2), "frac_of_fp32_peak": round(f / ms / 1e9 / FP32_PEAK_TFLOPS, 4)})
    for a in (sc, act, gy, ga, gw, gb):
        a.free()
    buf.free()
    return res


def bench_stack(T, be, rng, iters=100):
    """configs[3]: the 7 ternary projections of 30 decoder layers (hidden 2560, FFN 6912, 20 query
    heads and 5 KV heads of 128), W1.58A8, one launch for the whole stack with given inputs.
    tokens/s = batch / time of the projection path only."""
    h, f, kv, layers_n = 2560, 6912, 640, 30
    shapes = {"q": (h, h), "k": (kv, h), "v": (kv, h), "o": (h, h), "gate": (f, h), "up": (f, h), "down": (h, f)}
    hostw, hostt = {}, {}
    for name, (n, k) in shapes.items():
        key = (n, k)
        if key not in hostw:
            hostt[key] = ternary(rng, n, k, 0.4)
            hostw[key] = (T.pack_rows(hostt[key], n, k), rng.uniform(0.01, 0.1, n).astype(np.float32))
    res = {}
    lins = []
    for _ in range(layers_n):
        lins.append({name: be.linear([hostw[(n, k)][0]], [hostw[(n, k)][1]], n, k) for name, (n, k) in shapes.items()})
    code_bytes = layers_n * sum(n * ((k + 255) // 256) * 64 for n, k in shapes.values())
    nw = [[be.to_device(rng.uniform(0.5, 1.5, h).astype(np.float32), "f32") for _ in range(2)] for _ in range(layers_n)]
    for m in (1, 32):
        src_h = {key: f32_to_bf16_bits(rng.standard_normal((m, kk)).astype(np.float32)) for key, kk in (("hid", h), ("att", h), ("mid", f))}
        hid, att, mid = (be.to_device(src_h[key], "bf16") for key in ("hid", "att", "mid"))
        wiring = (("q", hid, "hid"), ("k", hid, "hid"), ("v", hid, "hid"), ("o", att, "att"), ("gate", hid, "hid"),
                  ("up", hid, "hid"), ("down", mid, "mid"))
        members, outs = [], []
        for L in lins:
            for name, src, _ in wiring:
                o = be.empty(m * shapes[name][0], "bf16")
                outs.append(o)
                members.append((L[name], src, m, o))
        g = be.group(members, 1, "bf16", "bf16")
        g.launch()
        be.sync()
        tok = sorted({0, m // 2, m - 1})
        ver = {}
        for j, (name, _, key) in enumerate(wiring):  # the last layer's seven projections
            n, k = shapes[name]
            ver[name] = check_a8(f"stack batch {m} {name}", outs[(layers_n - 1) * 7 + j].to_host().reshape(m, n)[tok],
                                 [hostt[(n, k)]], [hostw[(n, k)][1]], bf16_to_f32(src_h[key]).reshape(m, k)[tok], "bf16")
        ms = time_calls(be, lambda i: g.launch(), iters)
        g.launch_parts(True, False)
        ms_k = time_calls(be, lambda i: g.launch_parts(False, True), iters)
        res[f"batch{m}"] = {"ms_per_step_incl_quant": round(ms, 4), "tokens_per_s": round(m / ms * 1e3, 1),
                            "code_GB/s": round(code_bytes / ms / 1e6, 1),
                            "frac_of_hbm_peak": round(code_bytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                            "kernels_only_ms": round(ms_k, 4),
                            "kernels_only_frac_of_hbm_peak": round(code_bytes / ms_k / 1e6 / HBM_PEAK_GBS, 4),
                            "verified": ver}
        g.destroy()
        # the same step with the attention / FFN RMSNorms fused into the quantization of q,k,v and gate,up
        norms = []
        for li in range(layers_n):
            norms += [(nw[li][0], 1e-5, False)] * 3 + [None] + [(nw[li][1], 1e-5, False)] * 2 + [None]
        g = be.group(members, 1, "bf16", "bf16", norms=norms)
        ms = time_calls(be, lambda i: g.launch(), iters)
        res[f"batch{m}_rmsnorm_fused"] = {"ms_per_step_incl_norm_and_quant": round(ms, 4), "tokens_per_s": round(m / ms * 1e3, 1)}
        g.destroy()
        # the same projections in the order a decoder runs them, one dependent launch after the other: per layer the
        # q,k,v group (attention norm inside), o, the gate,up group (FFN norm inside), down -- 120 calls per step
        qkv, gu = [], []
        for li, L in enumerate(lins):
            base = li * 7
            qkv.append(be.group(members[base:base + 3], 1, "bf16", "bf16", norms=[(nw[li][0], 1e-5, False)] * 3))
            gu.append(be.group(members[base + 4:base + 6], 1, "bf16", "bf16", norms=[(nw[li][1], 1e-5, False)] * 2))

        def chain(_):
            for li, L in enumerate(lins):
                base = li * 7
                qkv[li].launch()
                be.linear_a8(L["o"], att, m, outs[base + 3])
                gu[li].launch()
                be.linear_a8(L["down"], mid, m, outs[base + 6])

        chain_ms = {}
        for label, fuse in (("two_launches_per_call", 0), ("default", -1)):
            be.set_fuse_tokens(fuse)
            chain_ms[label] = time_calls(be, chain, max(5, iters // 10))
        be.set_fuse_tokens(-1)
        res[f"batch{m}_layer_by_layer"] = {
            "ms_per_step": round(chain_ms["default"], 4), "tokens_per_s": round(m / chain_ms["default"] * 1e3, 1),
            "ms_per_step_with_every_call_as_two_launches": round(chain_ms["two_launches_per_call"], 4),
            "calls_per_step": 4 * layers_n}
        for grp in qkv + gu:
            grp.destroy()
        for x in outs + [hid, att, mid]:
            x.free()
    for L in lins:
        for l in L.values():
            l.free()
    for pair in nw:
        for w in pair:
            w.free()
    res["workload"] = ("30 layers x (q,k,v,o,gate,up,down), hidden 2560, FFN 6912, 20/5 heads of 128, 1 plane, "
                       "W1.58A8, bf16 in/out; 210 projections in one grouped launch on given inputs; "
                       "*_rmsnorm_fused: q,k,v and gate,up read RMSNorm(input), computed inside the quantization launch; "
                       "*_layer_by_layer: the same projections as 120 dependent calls in a decoder's order (q,k,v group with "
                       "its norm, o, gate,up group with its norm, down), launch-bound")
    res["code_bytes_per_step"] = code_bytes
    return res


def cpu_baseline(rng):
    """The CPU oracle (a restatement of tritium-cpu's dispatch: unpack per call, widest SIMD kernel,
    rows chunked across threads) on ONE pass of the headline sweep, on this host's cores."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib
    orc = oracle_lib.load()
    planes = [orc.pack_matrix(ternary(rng, N2, K2, p0), N2, K2, oracle_lib.FMT_TQ2_0) for p0 in (0.4, 0.7)]
    scs = [rng.uniform(0.01, 0.1, N2).astype(np.float32) for _ in range(PLANES2)]
    threads = min(os.cpu_count() or 1, 16)
    used_max, total_bytes, passes = 0, 0, 0
    acts = []
    for m in SWEEP:
        bits = f32_to_bf16_bits(rng.standard_normal((m, K2)).astype(np.float32))
        acts.append((bits.astype(np.uint32) << 16).view(np.float32).reshape(m, K2))
    t0 = time.perf_counter()
    while passes < 60 and time.perf_counter() - t0 < 9.0:  # a bounded sample: about 9 s of CPU work
        for m, act in zip(SWEEP, acts):
            out = None
            for p in range(PLANES2):
                o, used, _ = orc.cpu_mpgemm_fast(planes[p], oracle_lib.FMT_TQ2_0, act, scs[p], m, N2, K2, threads)
                out = o if out is None else out + o
                used_max = max(used_max, used)
            total_bytes += algorithmic_bytes(m, N2, K2, PLANES2, 2, 4)
        passes += 1
    dt = time.perf_counter() - t0
    res = {"value": round(total_bytes / dt / 1e9, 4), "unit": "GB/s", "cores": used_max, "kind": "port",
           "sample": f"{passes} passes of the sweep (batch {','.join(map(str, SWEEP))}) over ONE layer copy, "
                     f"{dt:.1f} s; C restatement of tritium-cpu (unpack per call, AVX-512 k-order f32 fold, rows "
                     f"chunked over threads: batch 1 gets a single worker, batch 16 gets {used_max})"}
    kernels = {0: "scalar", 1: "AVX2 f32 fold", 2: "AVX-512 f32 fold", 3: "AVX2 maddubs int8", 4: "AVX-VNNI dpbusd int8"}
    # configs[2]: what TernaryLinear::forward asks of tritium-cpu -- tokens quantized per token to int8 values, then
    # mpgemm, whose dispatch takes the integer kernel for such activations (crates/tritium-cpu/src/kernel.rs:577-664)
    m, k, n = 2048, 2560, 6912
    packed = orc.pack_matrix(ternary(rng, n, k, 0.4), n, k, oracle_lib.FMT_TQ2_0)
    sc = rng.uniform(0.01, 0.1, n).astype(np.float32)
    bits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    act = (bits.astype(np.uint32) << 16).view(np.float32).reshape(m, k)
    t0 = time.perf_counter()
    calls, used, kern = 0, 0, 0
    while calls < 20 and time.perf_counter() - t0 < 6.0:
        q, _ = orc.quantize_act_int8(act, m, k)
        _, used, kern = orc.cpu_mpgemm_fast(packed, oracle_lib.FMT_TQ2_0, np.ascontiguousarray(q, np.float32), sc, m, n, k, threads)
        calls += 1
    dt = time.perf_counter() - t0
    res["prefill_gemm"] = {"value": round(2.0 * m * n * k * calls / dt / 1e12, 4), "unit": "TOPS", "cores": used,
                           "kind": "port", "kernel": kernels.get(kern, str(kern)),
                           "sample": f"{calls} whole calls of M={m} K={k} N={n} (quantization, unpack and contraction), {dt:.1f} s"}
    # configs[3], batch 1: one token through q,k,v,o,gate,up,down of a layer; M = 1 gives the reference a single worker
    h, f, kv, sample_layers = 2560, 6912, 640, 2
    shapes = [(h, h), (kv, h), (kv, h), (h, h), (f, h), (f, h), (h, f)]
    layer = [(orc.pack_matrix(ternary(rng, nn, kk, 0.4), nn, kk, oracle_lib.FMT_TQ2_0), rng.uniform(0.01, 0.1, nn).astype(np.float32),
              nn, kk) for nn, kk in shapes]
    toks = {kk: np.ascontiguousarray(orc.quantize_act_int8(rng.standard_normal((1, kk)).astype(np.float32), 1, kk)[0], np.float32)
            for kk in (h, f)}
    t0 = time.perf_counter()
    done = 0
    while done < sample_layers or (time.perf_counter() - t0 < 4.0 and done < 30):
        for pk, scl, nn, kk in layer:
            _, used, kern = orc.cpu_mpgemm_fast(pk, oracle_lib.FMT_TQ2_0, toks[kk], scl, 1, nn, kk, threads)
        done += 1
    dt = time.perf_counter() - t0
    res["projection_stack_batch1"] = {"value": round(done / dt / 30.0, 3), "unit": "tokens/s", "cores": used, "kind": "port",
                                      "kernel": kernels.get(kern, str(kern)),
                                      "sample": f"{done} of the 30 layers' seven projections (tokens already int8-valued), {dt:.1f} s; "
                                                f"tokens/s = layers per second / 30"}
    return res


def summarize(out):
    """The five configurations in a few lines, as the LAST key of the record (a reader that keeps only the end of the
    line still has every headline figure): value, unit, fraction of the roofline that bounds it, kernel."""
    ex = out.get("extra", {})
    s = {"config2_decode_sweep_bf16": {"value": out["value"], "unit": "GB/s", "kernel_frac_of_hbm_peak": out["roofline"]["frac"],
                                       "kernel": "tk_flow_kernel / tk_flow32_kernel"}}
    c1 = ex.get("config1_f32_batch1")
    if c1:
        s["config1_batch1_f32"] = {"value": c1["step_GB/s_incl_digit_split"], "unit": "GB/s", "frac_of_hbm_peak": c1["step_frac_of_hbm_peak"],
                                   "kernel_frac_of_hbm_peak": c1["kernel_frac_of_hbm_peak"], "kernel": "tk_flow_kernel<1,1,2,2>"}
    a8 = ex.get("decode_sweep_int8_activations")
    if a8:
        s["config2_decode_sweep_int8_contract"] = {"value": a8["step_sweep_GB/s_incl_quant"], "unit": "GB/s",
                                                   "frac_of_hbm_peak": a8["step_frac_of_hbm_peak"],
                                                   "kernel_frac_of_hbm_peak": a8["kernel_frac_of_hbm_peak"]}
    pf = ex.get("prefill_gemm")
    if pf:
        s["config3_prefill"] = {"value": pf["TOPS"], "unit": "TOPS", "frac_of_int8_peak": pf["frac_of_int8_peak"],
                                "us_per_call_incl_quant": round(pf["ms_per_call_incl_quant"] * 1e3, 1), "kernel": pf.get("kernel")}
    st = ex.get("projection_stack")
    if st:
        s["config4_stack"] = {b: {"value": st[b]["tokens_per_s"], "unit": "tokens/s", "frac_of_hbm_peak": st[b]["frac_of_hbm_peak"]}
                              for b in ("batch1", "batch32") if b in st}
        for b in ("batch1", "batch32"):
            key = f"{b}_layer_by_layer"
            if key in st:
                s["config4_stack"][key] = {"value": st[key]["tokens_per_s"], "unit": "tokens/s"}
    c5 = ex.get("config5_three_planes")
    if c5:
        d = c5["decode_batch64"]
        s["config5"] = {"decode_batch64": {"value": d["GB/s"], "unit": "GB/s", "frac_of_hbm_peak": d["frac_of_hbm_peak"],
                                           "TOPS": d["kernels_only"]["TOPS"], "tokens_per_s": d["tokens_per_s"]}}
        for leg in ("prefill_4096_up", "prefill_4096_down"):
            if leg in c5:
                s["config5"][leg] = {"value": c5[leg]["TOPS"], "unit": "TOPS", "frac_of_int8_peak": c5[leg]["frac_of_int8_peak"]}
    cpu = out.get("cpu_baseline")
    if cpu:
        s["cpu_port"] = {"decode_sweep_GB/s": cpu["value"], "cores": cpu["cores"]}
        if "prefill_gemm" in cpu:
            s["cpu_port"]["prefill_TOPS"] = cpu["prefill_gemm"]["value"]
            s["cpu_port"]["prefill_cores"] = cpu["prefill_gemm"]["cores"]
        if "projection_stack_batch1" in cpu:
            s["cpu_port"]["stack_batch1_tokens_per_s"] = cpu["projection_stack_batch1"]["value"]
            s["cpu_port"]["stack_batch1_cores"] = cpu["projection_stack_batch1"]["cores"]
    return s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-extra", action="store_true", help="skip the legs under `extra`")
    ap.add_argument("--extra-legs", default="sweep_a8,config1,prefill,stack,config5,zero_skip,base3,salt,salt_v2,vjp,other_widths",
                    help="comma-separated subset of the `extra` legs to run (profiling runs name one)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain 1 GiB device copy kernel 3 times (scale for hardware traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the path would shard over output channels, each GPU "
                 "holding a slice of every plane, without any exchange); --gpus N with N > 1 is not supported.")
    import tritium_amd as T
    be = T.Mi355xBackend(0)
    info = be.info
    rng = np.random.default_rng(0)
    dec = bench_decode(T, be, args.steps, args.warmup, rng)
    out = {
        "metric": "decode GEMV HBM GB/s",
        "value": round(dec["value"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "prewarm_s": PREWARM_S,
        "ms_per_step": round(dec["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 MFMA (bf16 activations as 4 base-256 digits), int32 accumulate, f32 out",
        "data": "synthetic",
        "config": {"workload": f"two-plane additive ternary GEMV K={K2} N={N2}, P(0)=0.4/0.7, bf16 N(0,1) activations, "
                               f"per-channel f32 scales, batch sweep {','.join(map(str, SWEEP))}; one step = the sweep, "
                               f"each batch one launch over {COPIES} resident layer copies",
                   "copies": COPIES, "bytes_per_step": int(dec["bytes_per_launch_avg"] * len(SWEEP))},
        "roofline": {"bound": "hbm", "achieved": round(dec["kernel_gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dec["kernel_gbs"] / HBM_PEAK_GBS, 4), "traffic": DECODE_TRAFFIC_BYTES_PER_LAUNCH,
                     "kernel": "tk_flow_kernel<2,1,1,2> (batch 1), tk_flow_kernel<2,1,1,4> (batch 2), tk_flow_kernel<2,1,2,2> (batch 4), tk_flow32_kernel<2,1,2> (batch 8), tk_flow_kernel<2,4,2,2> (batch 16)", "avg_launch_ms": round(dec["kernel_avg_ms"], 4),
                     "algorithmic_bytes_per_launch": int(dec["bytes_per_launch_avg"])},
        "per_batch": dec["per_batch"],
        "verified": dec["verified"],
        "device": {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
                   "clock_mhz": info.clock_khz / 1000, "memory_clock_mhz": info.memory_clock_khz / 1000,
                   "memory_bus_bits": info.memory_bus_bits},
    }
    if args.copy_calibration:
        n = 1 << 30
        src, dst = be.empty(n // 4, "f32"), be.empty(n // 4, "f32")
        for _ in range(3):
            be.copy_kernel(dst, src, n)
        be.sync()
        src.free()
        dst.free()
    if not args.no_extra:
        legs = {"sweep_a8": ("decode_sweep_int8_activations", lambda: bench_sweep_a8(T, be, rng)),
                "config1": ("config1_f32_batch1", lambda: bench_config1(T, be, rng)),
                "prefill": ("prefill_gemm", lambda: bench_prefill(T, be, rng, 2048, 2560, 6912)),
                "stack": ("projection_stack", lambda: bench_stack(T, be, rng)),
                "config5": ("config5_three_planes", lambda: bench_config5(T, be, rng)),
                "zero_skip": ("zero_chunk_skip", lambda: bench_zero_skip(T, be, rng)),
                "base3": ("base3_stream_vs_two_bit", lambda: bench_base3(T, be, rng)),
                "salt": ("block_scale_planes", lambda: bench_salt(T, be, rng)),
                "salt_v2": ("salt_v2_exact", lambda: bench_salt_v2(T, be, rng)),
                "vjp": ("projected_vjp", lambda: bench_vjp(T, be, rng)),
                "other_widths": ("decode_other_widths", lambda: bench_other_widths(T, be, rng))}
        out["extra"] = {}
        for leg in [x for x in args.extra_legs.split(",") if x]:
            if leg not in legs:
                sys.exit(f"bench.py: unknown leg `{leg}` (choose from {','.join(legs)})")
            out["extra"][legs[leg][0]] = legs[leg][1]()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(np.random.default_rng(1))
    be.close()
    out["summary"] = summarize(out)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
