"""Host mirror of the caller of the path: `TernaryLinear` (crates/tritium-nn/src/layers/linear.rs:38-280).

`new` / `with_row_scales` pack rows with block scale 1.0 and upload once; `forward` is the W1.58A8
linear. Where the reference quantizes on the host and calls `mpgemm`, this goes through the fused
`mpgemm_with_act_quant`, whose result is bit-identical to that composition.
"""
import os

import numpy as np

from .backend import (GemmShape, InvalidInput, MpGemm, ShapeMismatch, TernaryFormat, pack_rows)


def weights_format():
    """`TRITIUM_WEIGHTS=tq1|tq2`, anything else rejected loudly (linear.rs:60-72)."""
    v = os.environ.get("TRITIUM_WEIGHTS")
    if v is None or v in ("tq2", ""):
        return TernaryFormat.Tq2_0
    if v == "tq1":
        return TernaryFormat.Tq1_0
    raise InvalidInput(f"TRITIUM_WEIGHTS={v!r} — use tq1 or tq2")


class TernaryLinear:
    def __init__(self, backend, trits, n_out, k_in, scales):
        trits = np.ascontiguousarray(trits, dtype=np.int8).reshape(-1)
        if trits.size != n_out * k_in:
            raise ShapeMismatch(n_out * k_in, trits.size)
        if k_in == 0:
            raise ShapeMismatch(1, 0)
        scales = np.ascontiguousarray(scales, dtype=np.float32).reshape(-1)
        if scales.size != n_out:
            raise ShapeMismatch(n_out, scales.size)
        self.n_out, self.k_in, self.scales = n_out, k_in, scales
        self.format = weights_format()
        packed = pack_rows(trits, n_out, k_in, self.format)
        self.weights = backend.upload_weights(packed, GemmShape(0, n_out, k_in), self.format)

    @classmethod
    def new(cls, backend, trits, n_out, k_in, weight_scale):
        return cls(backend, trits, n_out, k_in, np.full(n_out, weight_scale, np.float32))

    @classmethod
    def with_row_scales(cls, backend, trits, n_out, k_in, scales):
        return cls(backend, trits, n_out, k_in, scales)

    def replace_weights(self, backend, trits, scales):
        new = TernaryLinear(backend, trits, self.n_out, self.k_in, scales)
        self.weights, self.scales = new.weights, new.scales

    def shape(self, m):
        return GemmShape(m, self.n_out, self.k_in)

    def forward(self, backend, act, m, out):
        act = np.ascontiguousarray(act, dtype=np.float32).reshape(-1)
        if act.size != m * self.k_in:
            raise ShapeMismatch(m * self.k_in, act.size)
        if out.size != m * self.n_out:
            raise ShapeMismatch(m * self.n_out, out.size)
        backend.mpgemm_with_act_quant(MpGemm(act=act, weights=self.weights, scales=self.scales,
                                             shape=self.shape(m), format=self.format, out=out))
