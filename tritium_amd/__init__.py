"""tritium_amd — MI355X (gfx950) backend for Tritium's packed ternary linear layer.

The HIP kernel library (libtritium_mi355x.so, C ABI in include/tritium_mi355x.h) is the product;
this package is the thin host mirror of the reference's adapter interface over it.
"""
from . import _lib
from .backend import (BACKENDS, Backend, BackendEntry, BackendError, DeviceArray, DeviceBuffer, DeviceCaps,
                      GemmShape, InvalidInput, Linear, Mi355xBackend, Mi355xBuffer, MpGemm, MpGemmProjectedVjp, OutOfMemory,
                      Registry, ShapeMismatch, TernaryFormat, UnsupportedFormat, compute_zero_bitmaps, convert_i2s_to_tq2_0,
                      pack_rows, packed_len, unpack_rows,
                      SALT_V2_B3, SALT_V2_D2, SALT_V2_S34, SaltV2Tensor, salt_row_len, salt_row_unpack, salt_v2_pack,
                      salt_v2_payload_bytes, salt_v2_unpack, sparse_plane_to_tq2_0)
from .gguf import GgufError, GgufErrorKind, GgufFile, TensorInfo, read_gguf
from .linear import TernaryLinear

__all__ = [n for n in dir() if not n.startswith("_")]
