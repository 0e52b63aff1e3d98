"""ctypes binding of libtritium_mi355x.so (the C ABI in include/tritium_mi355x.h).

The library is required: there is no CPU fallback. If it has not been built, importing raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TRITIUM_MI355X_LIB") or os.path.join(HERE, "libtritium_mi355x.so")

TK_OK, TK_ERR_SHAPE_MISMATCH, TK_ERR_UNSUPPORTED_FORMAT, TK_ERR_OUT_OF_MEMORY, TK_ERR_INVALID_INPUT, TK_ERR_BACKEND = range(6)
TK_F32, TK_BF16, TK_I8, TK_I32 = range(4)
TK_MAX_PLANES = 4
TK_GROUP_FLOAT, TK_GROUP_A8 = 0, 1

vp = C.c_void_p
sz = C.c_size_t


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 32), ("total_memory_bytes", C.c_uint64),
                ("compute_units", C.c_int), ("clock_khz", C.c_int), ("memory_clock_khz", C.c_int),
                ("memory_bus_bits", C.c_int), ("wavefront_size", C.c_int), ("lds_bytes_per_cu", C.c_int)]


class LinearDesc(C.Structure):
    _fields_ = [("planes", vp * TK_MAX_PLANES), ("scales", vp * TK_MAX_PLANES), ("n_planes", C.c_int)]


class GroupMember(C.Structure):
    _fields_ = [("layer", LinearDesc), ("act", vp), ("m", sz), ("out", vp)]


class SaltDesc(C.Structure):
    _fields_ = [("planes", vp * TK_MAX_PLANES), ("n_planes", C.c_int)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_uint32), ("dims", C.c_uint64 * 8), ("ggml_type", C.c_uint32),
                ("offset", C.c_uint64), ("n_bytes", C.c_uint64)]


class RmsNorm(C.Structure):
    _fields_ = [("weight", vp), ("eps", C.c_float), ("zero_centered", C.c_int)]


# every symbol include/tritium_mi355x.h declares: (restype, argtypes)
SIGNATURES = {
    "tk_init": (C.c_int, [C.c_int, C.POINTER(vp)]),
    "tk_destroy": (None, [vp]),
    "tk_last_error": (C.c_char_p, []),
    "tk_last_mismatch": (None, [C.POINTER(sz), C.POINTER(sz)]),
    "tk_device_id": (C.c_char_p, [vp]),
    "tk_device_info_get": (C.c_int, [vp, C.POINTER(DeviceInfo)]),
    "tk_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "tk_packed_len": (sz, [sz, sz, C.c_int]),
    "tk_pack_rows": (C.c_int, [vp, sz, sz, sz, C.c_int, vp, sz]),
    "tk_unpack_rows": (C.c_int, [vp, sz, sz, sz, C.c_int, vp, sz]),
    "tk_compute_zero_bitmaps": (C.c_int, [vp, sz, sz, sz, sz, vp, sz]),
    "tk_upload_weights": (C.c_int, [vp, vp, sz, sz, sz, C.c_int, C.POINTER(vp)]),
    "tk_free_weights": (None, [vp]),
    "tk_weights_len_bytes": (sz, [vp]),
    "tk_weights_n": (sz, [vp]),
    "tk_weights_k": (sz, [vp]),
    "tk_weights_format": (C.c_int, [vp]),
    "tk_set_zero_skip": (C.c_int, [vp, C.c_int]),
    "tk_set_flow_operand_order": (C.c_int, [vp, C.c_int]),
    "tk_set_flow_workgroup_waves": (C.c_int, [vp, C.c_int]),
    "tk_set_prep_team_rows": (C.c_int, [vp, C.c_int]),
    "tk_set_gemm_two_by_two": (C.c_int, [vp, C.c_int]),
    "tk_set_base3_stream": (C.c_int, [vp, C.c_int]),
    "tk_weights_base3_bytes": (sz, [vp]),
    "tk_weights_zero_chunks": (C.c_int, [vp, C.POINTER(sz), C.POINTER(sz), C.POINTER(C.c_int)]),
    "tk_weights_download_trits": (C.c_int, [vp, vp, vp, sz]),
    "tk_mpgemm": (C.c_int, [vp, vp, sz, vp, vp, sz, sz, sz, sz, C.c_int, vp, sz]),
    "tk_mpgemm_with_act_quant": (C.c_int, [vp, vp, sz, vp, vp, sz, sz, sz, sz, C.c_int, vp, sz]),
    "tk_mpgemm_projected_vjp": (C.c_int, [vp, vp, sz, vp, vp, sz, vp, sz, sz, sz, sz, C.c_int, vp, sz, vp, sz, vp, sz]),
    "tk_projected_vjp": (C.c_int, [vp, vp, vp, vp, vp, sz, vp, vp, vp]),
    "tk_act_quant_i8": (C.c_int, [vp, vp, C.c_int, sz, sz, vp, vp, vp]),
    "tk_linear_float": (C.c_int, [vp, C.POINTER(LinearDesc), vp, C.c_int, sz, vp, C.c_int]),
    "tk_i2s_payload_len": (sz, [sz, sz]),
    "tk_convert_i2s_to_tq2_0": (C.c_int, [vp, sz, sz, sz, vp, sz, C.POINTER(C.c_float)]),
    "tk_upload_weights_i2s": (C.c_int, [vp, vp, sz, sz, sz, C.POINTER(vp), C.POINTER(C.c_float)]),
    "tk_gguf_open": (C.c_int, [vp, sz, C.POINTER(vp), C.POINTER(C.c_int), C.POINTER(C.c_uint64)]),
    "tk_gguf_close": (None, [vp]),
    "tk_gguf_version": (C.c_uint32, [vp]),
    "tk_gguf_alignment": (C.c_uint64, [vp]),
    "tk_gguf_tensor_data_offset": (C.c_uint64, [vp]),
    "tk_gguf_tensor_count": (sz, [vp]),
    "tk_gguf_metadata_count": (sz, [vp]),
    "tk_gguf_tensor_at": (C.c_int, [vp, sz, C.POINTER(GgufTensor)]),
    "tk_gguf_tensor_find": (C.c_int, [vp, C.c_char_p, C.POINTER(GgufTensor)]),
    "tk_gguf_meta_type": (C.c_int, [vp, C.c_char_p, C.c_longlong, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                                    C.POINTER(C.c_uint64)]),
    "tk_gguf_meta_u64": (C.c_int, [vp, C.c_char_p, C.c_longlong, C.POINTER(C.c_uint64)]),
    "tk_gguf_meta_i64": (C.c_int, [vp, C.c_char_p, C.c_longlong, C.POINTER(C.c_int64)]),
    "tk_gguf_meta_f64": (C.c_int, [vp, C.c_char_p, C.c_longlong, C.POINTER(C.c_double)]),
    "tk_gguf_meta_f32": (C.c_int, [vp, C.c_char_p, C.c_longlong, C.POINTER(C.c_float)]),
    "tk_gguf_meta_bool": (C.c_int, [vp, C.c_char_p, C.c_longlong, C.POINTER(C.c_int)]),
    "tk_gguf_meta_str": (C.c_int, [vp, C.c_char_p, C.c_longlong, C.POINTER(C.c_char_p), C.POINTER(sz)]),
    "tk_gguf_element_count": (C.c_int, [C.POINTER(GgufTensor), C.POINTER(C.c_uint64)]),
    "tk_gguf_tensor_payload": (C.c_int, [vp, sz, C.POINTER(GgufTensor), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "tk_gguf_ternary_shape": (C.c_int, [vp, C.c_char_p, C.POINTER(sz), C.POINTER(sz), C.POINTER(C.c_int)]),
    "tk_gguf_load_ternary": (C.c_int, [vp, vp, sz, C.c_char_p, vp, sz, vp, sz]),
    "tk_upload_weights_gguf": (C.c_int, [vp, vp, vp, sz, C.c_char_p, C.POINTER(vp), vp, sz]),
    "tk_upload_weights_scaled": (C.c_int, [vp, vp, sz, sz, sz, C.POINTER(vp)]),
    "tk_salt_row_len": (C.c_int, [vp, sz, C.POINTER(sz)]),
    "tk_salt_row_info": (C.c_int, [vp, sz, C.POINTER(sz), C.POINTER(sz), C.POINTER(C.c_int)]),
    "tk_salt_row_unpack": (C.c_int, [vp, sz, sz, vp, sz, C.POINTER(sz), C.POINTER(sz)]),
    "tk_sparse_plane_to_tq2_0": (C.c_int, [vp, sz, vp, sz, C.POINTER(sz)]),
    "tk_upload_salt_rows": (C.c_int, [vp, vp, sz, sz, sz, sz, C.POINTER(vp), C.POINTER(C.c_int)]),
    "tk_salt_v2_payload_bytes": (C.c_int, [C.c_int, sz, C.POINTER(sz)]),
    "tk_salt_v2_pack": (C.c_int, [C.c_int, vp, sz, vp, sz]),
    "tk_salt_v2_unpack": (C.c_int, [C.c_int, vp, sz, sz, vp]),
    "tk_salt_v2_upload": (C.c_int, [vp, C.c_int, sz, vp, sz, vp, sz, vp, sz, sz, sz, C.POINTER(vp)]),
    "tk_salt_v2_free": (None, [vp]),
    "tk_salt_v2_forward": (C.c_int, [vp, vp, vp, sz, vp]),
    "tk_salt_v2_gather_rows": (C.c_int, [vp, vp, vp, sz, vp]),
    "tk_linear_salt": (C.c_int, [vp, C.POINTER(SaltDesc), vp, C.c_int, sz, vp, C.c_int]),
    "tk_linear_salt_seq": (C.c_int, [vp, C.POINTER(SaltDesc), vp, C.c_int, sz, vp, C.c_int]),
    "tk_linear_a8": (C.c_int, [vp, C.POINTER(LinearDesc), vp, C.c_int, sz, vp, C.c_int]),
    "tk_linear_a8_noalloc": (C.c_int, [vp, C.POINTER(LinearDesc), vp, C.c_int, sz, vp, C.c_int]),
    "tk_rmsnorm_quant_i8": (C.c_int, [vp, vp, C.c_int, C.POINTER(RmsNorm), sz, sz, vp, vp, vp]),
    "tk_linear_rmsnorm_a8": (C.c_int, [vp, C.POINTER(LinearDesc), vp, C.c_int, C.POINTER(RmsNorm), sz, vp, C.c_int]),
    "tk_group_create_normed": (C.c_int, [vp, C.POINTER(GroupMember), C.POINTER(RmsNorm), sz, C.c_int, C.c_int,
                                         C.POINTER(vp)]),
    "tk_linear_i8": (C.c_int, [vp, C.POINTER(LinearDesc), vp, vp, sz, vp, C.c_int]),
    "tk_linear_a8_residual": (C.c_int, [vp, C.POINTER(LinearDesc), vp, C.c_int, sz, vp, vp, C.c_int]),
    "tk_linear_i8_residual": (C.c_int, [vp, C.POINTER(LinearDesc), vp, vp, sz, vp, vp, C.c_int]),
    "tk_linear_float_seq": (C.c_int, [vp, C.POINTER(LinearDesc), vp, C.c_int, sz, vp, C.c_int]),
    "tk_group_create": (C.c_int, [vp, C.POINTER(GroupMember), sz, C.c_int, C.c_int, C.c_int, C.POINTER(vp)]),
    "tk_group_launch": (C.c_int, [vp, vp]),
    "tk_group_launch_parts": (C.c_int, [vp, vp, C.c_int, C.c_int]),
    "tk_group_destroy": (None, [vp]),
    "tk_set_gemm_min_m": (C.c_int, [vp, C.c_int]),
    "tk_get_gemm_min_m": (C.c_int, [vp]),
    "tk_set_decode_kernel": (C.c_int, [vp, C.c_int]),
    "tk_set_flow_run_tiles": (C.c_int, [vp, C.c_int]),
    "tk_set_flow_ring": (C.c_int, [vp, C.c_int]),
    "tk_set_flow_mfma": (C.c_int, [vp, C.c_int]),
    "tk_set_gemm_tiles": (C.c_int, [vp, C.c_int]),
    "tk_set_gemm_ksplit": (C.c_int, [vp, C.c_int]),
    "tk_set_gemm_rows": (C.c_int, [vp, C.c_int]),
    "tk_set_gemm256_form": (C.c_int, [vp, C.c_int]),
    "tk_set_fuse_tokens": (C.c_int, [vp, C.c_int]),
    "tk_set_host_direct_bytes": (C.c_int, [vp, C.c_size_t]),
    "tk_get_fused_calls": (C.c_int, [vp, C.POINTER(C.c_ulonglong)]),
    "tk_last_kernel": (C.c_char_p, [vp]),
    "tk_set_group_overlap": (C.c_int, [vp, C.c_int]),
    "tk_set_stream_min_groups": (C.c_int, [vp, C.c_int]),
    "tk_get_stream_min_groups": (C.c_int, [vp]),
    "tk_set_exact_max_macs": (C.c_int, [vp, sz]),
    "tk_get_exact_max_macs": (sz, [vp]),
    "tk_malloc": (C.c_int, [vp, sz, C.POINTER(vp)]),
    "tk_free": (C.c_int, [vp, vp]),
    "tk_memcpy_h2d": (C.c_int, [vp, vp, vp, sz]),
    "tk_memcpy_d2h": (C.c_int, [vp, vp, vp, sz]),
    "tk_memset": (C.c_int, [vp, vp, C.c_int, sz]),
    "tk_sync": (C.c_int, [vp]),
    "tk_stream": (vp, [vp]),
    "tk_event_create": (C.c_int, [vp, C.POINTER(vp)]),
    "tk_event_record": (C.c_int, [vp, vp]),
    "tk_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
    "tk_event_destroy": (None, [vp]),
    "tk_copy_kernel": (C.c_int, [vp, vp, vp, sz]),
}

_lib = None


def load():
    """Load the library and bind every declared symbol. Raises if it is missing or incomplete."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -m tritium_amd.build` (hipcc, gfx950). "
            "This package has no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError names the missing symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
