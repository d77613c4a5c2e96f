"""ctypes binding of kvcomp_amd/lib/libkvcomp_hip.so (the C ABI of include/kvcomp_hip.h).

There is no CPU fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libkvcomp_hip.so")
_LIB = None

_i64, _int, _vp, _f32p, _u32 = C.c_int64, C.c_int, C.c_void_p, C.POINTER(C.c_float), C.c_uint32
_i64p, _intp = C.POINTER(C.c_int64), C.POINTER(C.c_int)

class CompressedDesc(C.Structure):
    """kvc_compressed_desc of include/kvcomp_hip.h."""
    _fields_ = [("d_luts", C.c_void_p), ("rows_per_codebook", C.c_int64),
                ("d_block_infos", C.c_void_p), ("block_infos_bytes", C.c_int64),
                ("d_thread_infos", C.c_void_p), ("thread_infos_bytes", C.c_int64),
                ("d_encoded", C.c_void_p), ("encoded_bytes", C.c_int64),
                ("d_quant_min_ints", C.c_void_p), ("d_quant_scales_f16", C.c_void_p),
                ("quant_mask", C.c_int64), ("max_tile_bytes", C.c_int64), ("max_stream_bytes", C.c_int64),
                ("max_code_bits", C.c_int64), ("tokens", C.c_int64),
                ("d_tail_f16", C.c_void_p), ("tail_tokens", C.c_int64)]


class EncodeJob(C.Structure):
    """kvc_encode_job of include/kvcomp_hip.h."""
    _fields_ = [("is_k", C.c_int32), ("quant_mask", C.c_int32), ("d_sym", C.c_void_p), ("d_x_f16", C.c_void_p),
                ("eb", C.c_float), ("d_min_i8", C.c_void_p), ("d_scale_f16", C.c_void_p),
                ("tokens", C.c_int64), ("batch", C.c_int64), ("heads", C.c_int64), ("head_dim", C.c_int64),
                ("d_encode_tables", C.c_void_p), ("encode_table_bytes", C.c_int64), ("table_stride_bytes", C.c_int64),
                ("rows_per_codebook", C.c_int64), ("d_codebook_meta", C.c_void_p),
                ("d_block_infos", C.c_void_p), ("d_thread_infos", C.c_void_p), ("d_encoded", C.c_void_p),
                ("encoded_cap", C.c_int64), ("base_global_offset", C.c_uint32),
                ("d_stream_bytes", C.c_void_p), ("d_result", C.c_void_p)]


# name -> argtypes (every function returns int unless listed in _RESTYPES)
_SIGNATURES = {
    "kvc_abi_version": [],
    "kvc_set_option": [C.c_char_p, _int],
    "kvc_get_option": [C.c_char_p, _intp],
    "kvc_calculate_buffer_size": [_i64, _i64, _int, _i64, _i64, _i64p],
    "kvc_histogram": [_vp, _i64, _vp, _vp],
    "kvc_build_codebook_host": [_i64p, _int, _intp, _vp, _i64, _i64p, _vp, _i64, _i64p],
    "kvc_codebook_tree_capacity": [_int],
    "kvc_histogram_chunks": [_vp, _i64, _i64, _vp, _vp],
    "kvc_build_codebook_device": [_vp, _i64, _int, _vp, _vp, _vp, _vp],
    "kvc_k_entropy_encode": [_vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _u32, _i64, _i64, _i64p, _i64p, _i64p, _vp],
    "kvc_v_entropy_encode": [_vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _u32, _i64, _i64, _i64p, _i64p, _i64p, _vp],
    "kvc_store_fused_supported": [_int, _int, _i64, _i64, _i64],
    "kvc_store_fused": [_int, _vp, _i64, _i64, _i64, _i64, _int, C.c_float, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64,
                        _u32, _i64p, _i64p, _i64p, _vp],
    "kvc_encode_async": [C.POINTER(EncodeJob), _vp],
    "kvc_encode_result": [_vp, _i64, _i64p, _i64p, _i64p, _i64p, _vp],
    "kvc_k_entropy_decode": [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _int, _vp, _i64, _i64, _i64, _i64, _f32p, _vp],
    "kvc_v_entropy_decode": [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _int, _vp, _i64, _i64, _i64, _i64, _f32p, _vp],
    "kvc_decode_dequant": [_int, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _int, _vp, _vp, _int, _i64, _vp, _i64, _i64, _i64,
                           _i64, _f32p, _vp],
    "kvc_k_decode_and_mat_vec_mul": [_vp, _i64, _int, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _int, _vp, _vp,
                                     _i64, _i64, _i64, _i64, _i64, _f32p, _vp],
    "kvc_v_decode_and_mat_vec_mul": [_vp, _i64, _int, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _int, _vp, _vp,
                                     _i64, _i64, _i64, _i64, _i64, _f32p, _vp],
    "kvc_lut_bytes": [],
    "kvc_build_lut": [_vp, _i64, _int, _i64, _i64, _vp, _vp],
    "kvc_k_scores_lut": [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64,
                         _int, _i64, _i64, _i64, _i64, _i64, _f32p, _vp],
    "kvc_v_partials_lut": [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _int, _vp, _vp, _int, _i64, _i64,
                           _int, _i64, _i64, _i64, _i64, _i64, _f32p, _vp],
    "kvc_k_mat_vec_mul": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32p, _vp],
    "kvc_quant_groups": [_i64, _i64, _i64, _i64, _i64, _int],
    "kvc_quant": [_vp, _i64, _i64, _i64, _i64, _i64, _int, C.c_float, _vp, _vp, _vp, _vp, _vp, _vp],
    "kvc_quant_error": [_vp, _i64, _i64, _i64, _i64, _i64, _int, C.c_float, _vp, _vp],
    "kvc_calibration_copy": [_vp, _vp, _i64, _vp],
    "kvc_h2_codes": [_i64p, _vp, _vp],
    "kvc_h2_scratch_bytes": [_i64],
    "kvc_h2_encode": [_vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _i64p, _vp],
    "kvc_attention_workspace_bytes": [_i64, _i64, _i64, _i64, _i64],
    "kvc_attention_decode": [C.POINTER(CompressedDesc), C.POINTER(CompressedDesc), _vp, C.c_float, _vp, _i64, _vp,
                             _i64, _i64, _i64, _i64, _f32p, _f32p, _vp],
    "kvc_attention_decode_static": [C.POINTER(CompressedDesc), C.POINTER(CompressedDesc), _vp, C.c_float, _vp,
                                    _i64, _i64, _i64, _i64, _vp],
    "kvc_dequant": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp],
}
_RESTYPES = {"kvc_quant_groups": _i64, "kvc_lut_bytes": _i64, "kvc_codebook_tree_capacity": _i64, "kvc_attention_workspace_bytes": _i64,
             "kvc_h2_scratch_bytes": _i64}

EXPORTED_SYMBOLS = sorted(list(_SIGNATURES) + ["kvc_last_error"])


class KvcompError(RuntimeError):
    pass


def lib():
    """Load the shared library (once).  Raises if it has not been built: there is no other code path."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise KvcompError("%s is missing: build it with `python -m kvcomp_amd.build` "
                              "(this package has no CPU fallback)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        L.kvc_last_error.restype = C.c_char_p
        L.kvc_last_error.argtypes = []
        for name, args in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _RESTYPES.get(name, _int)
        _LIB = L
    return _LIB


def set_option(name: str, value: int) -> int:
    """Set a tuning knob of the library (see include/kvcomp_hip.h); returns the previous value."""
    old = C.c_int(0)
    check(lib().kvc_get_option(name.encode(), C.byref(old)))
    check(lib().kvc_set_option(name.encode(), int(value)))
    return old.value


def check(rc):
    if rc != 0:
        raise KvcompError(lib().kvc_last_error().decode("utf-8", "replace") or "libkvcomp_hip call failed (%d)" % rc)
