"""ctypes binding of libmiq.so (the C ABI declared in include/miq.h).

The library is the only compute path of this package: if it has not been built the import fails with an error that
says how to build it.  There is no CPU or eager-PyTorch fallback.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmiq.so")

OK = 0
ROUND_NEAREST, ROUND_STOCHASTIC = 0, 1
QUANTIZATION_TF, QUANTIZATION_TF_ENHANCED = 0, 1
PDF_SIZE = 512


class MiqError(RuntimeError):
    """A libmiq entry point returned a non-zero status."""


class Encoding(C.Structure):
    """struct miq_encoding == DlQuantization::TfEncoding"""
    _fields_ = [("min", C.c_double), ("max", C.c_double), ("delta", C.c_double), ("offset", C.c_double),
                ("bw", C.c_int)]


class QdqSegment(C.Structure):
    """struct miq_qdq_segment: one tensor of a multi-tensor quantize-dequantize launch"""
    _fields_ = [("in_", C.c_void_p), ("out", C.c_void_p), ("num_element", C.c_int64), ("num_channel", C.c_int64),
                ("num_element_per_channel", C.c_int64), ("enc_min", C.c_void_p), ("enc_max", C.c_void_p),
                ("enc_delta", C.c_void_p), ("enc_offset", C.c_void_p), ("fd_magic", C.c_uint32),
                ("fd_shift", C.c_uint32), ("first_tile", C.c_int32), ("reserved", C.c_int32)]


_p = C.c_void_p
_i64 = C.c_int64
_int = C.c_int
_dbl = C.c_double
_flt = C.c_float

_SIGNATURES = {
    "miq_version": ([], _int),
    "miq_init": ([], _int),
    "miq_last_error": ([], C.c_char_p),
    "miq_fill_encoding_info": ([_int, _dbl, _dbl, C.POINTER(Encoding)], _int),
    "miq_get_computed_encodings": ([_int, _dbl, _dbl, _int, _int, _int, C.POINTER(Encoding)], _int),
    "miq_qdq_per_tensor_f32": ([_p, _p, _i64, _dbl, _dbl, _int, _int, _p], _int),
    "miq_qdq_per_tensor_bf16": ([_p, _p, _i64, _dbl, _dbl, _int, _int, _p], _int),
    "miq_quantize_per_tensor_f32": ([_p, _p, _i64, _dbl, _dbl, _int, _int, _int, _p], _int),
    "miq_qdq_codes_per_tensor_f32": ([_p, _p, _p, _i64, _dbl, _dbl, _int, _int, _p], _int),
    "miq_tf_encodings_per_channel_f32": ([_p, _p, _i64, _int, _int, _int, _int, _p, _p, _p, _p, _p, _p, _p, _p], _int),
    "miq_per_channel_params_f32": ([_p, _p, _i64, _dbl, _p, _p, _p, _p, _p], _int),
    "miq_qdq_per_channel_f32": ([_p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _int, _p], _int),
    "miq_qdq_per_channel_bf16": ([_p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _int, _p], _int),
    "miq_qdq_codes_per_channel_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _int, _int, _p], _int),
    "miq_qdq_broadcast_f32": ([_p, _p, _i64, _i64, C.POINTER(_i64), C.POINTER(_i64), _p, _p, _p, _p, _p], _int),
    "miq_ste_bwd_per_tensor_f32": ([_p, _p, _p, _i64, _flt, _flt, _p], _int),
    "miq_ste_bwd_per_tensor_bf16": ([_p, _p, _p, _i64, _flt, _flt, _p], _int),
    "miq_ste_bwd_per_channel_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _p], _int),
    "miq_ste_bwd_per_channel_bf16": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _p], _int),
    "miq_qdq_multi_plan": ([C.POINTER(QdqSegment), _int, _int], _i64),
    "miq_qdq_per_channel_multi_f32": ([_p, _int, _i64, _p], _int),
    "miq_qdq_per_channel_multi_bf16": ([_p, _int, _i64, _p], _int),
    "miq_ste_mask_bytes": ([_i64, _int], _i64),
    "miq_qdq_mask_per_tensor_f32": ([_p, _p, _p, _i64, _dbl, _dbl, _int, _flt, _flt, _p], _int),
    "miq_qdq_mask_per_tensor_bf16": ([_p, _p, _p, _i64, _dbl, _dbl, _int, _flt, _flt, _p], _int),
    "miq_qdq_mask_per_channel_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p, _p], _int),
    "miq_qdq_mask_per_channel_bf16": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p, _p], _int),
    "miq_v2_qdq_mask_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p], _int),
    "miq_v2_qdq_mask_bf16": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p], _int),
    "miq_ste_bwd_mask_f32": ([_p, _p, _p, _i64, _p], _int),
    "miq_ste_bwd_mask_bf16": ([_p, _p, _p, _i64, _p], _int),
    "miq_v2_qdq_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p], _int),
    "miq_v2_qdq_bf16": ([_p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p], _int),
    "miq_v2_qdq_bwd_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p], _int),
    "miq_v2_qdq_bwd_bf16": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p], _int),
    "miq_v2_qdq_bwd_params_workspace_bytes": ([_i64, _i64, _i64], _i64),
    "miq_v2_qdq_bwd_params_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p, _p, _p, _p], _int),
    "miq_v2_qdq_bwd_params_bf16": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _int, _int, _p, _p, _p, _p], _int),
    "miq_adaround_recon_grad_f32": ([_p, _p, _p, _i64, _i64, _i64, _int, C.c_float, _p, _p], _int),
    "miq_range_to_grid_f32": ([_p, _p, _i64, _int, _int, _int, _int, _p, _p], _int),
    "miq_qdq_bwd_range_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _int, _int, _int, _p, _p, _p, _p], _int),
    "miq_qdq_bwd_range_bf16": ([_p, _p, _p, _i64, _i64, _i64, _p, _int, _int, _int, _p, _p, _p, _p], _int),
    "miq_fp16_round_trip_f32": ([_p, _p, _i64, _p], _int),
    "miq_bf16_round_trip_f32": ([_p, _p, _i64, _p], _int),
    "miq_fp8_fake_cast_f32": ([_p, _p, _i64, _i64, _i64, _p, _p, _p, _int, _p], _int),
    "miq_float_fake_cast_f32": ([_p, _p, _i64, _i64, _i64, _p, _p, _p, _int, _p], _int),
    "miq_set_stochastic_seed": ([C.c_uint64], _int),
    "miq_get_stochastic_state": ([C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)], _int),
    "miq_minmax_workspace_bytes": ([_i64, _i64, _i64], _i64),
    "miq_minmax_f32": ([_p, _i64, _p, _p, _p], _int),
    "miq_minmax_per_channel_f32": ([_p, _i64, _i64, _i64, _p, _p, _p], _int),
    "miq_minmax_per_channel_static_f32": ([_p, _i64, _i64, _i64, _p, _p], _int),
    "miq_analyzer_create": ([_int, C.POINTER(_p)], _int),
    "miq_analyzer_state_bytes": ([], _i64),
    "miq_analyzer_create_in": ([_int, _p, C.POINTER(_p)], _int),
    "miq_analyzer_set_percentile": ([_p, C.c_float], _int),
    "miq_analyzer_destroy": ([_p], _int),
    "miq_analyzer_reset": ([_p, _p], _int),
    "miq_analyzer_update_stats_f32": ([_p, _p, _i64, _p], _int),
    "miq_analyzer_queue_encoding": ([_p, _int, _int, _int, _int, _p], _int),
    "miq_analyzer_compute_encoding": ([_p, _int, _int, _int, _int, C.POINTER(Encoding), C.POINTER(_int), _p], _int),
    "miq_analyzer_get_stats_histogram": ([_p, _p, _p, C.POINTER(_int), _p], _int),
    "miq_column_error_splits": ([_i64, _i64, _i64], _i64),
    "miq_column_error_f32": ([_p, _p, _i64, _i64, _i64, _int, _i64, _p, _p], _int),
    "miq_analyzer_entropy_histogram": ([_p, _p, _p, C.POINTER(_int), C.POINTER(_int), _p], _int),
    "miq_analyzer_last_batch_counts": ([_p, _p, _p], _int),
    "miq_analyzer_last_search": ([_p, _p, _p, _p, _int, C.POINTER(_int), C.POINTER(_int), _p], _int),
    "miq_adaround_soft_round_f32": ([_p, _p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _int, _p], _int),
    "miq_adaround_floor_f32": ([_p, _p, _i64, _i64, _i64, _p, _p], _int),
    "miq_adaround_floor_i8": ([_p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _p, _p], _int),
    "miq_adaround_floor_i16": ([_p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _p, _p], _int),
    "miq_adaround_init_alpha_f32": ([_p, _p, _i64, _i64, _i64, _p, _p], _int),
    "miq_adaround_bwd_adam_f32": ([_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _dbl, _dbl, _dbl,
                                   _dbl, _dbl, _dbl, _int, _p, _p], _int),
    "miq_adaround_bwd_f32": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _dbl, _dbl, _p, _p], _int),
    "miq_adaround_blocks": ([_i64], _int),
    "miq_adaround_eval_terms_f32": ([_p, _p, _i64, _int, _dbl, _p], _int),
    "miq_v2_hist_workspace_bytes": ([_i64, _i64, _int], _i64),
    "miq_v2_hist_update_f32": ([_p, _i64, _i64, _int, _int, _int, _p, _p, _p, _p, _p, _p, _p], _int),
    "miq_v2_sqnr_num_candidates": ([_dbl, _int, _int, _int, _int], _int),
    "miq_v2_sqnr_search_f32": ([_p, _p, _i64, _int, _dbl, _int, _dbl, _int, _int, _int, _p, _p, _p, _p, _p], _int),
    "miq_channel_analyzer_state_bytes": ([_i64], _i64),
    "miq_channel_analyzer_workspace_bytes": ([_i64, _i64, _i64], _i64),
    "miq_channel_analyzer_create": ([_int, _i64, _p, _p, C.POINTER(_p)], _int),
    "miq_channel_analyzer_destroy": ([_p], _int),
    "miq_channel_analyzer_reset": ([_p, _p], _int),
    "miq_channel_analyzer_set_percentile": ([_p, _flt], _int),
    "miq_channel_analyzer_update_stats_f32": ([_p, _p, _i64, _i64, _p, _p], _int),
    "miq_channel_analyzer_compute_encodings_device": ([_p, _int, _int, _int, _int, _p, _p, _p, _p, _p, _p, _p,
                                                        C.POINTER(_int), _p], _int),
    "miq_channel_analyzer_compute_encodings": ([_p, _int, _int, _int, _int, _p, C.POINTER(_int), _p], _int),
    "miq_channel_analyzer_get_stats_histogram": ([_p, _i64, _p, _p, C.POINTER(_int), _p], _int),
    "miq_adaround_linear_workspace_bytes": ([_i64, _i64, _i64], _i64),
    "miq_adaround_linear_blocks": ([_i64, _i64], _int),
    "miq_adaround_linear_fwd_f32": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _int,
                                     _p, _p, _p, _p, _p], _int),
    "miq_adaround_linear_bwd_adam_f32": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt,
                                          _dbl, _dbl, _dbl, _dbl, _dbl, _dbl, _int, _p, _p], _int),
    "miq_adaround_linear_fwd_i8": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _int,
                                    _p, _p, _p, _p, _p], _int),
    "miq_adaround_linear_bwd_adam_i8": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt,
                                         _dbl, _dbl, _dbl, _dbl, _dbl, _dbl, _int, _p, _p], _int),
    "miq_adaround_linear_fwd_i16": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _i64, _p, _i64, _i64, _i64, _p, _p, _flt, _flt, _int,
                                     _p, _p, _p, _p, _p], _int),
    "miq_adaround_linear_bwd_adam_i16": ([_p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64, _p, _p, _flt, _flt,
                                          _dbl, _dbl, _dbl, _dbl, _dbl, _dbl, _int, _p, _p], _int),
}

# Entry points declared in include/miq.h; the loader insists on every one of them.
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP kernels have not been built. Build them with "
            "`make -C aimet_amd/csrc` (or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "This package has no CPU fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (argtypes, restype) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise ImportError(f"{LIB_PATH} does not export {name}; rebuild it") from exc
        fn.argtypes = argtypes
        fn.restype = restype
    return lib


lib = _load()


def check(status):
    """Raise MiqError for a non-zero status (RuntimeError subclass, like the reference's pybind exceptions)."""
    if status != OK:
        msg = lib.miq_last_error()
        raise MiqError(f"libmiq status {status}: {msg.decode() if msg else ''}")
