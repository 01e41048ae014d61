"""ctypes binding of the C ABI declared in ``include/tracea.h``.

Nothing here computes: every call goes to ``libtracea.so``.  Loading fails
loudly when the library has not been built (``python -m tracea_amd.build``).
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TRACEA_LIB points at another build of the same library (kernel experiments).
LIB_PATH = os.environ.get("TRACEA_LIB") or os.path.join(_HERE, "lib", "libtracea.so")

# TraceaStatus
SUCCESS, INVALID_PARAMS, UNSUPPORTED_CONFIG, CUDA_ERROR, CPU_ERROR, UNKNOWN_ERROR = 0, 1, 2, 3, 4, 99
# TraceaDType
F32, F16, BF16, I32, I8 = 0, 1, 2, 3, 4
# TraceaEpilogueKind
(EPI_IDENTITY, EPI_BIAS_ADD, EPI_RELU, EPI_GELU, EPI_SILU, EPI_BIAS_RELU, EPI_BIAS_SILU,
 EPI_RESIDUAL, EPI_RESIDUAL_RELU) = range(9)
# TraceaEpilogueOpKind
(OP_NONE, OP_BIAS_ADD, OP_RELU, OP_GELU, OP_SILU, OP_RESIDUAL_ADD, OP_BIAS_ADD_SILU, OP_BATCHNORM,
 OP_SCALE_SHIFT) = range(9)
MAX_EPILOGUE_OPS = 4


class TensorView(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("rank", C.c_uint32), ("shape", C.POINTER(C.c_uint64)),
                ("stride", C.POINTER(C.c_int64)), ("dtype", C.c_int), ("device_id", C.c_int32)]


class Conv2dParams(C.Structure):
    _fields_ = [("stride_h", C.c_uint32), ("stride_w", C.c_uint32), ("padding_h", C.c_uint32),
                ("padding_w", C.c_uint32), ("dilation_h", C.c_uint32), ("dilation_w", C.c_uint32),
                ("groups", C.c_uint32), ("epilogue", C.c_int), ("stream", C.c_void_p)]


class ConvTranspose2dParams(C.Structure):
    _fields_ = [("stride_h", C.c_uint32), ("stride_w", C.c_uint32), ("padding_h", C.c_uint32),
                ("padding_w", C.c_uint32), ("output_padding_h", C.c_uint32),
                ("output_padding_w", C.c_uint32), ("dilation_h", C.c_uint32),
                ("dilation_w", C.c_uint32), ("groups", C.c_uint32), ("epilogue", C.c_int),
                ("stream", C.c_void_p)]


class GemmParams(C.Structure):
    _fields_ = [("epilogue", C.c_int), ("stream", C.c_void_p)]


class AttentionParams(C.Structure):
    _fields_ = [("causal", C.c_uint8), ("softmax_mode", C.c_int), ("scale", C.c_float),
                ("stream", C.c_void_p)]


class Result(C.Structure):
    _fields_ = [("success", C.c_bool), ("error_msg", C.c_void_p), ("score", C.c_float),
                ("config_ptr", C.c_void_p)]


class EpilogueOp(C.Structure):
    _fields_ = [("kind", C.c_int), ("dtype", C.c_int), ("p0", C.c_void_p), ("p1", C.c_void_p),
                ("p2", C.c_void_p), ("p3", C.c_void_p), ("epsilon", C.c_float), ("ld", C.c_int64)]


class ConvParamsBlock(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("batch", "h_in", "w_in", "c_in", "k_out", "h_out", "w_out", "r_sz", "s_sz",
                 "stride", "pad", "dilation")] + \
               [(n, C.c_uint32) for n in
                ("hw_m", "hw_s", "w_m", "w_s", "sic_m", "sic_s", "c_m", "c_s")]


# name -> (restype, argtypes); every symbol include/tracea.h declares
SIGNATURES = {
    "tracea_init": (C.c_int, []),
    "tracea_shutdown": (None, []),
    "tracea_free_string": (None, [C.c_void_p]),
    "tracea_conv2d": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), C.POINTER(TensorView),
                                C.POINTER(TensorView), Conv2dParams]),
    "tracea_conv_transpose2d": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView),
                                          C.POINTER(TensorView), C.POINTER(TensorView),
                                          ConvTranspose2dParams]),
    "tracea_gemm": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), C.POINTER(TensorView),
                              C.POINTER(TensorView), GemmParams]),
    "tracea_gemm_noalloc": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), C.POINTER(TensorView),
                                      C.POINTER(TensorView), GemmParams]),
    "tracea_attention": (C.c_int, [TensorView, TensorView, TensorView, C.POINTER(TensorView),
                                   AttentionParams]),
    "tracea_get_last_error": (C.c_int32, [C.c_char_p, C.c_size_t]),
    "tracea_clear_error": (None, []),
    "tracea_version_major": (C.c_uint32, []),
    "tracea_version_minor": (C.c_uint32, []),
    "tracea_version_patch": (C.c_uint32, []),
    "tracea_tune_gemm": (Result, [C.c_size_t, C.c_size_t, C.c_size_t]),
    "tracea_tune_fa2": (Result, [C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_bool]),
    "tracea_tune_conv2d": (Result, [C.c_size_t] * 10),
    "tracea_conv_transpose2d_ex": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), ConvTranspose2dParams,
                                             C.POINTER(EpilogueOp), C.c_uint32]),
    "tracea_conv2d_ex": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), Conv2dParams,
                                   C.POINTER(EpilogueOp), C.c_uint32]),
    "tracea_gemm_ex": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), GemmParams,
                                 C.POINTER(EpilogueOp), C.c_uint32]),
    "tracea_plan_compile": (C.c_void_p, [C.c_char_p, C.c_int]),
    "tracea_plan_destroy": (None, [C.c_void_p]),
    "tracea_plan_arena_size": (C.c_size_t, [C.c_void_p]),
    "tracea_plan_describe": (C.c_void_p, [C.c_void_p]),
    "tracea_plan_output": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "tracea_plan_bind": (C.c_int, [C.c_void_p, C.c_uint64, C.c_char_p, C.c_void_p]),
    "tracea_plan_bind_sized": (C.c_int, [C.c_void_p, C.c_uint64, C.c_char_p, C.c_void_p, C.c_size_t, C.c_int32]),
    "tracea_plan_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]),
    "tracea_apply_epilogue": (C.c_int, [TensorView, C.POINTER(TensorView), C.POINTER(EpilogueOp), C.c_uint32,
                                        C.c_void_p]),
    "tracea_softmax": (C.c_int, [TensorView, C.POINTER(TensorView), C.c_void_p]),
    "tracea_global_avg_pool": (C.c_int, [TensorView, C.POINTER(TensorView), C.c_void_p]),
    "tracea_linear": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), C.POINTER(TensorView), GemmParams]),
    "tracea_low_rank_mlp": (C.c_int, [TensorView, TensorView, TensorView, C.POINTER(TensorView),
                                      C.POINTER(TensorView), C.POINTER(TensorView), GemmParams]),
    "tracea_ttg_from_dense": (C.c_void_p, [C.c_uint32] * 6),
    "tracea_ttg_from_dense_k_split": (C.c_void_p, [C.c_uint32] * 7),
    "tracea_ttg_from_mask": (C.c_void_p, [C.c_uint32] * 6 + [C.c_void_p]),
    "tracea_ttg_from_diagonal": (C.c_void_p, [C.c_uint32] * 6),
    "tracea_ttg_from_random": (C.c_void_p, [C.c_uint32] * 6 + [C.c_double, C.c_uint64]),
    "tracea_ttg_from_low_rank": (C.c_void_p, [C.c_uint32] * 7),
    "tracea_ttg_from_tables": (C.c_void_p, [C.c_uint32] * 6 + [C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32]),
    "tracea_ttg_destroy": (None, [C.c_void_p]),
    "tracea_ttg_num_active_tiles": (C.c_uint32, [C.c_void_p]),
    "tracea_ttg_num_records": (C.c_uint32, [C.c_void_p]),
    "tracea_ttg_num_edges": (C.c_uint32, [C.c_void_p]),
    "tracea_ttg_l1_map": (C.c_uint32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "tracea_ttg_l1_map_ordered": (C.c_uint32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "tracea_ttg_l2_table": (C.c_uint32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "tracea_ttg_execution_order": (C.c_uint32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "tracea_ttg_edges": (C.c_uint32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "tracea_ttg_reuse_hints": (C.c_uint32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32]),
    "tracea_ttg_validate_order": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_uint32]),
    "tracea_ttg_device_size": (C.c_int, [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "tracea_ttg_upload_to": (C.c_int, [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p]),
    "tracea_gemm_ttg": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), C.POINTER(TensorView),
                                  C.POINTER(TensorView), GemmParams, C.c_void_p]),
    "tracea_gemm_ttg_ex": (C.c_int, [TensorView, TensorView, C.POINTER(TensorView), GemmParams,
                                     C.POINTER(EpilogueOp), C.c_uint32, C.c_void_p]),
    "tracea_set_split_k": (None, [C.c_int32]),
    "tracea_set_split_k_one_launch": (None, [C.c_int32]),
    "tracea_last_split_k_launches": (C.c_int32, []),
    "tracea_set_conv_transpose_by_phase": (None, [C.c_int32]),
    "tracea_set_conv_transpose_filter_cache": (None, [C.c_int32]),
    "tracea_conv_transpose_filter_cache_clear": (None, []),
    "tracea_last_split_k": (C.c_int32, []),
    "tracea_clock_probe": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "tracea_variant_count": (C.c_int32, [C.c_char_p]),
    "tracea_variant_name": (C.c_char_p, [C.c_char_p, C.c_int32]),
    "tracea_force_variant": (C.c_int32, [C.c_char_p, C.c_int32]),
    "tracea_select_variant": (C.c_int32, [C.c_char_p, C.c_int64, C.c_int64, C.c_int64]),
    "tracea_last_variant": (C.c_int32, [C.c_char_p]),
    "tracea_conv_params_pack": (C.c_int, [C.c_int32] * 10 + [C.POINTER(ConvParamsBlock)]),
    "tracea_conv_coords_device": (C.c_int, [C.POINTER(ConvParamsBlock), C.c_void_p, C.c_void_p,
                                            C.c_void_p, C.c_void_p]),
}

MEASURE_FN = C.CFUNCTYPE(C.c_float, C.c_char_p, C.c_void_p)
_STR = C.c_void_p  # char* the caller frees with tracea_free_string

# every symbol include/tracea_tuner.h declares
SIGNATURES.update({
    "tracea_pipeline_config_new": (_STR, [C.c_uint32] * 4),
    "tracea_pipeline_config_normalize": (_STR, [C.c_char_p]),
    "tracea_pipeline_config_validate": (C.c_int32, [C.c_char_p, C.POINTER(C.c_void_p)]),
    "tracea_pipeline_config_to_vector": (C.c_int32, [C.c_char_p, C.POINTER(C.c_float), C.c_int32]),
    "tracea_hardware_profile_json": (_STR, [C.c_char_p]),
    "tracea_check_feasibility": (C.c_int32, [C.c_char_p, C.c_char_p, C.c_uint64, C.POINTER(C.c_void_p)]),
    "tracea_estimate_occupancy": (C.c_float, [C.c_char_p, C.c_char_p]),
    "tracea_gp_create": (C.c_void_p, []),
    "tracea_gp_destroy": (None, [C.c_void_p]),
    "tracea_gp_set_noise_sigma": (None, [C.c_void_p, C.c_float]),
    "tracea_gp_set_exploration_beta": (None, [C.c_void_p, C.c_float]),
    "tracea_gp_observe": (C.c_int32, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_char_p, C.c_float,
                                      C.c_char_p]),
    "tracea_gp_predict": (C.c_int32, [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_char_p, C.c_char_p,
                                      C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "tracea_gp_acquisition": (C.c_float, [C.c_void_p, C.c_int32, C.c_uint32, C.c_uint32, C.c_uint32,
                                          C.c_char_p, C.c_char_p, C.c_float, C.c_uint64]),
    "tracea_gp_marginal_log_likelihood": (C.c_float, [C.c_void_p, C.c_char_p]),
    "tracea_gp_optimize_hyperparams": (None, [C.c_void_p, C.c_char_p]),
    "tracea_gp_length_scales": (C.c_int32, [C.c_void_p, C.POINTER(C.c_float), C.c_int32]),
    "tracea_gp_features": (C.c_int32, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_char_p, C.POINTER(C.c_float),
                                       C.c_int32]),
    "tracea_gp_roofline_prior": (C.c_float, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_char_p, C.c_char_p]),
    "tracea_propose_gemm_configs": (_STR, [C.c_uint32] * 3),
    "tracea_propose_conv_configs": (_STR, [C.c_uint32] * 3),
    "tracea_propose_attention_configs": (_STR, [C.c_uint32]),
    "tracea_search_space_enumerate": (_STR, [C.c_char_p]),
    "tracea_variant_for_config": (C.c_int32, [C.c_char_p]),
    "tracea_magic_number_strategy": (C.c_char_p, [C.c_uint64]),
    "tracea_tuning_cache_path": (_STR, []),
    "tracea_tuning_cache_get": (_STR, [C.c_char_p]),
    "tracea_tuning_cache_put": (C.c_int32, [C.c_char_p, C.c_char_p, C.c_float, C.c_uint64]),
    "tracea_tuning_cache_reload": (None, []),
    "tracea_tuning_history_path": (_STR, []),
    "tracea_tuning_history_record": (C.c_int32, [C.c_char_p, C.c_char_p, C.c_float, C.c_uint64, C.c_char_p]),
    "tracea_tuning_history_query": (_STR, [C.c_char_p]),
    "tracea_tuning_history_reload": (None, []),
    "tracea_tuning_key_gemm": (_STR, [C.c_uint64] * 3 + [C.c_char_p]),
    "tracea_tuning_key_conv2d": (_STR, [C.c_uint32] * 9 + [C.c_char_p]),
    "tracea_autotune_candidates": (Result, [C.c_char_p, C.c_char_p, MEASURE_FN, C.c_void_p]),
    "tracea_autotune_guided": (Result, [C.c_char_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_char_p,
                                        MEASURE_FN, C.c_void_p, C.c_uint32, C.c_int, C.c_uint64]),
    "tracea_autotune_gemm": (Result, [C.c_size_t] * 3 + [C.c_uint32]),
    "tracea_autotune_conv2d": (Result, [C.c_size_t] * 10 + [C.c_uint32]),
    # include/tracea_graph.h
    "tracea_graph_fuse": (_STR, [C.c_char_p]),
})

_lib = None


def lib():
    """The loaded library; raises if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libtracea.so is missing (%s); run `python -m tracea_amd.build`"
                               % LIB_PATH)
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def last_error():
    buf = C.create_string_buffer(1024)
    n = lib().tracea_get_last_error(buf, len(buf))
    return buf.raw[:n].decode("utf-8", "replace") if n > 0 else ""


class TraceaError(RuntimeError):
    def __init__(self, what, status):
        self.status = status
        super().__init__("%s failed (status %d): %s" % (what, status, last_error()))


def check(what, status):
    if status != SUCCESS:
        raise TraceaError(what, status)


def init():
    """tracea_init(); raises when no HIP device is usable."""
    if lib().tracea_init() != 0:
        raise RuntimeError("tracea_init failed: " + last_error())


_SHAPE_TYPES = [C.c_uint64 * n for n in range(9)]
_STRIDE_TYPES = [C.c_int64 * n for n in range(9)]


class View:
    """Owns the shape/stride arrays a TraceaTensorView borrows."""
    __slots__ = ("_shape", "_stride", "c")

    def __init__(self, ptr, shape, stride, dtype, device_id):
        n = len(shape)
        self._shape = _SHAPE_TYPES[n](*shape)
        self._stride = _STRIDE_TYPES[n](*stride) if stride is not None else None
        self.c = TensorView(ptr, n, self._shape, self._stride, dtype, device_id)


def take_result(res):
    """TraceaResult -> (success, score, config_json, error); frees the strings."""
    cfg = C.string_at(res.config_ptr).decode() if res.config_ptr else None
    err = C.string_at(res.error_msg).decode() if res.error_msg else None
    if res.config_ptr:
        lib().tracea_free_string(res.config_ptr)
    if res.error_msg:
        lib().tracea_free_string(res.error_msg)
    return bool(res.success), float(res.score), cfg, err


def take_string(ptr):
    """char* from the library -> str (None for NULL); frees it."""
    if not ptr:
        return None
    text = C.string_at(ptr).decode()
    lib().tracea_free_string(ptr)
    return text


def variants(op):
    n = lib().tracea_variant_count(op.encode())
    return [lib().tracea_variant_name(op.encode(), i).decode() for i in range(max(n, 0))]


def last_variant(op):
    """Name of the variant the latest call of `op` on this thread launched, or None."""
    i = lib().tracea_last_variant(op.encode())
    return variants(op)[i] if i >= 0 else None


def force_variant(op, index_or_name):
    if isinstance(index_or_name, str):
        index_or_name = variants(op).index(index_or_name)
    if lib().tracea_force_variant(op.encode(), int(index_or_name)) != 0:
        raise ValueError("bad variant %r for %s" % (index_or_name, op))
