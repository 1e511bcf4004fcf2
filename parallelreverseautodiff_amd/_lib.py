"""ctypes binding of libprad_hip.so (the C ABI declared in include/prad_hip.h).

The library is the product; this module only declares its signatures.  There is no CPU
fallback: if the shared library is missing or does not load, importing callers get an
ImportError that says how to build it.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# PRAD_HIP_LIBRARY names another build of the library (a tuning aid: two builds measured side by side).
LIB_PATH = os.environ.get("PRAD_HIP_LIBRARY") or os.path.join(_HERE, "libprad_hip.so")

PRAD_OK = 0
PRAD_ERR_NOT_INITIALIZED = -1
PRAD_ERR_SHAPE = -2
PRAD_ERR_ALLOC = -3
PRAD_ERR_LAUNCH = -4
PRAD_ERR_BAD_HANDLE = -5
PRAD_ERR_ARG = -6
PRAD_ERR_NOT_RECTANGULAR = -7
PRAD_ERR_DTYPE = -8
PRAD_ERR_RECORDING = -9

PRAD_F64 = 0
PRAD_F32 = 1

ACT_NONE, ACT_LEAKYRELU, ACT_SIGMOID, ACT_TANH, ACT_GELU, ACT_AMPLIFIED_SIGMOID = 0, 1, 2, 3, 4, 5

_c = ctypes
_i32, _i64, _f64, _vp = _c.c_int32, _c.c_int64, _c.c_double, _c.c_void_p
_vpp = _c.POINTER(_c.c_void_p)
_i64p = _c.POINTER(_c.c_int64)
_i32p = _c.POINTER(_c.c_int32)

# name -> (restype, argtypes); must list every function include/prad_hip.h declares.
SIGNATURES = {
    "prad_init": (_i32, [_i32]),
    "prad_shutdown": (_i32, []),
    "prad_is_initialized": (_i32, []),
    "prad_device_id": (_i32, []),
    "prad_last_error": (_c.c_char_p, []),
    "prad_stream_sync": (_i32, []),
    "prad_stream": (_vp, []),
    "prad_buf_alloc": (_i32, [_i32, _i64, _i64, _vpp]),
    "prad_buf_alloc_deep": (_i32, [_i32, _i64, _i64, _i64, _vpp]),
    "prad_buf_alloc_output": (_i32, [_i32, _i64, _i64, _i64, _vpp]),
    "prad_pool_trim": (_i32, []),
    "prad_alloc_stats": (_i32, [_i64p, _i64p, _i64p, _i64p, _i64p]),
    "prad_buf_wrap": (_i32, [_i32, _i64, _i64, _vp, _vpp]),
    "prad_buf_wrap_deep": (_i32, [_i32, _i64, _i64, _i64, _vp, _vpp]),
    "prad_buf_free": (_i32, [_vp]),
    "prad_buf_shape": (_i32, [_vp, _i64p, _i64p, _i64p, _i32p]),
    "prad_buf_device_ptr": (_vp, [_vp]),
    "prad_buf_zero": (_i32, [_vp]),
    "prad_zero_multi": (_i32, [_vp, _i32]),
    "prad_buf_upload_rows": (_i32, [_vp, _vpp, _i64p]),
    "prad_buf_download_rows": (_i32, [_vp, _vpp]),
    "prad_buf_upload": (_i32, [_vp, _vp, _i64]),
    "prad_buf_download": (_i32, [_vp, _vp, _i64]),
    "prad_buf_copy": (_i32, [_vp, _vp]),
    "prad_matmul_fwd": (_i32, [_vp, _vp, _vp]),
    "prad_matmul_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32]),
    "prad_matmul_fwd_fused": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _f64]),
    "prad_matmul_bwd_fused": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _vp, _f64]),
    "prad_matmul_batch_sum_fwd": (_i32, [_vp, _vp, _vp, _vp]),
    "prad_matmul_batch_sum_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp]),
    "prad_tensor_matmul_host": (_i32, [_i32, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f64]),
    "prad_tensor_matmul_reverse_host": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64]),
    "prad_matmul_bias_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _vp, _f64]),
    "prad_gemm": (_i32, [_i32, _i32, _vp, _vp, _vp, _i32]),
    "prad_gemm_batched": (_i32, [_i32, _i32, _vp, _vp, _vp, _i32]),
    "prad_gemm_f64": (_i32, [_i32, _i32, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i32]),
    "prad_gemm_f32": (_i32, [_i32, _i32, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _i32]),
    "prad_gemm_strided_batched_f64": (_i32, [_i32, _i32, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i32, _i32]),
    "prad_gemm_strided_batched_f32": (_i32, [_i32, _i32, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i32, _i32]),
    "prad_gemm_strided_batched_2d_f64": (_i32, [_i32, _i32, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i32, _i32, _i32]),
    "prad_gemm_strided_batched_2d_f32": (_i32, [_i32, _i32, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i32, _i32, _i32]),
    "prad_scale": (_i32, [_vp, _vp, _f64]),
    "prad_matmul_fwd_host": (_i32, [_i32, _vpp, _vpp, _vpp, _i64, _i64, _i64, _i64]),
    "prad_matmul_bwd_host": (_i32, [_i32, _vpp, _vpp, _vpp, _vpp, _vpp, _i64, _i64, _i64]),
    "prad_matmul_sum_fwd": (_i32, [_vp, _vp, _vp]),
    "prad_matmul_sum_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp]),
    "prad_act_fwd": (_i32, [_i32, _vp, _vp, _f64]),
    "prad_act_bwd": (_i32, [_i32, _vp, _vp, _vp, _f64]),
    "prad_hadamard_fwd": (_i32, [_vp, _vp, _vp]),
    "prad_hadamard_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp]),
    "prad_accumulate": (_i32, [_vp, _vp]),
    "prad_add_broadcast_fwd": (_i32, [_vp, _vp, _vp]),
    "prad_add_broadcast_bwd_bias": (_i32, [_vp, _vp]),
    "prad_add": (_i32, [_vp, _vp, _vp]),
    "prad_add_three": (_i32, [_vp, _vp, _vp, _vp]),
    "prad_transpose": (_i32, [_vp, _vp]),
    "prad_layernorm_fwd": (_i32, [_vp, _vp, _vp, _vp]),
    "prad_layernorm_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp]),
    "prad_softmax_fwd": (_i32, [_vp, _vp]),
    "prad_softmax_bwd": (_i32, [_vp, _vp, _vp]),
    "prad_softmax_scaled_fwd": (_i32, [_vp, _f64, _vp]),
    "prad_softmax_scaled_bwd": (_i32, [_vp, _vp, _f64, _vp]),
    "prad_cce_fwd": (_i32, [_vp, _vp, _vp]),
    "prad_cce_bwd": (_i32, [_vp, _vp, _vp]),
    "prad_mse_fwd": (_i32, [_vp, _vp, _vp]),
    "prad_mse_bwd": (_i32, [_vp, _vp, _vp]),
    "prad_mse": (_i32, [_vp, _vp, _vp, _vp]),
    "prad_lstm_cell_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp]),
    "prad_lstm_cell_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "prad_lstm_step_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "prad_lstm_step_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "prad_window_attention_supported": (_i32, [_i32, _i64, _i64]),
    "prad_window_attention_fwd": (_i32, [_vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_double]),
    "prad_window_attention_bwd": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_double]),
    "prad_lstm_sequence_supported": (_i32, [_i32, _i64, _i64, _i64]),
    "prad_lstm_sequence_enable": (_i32, [_i32]),
    "prad_lstm_sequence_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64]),
    "prad_lstm_sequence_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64]),
    "prad_buf_view_rows": (_i32, [_vp, _i64, _i64, _vpp]),
    "prad_softmax_cce": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp]),
    "prad_dense_softmax_cce": (_i32, [_vp] * 12 + [_i32, _i32, _vp, _f64]),
    "prad_graph_begin": (_i32, []),
    "prad_graph_end": (_i32, [_vpp]),
    "prad_graph_launch": (_i32, [_vp]),
    "prad_graph_set_adam_iteration": (_i32, [_vp, _f64]),
    "prad_graph_destroy": (_i32, [_vp]),
    "prad_clip": (_i32, [_vp, _f64, _f64]),
    "prad_adam": (_i32, [_vp, _vp, _vp, _vp, _f64, _f64, _f64, _f64, _f64]),
    "prad_clip_multi": (_i32, [_vpp, _i32, _f64, _f64]),
    "prad_adam_multi": (_i32, [_vpp, _vpp, _vpp, _vpp, _i32, _f64, _f64, _f64, _f64, _f64]),
    "prad_adam_revert_multi": (_i32, [_vpp, _vpp, _vpp, _vpp, _i32, _f64, _f64, _f64, _f64, _f64]),
    "prad_clip_adam_multi": (_i32, [_vpp, _vpp, _vpp, _vpp, _i32, _f64, _f64, _f64, _f64, _f64, _f64, _f64]),
    "prad_clip_adam_multi_noalloc": (_i32, [_vpp, _vpp, _vpp, _vpp, _i32, _f64, _f64, _f64, _f64, _f64, _f64, _f64]),
    "prad_event_create": (_i32, [_vpp]),
    "prad_event_destroy": (_i32, [_vp]),
    "prad_event_record": (_i32, [_vp]),
    "prad_event_elapsed_ms": (_i32, [_vp, _vp, _c.POINTER(_c.c_float)]),
}

_lib = None


def load():
    """Loads libprad_hip.so once and returns the ctypes handle with typed entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libprad_hip.so is not built (%s missing). Build it with "
            "`python -m parallelreverseautodiff_amd.build`; there is no CPU fallback." % LIB_PATH)
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as exc:  # missing HIP runtime, wrong arch, ...
        raise ImportError("libprad_hip.so failed to load: %s" % exc)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib
