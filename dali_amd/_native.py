"""Loads the two native libraries and declares their C signatures."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIBDIR = os.path.join(_HERE, "lib")


class DaliError(RuntimeError):
    pass


def lib_paths():
    return os.path.join(_LIBDIR, "libdali_hip.so"), os.path.join(_LIBDIR, "libdali_front.so")


def _load():
    hip_path, front_path = lib_paths()
    for p in (hip_path, front_path):
        if not os.path.exists(p):
            raise ImportError(
                "native library %s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "from the repository root (there is no fallback path)" % p)
    hip_lib = C.CDLL(hip_path, mode=C.RTLD_GLOBAL)
    front_lib = C.CDLL(front_path, mode=C.RTLD_GLOBAL)
    return hip_lib, front_lib


hip, front = _load()

H = C.c_void_p
_i = C.c_int
_ip = C.POINTER(C.c_int)
_sz = C.c_size_t
_u64 = C.c_uint64


class LaunchPlan(C.Structure):
    _fields_ = [
        ("n_arrays", C.c_int32), ("n_scalars", C.c_int32), ("n_shapes", C.c_int32),
        ("array_ndim", C.POINTER(C.c_int32)), ("array_strided", C.POINTER(C.c_int32)),
        ("array_elsize", C.POINTER(C.c_int32)), ("scalar_dtype", C.POINTER(C.c_int32)),
        ("shape_ndim", C.POINTER(C.c_int32)),
        ("block_threads", C.c_int32), ("grid_kind", C.c_int32), ("work_begin", C.c_int32),
        ("work_count", C.c_int32), ("work_per_block", C.c_int32), ("max_blocks", C.c_int32),
        ("work2_begin", C.c_int32), ("work2_per_block", C.c_int32), ("max_blocks2", C.c_int32),
        ("ws_elsize", C.c_int32),
    ]


def _sig(lib, name, restype, argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = argtypes
    return fn


# ---- include/dali_hip.h
HIP_SYMBOLS = {
    "dali_hip_last_error": (C.c_char_p, []),
    "dali_hip_device_count": (_i, [_ip]),
    "dali_hip_init": (_i, [_i]),
    "dali_hip_device_name": (_i, [_i, C.c_char_p, _sz, C.c_char_p, _sz]),
    "dali_hip_mem_info": (_i, [C.POINTER(_sz), C.POINTER(_sz)]),
    "dali_hip_sync": (_i, []),
    "dali_hip_stream": (H, []),
    "dali_hip_malloc": (_i, [C.POINTER(H), _sz]),
    "dali_hip_free": (_i, [H]),
    "dali_hip_bank_allocate": (_i, [C.POINTER(H), _sz]),
    "dali_hip_bank_deposit": (_i, [H, _sz]),
    "dali_hip_bank_clear": (_i, []),
    "dali_hip_bank_stats": (_i, [C.POINTER(_sz), C.POINTER(_sz)]),
    "dali_hip_memset_async": (_i, [H, _i, _sz]),
    "dali_hip_memcpy_h2d": (_i, [H, H, _sz]),
    "dali_hip_memcpy_d2h": (_i, [H, H, _sz]),
    "dali_hip_memcpy_d2d": (_i, [H, H, _sz]),
    "dali_hip_host_alloc": (_i, [C.POINTER(H), _sz]),
    "dali_hip_host_free": (_i, [H]),
    "dali_hip_memcpy_h2d_async": (_i, [H, H, _sz, H]),
    "dali_hip_memcpy_d2h_async": (_i, [H, H, _sz, H]),
    "dali_hip_module_load": (_i, [_u64, C.c_char_p, C.c_char_p, C.POINTER(LaunchPlan), _ip]),
    "dali_hip_module_is_loaded": (_i, [_u64]),
    "dali_hip_launch": (_i, [_u64, C.POINTER(H), _ip, C.POINTER(_ip), C.POINTER(_ip), C.POINTER(H), C.POINTER(_ip)]),
    "dali_hip_compile_only": (_i, [C.c_char_p, C.POINTER(_sz)]),
    "dali_hip_rtc_options": (C.c_char_p, []),
    "dali_hip_jit_stats": (_i, [C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_u64)]),
    "dali_hip_set_cache_dir": (_i, [C.c_char_p]),
    "dali_hip_cache_warm": (_i, [C.POINTER(_i)]),
    "dali_hip_sgemm": (_i, [_i, _i, _i, _i, _i, C.c_float, H, _i, H, _i, C.c_float, H, _i]),
    "dali_hip_dgemm": (_i, [_i, _i, _i, _i, _i, C.c_double, H, _i, H, _i, C.c_double, H, _i]),
    "dali_hip_sgemm_pair": (_i, [_i, _i, _i, _i, _i, _i, _i, _i, C.c_float, H, _i, H, _i, H, _i, H, _i, C.c_float, H, _i]),
    "dali_hip_sgemm_terms": (_i, [_i, _i, _i, _i, _i, _ip, C.POINTER(H), _i, C.POINTER(H), _i, C.c_float, C.c_float, H, _i, _ip]),
    "dali_hip_lstm_step": (_i, [_i, _i, _i, H, _i, H, _i, H, H, _i, H, _i, H, H, H]),
    "dali_hip_lstm_step_small": (_i, [_i, _i, _i, H, _i, H, _i, H, H, _i, H, _i, H, H, H]),
    "dali_hip_lstm_recurrent_persistent": (_i, [_i, _i, _i, H, H, _i, H, H, H, H]),
    "dali_hip_lstm_recurrent_persistent_supported": (_i, [_i, _i]),
    "dali_hip_gru_recurrent_persistent": (_i, [_i, _i, _i, H, H, _i, H, H, H]),
    "dali_hip_gru_recurrent_persistent_supported": (_i, [_i, _i]),
    "dali_hip_softmax_axis": (_i, [H, H, C.c_int64, _i, C.c_int64]),
    "dali_hip_softmax_axis_supported": (_i, [C.c_int64, _i, C.c_int64]),
    "dali_hip_argsort_i32": (_i, [H, C.c_int64, C.c_int32, H, H]),
    "dali_hip_argsort_i32_noalloc": (_i, [H, C.c_int64, C.c_int32, H, H]),
    "dali_hip_topk_rows": (_i, [H, _i, C.c_int64, C.c_int32, C.c_int32, _i, _i, H]),
    "dali_hip_capture_begin": (_i, []),
    "dali_hip_capture_end": (_i, [C.POINTER(H)]),
    "dali_hip_graph_launch": (_i, [H]),
    "dali_hip_graph_destroy": (_i, [H]),
    "dali_hip_event_create": (_i, [C.POINTER(H)]),
    "dali_hip_event_record": (_i, [H]),
    "dali_hip_event_elapsed_ms": (_i, [H, H, C.POINTER(C.c_float)]),
    "dali_hip_event_destroy": (_i, [H]),
    "dali_hip_stream_wait_event": (_i, [H]),
    "dali_hip_event_synchronize": (_i, [H]),
    "dali_hip_event_query": (_i, [H, C.POINTER(_i)]),
}
for _name, (_res, _args) in HIP_SYMBOLS.items():
    _sig(hip, _name, _res, _args)

# ---- include/dali_front.h
_HP = C.POINTER(H)
FRONT_SYMBOLS = {
    "dali_fe_last_error": (C.c_char_p, []),
    "dali_fe_from_host": (H, [H, _ip, _i, _i]),
    "dali_fe_from_host_pinned": (H, [H, _ip, _i, _i]),
    "dali_fe_prefetch": (_i, [H, _i]),
    "dali_fe_empty": (H, [_ip, _i, _i]),
    "dali_fe_zeros": (H, [_ip, _i, _i]),
    "dali_fe_scalar_double": (H, [C.c_double]),
    "dali_fe_scalar_float": (H, [C.c_float]),
    "dali_fe_scalar_int": (H, [_i]),
    "dali_fe_clone_handle": (H, [H]),
    "dali_fe_release": (None, [H]),
    "dali_fe_ndim": (_i, [H]),
    "dali_fe_shape": (_i, [H, _ip]),
    "dali_fe_dtype": (_i, [H]),
    "dali_fe_is_buffer": (_i, [H]),
    "dali_fe_is_contiguous": (_i, [H]),
    "dali_fe_strides": (_i, [H, _ip]),
    "dali_fe_offset": (_i, [H]),
    "dali_fe_transpose": (H, [H, _ip, _i]),
    "dali_fe_pluck_axis": (H, [H, _i, _i]),
    "dali_fe_slice": (H, [H, _i, _i, _i, _i]),
    "dali_fe_reshape": (H, [H, _ip, _i]),
    "dali_fe_expand_dims": (H, [H, _i]),
    "dali_fe_squeeze": (H, [H, _i]),
    "dali_fe_ascontiguousarray": (H, [H]),
    "dali_fe_unary": (H, [C.c_char_p, H]),
    "dali_fe_binary": (H, [C.c_char_p, H, H]),
    "dali_fe_astype": (H, [H, _i]),
    "dali_fe_all_reduce": (H, [C.c_char_p, H]),
    "dali_fe_axis_reduce": (H, [C.c_char_p, H, _ip, _i, _i]),
    "dali_fe_arg_all_reduce": (H, [C.c_char_p, H]),
    "dali_fe_arg_axis_reduce": (H, [C.c_char_p, H, _i]),
    "dali_fe_mean_all": (H, [H]),
    "dali_fe_mean_axes": (H, [H, _ip, _i, _i]),
    "dali_fe_softmax": (H, [H, _i]),
    "dali_fe_softmax_naive": (H, [H, _i]),
    "dali_fe_gather_from_rows": (H, [H, H]),
    "dali_fe_gather": (H, [H, H]),
    "dali_fe_axis_scan": (H, [H, C.c_char_p, _i]),
    "dali_fe_arange": (H, [H, H, H]),
    "dali_fe_diag": (H, [H, _i, _i]),
    "dali_fe_outer": (H, [H, H]),
    "dali_fe_circular_convolution": (H, [H, H]),
    "dali_fe_concatenate": (H, [_HP, _i, _i]),
    "dali_fe_im2col": (H, [H] + [_i] * 8 + [C.c_char_p]),
    "dali_fe_col2im": (H, [H, _ip, _i, _i, _i, _i, _i, C.c_char_p]),
    "dali_fe_conv2d": (H, [H, H, _i, _i, _i, C.c_char_p]),
    "dali_fe_conv2d_backward_input": (H, [H, H, _i, _i, _ip, _i, C.c_char_p]),
    "dali_fe_conv2d_backward_filters": (H, [H, H, _i, _i, _ip, _i, C.c_char_p]),
    "dali_fe_conv2d_backward_bias": (H, [H, C.c_char_p]),
    "dali_fe_pool2d": (H, [H, _i, _i, _i, _i, _i, _i, C.c_char_p]),
    "dali_fe_pool2d_backward": (H, [H, H, H, _i, _i, _i, _i, _i, _i, C.c_char_p]),
    "dali_fe_autoreduce_assign": (_i, [H, H]),
    "dali_fe_one_hot": (H, [H, _i, H, H]),
    "dali_fe_dot": (H, [H, H]),
    "dali_fe_inner": (H, [H, H]),
    "dali_fe_matrix_vector_dot": (H, [H, H]),
    "dali_fe_ceil": (H, [H]),
    "dali_fe_softmax_temperature": (H, [H, H, _i]),
    "dali_fe_top_k": (H, [H, _i, _i, _i]),
    "dali_fe_argsort": (H, [H, _i, _i]),
    "dali_fe_tensordot": (H, [H, H, _i, _ip, _ip]),
    "dali_fe_softmax_cross_entropy": (_i, [H, H, _HP, _HP, _HP]),
    "dali_fe_lstm_step": (_i, [H, H, H, H, H, H, _HP, _HP]),
    "dali_fe_lstm_sequence": (_i, [H, H, H, H, H, H, _HP, _HP, _HP]),
    "dali_fe_gru_step": (H, [H, H, H, H, H]),
    "dali_fe_gru_sequence": (_i, [H, H, H, H, H, _HP, _HP]),
    "dali_fe_stacked_lstm_step": (_i, [H, _i, _HP, _HP, _HP, _HP, _HP, _i, _HP, _HP]),
    "dali_fe_stacked_lstm_sequence": (_i, [H, _i, _HP, _HP, _HP, _HP, _HP, _i, _HP, _HP, _HP]),
    "dali_fe_eval": (_i, [H]),
    "dali_fe_eval_together": (_i, [_HP, _i]),
    "dali_fe_assign": (_i, [H, _i, H]),
    "dali_fe_to_host": (_i, [H, H]),
    "dali_fe_device_ptr": (H, [H]),
    "dali_fe_stats": (_i, [C.POINTER(_u64)] * 4),
    "dali_fe_plan_cache_stats": (_i, [C.POINTER(_u64)] * 2),
    "dali_fe_scope_observe": (_i, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "dali_fe_scope_unobserve": (None, [_i]),
    "dali_fe_last_kernel_kinds": (C.c_char_p, []),
    "dali_fe_last_kernel_names": (C.c_char_p, []),
    "dali_fe_last_source": (C.c_char_p, []),
    "dali_fe_generated_source": (C.c_char_p, [C.c_int]),
    "dali_fe_generate_only": (_i, [_HP, _i, _i]),
    "dali_fe_set_dry_run": (_i, [_i, _i]),
    "dali_fe_record_begin": (H, []),
    "dali_fe_record_end": (_i, [H]),
    "dali_fe_record_make_graph": (_i, [H]),
    "dali_fe_replay": (_i, [H, _i]),
    "dali_fe_record_free": (None, [H]),
}
for _name, (_res, _args) in FRONT_SYMBOLS.items():
    _sig(front, _name, _res, _args)


def hip_check(status, what="dali_hip call"):
    if status != 0:
        raise DaliError("%s failed: %s" % (what, hip.dali_hip_last_error().decode()))


def fe_error(what):
    return DaliError("%s failed: %s" % (what, front.dali_fe_last_error().decode()))
