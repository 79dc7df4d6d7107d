"""ctypes binding of libtorpor_amd.so (declared in include/torpor_amd.h).

The library is the product: if it is missing or fails to load this module raises,
there is no other execution path.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtorpor_amd.so")


class TorporError(RuntimeError):
    def __init__(self, code, what=""):
        self.code = code
        msg = lib().tp_strerror(code).decode() if _lib is not None else "error"
        super().__init__(f"{what}: {msg} ({code})" if what else f"{msg} ({code})")


class Config(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32),
        ("device", C.c_int32),
        ("mem_limit_bytes", C.c_uint64),
        ("pool_bytes", C.c_uint64),
        ("chunk_bytes", C.c_uint64),
        ("chunk_max_bytes", C.c_uint64),
        ("workspace_bytes", C.c_uint64),
        ("flags", C.c_int32),
        ("request_timeout_ms", C.c_int32),
        ("copy_streams", C.c_int32),
        ("reserved0", C.c_int32),
    ]


class Epilogue(C.Structure):
    _fields_ = [
        ("alpha", C.c_float),
        ("beta", C.c_float),
        ("bias", C.c_uint64),
        ("bn_scale", C.c_uint64),
        ("bn_bias", C.c_uint64),
        ("bn_mean", C.c_uint64),
        ("bn_var", C.c_uint64),
        ("bn_eps", C.c_float),
        ("act", C.c_int32),
        ("residual", C.c_uint64),
        ("ldr", C.c_int64),
    ]


class GemmDesc(C.Structure):
    _fields_ = [
        ("x", C.c_uint64), ("y", C.c_uint64), ("c", C.c_uint64),
        ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
        ("xs_r", C.c_int64), ("xs_k", C.c_int64), ("ys_c", C.c_int64), ("ys_k", C.c_int64), ("ldc", C.c_int64),
        ("nb0", C.c_int32), ("nb1", C.c_int32),
        ("xb0", C.c_int64), ("xb1", C.c_int64), ("yb0", C.c_int64), ("yb1", C.c_int64),
        ("cb0", C.c_int64), ("cb1", C.c_int64),
        ("ep", Epilogue),
    ]


class ConvDesc(C.Structure):
    _fields_ = [
        ("x", C.c_uint64), ("w", C.c_uint64), ("y", C.c_uint64),
        ("n", C.c_int32), ("h", C.c_int32), ("w_in", C.c_int32), ("cin", C.c_int32), ("cout", C.c_int32),
        ("kh", C.c_int32), ("kw", C.c_int32),
        ("stride_h", C.c_int32), ("stride_w", C.c_int32), ("pad_h", C.c_int32), ("pad_w", C.c_int32),
        ("groups", C.c_int32),
        ("x_layout", C.c_int32), ("y_layout", C.c_int32),
        ("x_pitch", C.c_int64), ("y_pitch", C.c_int64),
        ("ep", Epilogue),
    ]


class PoolStats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in (
        "capacity", "used", "largest_free", "live_extents", "free_extents",
        "lru_budget", "lru_used", "lru_models", "evictions", "swap_ins", "fragmentation_evictions",
        "host_image_bytes", "host_transfer_bytes", "host_staging_bytes", "device_staging_bytes",
        "device_workspace_bytes", "pool_cached_bytes", "pool_idle_extents")]


class ModelInfo(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("registered", "resident", "level", "n_params", "n_chunks", "n_ops")] + \
               [(n, C.c_uint64) for n in ("image_bytes", "param_bytes", "act_bytes", "total_bytes",
                                          "weight_off", "act_off")]


class SwapStats(C.Structure):
    _fields_ = [("bytes", C.c_uint64), ("copy_ms", C.c_double), ("alloc_us", C.c_double),
                ("evict_us", C.c_double), ("chunks", C.c_uint32), ("gate_waits", C.c_uint32),
                ("copy_streams", C.c_uint32), ("host_gathers", C.c_uint32), ("deferred_bytes", C.c_uint64),
                ("issue_ms", C.c_double), ("max_call_us", C.c_double), ("max_call_group", C.c_uint32),
                ("max_call_kind", C.c_uint32)]


class KernelStat(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("launches", C.c_uint64), ("total_us", C.c_double),
                ("flops", C.c_double), ("bytes", C.c_double)]


# every symbol include/torpor_amd.h declares: name -> (restype, argtypes)
_P = C.c_void_p
_U64 = C.c_uint64
_I32 = C.c_int32
_I64 = C.c_int64
SYMBOLS = {
    "tp_server_create": (C.c_int, [C.POINTER(Config), C.POINTER(_P)]),
    "tp_server_destroy": (None, [_P]),
    "tp_strerror": (C.c_char_p, [C.c_int]),
    "tp_version": (C.c_char_p, []),
    "tp_signal": (C.c_int, [_P, _I32, C.c_char_p, C.c_char_p, C.POINTER(_I32), C.POINTER(_I32), C.POINTER(_I32)]),
    "tp_take_deferred_ack": (C.c_int, [_P, C.POINTER(_I32), C.POINTER(_I32)]),
    "tp_signal_ticket": (C.c_int, [_P, _I32, C.c_char_p, C.c_char_p, C.POINTER(_I32), C.POINTER(_I32),
                                   C.POINTER(_I32), C.POINTER(_U64)]),
    "tp_take_deferred_ack_ticket": (C.c_int, [_P, C.POINTER(_I32), C.POINTER(_I32), C.POINTER(_U64)]),
    "tp_cancel_deferred": (C.c_int, [_P, _U64]),
    "tp_check_address": (C.c_int, [_P, _I32, _U64, _U64]),
    "tp_poll": (C.c_int, [_P]),
    "tp_malloc": (C.c_int, [_P, _I32, _U64, C.POINTER(_U64)]),
    "tp_free": (C.c_int, [_P, _I32, _U64]),
    "tp_memcpy_h2d": (C.c_int, [_P, _I32, _U64, _P, _U64]),
    "tp_memcpy_d2h_async": (C.c_int, [_P, _I32, _P, _U64, _U64]),
    "tp_memcpy_d2h": (C.c_int, [_P, _I32, _P, _U64, _U64]),
    "tp_memcpy_d2d": (C.c_int, [_P, _I32, _U64, _U64, _U64]),
    "tp_memset_async": (C.c_int, [_P, _I32, _U64, _I32, _U64]),
    "tp_device_synchronize": (C.c_int, [_P, _I32]),
    "tp_stream_synchronize": (C.c_int, [_P, _I32]),
    "tp_sgemm": (C.c_int, [_P, _I32, _I32, _I32, _I32, _I32, _I32, C.c_float, _U64, _I32, _U64, _I32,
                           C.c_float, _U64, _I32]),
    "tp_sgemm_strided_batched": (C.c_int, [_P, _I32, _I32, _I32, _I32, _I32, _I32, C.c_float, _U64, _I32, _I64,
                                           _U64, _I32, _I64, C.c_float, _U64, _I32, _I64, _I32]),
    "tp_gemm": (C.c_int, [_P, _I32, C.POINTER(GemmDesc)]),
    "tp_gemm_noalloc": (C.c_int, [C.POINTER(GemmDesc), _P]),
    "tp_conv_forward": (C.c_int, [_P, _I32, C.POINTER(ConvDesc)]),
    "tp_bn_inference": (C.c_int, [_P, _I32, _U64, _U64, _U64, _U64, _U64, _U64, C.c_double, _I64, _I32, _I64,
                                  _I32, _I32]),
    "tp_bn_inference_pitched": (C.c_int, [_P, _I32, _U64, _U64, _U64, _U64, _U64, _U64, C.c_double, _I64, _I32,
                                          _I64, _I32, _I32, _I64]),
    "tp_launch": (C.c_int, [_P, _I32, _I32, C.POINTER(_U64), _I32, C.POINTER(_I64), _I32,
                            C.POINTER(C.c_float), _I32]),
    "tp_replay": (C.c_int, [_P, _I32, _P, _U64, _P, _U64]),
    "tp_model_resident": (C.c_int, [_P, _I32]),
    "tp_model_loaded": (C.c_int, [_P, _I32]),
    "tp_get_load_estimate": (C.c_int, [_P, _I32, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "tp_get_model_info": (C.c_int, [_P, _I32, C.POINTER(ModelInfo)]),
    "tp_get_pool_stats": (C.c_int, [_P, C.POINTER(PoolStats)]),
    "tp_get_swap_stats": (C.c_int, [_P, _I32, C.POINTER(SwapStats)]),
    "tp_readback_weights": (C.c_int, [_P, _I32, _P, _U64]),
    "tp_host_weights": (C.c_int, [_P, _I32, C.POINTER(_P), C.POINTER(_U64)]),
    "tp_weight_offset": (C.c_int, [_P, _I32, _U64, C.POINTER(_U64)]),
    "tp_last_kernel": (C.c_char_p, []),
    "tp_measure_h2d": (C.c_int, [_P, _U64, _I32, C.POINTER(C.c_double)]),
    "tp_time_op": (C.c_int, [_P, _I32, _I32, _I32, C.POINTER(C.c_double)]),
    "tp_profile_begin": (C.c_int, [_P]),
    "tp_profile_end": (C.c_int, [_P]),
    "tp_profile_read": (C.c_int, [_P, _I32, C.POINTER(KernelStat)]),
    "tp_pool_create": (_P, [_U64]),
    "tp_pool_create_policy": (_P, [_U64, _I32]),
    "tp_pool_cached": (C.c_int, [_P, C.POINTER(_U64), C.POINTER(_U64)]),
    "tp_pool_trim": (C.c_int, [_P]),
    "tp_pool_destroy": (None, [_P]),
    "tp_pool_alloc": (_U64, [_P, _U64]),
    "tp_pool_release": (C.c_int, [_P, _U64]),
    "tp_pool_query": (C.c_int, [_P] + [C.POINTER(_U64)] * 5),
    "tp_lru_create": (_P, [_U64]),
    "tp_lru_destroy": (None, [_P]),
    "tp_lru_check_and_add": (C.c_int, [_P, C.c_char_p, _U64, C.c_char_p, _U64, C.POINTER(_I32), C.POINTER(_I32)]),
    "tp_lru_force_evict": (C.c_int, [_P, C.c_char_p]),
    "tp_lru_lock": (C.c_int, [_P, C.c_char_p]),
    "tp_lru_unlock": (C.c_int, [_P, C.c_char_p]),
    "tp_lru_used": (_U64, [_P]),
    "tp_evictor_create": (_P, [_I32, _I32, _U64]),
    "tp_evictor_destroy": (None, [_P]),
    "tp_evictor_set_level": (C.c_int, [_P, C.c_char_p, _I32]),
    "tp_evictor_check_and_add": (C.c_int, [_P, _I32, C.c_char_p, _U64, C.c_char_p, _U64, C.POINTER(_I32),
                                           C.POINTER(_I32)]),
    "tp_evictor_force_evict": (C.c_int, [_P, _I32, C.c_char_p]),
    "tp_evictor_lock": (C.c_int, [_P, _I32, C.c_char_p]),
    "tp_evictor_unlock": (C.c_int, [_P, _I32, C.c_char_p]),
    "tp_evictor_used": (_U64, [_P, _I32]),
    "tp_evictor_is_protected": (C.c_int, [_P, _I32, C.c_char_p]),
    "tp_evictor_order": (C.c_int, [_P, _I32, C.c_char_p, _U64]),
    "tp_sched_create": (_P, [_I32]),
    "tp_sched_destroy": (None, [_P]),
    "tp_sched_set_sibling": (C.c_int, [_P, _I32, _I32]),
    "tp_sched_set_link": (C.c_int, [_P, _I32, _I32, _I32]),
    "tp_sched_set_status": (C.c_int, [_P, _I32, _I32]),
    "tp_sched_set_level": (C.c_int, [_P, C.c_char_p, _I32]),
    "tp_sched_set_resident": (C.c_int, [_P, C.c_char_p, _I32, _I32]),
    "tp_sched_placement": (C.c_int, [_P]),
    "tp_sched_decide": (C.c_int, [_P, _I32, C.c_char_p, C.c_uint32, C.POINTER(_I32), C.POINTER(_I32),
                                  C.POINTER(_I32)]),
    "tp_host_alloc": (C.c_int, [_P, _U64, C.POINTER(_P)]),
    "tp_host_free": (C.c_int, [_P, _P]),
    "tp_pack_bound": (_U64, [_U64]),
    "tp_pack_blocks": (_U64, [_U64]),
    "tp_pack_words": (C.c_int, [_P, _U64, _P, C.POINTER(_I32), _P, _U64, C.POINTER(_U64), _P]),
    "tp_unpack_words": (C.c_int, [_P, _U64, _I32, _P, _U64, _P]),
    "tp_unpack_words_device": (C.c_int, [_P, _P, _U64, _I32, _P, _U64, _P, _U64, _U64, _P]),
}

_lib = None


def _share_hip_runtime_with_torch():
    """One HIP runtime per process.  A PyTorch wheel for ROCm carries its own libamdhip64 (soname
    libamdhip64.so.7, the one this library asks for too) and finds it by file name: loaded after this library
    it would come in as a second runtime beside the system's, and the second one to initialise sees no
    device.  So where torch is installed but not imported yet, its copy is loaded first and this library binds
    to it, which is what happens anyway when torch is imported first; either import order then works."""
    import importlib.util
    import sys
    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        return
    if spec is None or not spec.submodule_search_locations:
        return
    path = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libamdhip64.so")
    if os.path.exists(path):
        try:
            C.CDLL(path, mode=C.RTLD_GLOBAL)
        except OSError:
            pass    # not loadable here: the system's runtime serves this library alone


def lib():
    """Load the shared library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C torpor_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback path")
        _share_hip_runtime_with_torch()
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(l, name)  # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib
