"""Loader and ctypes prototypes of libeddlhip.so (the C ABI declared in include/eddlhip.h).

There is no fallback: when the library has not been built, or cannot be loaded, importing
this module raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("EDDLHIP_LIBRARY") or os.path.join(_HERE, "libeddlhip.so")

c_int, c_float, c_size_t, c_void_p = ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_void_p
P = c_void_p  # device pointers travel as integers
intp = ctypes.POINTER(c_int)

# name -> argument types; every entry returns int unless listed in _RESTYPE
PROTOTYPES = {
    "eddlhip_version": [],
    "eddlhip_last_error": [],
    "eddlhip_device_count": [intp],
    "eddlhip_init": [c_int],
    "eddlhip_shutdown": [c_int],
    "eddlhip_device_name": [c_int, ctypes.c_char_p, c_size_t],
    "eddlhip_set_stream": [c_int, c_void_p],
    "eddlhip_synchronize": [c_int],
    "eddlhip_malloc": [c_int, c_size_t, ctypes.POINTER(c_void_p)],
    "eddlhip_free": [c_int, P],
    "eddlhip_memcpy_h2d": [c_int, P, c_void_p, c_size_t],
    "eddlhip_memcpy_d2h": [c_int, c_void_p, P, c_size_t],
    "eddlhip_memcpy_d2d": [c_int, P, P, c_size_t],
    "eddlhip_fill": [c_int, P, c_size_t, c_float],
    "eddlhip_workspace_bytes": [c_int, ctypes.POINTER(c_size_t)],
    "eddlhip_workspace_trim": [c_int],
    "eddlhip_event_create": [c_int, ctypes.POINTER(c_void_p)],
    "eddlhip_event_destroy": [c_int, c_void_p],
    "eddlhip_event_record": [c_int, c_void_p],
    "eddlhip_event_elapsed_ms": [c_int, c_void_p, c_void_p, ctypes.POINTER(c_float)],
    "eddlhip_host_malloc": [c_int, ctypes.POINTER(c_void_p), c_size_t],
    "eddlhip_host_free": [c_int, c_void_p],
    "eddlhip_memcpy_h2d_async": [c_int, P, c_void_p, c_size_t, c_void_p],
    "eddlhip_memcpy_d2h_async": [c_int, c_void_p, P, c_size_t, c_void_p],
    "eddlhip_stream_wait_event": [c_int, c_void_p],
    "eddlhip_upload_wait_event": [c_int, c_void_p],
    "eddlhip_download_wait_event": [c_int, c_void_p],
    "eddlhip_event_synchronize": [c_int, c_void_p],
    "eddlhip_graph_begin": [c_int],
    "eddlhip_graph_end": [c_int, ctypes.POINTER(c_void_p)],
    "eddlhip_graph_launch": [c_int, c_void_p],
    "eddlhip_graph_destroy": [c_int, c_void_p],
    "eddlhip_conv2d_fwd": [c_int, P, P, P, P] + [c_int] * 13 + [P, P, P, P, c_float, P, c_int],
    "eddlhip_conv2d_fwd_noalloc": [c_int, P, P, P, P] + [c_int] * 13 + [P, P, P, P, c_float, P, c_int],
    "eddlhip_conv2d_fwd_concat": [c_int, P, P, P, P, P] + [c_int] * 13 + [P, P, P, P, c_float, P, c_int],
    "eddlhip_conv2d_fwd_upsampled": [c_int, P, c_int, c_int, P, P, P] + [c_int] * 13 + [P, P, P, P, c_float, P, c_int],
    "eddlhip_conv2d_fwd_maxpool": [c_int, P, P, c_int, c_int, P, P, P] + [c_int] * 13 + [P, P, P, P, c_float, P, c_int, P, P, P, c_int],
    "eddlhip_conv2d_cache_filters": [c_int, P, c_int, c_int, c_int, c_int],
    "eddlhip_conv2d_uncache_filters": [c_int, P],
    "eddlhip_conv2d_set_algo": [c_int],
    "eddlhip_conv2d_last_kernel": [],
    "eddlhip_conv2d_force_plan": [c_int, c_int],
    "eddlhip_conv2d_profile": [c_int],
    "eddlhip_conv2d_profile_read": [intp, ctypes.POINTER(c_float)],
    "eddlhip_conv2d_trace": [P, ctypes.c_longlong],
    "eddlhip_conv2d_autotune": [c_int],
    "eddlhip_conv2d_tuned_plans": [c_int],
    "eddlhip_conv2d_tuned_save": [c_int, ctypes.c_char_p],
    "eddlhip_conv2d_tuned_load": [c_int, ctypes.c_char_p],
    "eddlhip_batchnorm_inference": [c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P, c_float],
    "eddlhip_relu": [c_int, P, P, c_size_t],
    "eddlhip_sigmoid": [c_int, P, P, c_size_t],
    "eddlhip_softmax": [c_int, P, P, c_int, c_int, c_int, c_int],
    "eddlhip_pool2d_out_dims": [c_int] * 10 + [intp, intp],
    "eddlhip_maxpool2d": [c_int, P, P, P, P] + [c_int] * 12,
    "eddlhip_avgpool2d": [c_int, P, P] + [c_int] * 12,
    "eddlhip_scale_nearest": [c_int, P, P] + [c_int] * 8,
    "eddlhip_concat": [c_int, P, ctypes.POINTER(c_void_p), intp, c_int, c_int, c_int],
    "eddlhip_add": [c_int, c_float, P, c_float, P, P, c_int, c_size_t],
    "eddlhip_inc": [c_int, P, P, c_size_t],
    "eddlhip_pad": [c_int, P, P] + [c_int] * 8,
    "eddlhip_rand_uniform": [c_int, P, c_size_t, c_float, ctypes.c_ulonglong],
    "eddlhip_rand_signed_uniform": [c_int, P, c_size_t, c_float, ctypes.c_ulonglong],
    "eddlhip_rand_binary": [c_int, P, c_size_t, c_float, ctypes.c_ulonglong],
    "eddlhip_rand_normal": [c_int, P, c_size_t, c_float, c_float, ctypes.c_ulonglong],
    "eddlhip_rand_words": [c_int, P, c_size_t, ctypes.c_ulonglong, ctypes.c_ulonglong, ctypes.c_ulonglong],
    "eddlhip_mult_scalar": [c_int, P, P, c_size_t, c_float],
    "eddlhip_add_scalar": [c_int, P, P, c_size_t, c_float],
    "eddlhip_mult2d": [c_int, P, P, P, c_int, c_int, c_int, c_int],
    "eddlhip_sum2d_rowwise": [c_int, P, P, P, c_int, c_int],
    "eddlhip_dense_fwd": [c_int, P, P, P, P, c_int, c_int, c_int, c_int],
}
_RESTYPE = {"eddlhip_version": ctypes.c_char_p, "eddlhip_last_error": ctypes.c_char_p,
            "eddlhip_conv2d_last_kernel": ctypes.c_char_p}


# include/eddlhip_probe.h: the benchmark's device probes, in libeddlhip_probe.so
PROBE_PROTOTYPES = {
    "eddlhip_probe_mfma_f32": [c_int, c_int, c_int, ctypes.POINTER(c_float), ctypes.POINTER(c_float), ctypes.POINTER(c_float)],
    "eddlhip_probe_hbm": [c_int, c_size_t, ctypes.POINTER(c_float), ctypes.POINTER(c_float), ctypes.POINTER(c_float)],
}
PROBE_LIB_PATH = os.path.join(os.path.dirname(LIB_PATH), "libeddlhip_probe.so")


def load_probe():
    """The probe library (loads libeddlhip.so, which it is linked against, through its run path)."""
    if not os.path.exists(PROBE_LIB_PATH):
        raise ImportError("%s is missing: build it with `python -m eddl_amd.build` (hipcc, gfx950)." % PROBE_LIB_PATH)
    ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    lib = ctypes.CDLL(PROBE_LIB_PATH)
    for name, args in PROBE_PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    return lib


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python -m eddl_amd.build` (hipcc, gfx950). "
            "There is no CPU fallback." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, args in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.argtypes = args
        fn.restype = _RESTYPE.get(name, c_int)
    return lib
