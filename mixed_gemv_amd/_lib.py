"""ctypes binding of libmixed_gemv_amd.so (the C-ABI declared in include/mixed_gemv.h).

There is no fallback: if the HIP library has not been built, importing a device entry point
raises.  Build it with `python -m mixed_gemv_amd.build`.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "lib", "libmixed_gemv_amd.so")

_c = ctypes
_u16p = _c.c_void_p  # fp16 bit patterns; passed as raw addresses (host numpy or device pointers)
_vp = _c.c_void_p
_szp = _c.POINTER(_c.c_size_t)

# name -> (restype, argtypes); must list every function include/mixed_gemv.h declares
SIGNATURES = {
    "mgemv_status_string": (_c.c_char_p, [_c.c_int]),
    "mgemv_version": (_c.c_int, []),
    "mgemv_pack_int4": (_c.c_int, [_vp, _vp, _c.c_size_t]),
    "mgemv_unpack_int4": (_c.c_int, [_vp, _vp, _c.c_size_t]),
    "mgemv_fold_zero_points": (_c.c_int, [_u16p, _u16p, _vp, _c.c_size_t]),
    "mgemv_preprocessed_size": (_c.c_size_t, [_szp, _c.c_int, _c.c_int]),
    "mgemv_preprocess_weights": (_c.c_int, [_vp, _vp, _szp, _c.c_int, _c.c_int, _c.c_int]),
    "mgemv_unpreprocess_weights": (_c.c_int, [_vp, _vp, _szp, _c.c_int, _c.c_int]),
    "mgemv_gemv": (_c.c_int, [_vp, _u16p, _u16p, _u16p, _u16p, _u16p] + [_c.c_int] * 6 + [_vp]),
    "mgemv_gemv_batched": (_c.c_int, [_vp, _u16p, _u16p, _u16p, _u16p, _u16p] + [_c.c_int] * 7
                           + [_c.c_int64] * 5 + [_vp]),
    "mgemv_gemv_routed": (_c.c_int, [_vp, _u16p, _u16p, _u16p, _u16p, _u16p, _vp] + [_c.c_int] * 8
                          + [_c.c_int64] * 5 + [_vp]),
    "mgemv_gemv_routed_bf16": (_c.c_int, [_vp, _u16p, _u16p, _u16p, _u16p, _u16p, _vp] + [_c.c_int] * 8
                               + [_c.c_int64] * 5 + [_vp]),
    "mgemv_dequantize": (_c.c_int, [_vp, _u16p, _u16p, _u16p] + [_c.c_int] * 5 + [_vp]),
    "mgemv_gemv_bf16": (_c.c_int, [_vp, _u16p, _u16p, _u16p, _u16p, _u16p] + [_c.c_int] * 6 + [_vp]),
    "mgemv_gemv_batched_bf16": (_c.c_int, [_vp, _u16p, _u16p, _u16p, _u16p, _u16p] + [_c.c_int] * 7
                                + [_c.c_int64] * 5 + [_vp]),
    "mgemv_dequantize_bf16": (_c.c_int, [_vp, _u16p, _u16p, _u16p] + [_c.c_int] * 5 + [_vp]),
    "mgemv_fold_zero_points_bf16": (_c.c_int, [_u16p, _u16p, _vp, _c.c_size_t]),
    "mgemv_set_launch_override": (_c.c_int, [_c.c_int, _c.c_int, _c.c_int, _c.c_int]),
    "mgemv_set_matrix_core_threshold": (_c.c_int, [_c.c_int]),
    "mgemv_set_dequant_form": (_c.c_int, [_c.c_int]),
    "mgemv_set_matrix_core_variant": (_c.c_int, [_c.c_int]),
    "mgemv_query_launch": (_c.c_int, [_c.c_int] * 5 + [_c.POINTER(_c.c_int * 8)]),
    "mgemv_query_launch_bf16": (_c.c_int, [_c.c_int] * 5 + [_c.POINTER(_c.c_int * 8)]),
    "mgemv_query_launch_for": (_c.c_int, [_c.c_int] * 7 + [_c.POINTER(_c.c_int * 12)]),
    "mgemv_set_prefetch_stages": (_c.c_int, [_c.c_int]),
    "mgemv_plan_coverage": (_c.c_int, [_c.c_int] * 7 + [_c.POINTER(_c.c_int64 * 8)]),
    "mgemv_gemv_arguments": (_c.c_int, [_vp, _vp]),
    "mgemv_probe_empty_launch": (_c.c_int, [_vp]),
    "mgemv_probe_empty_grid": (_c.c_int, [_c.c_int, _c.c_int, _vp]),
    "mgemv_probe_stream_read": (_c.c_int, [_vp, _c.c_size_t, _c.c_int, _c.c_int, _c.c_int, _vp, _vp]),
    "mgemv_probe_gemv": (_c.c_int, [_c.c_int, _vp, _c.c_size_t, _vp, _u16p, _u16p, _u16p, _u16p, _c.c_int, _c.c_int, _c.c_int, _vp]),
    "mgemv_probe_gemv_rows": (_c.c_int, [_c.c_int, _c.c_int, _vp, _u16p, _u16p, _u16p, _u16p, _c.c_int, _c.c_int, _c.c_int,
                                         _vp]),
    "mgemv_host_gemv": (_c.c_int, [_c.c_int] * 5 + [_vp] * 6 + [_c.c_int] * 2),
    "mgemv_host_gemv_static": (_c.c_int, [_c.c_int] * 5 + [_vp] * 6 + [_c.c_int] * 2),
    "mgemv_static_scratch_bytes_needed": (_c.c_size_t, [_c.c_int] * 7),
    "mgemv_tuned_plan_set": (_c.c_int, [_c.POINTER(_c.c_int * 12)]),
    "mgemv_tuned_plan_erase": (_c.c_int, [_c.POINTER(_c.c_int * 12)]),
    "mgemv_tuned_plan_clear": (_c.c_int, []),
    "mgemv_set_default_plans": (_c.c_int, [_c.c_int]),
    "mgemv_default_plan_count": (_c.c_int, []),
    "mgemv_tuned_plan_count": (_c.c_int, []),
}

_lib = None


class MixedGemvError(RuntimeError):
    def __init__(self, status, where):
        self.status = int(status)
        text = lib().mgemv_status_string(self.status).decode()
        super().__init__(f"{where}: status {self.status} ({text})")


def lib():
    """Loads the shared library once; raises if it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} not found: the HIP library is not built "
                "(run `python -m mixed_gemv_amd.build`); there is no CPU fallback")
        # PyTorch ships a HIP runtime of its own.  The library must bind to the runtime that owns the memory of the
        # tensors it is handed, so that runtime has to be in the process before the library is loaded: loaded first,
        # the library would bring in the system's runtime beside it, and every launch on a tensor would then fail
        # with "no usable gfx950 device".
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status, where):
    if status != 0:
        raise MixedGemvError(status, where)
