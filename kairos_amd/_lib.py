"""ctypes binding of libkairos_mi.so (the C ABI declared in include/kairos_mi.h).

The library is the only compute path: if it is missing this module raises, nothing falls back to
PyTorch or to the CPU.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkairos_mi.so")

_P = ctypes.c_void_p
_I = ctypes.c_int
_Z = ctypes.c_size_t
_IP = ctypes.POINTER(ctypes.c_int)

# name -> argument types (every function returns int unless listed in _RESTYPE)
SIGNATURES = {
    "kmi_version": [],
    "kmi_get_last_error_string": [],
    "kmi_cvt_i4_to_f16": [_P, _P, _P, _P, _I, _I, _I, _P],
    "kmi_cvt_i4_to_i8": [_P, _P, _P, _P, _I, _I, _I, _P],
    "kmi_cvt_i4_to_f16_tiled": [_P, _P, _P, _P, _I, _I, _I, _P],
    "kmi_cvt_i4_to_i8_tiled": [_P, _P, _P, _P, _I, _I, _I, _P],
    "kmi_untile": [_P, _P, _I, _I, _I, _P],
    "kmi_quant_act_i8": [_P, _P, _P, _I, _I, _P],
    "kmi_prep_w8a8": [_P, _I, _P, _P, _P, _I, _I, _I, _P, _P, _P, _I, _P],
    "kmi_rmsnorm_quant_act": [_P, _P, _P, _P, _P, _P, _P, ctypes.c_float, _I, _I, _P],
    "kmi_silu_mul_quant_act": [_P, _P, _P, _P, _I, _I, _P],
    "kmi_prepare_weight": [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P],
    "kmi_padded_groups": [_I, _I],
    "kmi_trans_layout_w4a8": [_P, _P, _I, _I, _P],
    "kmi_gemv_w4a16": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemv_w4a16_cfg": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemv_w4a16_ring_cfg": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemv_w4a16_plan": [_I, _I, _I, _Z, _IP, _IP, _IP, _IP, _IP],
    "kmi_gemv_ws_reset": [_P, _Z, _P],
    # GEMMs end with (workspace pointer, workspace bytes, stream)
    "kmi_gemm_w4a16": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w4a16_noalloc": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "kmi_gemm_w8a16": [_P, _P, _P, _P, _P, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w8a8": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w8a8_acc_i32": [_P, _P, _P, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w4a8": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w4a8_acc_i32": [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w4a8_pick_tile": [_I, _I, _I],
    "kmi_gemm_w4a8_int": [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w4a8_int_acc_i32": [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_f16": [_P, _P, _P, _P, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_w8a8_tiled": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_f16_tiled": [_P, _P, _P, _P, _I, _I, _I, _P, _Z, _P],
    "kmi_gemm_force_tile": [_I],
    "kmi_gemm_pick_tile": [_I, _I, _I],
    "kmi_gemm_w4a16_wp_rows": [_I, _I, _I],
    "kmi_gemm_splits_for": [_I, _I, _I, _I, _Z],
    "kmi_gemm_force_splits": [_I],
    "kmi_gemm_force_group_m": [_I],
    "kmi_lut_new": [],
    "kmi_lut_free": [_P],
    "kmi_lut_record": [_P, _I, _I],
    "kmi_lut_get": [_P, _I],
    "kmi_lut_shrink_to_fit": [_P],
    "kmi_lut_size": [_P],
    "kmi_probe_empty": [_P],
    "kmi_probe_stream_read": [_P, _Z, _P],
    "kmi_probe_gemv_read": [_P, _I, _I, _I, _I, _P],
    "kmi_probe_mfma_stream": [_I, _P, _Z, _I, _I, _P, _P],
    "kmi_probe_pipe_overlap": [_I, _P, _P],
    "kmi_cache_create": [_P, _Z],
    "kmi_cache_destroy": [_P],
    "kmi_cache_acquire": [_P, ctypes.c_uint64, _I, _Z, ctypes.POINTER(_P)],
    "kmi_cache_invalidate": [_P],
    "kmi_cache_stats": [_P, ctypes.POINTER(_Z), ctypes.POINTER(_Z), ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64)],
}
_RESTYPE = {"kmi_get_last_error_string": ctypes.c_char_p, "kmi_lut_new": _P, "kmi_lut_free": None,
            "kmi_cache_create": _P, "kmi_cache_destroy": None,
            "kmi_gemm_force_tile": None, "kmi_gemm_force_splits": None, "kmi_gemm_force_group_m": None}

_lib = None


class KairosMiError(RuntimeError):
    """A C-ABI call returned a negative status; mirrors the RuntimeError pybind raises in the reference."""

    def __init__(self, code, message):
        super().__init__(f"[kairos_mi {code}] {message}")
        self.code = code


def load():
    global _lib
    if _lib is not None:
        return _lib
    # PyTorch ships its own HIP runtime under the same soname as the system one.  It must be the
    # first (and only) copy in the process, so that streams, events and allocations are shared
    # between torch and this library: load torch before dlopen-ing anything that needs the runtime.
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m kairos_amd.build` "
            "(the HIP library is the only compute path; there is no fallback)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if a declared symbol is not exported
        fn.argtypes = args
        fn.restype = _RESTYPE.get(name, _I)
    _lib = lib
    return lib


def check(rc):
    if rc < 0:
        raise KairosMiError(rc, load().kmi_get_last_error_string().decode())
    return rc
