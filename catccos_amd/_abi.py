"""ctypes view of libcatccos_hip.so (the C ABI declared in include/catccos_hip.h).

The library must exist: there is no CPU fallback.  Build it with
``python -m catccos_amd.build``.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libcatccos_hip.so")

OK, EINVAL, EHIP, ENODEV, ENOSUP = 0, -1, -2, -3, -4
FMT_E4M3, FMT_E5M2, FMT_E2M1, FMT_E1M2 = 0, 1, 2, 3
ROUND_RNE, ROUND_LUT = 0, 1

c = ctypes
_P, _I64, _I, _SZ = c.c_void_p, c.c_int64, c.c_int, c.c_size_t

# name -> argument types; every entry returns int unless listed in _RESTYPE
PROTOTYPES = {
    "cch_init": [_I],
    "cch_last_error": [],
    "cch_device_info": [c.c_char_p, _SZ, c.POINTER(_I), c.POINTER(_I), c.POINTER(c.c_uint64)],
    "cch_malloc": [c.POINTER(_P), _SZ],
    "cch_free": [_P],
    "cch_malloc_host": [c.POINTER(_P), _SZ],
    "cch_free_host": [_P],
    "cch_memcpy_h2d": [_P, _P, _SZ],
    "cch_memcpy_d2h": [_P, _P, _SZ],
    "cch_memset": [_P, _I, _SZ],
    "cch_stream_create": [c.POINTER(_P)],
    "cch_stream_sync": [_P],
    "cch_stream_destroy": [_P],
    "cch_mx_quant_rows": [_P, _P, _P, _I64, _I64, _I, _I, _P],
    "cch_mx_quant_rows_f16": [_P, _P, _P, _I64, _I64, _I, _I, _P],
    "cch_mx_quant_b": [_P, _P, _P, _I64, _I64, _I, _I, _I, _P],
    "cch_mx_quant_scatter_packed": [_P, _P, _P, _I64, _I64, _I, _I, _I, _P],
    "cch_mx_quant_scatter_packed_rows": [_P, _P, _P, _I64, _I64, _I64, _I, _I, _I, _P],
    "cch_moe_token_unpermute": [_P, _P, _P, _P, _I64, _I64, _I64, _I, _P],
    "cch_moe_init_routing_workspace_bytes": [_I64, _I],
    "cch_moe_init_routing": [_P, _I64, _I, _P, _P, _P, _I, _P, _I64, _P],
    "cch_moe_init_routing_noalloc": [_P, _I64, _I, _P, _P, _P, _I, _P],
    "cch_dyn_quant_i8_rows": [_P, _P, _P, _P, _I64, _I64, _I64, _I, _I, _P],
    "cch_dyn_quant_i8_rows_smooth": [_P, _P, _P, _P, _I64, _P, _P, _I64, _I64, _I64, _I, _I, _P],
    "cch_gemm_i8_dequant": [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I, _P],
    "cch_gemm_i8_dequant_out": [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I, _I, _P],
    "cch_gmm_i8_dequant_out": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _I, _P],
    "cch_gmm_i8_dequant_swiglu_out": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _I, _P],
    "cch_gmm_i8_dequant_swiglu_mx": [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _I, _P],
    "cch_mx_gmm_swiglu": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _I, _I, _P],
    "cch_mx_gmm_swiglu_mx_packed": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _I, _I, _P],
    "cch_mx_gmm_swiglu_mx": [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _I, _I, _P],
    "cch_mx_gemm_out": [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I, _I, _I, _P],
    "cch_gmm_i8_dequant": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _P],
    "cch_gmm_i8_dequant_swiglu": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _P],
    "cch_mx_gemm": [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I, _I, _P],
    "cch_mx_gmm": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I, _I, _P],
    "cch_mx_gmm_mapped": [_P, _P, _P, _P, _P, _P, _P, _I64, _I, _I64, _I64, _I64, _I64, _I, _I, _P],
    "cch_set_option": [c.c_char_p, _I],
}
_RESTYPE = {"cch_last_error": c.c_char_p, "cch_moe_init_routing_workspace_bytes": _I64}

_lib = None


class CatccosError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("catccos_hip error %d: %s" % (code, msg))
        self.code = code


def lib():
    """Loads the library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                LIB_PATH + " is missing: build it with `python -m catccos_amd.build` (no CPU fallback exists)")
        L = ctypes.CDLL(LIB_PATH)
        for name, args in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _RESTYPE.get(name, _I)
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise CatccosError(rc, lib().cch_last_error().decode())
    return rc
