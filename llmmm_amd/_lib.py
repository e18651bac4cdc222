"""ctypes binding of ``libllmmm.so`` (the C ABI declared in ``include/llmmm.h``).

The library is the product: there is no Python or CPU fallback.  If it is missing, importing
this module raises, so nothing can silently run on another path.
"""
import ctypes
import os

# torch must be loaded first: it brings its own libamdhip64.so (soname libamdhip64.so.7) and
# libllmmm.so then binds to that already-loaded runtime.  Loaded the other way round the process
# ends up with two HIP runtimes, and launches on torch's streams from the second one fail.
import torch  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libllmmm.so")

OK, ERR_NOT_ALIGNED, ERR_UNSUPPORTED_TYPE, ERR_INVALID_ARGUMENT, ERR_WORKSPACE, ERR_RUNTIME = range(6)
DTYPE_F16, DTYPE_BF16, DTYPE_F32 = 0, 1, 2
B_ROW_MAJOR, B_TRANSPOSED = 0, 1
OUT_F32, OUT_BF16, OUT_FP8Q, OUT_FP8Q_SWIGLU = 0, 1, 2, 3
QUANT_1x128_T, QUANT_128x128, QUANT_1x128, QUANT_128x128_T = 0, 1, 2, 3
FP8_B_ROWS, FP8_B_PRESHUFFLED = 0, 1
FP8_A_QUANTISED, FP8_A_SWIGLU_F32, FP8_A_PLANES_RMSNORM = 0, 1, 2


class APlanesRmsnorm(ctypes.Structure):
    """llmmm_a_planes_rmsnorm: the A operand of cfg.a_layout = FP8_A_PLANES_RMSNORM."""
    _fields_ = [("planes", ctypes.c_void_p), ("splits", ctypes.c_int), ("hidden_dtype", ctypes.c_int), ("residual", ctypes.c_void_p),
                ("hidden_out", ctypes.c_void_p), ("norm_weight", ctypes.c_void_p), ("eps", ctypes.c_float)]
PROBE_FP8 = 2
STATIC_WS_BYTES = 16 << 20
TILE_AUTO, TILE_256x256, TILE_128x256, TILE_256x128, TILE_128x128, TILE_64x128, TILE_128x160, TILE_SKINNY, TILE_STRIP = -1, 0, 1, 2, 3, 4, 5, 8, 9


class GemmCfg(ctypes.Structure):
    _fields_ = [("tile", ctypes.c_int), ("split_k", ctypes.c_int), ("b_layout", ctypes.c_int), ("a_layout", ctypes.c_int)]


# name -> (restype, argtypes); must list every symbol include/llmmm.h declares
_c = ctypes
_vp, _fp, _i, _sz = _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_size_t
SIGNATURES = {
    "llmmm_fp16_gemm": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "llmmm_fp16_gemm_ex": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _c.POINTER(GemmCfg), _vp]),
    "llmmm_fp8_gemm": (_i, [_i, _vp, _fp, _vp, _fp, _vp, _fp, _i, _i, _i, _vp, _sz, _vp]),
    "llmmm_fp8_gemm_ex": (_i, [_i, _vp, _fp, _vp, _fp, _vp, _fp, _i, _i, _i, _vp, _sz, _c.POINTER(GemmCfg), _vp]),
    "llmmm_fp8_gemm_static_ws": (_i, [_i, _vp, _fp, _vp, _fp, _vp, _fp, _i, _i, _i, _vp]),
    "llmmm_fp8_gemm_workspace": (_sz, [_i, _i, _i, _i]),
    "llmmm_fp8_gemm_query": (_i, [_i, _i, _i, _i, _c.POINTER(GemmCfg)]),
    "llmmm_quant_fp8": (_i, [_i, _fp, _vp, _fp, _i, _i, _vp]),
    "llmmm_rmsnorm_quant_fp8": (_i, [_i, _vp, _fp, _c.c_float, _vp, _fp, _i, _i, _vp]),
    "llmmm_fp8_gemm_add_rmsnorm_quant": (_i, [_vp, _fp, _vp, _fp, _i, _vp, _vp, _fp, _c.c_float, _vp, _fp, _i, _i, _i, _vp, _sz,
                                              _c.POINTER(GemmCfg), _vp]),
    "llmmm_fp8_gemm_add_rmsnorm_quant_workspace": (_sz, [_i, _i, _i]),
    "llmmm_fp8_gemm_qkv_rope": (_i, [_i, _vp, _fp, _vp, _fp, _vp, _fp, _fp, _fp, _c.c_float, _fp, _fp, _i, _vp, _i, _i, _i, _i, _i, _vp, _sz,
                                     _c.POINTER(GemmCfg), _vp]),
    "llmmm_fp8_gemm_qkv_rope_workspace": (_sz, [_i, _i, _i]),
    "llmmm_fp8_swiglu_a_workspace": (_sz, [_i, _i, _i]),
    "llmmm_fp8_gemm_planes": (_i, [_vp, _fp, _vp, _fp, _i, _i, _i, _vp, _sz, _c.POINTER(_c.c_int), _vp, _sz, _c.POINTER(GemmCfg), _vp]),
    "llmmm_fp8_gemm_planes_bytes": (_sz, [_i, _i, _i]),
    "llmmm_fp8_planes_rmsnorm_a_workspace": (_sz, [_i, _i, _i]),
    "llmmm_fp8_preshuffle_b": (_i, [_vp, _vp, _i, _i, _vp]),
    "llmmm_fp8_unshuffle_b": (_i, [_vp, _vp, _i, _i, _vp]),
    "llmmm_transpose": (_i, [_i, _vp, _vp, _i, _i, _vp]),
    "llmmm_probe_mfma": (_i, [_i, _vp, _fp, _i, _i, _vp]),
    "llmmm_probe_mfma_flops": (_c.c_double, [_i, _i, _i]),
    "llmmm_probe_hbm_read": (_i, [_vp, _sz, _fp, _i, _vp]),
    "llmmm_probe_strip_exchange_timeouts": (_i, [_c.POINTER(_c.c_uint)]),
    "llmmm_probe_phases_bytes": (_sz, [_i, _i]),
    "llmmm_probe_fp8_gemm_phases": (_i, [_vp, _fp, _vp, _fp, _vp, _fp, _i, _i, _i, _vp, _sz, _vp]),
    "llmmm_probe_fp16_gemm_phases": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _vp, _sz, _vp]),
    "llmmm_error_string": (_c.c_char_p, [_i]),
    "llmmm_last_error": (_c.c_char_p, []),
    "llmmm_version": (_i, []),
}


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python llmmm_amd/build.py` (hipcc, gfx950). "
            "There is no fallback path." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise ImportError("%s lacks %s: it is older than the sources, rebuild it with "
                              "`python llmmm_amd/build.py`" % (LIB_PATH, name)) from None
        fn.restype, fn.argtypes = res, args
    return lib


lib = load()


def check(code):
    """Turn a status code into the exception the reference's launchers throw.

    Codes 1 and 2 carry the reference's own texts (src/mm/fp16/mm.cu:15-21, src/base/base.cu:127-129, :265-267)."""
    if code == OK:
        return
    text = lib.llmmm_error_string(code).decode()
    detail = lib.llmmm_last_error().decode()
    if code in (ERR_NOT_ALIGNED, ERR_UNSUPPORTED_TYPE):
        raise RuntimeError(detail or text)  # the detail is the reference's text for the entry point that failed
    raise RuntimeError("%s: %s" % (text, detail) if detail else text)
