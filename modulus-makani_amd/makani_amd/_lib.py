"""ctypes binding of libsfno_spectral.so (the C ABI declared in include/sfno_spectral.h).

The library is built in-tree next to this file by ``build.py`` (hipcc, gfx950).  There is
no fallback implementation: if the shared object is missing, importing this module
raises, and every compute entry point raises on a non-zero return code.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsfno_spectral.so")

GRID = {"legendre-gauss": 0, "lobatto": 1, "equiangular": 2, "planar": 3}
NORM = {"ortho": 0, "four-pi": 1, "schmidt": 2}
DIR_FORWARD, DIR_INVERSE, DIR_FORWARD_ADJOINT, DIR_INVERSE_ADJOINT = 1, 2, 4, 8
COMPUTE_FP32, COMPUTE_BF16, COMPUTE_FP32_MFMA, COMPUTE_FP32_BF16X3 = 0, 1, 2, 3
DTYPE_F32, DTYPE_BF16 = 0, 1
ACT_NONE, ACT_GELU = 0, 1


class SfnoError(RuntimeError):
    pass


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build the HIP library first (python modulus-makani_amd/build.py); "
            "this package has no CPU or PyTorch fallback"
        )
    lib = ctypes.CDLL(LIB_PATH)
    c = ctypes
    vp, i32, i64, sz = c.c_void_p, c.c_int, c.c_int64, c.c_size_t
    dp = c.POINTER(c.c_double)
    sig = {
        "sfno_strerror": (c.c_char_p, [i32]),
        "sfno_version": (i32, []),
        "sfno_quadrature": (i32, [i32, i32, dp, dp]),
        "sfno_legendre_table": (i32, [i32, i32, i32, dp, i32, i32, i32, dp]),
        "sfno_legendre_stream_skips": (i64, [i32, i32, i32, dp, dp, i32, i32, i32, i32, c.POINTER(c.c_int32), i64]),
        "sfno_sht_plan_create": (i32, [i32, i32, i32, i32, i32, i32, i32, i32, i32, c.POINTER(vp)]),
        "sfno_sht_plan_destroy": (i32, [vp]),
        "sfno_spectral_ld": (i64, [i64]),
        "sfno_spectral_elems": (i64, [vp, i64]),
        "sfno_sht_workspace_bytes": (sz, [vp, i64]),
        "sfno_sht_forward": (i32, [vp, vp, vp, i64, vp, sz, vp]),
        "sfno_sht_inverse": (i32, [vp, vp, vp, i64, vp, sz, vp]),
        "sfno_sht_forward_static": (i32, [vp, vp, vp, i64, vp]),
        "sfno_sht_io_dtype_supported": (i32, [vp, i32]),
        "sfno_sht_analysis": (i32, [vp, vp, i32, vp, i64, vp, sz, vp]),
        "sfno_sht_synthesis": (i32, [vp, vp, vp, i32, i64, vp, sz, vp]),
        "sfno_sht_lat_stats_supported": (i32, [vp]),
        "sfno_sht_synthesis_lat_stats": (i32, [vp, vp, vp, i32, i64, vp, sz, vp, vp]),
        "sfno_sht_forward_adjoint": (i32, [vp, vp, vp, i64, vp, sz, vp]),
        "sfno_sht_inverse_adjoint": (i32, [vp, vp, vp, i64, vp, sz, vp]),
        "sfno_sht_analysis_adjoint": (i32, [vp, vp, vp, i32, i64, vp, sz, vp]),
        "sfno_sht_synthesis_adjoint": (i32, [vp, vp, i32, vp, i64, vp, sz, vp]),
        "sfno_rfft": (i32, [vp, vp, i32, vp, i64, vp]),
        "sfno_irfft": (i32, [vp, vp, vp, i32, i64, vp]),
        "sfno_legendre_analysis": (i32, [vp, vp, vp, i64, vp]),
        "sfno_legendre_synthesis": (i32, [vp, vp, vp, i64, vp]),
        "sfno_fourier_elems": (i64, [vp, i64]),
        "sfno_coeffs_to_spectral": (i32, [vp, vp, i64, i32, i32, i32, vp]),
        "sfno_spectral_to_coeffs": (i32, [vp, vp, i64, i32, i32, i32, vp]),
        "sfno_dhconv_weights_create": (i32, [i32, i32, i32, i32, c.POINTER(vp)]),
        "sfno_dhconv_weights_update": (i32, [vp, vp, vp]),
        "sfno_dhconv_weights_destroy": (i32, [vp]),
        "sfno_dhconv_weights_update_adjoint": (i32, [vp, vp, vp]),
        "sfno_dhconv_weight_grad": (i32, [i32, i32, i32, vp, vp, vp, i32, i32, i32, vp]),
        "sfno_dhconv_spectral": (i32, [vp, vp, vp, i32, i32, i32, vp]),
        "sfno_dhconv_workspace_bytes": (sz, [vp, i32, i32]),
        "sfno_dhconv": (i32, [vp, vp, vp, i32, i32, i32, vp, sz, vp]),
        "sfno_degree_power": (i32, [vp, vp, i64, i32, i32, vp]),
        "sfno_degree_power_grad": (i32, [vp, vp, vp, i64, i32, i32, vp]),
        "sfno_diagonal_contract": (i32, [vp, vp, vp, i32, i32, i32, i64, i32, vp]),
        "sfno_diagonal_weight_grad": (i32, [vp, vp, vp, i32, i32, i32, i64, vp]),
        "sfno_pointwise_weight_elems": (i64, [i32, i32]),
        "sfno_pointwise_pack_weight": (i32, [vp, vp, i32, i32, vp]),
        "sfno_pointwise_conv": (i32, [vp, vp, vp, vp, i32, i32, i32, i64, i32, vp, vp, vp, vp]),
        "sfno_pointwise_conv_cat": (i32, [vp, i32, vp, i32, vp, vp, vp, i32, i32, i64, i32, vp]),
        "sfno_pointwise_weight_grad_workspace_bytes": (sz, [i32, i32, i32, i64, i32]),
        "sfno_pointwise_weight_grad": (i32, [vp, vp, vp, vp, i32, i32, i32, i64, vp, sz, vp]),
        "sfno_instance_norm_workspace_bytes": (sz, [i64, i64]),
        "sfno_instance_norm_coeffs": (i32, [vp, vp, vp, vp, vp, i64, i32, i64, c.c_float, vp, sz, vp]),
        "sfno_instance_norm_coeffs_lat": (i32, [vp, vp, vp, vp, vp, i64, i32, i32, c.c_float, vp]),
        "sfno_scale_shift_act": (i32, [vp, vp, vp, vp, i64, i64, i32, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib, tuple(sig)


lib, EXPORTS = _load()


def check(code, what):
    if code != 0:
        raise SfnoError(f"{what} failed: {lib.sfno_strerror(code).decode()} ({code})")
