"""ctypes binding of libcubework_hip.so (declared in include/cubework_hip.h).

The library is the only compute path of this package: if it cannot be loaded
the import of any operator fails with an error instead of falling back to
torch.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# CUBEWORK_HIP_LIB selects another build of the library (kernel experiments).
LIB_PATH = os.environ.get("CUBEWORK_HIP_LIB") or os.path.join(_HERE, "libcubework_hip.so")

# enums of include/cubework_hip.h
CW_BF16, CW_F32, CW_F16 = 0, 1, 2
CW_NN, CW_NT, CW_TN = 0, 1, 2
CW_EPI_NONE, CW_EPI_BIAS, CW_EPI_BIAS_GELU_TANH, CW_EPI_BIAS_GELU_ERF, CW_EPI_BIAS_RELU = 0, 1, 2, 3, 4
CW_ACT_NONE, CW_ACT_GELU_TANH, CW_ACT_GELU_ERF, CW_ACT_RELU = 0, 2, 3, 4
CW_LN_ONE_PASS, CW_LN_TWO_PASS = 0, 1
CW_MAX_KSTEPS, CW_MAX_ADDENDS = 16, 8
CW_ERR_INVALID, CW_ERR_ALIGNMENT, CW_ERR_UNSUPPORTED, CW_ERR_LAUNCH, CW_ERR_DEVICE = -1, -2, -3, -4, -5

_i64 = ctypes.c_int64
_int = ctypes.c_int
_ptr = ctypes.c_void_p
_f32 = ctypes.c_float
_pp = ctypes.POINTER(ctypes.c_void_p)

# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "cw_version": (ctypes.c_char_p, []),
    "cw_device_arch": (ctypes.c_char_p, []),
    "cw_last_error": (ctypes.c_char_p, []),
    "cw_gemm_ksteps": (_int, [_int, _i64, _i64, _i64, _int, _pp, _i64, _pp, _i64, _ptr, _int, _ptr, _i64, _ptr, _i64,
                              _pp, _int, _i64, _int, _ptr]),
    "cw_gemm_workspace_bytes": (_i64, [_int, _i64, _i64, _i64, _int, _int]),
    "cw_gemm_ksteps_ws": (_int, [_int, _i64, _i64, _i64, _int, _pp, _i64, _pp, _i64, _ptr, _int, _ptr, _i64, _ptr, _i64,
                                 _pp, _int, _i64, _ptr, _i64, _int, _ptr]),
    "cw_multi_norm_workspace_bytes": (_i64, [_int, _ptr]),
    "cw_multi_norm_partials": (_int, [_int, _pp, _ptr, _ptr, _ptr, _f32, _ptr, _ptr, _i64, _int, _ptr]),
    "cw_clip_coef": (_int, [_int, _ptr, _f32, _f32, _f32, _ptr, _ptr]),
    "cw_multi_scale": (_int, [_int, _pp, _ptr, _ptr, _int, _ptr]),
    "cw_multi_norm_partial_count": (_i64, [_int, _ptr]),
    "cw_clip_scale": (_int, [_int, _pp, _ptr, _int, _int, _ptr, _i64, _ptr, _f32, _f32, _f32, _ptr, _ptr]),
    "cw_embed_fwd": (_int, [_i64, _i64, _ptr, _i64, _i64, _ptr, _i64, _ptr, _i64, _int, _ptr]),
    "cw_embed_sort_workspace_bytes": (_i64, [_i64]),
    "cw_embed_sort_ids": (_int, [_i64, _ptr, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr]),
    "cw_embed_bwd": (_int, [_i64, _i64, _ptr, _ptr, _i64, _i64, _i64, _ptr, _i64, _ptr, _i64, _int, _ptr]),
    "cw_embed_bwd_ids_supported": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _int]),
    "cw_embed_bwd_ids": (_int, [_i64, _i64, _ptr, _i64, _i64, _i64, _ptr, _i64, _ptr, _i64, _int, _ptr]),
    "cw_attn_fwd": (_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _i64, _i64, _f32, _int, _ptr, _i64, _i64, _i64,
                           _ptr, _int, _ptr]),
    "cw_attn_bwd_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "cw_attn_bwd": (_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr, _i64, _i64, _i64, _ptr,
                           _f32, _int, _ptr, _ptr, _ptr, _i64, _i64, _i64, _ptr, _i64, _int, _ptr]),
    "cw_colsum_workspace_bytes": (_i64, [_i64, _i64]),
    "cw_colsum": (_int, [_i64, _i64, _ptr, _i64, _ptr, _int, _ptr, _i64, _int, _ptr]),
    "cw_colsum_static_max_bytes": (_i64, []),
    "cw_colsum_static": (_int, [_i64, _i64, _ptr, _i64, _ptr, _int, _int, _ptr]),
    "cw_act_bwd_colsum": (_int, [_int, _i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _int, _ptr, _i64, _int, _ptr]),
    "cw_ln_partial_stats": (_int, [_i64, _i64, _ptr, _i64, _int, _ptr, _ptr, _int, _ptr]),
    "cw_ln_normalize": (_int, [_i64, _i64, _ptr, _i64, _ptr, _int, _i64, _f32, _ptr, _ptr, _ptr, _i64, _ptr, _int,
                               _ptr]),
    "cw_ln_forward_fused": (_int, [_i64, _i64, _ptr, _i64, _int, _f32, _ptr, _ptr, _ptr, _i64, _ptr, _int, _ptr]),
    "cw_ln_bwd_partials": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _i64, _int,
                                  _ptr]),
    "cw_ln_backward_fused": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr,
                                    _int, _ptr, _i64, _int, _ptr]),
    "cw_ln_bwd_dx": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _int, _ptr]),
    "cw_ln_bwd_partials_open": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _int, _ptr]),
    "cw_ln_bwd_dx_close": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr,
                                  _ptr, _int, _int, _ptr]),
    "cw_vpce_fwd_local": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr]),
    "cw_vpce_finalize": (_int, [_i64, _int, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "cw_vpce_bwd": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _f32, _ptr, _i64, _int, _int, _ptr]),
}

_lib = None


class CubeworkHipError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


def load():
    """Load (once) and return the shared library; raise if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libcubework_hip.so is not built (expected at %s). Run `python -m cubework_amd.build`; "
            "there is no fallback compute path." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status, what):
    if status != 0:
        msg = load().cw_last_error().decode("utf-8", "replace")
        raise CubeworkHipError("%s failed (status %d): %s" % (what, status, msg))
