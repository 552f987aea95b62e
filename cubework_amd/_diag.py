"""ctypes binding of libcubework_diag.so: measurement aids for bench.py (and their tests), built from
csrc/diag.hip and csrc/diag_gemm.hip. Not part of the product: nothing under cubework_amd/ but this file loads
it, the operators never call it, and libcubework_hip.so exports none of its symbols.

  cw_diag_mfma_rate(iters, mode, sink, stream)   the GEMM's matrix instruction back to back from registers
                                                 (mode 0 random operands, 1 zeros, 2 random operands read from LDS,
                                                 3 random operands, the 16 x 16 x 32 instruction)
  cw_diag_mfma_rate_flop(iters)                  FLOP of one such call
  cw_diag_overlap(iters, roles, vop, sink, stream)
                                                 two wavefronts per SIMD, one issuing MFMAs (roles bit 0), one vector
                                                 instructions (bit 1; vop 0 v_fma_f32, 1 v_exp_f32): how far they overlap
  cw_diag_lds_rate(iters, transposing, sink, stream), cw_diag_lds_rate_bytes(iters)
                                                 LDS read rate of a compute unit: ds_read_b128 / ds_read_b64_tr_b16
  cw_diag_gemm_part(part, M, N, K, n_steps, A_steps, lda, B_steps, ldb, bias, C, ldc, stream)
                                                 the ring kernel of the block GEMM (NN, bf16, bias + GeLU-tanh) whole
                                                 (part 0) or without its operand loads (1), its epilogue (2), its LDS
                                                 fragment reads (3)
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcubework_diag.so")

_i64, _int, _ptr = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
_pp = ctypes.POINTER(ctypes.c_void_p)

SIGNATURES = {
    "cw_last_error": (ctypes.c_char_p, []),
    "cw_diag_mfma_rate_flop": (_i64, [_int]),
    "cw_diag_mfma_rate": (_int, [_int, _int, _ptr, _ptr]),
    "cw_diag_overlap": (_int, [_int, _int, _int, _ptr, _ptr]),
    "cw_diag_lds_rate_bytes": (_i64, [_int]),
    "cw_diag_lds_rate": (_int, [_int, _int, _ptr, _ptr]),
    "cw_diag_gemm_part": (_int, [_int, _i64, _i64, _i64, _int, _pp, _i64, _pp, _i64, _ptr, _ptr, _i64, _ptr]),
}

_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("libcubework_diag.so is not built (expected at %s). Run `python -m cubework_amd.build`." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib
