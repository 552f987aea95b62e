"""The C-ABI library loads on a machine without a GPU and exports exactly the
entry points include/cubework_hip.h declares; argument validation that needs
no device works. No compute is launched here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cubework_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cw_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    from cubework_amd import _lib
    assert _declared_functions() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    from cubework_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libcubework_hip.so not built yet (python -m cubework_amd.build)")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(lib, name), name
    lib = _lib.load()
    assert b"gfx950" in lib.cw_version()


def test_argument_validation_without_a_device():
    from cubework_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libcubework_hip.so not built yet")
    lib = _lib.load()
    assert lib.cw_gemm_ksteps(9, 8, 8, 8, 1, None, 8, None, 8, None, 0, None, 8, None, 0, None, 0, 0, 0, None) == -1
    assert b"layout" in lib.cw_last_error()
    assert lib.cw_gemm_ksteps(0, 8, 8, 8, 99, None, 8, None, 8, None, 0, None, 8, None, 0, None, 0, 0, 0, None) == -1
    assert b"n_steps" in lib.cw_last_error()
    assert lib.cw_gemm_ksteps(0, 0, 8, 8, 1, None, 8, None, 8, None, 0, None, 8, None, 0, None, 0, 0, 0, None) == 0
    assert lib.cw_ln_partial_stats(4, 0, None, 0, 0, None, None, 0, None) == -1
    assert lib.cw_ln_partial_stats(0, 8, None, 8, 0, None, None, 0, None) == 0  # empty input is fine
    assert lib.cw_vpce_fwd_local(4, 8, None, 8, None, -1, None, None, None, None, 0, None) == -1
    assert b"vocab_start" in lib.cw_last_error()
    assert lib.cw_vpce_bwd(4, 8, None, 8, None, 0, None, None, None, 1.0, None, 8, 1, 0, None) == -3
    assert lib.cw_colsum_workspace_bytes(8192, 2048) >= 512 * 2048 * 4
    with pytest.raises(_lib.CubeworkHipError):
        _lib.check(-1, "example")
