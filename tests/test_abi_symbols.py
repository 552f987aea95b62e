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


def test_scratch_sizes_and_refusals_of_the_later_entry_points():
    """Host-only parts of the entry points added after the first set: scratch sizing and the argument checks
    that come before any device work."""
    import ctypes as C
    from cubework_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libcubework_hip.so not built yet")
    lib = _lib.load()
    NN, NT, TN, BF16, F32 = 0, 1, 2, 0, 1
    # split-k: few tiles, long reduction (config-2 weight gradient: 64 tiles x 4 slices of fp32 partials)
    assert lib.cw_gemm_workspace_bytes(TN, 2048, 2048, 8192, 2, BF16) == 4 * 2048 * 2048 * 4
    assert lib.cw_gemm_workspace_bytes(NN, 8192, 2048, 2048, 2, BF16) == 0
    assert lib.cw_gemm_workspace_bytes(TN, 2048, 2048, 2048, 1, BF16) == 0    # 256 tiles of 128 x 128: the small-tile ring kernel
    assert lib.cw_gemm_workspace_bytes(TN, 1024, 1024, 2048, 1, BF16) > 0     # 64 small tiles: split k
    assert lib.cw_gemm_workspace_bytes(TN, 2048, 2048, 8192, 2, F32) == 0
    # reduction length that is not a multiple of 32 with B stored [K, N]: 32 rows of B
    assert lib.cw_gemm_workspace_bytes(NN, 8192, 2048, 12568, 1, BF16) == 32 * 2048 * 2
    assert lib.cw_gemm_workspace_bytes(TN, 8192, 2048, 12568, 1, BF16) == 32 * 2048 * 2
    assert lib.cw_gemm_workspace_bytes(NT, 8192, 2048, 12568, 1, BF16) == 0   # B is [N, K]: not provided
    assert lib.cw_gemm_workspace_bytes(NN, 8192, 2048, 12568, 2, BF16) == 0   # one step only
    assert lib.cw_gemm_workspace_bytes(NN, 512, 512, 12568, 1, BF16) == 0     # small outputs keep the guarded kernel
    # token order: direct ranks need no scratch, the sorting network one 64-bit key per padded token
    assert lib.cw_embed_sort_workspace_bytes(16384) == 0
    assert lib.cw_embed_sort_workspace_bytes(16385) == 32768 * 8
    assert lib.cw_embed_sort_ids(-1, None, 0, 8, None, None, None, 0, None) == -1
    assert lib.cw_embed_sort_ids(4, None, 0, 0, None, None, None, 0, None) == -1
    assert b"V_loc" in lib.cw_last_error()
    assert lib.cw_embed_sort_ids(0, None, 0, 8, None, None, None, 0, None) == 0
    assert lib.cw_embed_sort_ids(20000, None, 0, 8, None, None, None, 0, None) == -1  # null pointers
    # gradient-norm clipping
    numels = (C.c_int64 * 3)(65536, 1, 65537)
    assert lib.cw_multi_norm_workspace_bytes(3, C.cast(numels, C.c_void_p)) == (1 + 1 + 2) * 2 * 4
    assert lib.cw_clip_coef(0, None, 1.0, 2.0, 1.0, None, None) == -1
    assert lib.cw_clip_coef(1, None, 1.0, 2.0, 1.0, None, None) == -1
    assert lib.cw_multi_norm_partial_count(3, C.cast(numels, C.c_void_p)) == 1 + 1 + 2
    assert lib.cw_multi_norm_partial_count(0, None) == 0
    assert lib.cw_clip_scale(0, None, None, BF16, 1, None, 0, None, 1.0, 2.0, 1.0, None, None) == -1
    # attention: head sizes other than 64 / 128 and fp32 are refused before any launch
    assert lib.cw_attn_bwd_workspace_bytes(4, 32, 2048) == 4 * 32 * 2048 * 4
    args = [1, 1, 8, 80, None, None, None, 240, 240, 240, 0.1, 1, None, 80, 80, 80, None, BF16, None]
    assert lib.cw_attn_fwd(*args) == -3
    assert b"head size" in lib.cw_last_error()
    args[3], args[17] = 64, F32
    assert lib.cw_attn_fwd(*args) == -3
    # fused LayerNorm backward: the two column outputs come together
    assert lib.cw_ln_backward_fused(4, 8, None, 8, None, 8, None, None, None, None, 8, None, 0, None, C.c_void_p(16), F32, None, 0, BF16, None) == -1
    assert b"both" in lib.cw_last_error()


def test_no_usable_device_is_reported_as_such():
    """Without a GPU (or on one that is not gfx950) a call that passes its argument checks returns
    CW_ERR_DEVICE before anything is launched; the pointers are never touched."""
    import ctypes as C
    import torch
    from cubework_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libcubework_hip.so not built yet")
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible: the refusal path needs a machine without one")
    lib = _lib.load()
    p = C.c_void_p(256)
    assert lib.cw_colsum(8, 8, p, 8, p, _lib.CW_F32, p, 1 << 20, _lib.CW_F32, None) == -5
    assert b"device" in lib.cw_last_error().lower()
    assert lib.cw_colsum_static(8, 8, p, 8, p, _lib.CW_F32, _lib.CW_F32, None) == -5
    assert lib.cw_ln_partial_stats(4, 8, p, 8, _lib.CW_LN_ONE_PASS, None, p, _lib.CW_BF16, None) == -5
    tab = (C.c_void_p * 1)(256)
    assert lib.cw_gemm_ksteps(_lib.CW_NN, 8, 8, 8, 1, tab, 8, tab, 8, None, 0, p, 8, None, 0, None, 0, 0, _lib.CW_BF16, None) == -5
    assert lib.cw_vpce_finalize(4, 1, p, p, p, p, p, p, p, None) == -5
    assert lib.cw_device_arch() == b""


def test_measurement_library_is_separate_from_the_boundary():
    """The measurement aids bench.py uses (MFMA rate loop, the ring kernel with one part taken out) live in a
    library of their own: the product library exports none of them, and their host-side checks work without a
    device."""
    from cubework_amd import _diag, _lib
    if not os.path.exists(_lib.LIB_PATH) or not os.path.exists(_diag.LIB_PATH):
        pytest.skip("libraries not built yet")
    product = ctypes.CDLL(_lib.LIB_PATH)
    for name in _diag.SIGNATURES:
        if name.startswith("cw_diag"):
            assert not hasattr(product, name), name
    diag = _diag.load()
    assert diag.cw_diag_mfma_rate(0, 0, None, None) == -1
    assert diag.cw_diag_mfma_rate(10, 4, None, None) == -1
    assert b"mode" in diag.cw_last_error()
    assert diag.cw_diag_overlap(10, 0, 0, None, None) == -1
    assert diag.cw_diag_lds_rate(10, 2, None, None) == -1
    assert diag.cw_diag_lds_rate_bytes(3) == 3 * 65536
    assert diag.cw_diag_mfma_rate_flop(2) == 2 * 1024 * 16 * 32768
    assert diag.cw_diag_gemm_part(7, 8192, 2048, 2048, 2, None, 2048, None, 2048, None, None, 2048, None) == -1
    tab = (ctypes.c_void_p * 2)(256, 256)
    p = ctypes.c_void_p(256)
    assert diag.cw_diag_gemm_part(1, 8192, 2000, 2048, 2, tab, 2048, tab, 2048, p, p, 2048, None) == -3
