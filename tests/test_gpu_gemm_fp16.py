"""GPU parity of the float16 flavour of cw_gemm_ksteps / cw_colsum / cw_act_bwd_colsum (through the C ABI)
against the CPU oracle: the dtype torch's autocast hands the reference's GEMM-type Functions
(custom_fwd(cast_inputs=torch.float16), cubework/module/parallel_2d/_operation.py:17,96,176,255,363).

Bar: <= 1e-3 relative to the largest magnitude of the expected result (fp32 accumulation, one rounding to
float16), the rtol of the reference's own tests (tests/test_2d/check_2d_modules.py).
"""
import pytest
import torch

from tests.test_gpu_gemm import LAYOUTS, _run
from tests.util import assert_parity, rand_uniform, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F16 = torch.float16


@pytest.mark.parametrize("layout", LAYOUTS)
def test_f16_exact_tiles_small_and_big_config(layout):
    _run(layout, 256, 384, 192, 2, F16, act=None)                   # 128x128 tiles
    _run(layout, 4096, 2048, 256, 2, F16, act="gelu_tanh")          # LDS-DMA kernel, 256x256 tiles


@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("shape", [(300, 200, 100), (1, 8, 8), (129, 1, 3), (64, 130, 520)])
def test_f16_ragged(layout, shape):
    M, N, K = shape
    _run(layout, M, N, K, 3, F16, act="relu", seed=3)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_f16_ragged_around_aligned_core(layout):
    _run(layout, 4104, 8200, 64, 2, F16, act="gelu_tanh", n_add=1, preact=True, seed=5)
    _run(layout, 4100, 2056, 136, 2, F16, act="gelu_erf", seed=5)   # guarded 256x256 tiles


@pytest.mark.parametrize("layout", LAYOUTS)
def test_f16_mostly_empty_last_round_goes_to_small_tiles(layout):
    _run(layout, 4096, 4376, 128, 2, F16, act="gelu_tanh", n_add=1, preact=True, seed=11)   # 280 columns peeled
    _run(layout, 8472, 2048, 64, 1, F16, act="relu", seed=12)                               # 280 rows peeled


@pytest.mark.parametrize("layout", ["NN", "TN"])
def test_f16_ragged_reduction_length(layout):
    _run(layout, 4096, 8192, 344, 1, F16, act="relu", n_add=1, preact=True, seed=7)


@pytest.mark.parametrize("act", [None, "gelu_tanh", "gelu_erf", "relu"])
def test_f16_epilogues_with_preact_and_addends(act):
    _run("NN", 384, 256, 128, 2, F16, act=act, n_add=2, preact=True, seed=7)
    _run("NT", 130, 70, 50, 2, F16, act=act, pad_a=3, pad_b=5, seed=12)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_f16_split_k_long_reduction(layout):
    from cubework_amd import _lib
    from cubework_amd.ops import LAYOUTS as CODES

    assert _lib.load().cw_gemm_workspace_bytes(CODES[layout], 512, 768, 1024, 2, _lib.CW_F16) > 0
    _run(layout, 512, 768, 1024, 2, F16, act="gelu_tanh", n_add=1, preact=True, seed=5)


def test_f16_differs_from_bf16_reading_of_the_same_bits():
    """The element type reaches the kernel: the same 16-bit patterns multiplied as float16 and as bfloat16
    give the products of the respective values."""
    from cubework_amd import ops

    a = randn((256, 128), F16, 1).to(DEV)
    b = randn((128, 256), F16, 2).to(DEV)
    as_f16 = ops.gemm_ksteps("NN", [a], [b])
    as_bf16 = ops.gemm_ksteps("NN", [a.view(torch.bfloat16)], [b.view(torch.bfloat16)])
    torch.cuda.synchronize()
    want_f16 = a.float().cpu() @ b.float().cpu()
    want_bf16 = a.view(torch.bfloat16).float().cpu() @ b.view(torch.bfloat16).float().cpu()
    assert_parity(as_f16, want_f16, F16, "float16 reading")
    assert_parity(as_bf16, want_bf16, torch.bfloat16, "bfloat16 reading")


def test_f16_overflow_rounds_to_infinity_like_torch():
    from cubework_amd import ops

    a = torch.full((128, 64), 60.0, dtype=F16, device=DEV)
    b = torch.full((64, 128), 60.0, dtype=F16, device=DEV)          # 64 * 3600 = 230400 > 65504
    got = ops.gemm_ksteps("NN", [a], [b])
    torch.cuda.synchronize()
    assert torch.isinf(got).all() and (got > 0).all()
    assert torch.equal(got.cpu(), (a.float().cpu() @ b.float().cpu()).to(F16))


@pytest.mark.parametrize("shape", [(8192, 2048), (100, 1000), (5, 7), (1000, 520)])
def test_f16_colsum_and_act_bwd(shape):
    import oracle
    from cubework_amd import ops

    M, N = shape
    dy = randn((M, N), F16, 1)
    got = ops.colsum(dy.to(DEV))
    with oracle.precision(torch.float64):
        want = oracle.colsum(dy)
    assert_parity(got, want, torch.float32, "colsum")
    pre = randn((M, N), F16, 3, std=1.5)
    for act in ("gelu_tanh", "relu"):
        dpre, dbias = ops.act_bwd_colsum(act, dy.to(DEV), pre.to(DEV))
        with oracle.precision(torch.float64):
            want_dpre, want_dbias = oracle.act_bwd_colsum(act, dy, pre)
        assert_parity(dpre, want_dpre, F16, "dPre %s" % act)
        assert_parity(dbias, want_dbias, torch.float32, "dbias %s" % act)


def test_half_model_layernorm():
    """model.half() without autocast: nothing casts, so the reference's LayerNorm Functions receive float16
    (custom_fwd casts only inside an autocast region). The kernels read float16, compute in fp32 and write
    float16; against F.layer_norm in fp32 on the same values."""
    from cubework_amd import module as cube_nn
    from cubework_amd.distributed import initialize

    initialize("2d", 1)
    torch.manual_seed(0)
    ln = cube_nn.LayerNorm(768, dtype=F16).to(DEV)
    with torch.no_grad():
        ln.weight.copy_(rand_uniform((768,), F16, 2, 0.9, 1.1))
        ln.bias.copy_(randn((768,), F16, 3, std=0.02))
    x = randn((4, 33, 768), F16, 4).to(DEV).requires_grad_(True)
    dy = randn((4, 33, 768), F16, 5).to(DEV)
    y = ln(x)
    assert y.dtype == F16
    y.backward(dy)
    xr = x.detach().float().requires_grad_(True)
    wr = ln.weight.detach().float().requires_grad_(True)
    br = ln.bias.detach().float().requires_grad_(True)
    torch.nn.functional.layer_norm(xr, (768,), wr, br, 1e-5).backward(dy.float())
    assert_parity(y, torch.nn.functional.layer_norm(xr, (768,), wr, br, 1e-5).detach().to(F16), F16, "y")
    assert_parity(x.grad, xr.grad.to(F16), F16, "dx")
    assert_parity(ln.weight.grad, wr.grad.to(F16), F16, "dgamma")
    assert_parity(ln.bias.grad, br.grad.to(F16), F16, "dbeta")


@pytest.mark.parametrize("amp_dtype", [torch.float16, torch.bfloat16])
def test_linear2d_under_autocast(amp_dtype):
    """fp32 parameters and activations inside torch.autocast: the GEMM-type Functions cast to the autocast
    dtype (float16 by default, as the reference's custom_fwd does), the gradients come back in fp32."""
    import oracle
    from cubework_amd import module as cube_nn
    from cubework_amd.distributed import initialize

    initialize("2d", 1)
    torch.manual_seed(0)
    lin = cube_nn.Linear(256, 384).to(DEV)
    x = randn((4, 64, 256), torch.float32, 5).to(DEV).requires_grad_(True)
    with torch.autocast("cuda", dtype=amp_dtype):
        y = lin(x)
    assert y.dtype == amp_dtype
    w, b = lin.weight.detach().cpu(), lin.bias.detach().cpu()
    xh, wh = x.detach().cpu().to(amp_dtype), w.to(amp_dtype)
    want = oracle.gemm_ksteps("NN", [xh.reshape(-1, 256)], [wh], b.to(amp_dtype), None)
    assert_parity(y.reshape(-1, 384), want, amp_dtype, "Linear2D under autocast(%s)" % amp_dtype)
    dy = randn((4, 64, 384), torch.float32, 6).to(DEV)
    y.backward(dy.to(amp_dtype))
    assert x.grad.dtype == torch.float32 and lin.weight.grad.dtype == torch.float32
    dyh = dy.cpu().to(amp_dtype).float().reshape(-1, 384)
    assert_parity(x.grad.reshape(-1, 256), (dyh @ wh.float().t()).to(amp_dtype).float(), amp_dtype, "dX")
    assert_parity(lin.weight.grad, (xh.float().reshape(-1, 256).t() @ dyh).to(amp_dtype).float(), amp_dtype, "dW")
    assert_parity(lin.bias.grad, dyh.sum(0), amp_dtype, "dbias")
