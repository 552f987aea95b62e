"""CPU oracle: a restatement, in plain torch on the CPU, of the per-rank math of
Cubework's tensor-parallel layers (reference tree: kurisusnowdeng/Cubework).

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT A COMPUTE PATH. Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import it, and
only as the checker. The product (cubework_amd) never imports it and has no
CPU fallback.

Why torch and not C: the reference has no native code; every operation on the
path is a stock torch op (torch.addmm, torch.matmul, F.linear, torch.sum,
torch.exp, advanced indexing) and the reference's own tests compare against
single-device torch. The oracle therefore follows the reference's statements
line by line in torch, and is pinned by
  * brute-force float64 golden vectors (tests/golden/, pure-Python loops),
  * torch library routines the reference's tests use as their own oracle
    (A @ W + b, nn.LayerNorm, F.cross_entropy),
  * for the attention core: pure-Python float64 loops, F.scaled_dot_product_attention and its autograd,
  * for the OPT decoder layer: the composition of the functions above, its residual paths (identity with
    zeroed branch outputs), causality, and the agreement of both weight orientations,
  * invariants (split-invariance of statistics, sum of softmax gradient = 0,
    k-step sum == concatenated GEMM, grid composition == master result).
Parity status: every function below is pinned by at least one such check in
tests/test_oracle_*.py; none is "parity unpinned". Initial parameter values
drawn under the reference's per-rank RNG fork are deliberately not restated.

Precision convention for bf16 inputs: evaluate the reference formulas in fp32
(float64 where noted) on the bf16-rounded inputs and round the result once.
"""
from ._precision import precision, compute_dtype  # noqa: F401
from .summa import (gemm_ksteps, summa_ab_rank, summa_abt_rank, summa_atb_rank, summa_ab_reference_dtype,  # noqa: F401
                    activation, activation_grad, act_bwd_colsum, colsum)
from .layernorm import (ln2d_partial_stats, ln2d_mean_rstd, ln2d_normalize, ln2d_backward_partials, ln2d_backward_dx,  # noqa: F401
                        ln3d_forward, ln3d_backward, ln_forward_full, ln_backward_full)
from .vpce import vpce_fwd_local, vpce_finalize, vpce_bwd, vpce_reference_full  # noqa: F401
from .attention import split_qkv, attention_core, attention_core_backward, attention_brute_force  # noqa: F401
from .embedding import vocab_embedding_fwd, vocab_embedding_bwd  # noqa: F401
from .clip_grad import clip_grad_norm  # noqa: F401
from .opt_block import opt_block_reference  # noqa: F401
from . import grid  # noqa: F401
